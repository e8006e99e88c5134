// A feed-forward that sends every token to a few of many small experts.
//
//   route      per token: router logits (float, computed by a 32-bit product) plus
//              a bias, the `top` largest, and the softmax over those alone.
//   sort       the (token, choice) pairs in order of their expert: where each
//              expert's run starts, which pair stands at each place, the place
//              of each pair, and the list of row tiles (expert, first place) the
//              products walk.  One workgroup; the order inside a run is that of
//              the pairs, whatever the timing.  Nothing goes back to the host: the
//              products' grids are sized for the most tiles there can be.
//   product    a tile of one expert's rows times a tile of that expert's matrix,
//              on the matrix cores (through LDS for many rows an expert, straight
//              from memory for few).  GATED: rows are gathered from
//              the step's activations by token, the gate's and the up
//              projection's columns are computed side by side and the epilogue
//              writes  min(g, limit) * sigmoid(alpha * min(g, limit)) * (clamp(u, -limit, limit) + 1).
//              Otherwise rows are read by place and the product is stored.
//   combine    out[t] = addend[t] + shared[t] + sum_k weight[t, k] * y[place(t, k)],
//              in 32-bit, in the order of k.
//
// Every row's sums run over the inner dimension in the same order wherever the
// row stands in its tile, so a token's result does not depend on what else is in
// the batch.
#include <algorithm>

#include "common.h"

namespace lyp {

constexpr int kRouteRegs = 8;            // experts per lane: up to 64 * 8 experts
constexpr int kMostExperts = 64 * kRouteRegs;
constexpr int kMostTop = 32;

// One wave chooses for one row: z points at the row's E logits (bias not yet added).
// `always` >= 0: one more pair is written after the chosen ones, expert `always` with weight 1 (an
// expert every token uses, kept as one more matrix behind the routed ones).
// `parts` > 1: the logits are the sum of that many partial sums, `part_stride` floats apart.
__device__ __forceinline__ void route_row(const float* z, const float* __restrict__ bias, int E, int top,
                                          int32_t* __restrict__ idx, float* __restrict__ wgt, int lane, int always,
                                          int parts = 1, size_t part_stride = 0) {
  float v[kRouteRegs];
#pragma unroll
  for (int r = 0; r < kRouteRegs; ++r) {
    const int e = lane + kWave * r;
    if (e < E) {
      // four partial sums asked for at a time, added in their order
      float sum = 0.f;
      for (int p0 = 0; p0 < parts; p0 += 4) {
        float t[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) t[i] = p0 + i < parts ? z[(p0 + i) * part_stride + e] : 0.f;
#pragma unroll
        for (int i = 0; i < 4; ++i) sum += t[i];
      }
      v[r] = sum + (bias != nullptr ? bias[e] : 0.f);
    } else {
      v[r] = LYP_NEG_INF;
    }
  }
  float chosen_v = 0.f;      // lane k keeps the k-th choice
  int chosen_e = 0;
  for (int k = 0; k < top; ++k) {
    ArgMax best{LYP_NEG_INF, 0x7fffffff};
#pragma unroll
    for (int r = 0; r < kRouteRegs; ++r) best = better(best, ArgMax{v[r], lane + kWave * r});
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      ArgMax o{__shfl_xor(best.v, off, kWave), __shfl_xor(best.i, off, kWave)};
      best = better(best, o);
    }
#pragma unroll
    for (int r = 0; r < kRouteRegs; ++r)
      if (lane + kWave * r == best.i) v[r] = LYP_NEG_INF;
    if (lane == k) {
      chosen_v = best.v;
      chosen_e = best.i;
    }
  }
  const float m = __shfl(chosen_v, 0, kWave);      // the first choice is the largest
  const float p = lane < top ? expf(chosen_v - m) : 0.f;
  const float total = wave_sum(p);
  if (lane < top) {
    idx[lane] = chosen_e;
    wgt[lane] = p / total;
  }
  if (always >= 0 && lane == top) {
    idx[top] = always;
    wgt[top] = 1.0f;
  }
}

// z [rows, E] float logits without bias.  One wave per row.
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ z, const float* __restrict__ bias,
                                                        int rows, int E, int top, int32_t* __restrict__ idx,
                                                        float* __restrict__ wgt, int always, int parts) {
  const int lane = threadIdx.x % kWave;
  const int row = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (row >= rows) return;
  const int per = top + (always >= 0 ? 1 : 0);
  route_row(z + static_cast<size_t>(row) * E, bias, E, top, idx + static_cast<size_t>(row) * per,
            wgt + static_cast<size_t>(row) * per, lane, always, parts, static_cast<size_t>(rows) * E);
}

// The router's product and the choice in one kernel: x [rows, K] in T, the router's matrix
// w [E, K] in float; logits in 32-bit on the float matrix instruction.  A workgroup takes 16 rows;
// its eight waves share the inner dimension (an eighth each, added up in the order of the waves),
// walk the experts in blocks of 16, four blocks a pass, and then choose for two rows each.  A wave
// asks for four steps' operands at once: the kernel is as long as its chain of loads.
constexpr int kRouteBlocks = 4;   // blocks of 16 experts whose sums a wave holds at a time
constexpr int kRouteWaves = 8;
constexpr int kRouteAhead = 4;    // steps of 16 inner values whose loads are in flight together

template <typename T>
__global__ __launch_bounds__(kRouteWaves* kWave) void moe_route_fused_kernel(
    const T* __restrict__ x, int ldx, const float* __restrict__ w, const float* __restrict__ bias, int rows, int E,
    int K, int top, int32_t* __restrict__ idx, float* __restrict__ wgt, int always, int vec_ok,
    float* __restrict__ part) {
  extern __shared__ float s_route[];                 // [waves][kRouteBlocks][64 lanes][4], then z [16][E]
  float* s_part = s_route;
  float* s_z = s_route + kRouteWaves * kRouteBlocks * kWave * 4;
  typedef T XVec __attribute__((ext_vector_type(4)));
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int t0 = blockIdx.x * 16;
  const int r = lane % 16, grp = lane / 16;
  const int row = t0 + r;
  const T* xrow = x + static_cast<size_t>(min(row, rows - 1)) * ldx;
  // this wave's share of the inner dimension, in steps of 16
  // (grid y > 1: the workgroups of a row block share the inner dimension too, each leaves its sums in
  // `part` [y][rows][E], and moe_route_kernel adds them up and chooses)
  const int steps = (K + 15) / 16;
  const int ks = gridDim.y, ky = blockIdx.y;
  const int wg_begin = steps * ky / ks, wg_steps = steps * (ky + 1) / ks - wg_begin;
  const int s_begin = wg_begin + wg_steps * wave / kRouteWaves, s_end = wg_begin + wg_steps * (wave + 1) / kRouteWaves;
  const int e_blocks = (E + 15) / 16;
  auto load_x = [&](int st) {
    const int k = st * 16 + grp * 4;
    f32x4 xf = f32x4{0.f, 0.f, 0.f, 0.f};
    if (row < rows) {
      if (vec_ok && k + 4 <= K) {
        const XVec v = *reinterpret_cast<const XVec*>(xrow + k);
#pragma unroll
        for (int i = 0; i < 4; ++i) xf[i] = to_f32(v[i]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (k + i < K) xf[i] = to_f32(xrow[k + i]);
      }
    }
    return xf;
  };
  auto load_w = [&](int st, int eb) {
    const int k = st * 16 + grp * 4;
    const int e = eb * 16 + r;
    f32x4 wf = f32x4{0.f, 0.f, 0.f, 0.f};
    if (e < E) {
      const float* wrow = w + static_cast<size_t>(e) * K;
      if (vec_ok && k + 4 <= K) {
        wf = *reinterpret_cast<const f32x4*>(wrow + k);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (k + i < K) wf[i] = wrow[k + i];
      }
    }
    return wf;
  };
  for (int eb0 = 0; eb0 < e_blocks; eb0 += kRouteBlocks) {
    f32x4 acc[kRouteBlocks];
#pragma unroll
    for (int b = 0; b < kRouteBlocks; ++b) acc[b] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int st0 = s_begin; st0 < s_end; st0 += kRouteAhead) {
      f32x4 xf[kRouteAhead], wf[kRouteAhead][kRouteBlocks];
#pragma unroll
      for (int a = 0; a < kRouteAhead; ++a) {
        const int st = st0 + a;
        xf[a] = st < s_end ? load_x(st) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int b = 0; b < kRouteBlocks; ++b)
          wf[a][b] = (st < s_end && eb0 + b < e_blocks) ? load_w(st, eb0 + b) : f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int a = 0; a < kRouteAhead; ++a)
#pragma unroll
        for (int b = 0; b < kRouteBlocks; ++b)
          acc[b] = Mma16<float>::mma(wf[a][b], xf[a], acc[b]);   // acc[i]: row l % 16, the block's expert 4 * (l / 16) + i
    }
#pragma unroll
    for (int b = 0; b < kRouteBlocks; ++b)
      *reinterpret_cast<f32x4*>(&s_part[((wave * kRouteBlocks + b) * kWave + lane) * 4]) = acc[b];
    __syncthreads();
    // the waves' shares added up in their order; thread -> (block, lane)
    for (int p = threadIdx.x; p < kRouteBlocks * kWave; p += kRouteWaves * kWave) {
      const int b = p / kWave, l = p % kWave;
      if (eb0 + b >= e_blocks) continue;
      f32x4 sum = *reinterpret_cast<const f32x4*>(&s_part[(b * kWave + l) * 4]);
#pragma unroll
      for (int wv = 1; wv < kRouteWaves; ++wv) {
        const f32x4 o = *reinterpret_cast<const f32x4*>(&s_part[((wv * kRouteBlocks + b) * kWave + l) * 4]);
#pragma unroll
        for (int i = 0; i < 4; ++i) sum[i] += o[i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = (eb0 + b) * 16 + 4 * (l / 16) + i;
        if (e < E) s_z[(l % 16) * E + e] = sum[i];
      }
    }
    __syncthreads();
  }
  if (ks > 1) {
    for (int i = threadIdx.x; i < 16 * E; i += kRouteWaves * kWave) {
      const int rr = t0 + i / E;
      if (rr < rows) part[(static_cast<size_t>(ky) * rows + rr) * E + i % E] = s_z[i];
    }
    return;
  }
  const int per = top + (always >= 0 ? 1 : 0);
  for (int q = wave; q < 16; q += kRouteWaves) {
    const int rr = t0 + q;
    if (rr >= rows) break;
    route_row(s_z + q * E, bias, E, top, idx + static_cast<size_t>(rr) * per, wgt + static_cast<size_t>(rr) * per, lane,
              always);
  }
}

// The lanes of the wave that hold the same value as this one, as a mask: one ballot per bit of the
// values (`bits` of them) instead of one look at every lane.
__device__ __forceinline__ unsigned long long wave_same(int v, int bits) {
  unsigned long long mask = ~0ull;
  for (int b = 0; b < bits; ++b) {
    const unsigned long long set = __builtin_amdgcn_ballot_w64(((v >> b) & 1) != 0);
    mask &= ((v >> b) & 1) ? set : ~set;
  }
  return mask;
}

constexpr int kSortThreads = 1024;
constexpr int kSortWaves = kSortThreads / kWave;

// What the sort may do first, for steps of few rows (one kernel less): add up the router's partial
// sums and choose, as moe_route_kernel does, a wave a row.
struct RouteFirst {
  const float* part;     // nullptr: the choices are there already
  const float* bias;
  float* wgt;
  int parts, rows, experts, top, always;
};

__global__ __launch_bounds__(kSortThreads) void moe_sort_kernel(
    int32_t* __restrict__ idx, int P, int E, int tile_rows, int32_t* __restrict__ expert_off,
    int32_t* __restrict__ sorted_pair, int32_t* __restrict__ place_of, int32_t* __restrict__ tile_expert,
    int32_t* __restrict__ tile_row0, int32_t* __restrict__ n_tiles, RouteFirst first) {
  extern __shared__ int32_t s_sort[];
  int32_t* cnt = s_sort;               // [E]
  int32_t* base = cnt + E;             // [E]
  int32_t* tbase = base + E;           // [E + 1]
  int32_t* wcnt = tbase + E + 1;       // [kSortWaves][E]
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  int bits = 1;                       // bits that tell the experts (and -1) apart
  while ((1 << bits) <= E) ++bits;
  if (first.part != nullptr) {
    const int per = first.top + (first.always >= 0 ? 1 : 0);
    for (int row = wave; row < first.rows; row += kSortWaves)
      route_row(first.part + static_cast<size_t>(row) * first.experts, first.bias, first.experts, first.top,
                idx + static_cast<size_t>(row) * per, first.wgt + static_cast<size_t>(row) * per, lane, first.always,
                first.parts, static_cast<size_t>(first.rows) * first.experts);
    __syncthreads();   // the choices are read back below by other threads of this workgroup
  }
  for (int e = tid; e < E; e += kSortThreads) cnt[e] = 0;
  __syncthreads();
  // counts: a wave first finds out how many of its 64 pairs go to each expert, and one lane per expert
  // adds that to the expert's count (integers: no order to depend on; 64 lanes adding to a few dozen
  // places one by one is what this pass would otherwise wait for)
  for (int p0 = 0; p0 < P; p0 += kSortThreads) {
    const int p = p0 + tid;
    const int e = p < P ? idx[p] : -1;                       // (-1: all bits set, a value no expert has)
    const unsigned long long mates = wave_same(e, bits);
    const bool last = (mates >> lane) == 1ull;               // no later lane holds the same expert
    if (e >= 0 && last) atomicAdd(&cnt[e], __builtin_popcountll(mates));
  }
  __syncthreads();
  if (tid == 0) {
    int run = 0, tiles = 0;
    for (int e = 0; e < E; ++e) {
      base[e] = run;
      tbase[e] = tiles;
      run += cnt[e];
      tiles += (cnt[e] + tile_rows - 1) / tile_rows;
    }
    tbase[E] = tiles;
    n_tiles[0] = tiles;
  }
  __syncthreads();
  for (int e = tid; e <= E; e += kSortThreads) expert_off[e] = e < E ? base[e] : P;
  for (int e = tid; e < E; e += kSortThreads) {
    const int n = tbase[e + 1] - tbase[e];
    for (int i = 0; i < n; ++i) {
      tile_expert[tbase[e] + i] = e;
      tile_row0[tbase[e] + i] = base[e] + i * tile_rows;
    }
  }
  // a thread's experts of the next rounds are asked for ahead, kAhead rounds at a time
  constexpr int kAhead = 8;
  int mine[kAhead];
  for (int p0 = 0; p0 < P; p0 += kSortThreads) {
    const int round = p0 / kSortThreads;
    if (round % kAhead == 0) {
#pragma unroll
      for (int a = 0; a < kAhead; ++a) {
        const int pa = p0 + a * kSortThreads + tid;
        mine[a] = pa < P ? idx[pa] : -1;
      }
    }
    __syncthreads();
    for (int i = tid; i < kSortWaves * E; i += kSortThreads) wcnt[i] = 0;
    __syncthreads();
    const int p = p0 + tid;
    int e = -1;
#pragma unroll
    for (int a = 0; a < kAhead; ++a)
      if (round % kAhead == a) e = mine[a];
    const unsigned long long mates = wave_same(e, bits);
    const int rank = __builtin_popcountll(mates & ((1ull << lane) - 1ull));   // earlier lanes with the same expert
    const bool last = (mates >> lane) == 1ull;
    if (e >= 0 && last) wcnt[wave * E + e] = rank + 1;
    __syncthreads();
    if (e >= 0) {
      int at = base[e] + rank;
      for (int w = 0; w < wave; ++w) at += wcnt[w * E + e];
      sorted_pair[at] = p;
      place_of[p] = at;
    }
    __syncthreads();
    for (int x = tid; x < E; x += kSortThreads) {
      int add = 0;
      for (int w = 0; w < kSortWaves; ++w) add += wcnt[w * E + x];
      base[x] += add;
    }
  }
}

// ------------------------------------------------------- choice within groups
// Sigmoid scores s = sigmoid(x W^T) in 32-bit; the choice goes by s + correction, the weights by s
// alone.  The experts form n_groups equal groups of neighbours; a group's score is the sum of its
// two largest choice scores (its one score when a group is one expert), and only experts of the
// `keep` best groups can be chosen.  The `top` largest choice scores among those are taken (of
// equal ones the first); their weights are s over the sum of the chosen s (+ 1e-20), times scale.
// A wave forms a row's product with a block of experts at a time (the block's loads all in flight,
// the lanes sharing the inner dimension in a fixed order that does not depend on the launch); a
// workgroup's four waves take four rows, or, when the step has few rows, share one row's experts.
// Then one wave per row chooses: group scores a lane each, maxima over the wave.
constexpr int kGroupedRows = 4;   // waves a workgroup
constexpr int kRouteBlock = 8;    // experts whose products a wave forms side by side

template <typename T>
__device__ __forceinline__ f32x4 route_load4(const T* p);
template <>
__device__ __forceinline__ f32x4 route_load4<float>(const float* p) {
  return *reinterpret_cast<const f32x4*>(p);
}
template <>
__device__ __forceinline__ f32x4 route_load4<bf16_t>(const bf16_t* p) {
  const bf16x4 v = *reinterpret_cast<const bf16x4*>(p);
  return f32x4{static_cast<float>(v[0]), static_cast<float>(v[1]), static_cast<float>(v[2]), static_cast<float>(v[3])};
}

__device__ __forceinline__ ArgMax wave_argmax(ArgMax m) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    ArgMax o;
    o.v = __shfl_xor(m.v, off, kWave);
    o.i = __shfl_xor(m.i, off, kWave);
    m = better(m, o);
  }
  return m;
}

// One wave chooses for a row: c [E] choice scores (set to minus infinity as experts are chosen), sc [E] plain scores, both in LDS.
__device__ __forceinline__ void choose_grouped(float* c, const float* sc, int lane, int row, int E, int top, int n_groups,
                                               int keep, float scale, int32_t* __restrict__ idx, float* __restrict__ wgt) {
  const int per = E / n_groups;
  // a lane a group: the sum of its two largest choice scores (its one score for a group of one)
  float gs = LYP_NEG_INF;
  if (lane < n_groups) {
    float a = LYP_NEG_INF, b = LYP_NEG_INF;
    for (int i = 0; i < per; ++i) {
      const float v = c[lane * per + i];
      if (v > a) {
        b = a;
        a = v;
      } else if (v > b) {
        b = v;
      }
    }
    gs = per > 1 ? a + b : a;
  }
  unsigned long long kept = 0ull;
  bool mine_taken = lane >= n_groups;
  for (int n = 0; n < keep; ++n) {
    ArgMax m{mine_taken ? LYP_NEG_INF : gs, mine_taken ? 0x7fffffff : lane};
    m = wave_argmax(m);
    kept |= 1ull << m.i;
    if (lane == m.i) mine_taken = true;
  }
  float total = 0.f;
  int chosen = 0;   // lane n keeps the n-th choice
  for (int n = 0; n < top; ++n) {
    ArgMax m{LYP_NEG_INF, 0x7fffffff};
    for (int e = lane; e < E; e += kWave)
      if ((kept >> (e / per)) & 1ull) m = better(m, ArgMax{c[e], e});
    m = wave_argmax(m);
    if (lane == n) chosen = m.i;
    if (lane == 0) c[m.i] = LYP_NEG_INF;
    total += sc[m.i];
    // the wave's lanes run together: the store above is seen by the next round's reads
    __builtin_amdgcn_wave_barrier();
  }
  if (lane < top) {
    idx[static_cast<size_t>(row) * top + lane] = chosen;
    wgt[static_cast<size_t>(row) * top + lane] = sc[chosen] / (total + 1e-20f) * scale;
  }
}

template <typename T>
__global__ __launch_bounds__(kGroupedRows* kWave) void moe_route_grouped_kernel(
    const T* __restrict__ x, int ldx, const float* __restrict__ w, const float* __restrict__ correction, int rows, int E,
    int K, int top, int n_groups, int keep, float scale, int32_t* __restrict__ idx, float* __restrict__ wgt, int rpb,
    int vec_ok) {
  __shared__ float s_score[kGroupedRows][kMostExperts];    // s
  __shared__ float s_choice[kGroupedRows][kMostExperts];   // s + correction; minus infinity once chosen
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int slot = wave % rpb, share = wave / rpb, shares = kGroupedRows / rpb;
  const int row = blockIdx.x * rpb + slot;
  if (row < rows) {
    const T* xr = x + static_cast<size_t>(row) * ldx;
    for (int e0 = share * kRouteBlock; e0 < E; e0 += shares * kRouteBlock) {
      float acc[kRouteBlock];
      const float* we[kRouteBlock];
#pragma unroll
      for (int j = 0; j < kRouteBlock; ++j) {
        acc[j] = 0.f;
        we[j] = w + static_cast<size_t>(min(e0 + j, E - 1)) * K;   // past the last expert: worked out, not kept
      }
      if (vec_ok) {
        // four steps of the inner dimension at a time, their loads all issued before the first is used
        constexpr int U = 4;
        for (int k0 = lane * 4; k0 < K; k0 += kWave * 4 * U) {
          f32x4 xv[U], wv[U][kRouteBlock];
#pragma unroll
          for (int u = 0; u < U; ++u) {
            const int k = k0 + u * kWave * 4;
            const bool in = k < K;
            xv[u] = in ? route_load4<T>(xr + k) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int j = 0; j < kRouteBlock; ++j)
              wv[u][j] = in ? *reinterpret_cast<const f32x4*>(we[j] + k) : f32x4{0.f, 0.f, 0.f, 0.f};
          }
#pragma unroll
          for (int u = 0; u < U; ++u) {
#pragma unroll
            for (int j = 0; j < kRouteBlock; ++j)
              acc[j] += xv[u][0] * wv[u][j][0] + xv[u][1] * wv[u][j][1] + xv[u][2] * wv[u][j][2] + xv[u][3] * wv[u][j][3];
          }
        }
      } else {
        for (int k = lane; k < K; k += kWave) {
          const float xv = to_f32(xr[k]);
#pragma unroll
          for (int j = 0; j < kRouteBlock; ++j) acc[j] += xv * we[j][k];
        }
      }
#pragma unroll
      for (int j = 0; j < kRouteBlock; ++j) {
        const float sum = wave_sum(acc[j]);
        if (lane == 0 && e0 + j < E) {
          const float sg = 1.0f / (1.0f + expf(-sum));
          s_score[slot][e0 + j] = sg;
          s_choice[slot][e0 + j] = sg + (correction != nullptr ? correction[e0 + j] : 0.f);
        }
      }
    }
  }
  __syncthreads();
  if (share != 0 || row >= rows) return;
  choose_grouped(s_choice[slot], s_score[slot], lane, row, E, top, n_groups, keep, scale, idx, wgt);
}

// The choice alone, from logits that the router's product kernel left as partial sums `part` [parts][rows][E]
// (added up here in their order): a wave a row.
__global__ __launch_bounds__(kGroupedRows* kWave) void moe_choose_grouped_kernel(
    const float* __restrict__ part, int parts, const float* __restrict__ correction, int rows, int E, int top,
    int n_groups, int keep, float scale, int32_t* __restrict__ idx, float* __restrict__ wgt) {
  __shared__ float s_score[kGroupedRows][kMostExperts];
  __shared__ float s_choice[kGroupedRows][kMostExperts];
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int row = blockIdx.x * kGroupedRows + wave;
  if (row >= rows) return;
  for (int e = lane; e < E; e += kWave) {
    float z = part[static_cast<size_t>(row) * E + e];
    for (int p = 1; p < parts; ++p) z += part[(static_cast<size_t>(p) * rows + row) * E + e];
    const float sg = 1.0f / (1.0f + expf(-z));
    s_score[wave][e] = sg;
    s_choice[wave][e] = sg + (correction != nullptr ? correction[e] : 0.f);
  }
  __builtin_amdgcn_wave_barrier();
  choose_grouped(s_choice[wave], s_score[wave], lane, row, E, top, n_groups, keep, scale, idx, wgt);
}


// ------------------------------------------------------------------- product
// Two kernels: tiles of up to 16 rows for experts that see few rows (moe_gemm_few_kernel), tiles of
// 128 rows through LDS on the 32x32 instruction for experts that see many (moe_gemm_wide_kernel).
// Both read a row's operands over the inner dimension in a fixed order, whatever the row's place.
//
// Launches of few tiles (a decode step: a handful of pairs, each expert's matrix read for one or two
// rows).  A workgroup takes a tile of up to 16 rows and only 16 output columns
// (GATED: 16 gate rows and their 16 up rows of the matrix), so that there are many workgroups to pull
// the matrices through; its four waves share the inner dimension, step by step in turn, take their
// operands straight from memory into the matrix instruction's registers, four steps' loads in flight,
// and add their sums up through LDS in the order of the waves.
constexpr int kFewAhead = 4;
// what a product without a gate may do besides: take its rows by token (as a gated one does) and square
// the positive part of its result
enum MoeFlags : int { kMoeGather = 1, kMoeRelu2 = 2 };

template <typename T, bool GATED>
__global__ __launch_bounds__(256) void moe_gemm_few_kernel(
    const T* __restrict__ a, int lda, const T* __restrict__ w, long long w_expert_stride, int ldw,
    T* __restrict__ out, int ldo, const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_row0,
    const int32_t* __restrict__ n_tiles, const int32_t* __restrict__ expert_off,
    const int32_t* __restrict__ sorted_pair, int top, int N, int K, int up_offset, float limit, float alpha,
    int vec_ok, int flags) {
  using MW = Mma16Wide<T>;
  constexpr int KE = MW::kElems, STEP = 4 * KE;
  __shared__ float s_red[4][2][kWave][4];
  const int tile = blockIdx.x;
  if (tile >= n_tiles[0]) return;
  const int e = tile_expert[tile];
  const int row0 = tile_row0[tile];
  const int row_end = expert_off[e + 1];
  const int c0 = blockIdx.y * 16;
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int r = lane % 16, grp = lane / 16;
  const T* we = w + static_cast<size_t>(e) * w_expert_stride;
  const int place = row0 + r;
  const T* x_row = nullptr;
  if (place < row_end) x_row = a + static_cast<size_t>((GATED || (flags & kMoeGather)) ? sorted_pair[place] / top : place) * lda;
  const int col = c0 + r;
  const T* g_row = col < N ? we + static_cast<size_t>(col) * ldw : nullptr;
  const T* u_row = GATED && col < N ? we + static_cast<size_t>(col + up_offset) * ldw : nullptr;
  auto fetch = [&](const T* src, int k) {
    typename MW::Frag f;
#pragma unroll
    for (int i = 0; i < KE; ++i) f[i] = from_f32<T>(0.f);
    if (src != nullptr) {
      if (vec_ok && k + KE <= K) {
        f = *reinterpret_cast<const typename MW::Frag*>(src + k);
      } else {
#pragma unroll
        for (int i = 0; i < KE; ++i)
          if (k + i < K) f[i] = src[k + i];
      }
    }
    return f;
  };
  f32x4 acc_g = f32x4{0.f, 0.f, 0.f, 0.f}, acc_u = f32x4{0.f, 0.f, 0.f, 0.f};
  const int steps = (K + STEP - 1) / STEP;
  for (int s0 = wave; s0 < steps; s0 += 4 * kFewAhead) {
    typename MW::Frag xf[kFewAhead], gf[kFewAhead], uf[kFewAhead];
#pragma unroll
    for (int t = 0; t < kFewAhead; ++t) {
      const int k = (s0 + 4 * t) * STEP + grp * KE;      // beyond K: zeros
      xf[t] = fetch(x_row, k);
      gf[t] = fetch(g_row, k);
      if constexpr (GATED) uf[t] = fetch(u_row, k);
    }
#pragma unroll
    for (int t = 0; t < kFewAhead; ++t) {
      acc_g = MW::mma(gf[t], xf[t], acc_g);
      if constexpr (GATED) acc_u = MW::mma(uf[t], xf[t], acc_u);
    }
  }
  *reinterpret_cast<f32x4*>(&s_red[wave][0][lane][0]) = acc_g;
  if constexpr (GATED) *reinterpret_cast<f32x4*>(&s_red[wave][1][lane][0]) = acc_u;
  __syncthreads();
  if (wave != 0 || place >= row_end) return;
  // lane l: token row l % 16, features c0 + 4 * (l / 16) + {0..3}
  T* orow = out + static_cast<size_t>(place) * ldo;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = c0 + 4 * grp + i;
    if (c >= N) continue;
    float y = s_red[0][0][lane][i] + s_red[1][0][lane][i] + s_red[2][0][lane][i] + s_red[3][0][lane][i];
    if constexpr (GATED) {
      const float up = s_red[0][1][lane][i] + s_red[1][1][lane][i] + s_red[2][1][lane][i] + s_red[3][1][lane][i];
      const float g = fminf(y, limit);
      const float u = fminf(fmaxf(up, -limit), limit);
      y = g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
    } else if (flags & kMoeRelu2) {
      y = fmaxf(y, 0.f);
      y *= y;
    }
    orow[c] = from_f32<T>(y);
  }
}

template <typename T, int NW>
struct MoeWide {
  static constexpr int kKT = 128 / sizeof(T);
  static constexpr int kLD = kKT + (sizeof(T) == 2 ? 8 : 4);
  static constexpr int kBRows = 128;                                 // matrix rows a tile
  static constexpr int kBytes = 2 * (128 + kBRows) * kLD * sizeof(T);   // both buffers
};

// Many rows an expert: tiles of 128 rows and 128 matrix rows (GATED: 64 gate
// columns and their 64 up columns) on the 32x32 instruction.  NW = 4 waves in 2 x 2: a wave takes two
// blocks of 32 rows x two blocks of 32 matrix rows, so that a fragment read from LDS feeds two
// products.  NW = 8 waves in 4 x 2: a wave takes one block of rows x two blocks of matrix rows: half
// the sums a wave, twice the waves a compute unit to fill each other's waits.
template <typename T, bool GATED, int NW>
__global__ __launch_bounds__(NW * 64) void moe_gemm_wide_kernel(
    const T* __restrict__ a, int lda, const T* __restrict__ w, long long w_expert_stride, int ldw,
    T* __restrict__ out, int ldo, const int32_t* __restrict__ tile_expert, const int32_t* __restrict__ tile_row0,
    const int32_t* __restrict__ n_tiles, const int32_t* __restrict__ expert_off,
    const int32_t* __restrict__ sorted_pair, int top, int N, int K, int up_offset, float limit, float alpha,
    int vec_ok, int flags) {
  using MW = Mma32<T>;
  constexpr int VEC = 16 / sizeof(T);
  constexpr int KT = MoeWide<T, NW>::kKT;             // inner values a round: 128 bytes of every row
  constexpr int LD = MoeWide<T, NW>::kLD;
  constexpr int TM = 128, BROWS = MoeWide<T, NW>::kBRows, THREADS = NW * 64;
  constexpr int TN = GATED ? BROWS / 2 : BROWS;       // output columns a workgroup
  constexpr int STEPS = KT / (2 * MW::kElems);
  constexpr int A_PER = TM * KT / VEC / THREADS;      // 16-byte pieces of the two tiles per thread
  constexpr int B_PER = BROWS * KT / VEC / THREADS;
  typedef T VecT __attribute__((ext_vector_type(VEC)));
  extern __shared__ __attribute__((aligned(16))) unsigned char s_wide[];   // two buffers of (A tile, B tile)
  auto a_tile = [&](int buf) { return reinterpret_cast<T*>(s_wide) + buf * (TM + BROWS) * LD; };
  auto b_tile = [&](int buf) { return a_tile(buf) + TM * LD; };

  // Which (row tile, column tile) this workgroup takes.  Workgroups go to the chip's eight dies in
  // turn by their number, and a die has a second-level cache of its own: every die gets one stretch of
  // the work in the order (column tile, row tile), so that the row tiles of one expert, which read the
  // same piece of its matrix, run on one die one after the other and the piece comes from memory once.
  constexpr int kDies = 8;
  const int total = gridDim.x * gridDim.y;
  const int number = blockIdx.x + gridDim.x * blockIdx.y;
  const int die = number % kDies;   // die d gets the numbers d, d + 8, ...: total / 8 of them, one more for the first total % 8
  const int work = die * (total / kDies) + min(die, total % kDies) + number / kDies;
  const int tile = work % static_cast<int>(gridDim.x);
  if (tile >= n_tiles[0]) return;
  const int e = tile_expert[tile];
  const int row0 = tile_row0[tile];
  const int row_end = expert_off[e + 1];
  const int c0 = (work / static_cast<int>(gridDim.x)) * TN;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  constexpr int RB = 8 / NW;           // blocks of 32 rows a wave: 2 or 1
  constexpr int WM = 4 / RB;           // waves side by side over the tile's rows
  const int wm = wave % WM, wn = wave / WM;
  // this wave's blocks of 32 rows: wm (and wm + 2), so that a tile whose last rows are missing
  // (an expert's tail) leaves every wave with less to do, not some with nothing
  const int rb[2] = {wm, wm + WM};
  const bool rb_live[2] = {row0 + rb[0] * 32 < row_end, RB > 1 && row0 + rb[1] * 32 < row_end};
  const T* we = w + static_cast<size_t>(e) * w_expert_stride;

  const T* a_src[A_PER];
  const T* b_src[B_PER];
  int a_k[A_PER], a_lds[A_PER], b_k[B_PER], b_lds[B_PER];
#pragma unroll
  for (int n = 0; n < A_PER; ++n) {
    const int v = tid + n * THREADS;
    const int r = v / (KT / VEC), kc = (v % (KT / VEC)) * VEC;
    a_k[n] = kc;
    a_lds[n] = r * LD + kc;
    a_src[n] = nullptr;
    if (row0 + r < row_end) {
      const int place = row0 + r;
      a_src[n] = a + static_cast<size_t>((GATED || (flags & kMoeGather)) ? sorted_pair[place] / top : place) * lda;
    }
  }
#pragma unroll
  for (int n = 0; n < B_PER; ++n) {
    const int v = tid + n * THREADS;
    const int r = v / (KT / VEC), kc = (v % (KT / VEC)) * VEC;
    b_k[n] = kc;
    b_lds[n] = r * LD + kc;
    // matrix rows of the tile: GATED: the gate rows, then the up rows that go with them
    const int col = GATED ? c0 + r % (BROWS / 2) : c0 + r;
    b_src[n] = col < N ? we + static_cast<size_t>(col + (GATED && r >= BROWS / 2 ? up_offset : 0)) * ldw : nullptr;
  }
  auto fetch = [&](const T* src, int k) {
    VecT x;
#pragma unroll
    for (int i = 0; i < VEC; ++i) x[i] = from_f32<T>(0.f);
    if (src != nullptr) {
      if (vec_ok && k + VEC <= K) {
        x = *reinterpret_cast<const VecT*>(src + k);
      } else {
#pragma unroll
        for (int i = 0; i < VEC; ++i)
          if (k + i < K) x[i] = src[k + i];
      }
    }
    return x;
  };
  // Two sets of registers: while round r is computed from LDS, round r + 1 waits in one set and round
  // r + 2 is on its way from memory into the other (the kernel's speed is what it has in flight).
  struct Regs {
    VecT a[A_PER], b[B_PER];
  };
  auto load = [&](Regs& rg, int k0) {
#pragma unroll
    for (int n = 0; n < A_PER; ++n) rg.a[n] = fetch(a_src[n], k0 + a_k[n]);
#pragma unroll
    for (int n = 0; n < B_PER; ++n) rg.b[n] = fetch(b_src[n], k0 + b_k[n]);
  };
  auto stash = [&](const Regs& rg, int buf) {
#pragma unroll
    for (int n = 0; n < A_PER; ++n) *reinterpret_cast<VecT*>(a_tile(buf) + a_lds[n]) = rg.a[n];
#pragma unroll
    for (int n = 0; n < B_PER; ++n) *reinterpret_cast<VecT*>(b_tile(buf) + b_lds[n]) = rg.b[n];
  };
  // this wave: row blocks rb[0], rb[1]; matrix-row blocks fb[0], fb[1] of the tile
  const int fb[2] = {GATED ? wn * 32 : wn * 64, GATED ? BROWS / 2 + wn * 32 : wn * 64 + 32};
  f32x16 acc[RB][2];
#pragma unroll
  for (int i = 0; i < RB; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  auto compute = [&](int buf) {
    const T* As = a_tile(buf);
    const T* Bs = b_tile(buf);
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int kk = s * 2 * MW::kElems + (lane / 32) * MW::kElems;
      typename MW::Frag xf[RB], wf[2];
#pragma unroll
      for (int i = 0; i < RB; ++i)
        if (rb_live[i]) xf[i] = *reinterpret_cast<const typename MW::Frag*>(As + (rb[i] * 32 + lane % 32) * LD + kk);
#pragma unroll
      for (int j = 0; j < 2; ++j) wf[j] = *reinterpret_cast<const typename MW::Frag*>(Bs + (fb[j] + lane % 32) * LD + kk);
#pragma unroll
      for (int i = 0; i < RB; ++i) {
        if (!rb_live[i]) continue;
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = MW::mma(wf[j], xf[i], acc[i][j]);
      }
    }
  };
  // one round: LDS buffer `buf` holds round k0; `next` holds round k0 + KT; `far` takes round k0 + 2 KT
  auto round = [&](int k0, int buf, Regs& next, Regs& far) {
    if (k0 + 2 * KT < K) load(far, k0 + 2 * KT);
    compute(buf);
    if (k0 + KT < K) stash(next, buf ^ 1);
    __syncthreads();
  };
  Regs ra, rb2;
  load(ra, 0);
  if (KT < K) load(rb2, KT);
  stash(ra, 0);
  __syncthreads();
  for (int k0 = 0; k0 < K; k0 += 2 * KT) {
    round(k0, 0, rb2, ra);
    if (k0 + KT >= K) break;
    round(k0 + KT, 1, ra, rb2);
  }

  // register v of lane l: matrix row 8 * (v / 4) + 4 * (l / 32) + v % 4 of the block, token l % 32
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    const int place = row0 + rb[i] * 32 + lane % 32;
    if (place >= row_end) continue;
    T* orow = out + static_cast<size_t>(place) * ldo;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int f = 8 * (v / 4) + 4 * (lane / 32) + v % 4;
      if constexpr (GATED) {
        const int col = c0 + wn * 32 + f;
        if (col >= N) continue;
        const float g = fminf(acc[i][0][v], limit);
        const float u = fminf(fmaxf(acc[i][1][v], -limit), limit);
        orow[col] = from_f32<T>(g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
      } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int col = c0 + wn * 64 + j * 32 + f;
          if (col >= N) continue;
          float y = acc[i][j][v];
          if (flags & kMoeRelu2) {
            y = fmaxf(y, 0.f);
            y *= y;
          }
          orow[col] = from_f32<T>(y);
        }
      }
    }
  }
}

// gate_up [rows, 2 I] (gates first) -> out [rows, I], the experts' activation
template <typename T>
__global__ void glu_clamped_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int rows, int I, float limit,
                                   float alpha) {
  const size_t total = static_cast<size_t>(rows) * I;
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t r = i / I, c = i % I;
    const float g = fminf(to_f32(gate_up[r * 2 * I + c]), limit);
    const float u = fminf(fmaxf(to_f32(gate_up[r * 2 * I + I + c]), -limit), limit);
    out[i] = from_f32<T>(g / (1.0f + expf(-alpha * g)) * (u + 1.0f));
  }
}

// out [rows, H] float = addend + shared + sum_k wgt[row, k] * y[place_of[row * top + k]]
// One workgroup a row; the row's places and weights are read once; a thread takes V neighbouring
// columns at a time (V = 4 where rows are whole multiples of that, else 1), two such groups in flight.
template <typename T, int V>
__global__ void moe_combine_kernel(const T* __restrict__ y, const int32_t* __restrict__ place_of,
                                   const float* __restrict__ wgt, int top, const T* __restrict__ addend,
                                   const T* __restrict__ shared, float* __restrict__ out, int rows, int H) {
  __shared__ int32_t s_at[kMostTop];
  __shared__ float s_w[kMostTop];
  typedef T VecT __attribute__((ext_vector_type(V)));
  typedef float VecF __attribute__((ext_vector_type(V)));
  const int row = blockIdx.x;
  if (threadIdx.x < top) {
    s_at[threadIdx.x] = place_of[static_cast<size_t>(row) * top + threadIdx.x];
    s_w[threadIdx.x] = wgt[static_cast<size_t>(row) * top + threadIdx.x];
  }
  __syncthreads();
  constexpr int U = 2;
  const int stride = blockDim.x * V;
  auto get = [&](const T* p) {
    VecF f;
    if constexpr (V == 1) {
      f[0] = to_f32(p[0]);
    } else {
      const VecT v = *reinterpret_cast<const VecT*>(p);
#pragma unroll
      for (int i = 0; i < V; ++i) f[i] = to_f32(v[i]);
    }
    return f;
  };
  for (int c0 = threadIdx.x * V; c0 < H; c0 += U * stride) {
    VecF v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u * stride;
#pragma unroll
      for (int i = 0; i < V; ++i) v[u][i] = 0.f;
      if (c >= H) continue;
      if (addend != nullptr) v[u] += get(addend + static_cast<size_t>(row) * H + c);
      if (shared != nullptr) v[u] += get(shared + static_cast<size_t>(row) * H + c);
    }
    for (int k = 0; k < top; ++k) {
      const size_t base = static_cast<size_t>(s_at[k]) * H;
      const float wk = s_w[k];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = c0 + u * stride;
        if (c < H) v[u] += wk * get(y + base + c);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u * stride;
      if (c >= H) continue;
      if constexpr (V == 1) out[static_cast<size_t>(row) * H + c] = v[u][0];
      else *reinterpret_cast<VecF*>(out + static_cast<size_t>(row) * H + c) = v[u];
    }
  }
}

}  // namespace lyp

using namespace lyp;

extern "C" {

int lyp_moe_most_experts() { return kMostExperts; }

int lyp_moe_route(const float* z, const float* bias, int rows, int E, int top, int32_t* idx, float* wgt, int always,
                  hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && E > 0 && E <= kMostExperts && top > 0 && top <= E && top <= kMostTop,
              "moe_route: %d rows, %d experts (at most %d), %d chosen (at most %d)", rows, E, kMostExperts, top,
              kMostTop);
  if (rows == 0) return 0;
  LYP_REQUIRE(top < kMostTop || always < 0, "moe_route: %d chosen and one more", top);
  moe_route_kernel<<<(rows + 3) / 4, 256, 0, stream>>>(z, bias, rows, E, top, idx, wgt, always, 1);
  LYP_LAUNCH_CHECK("moe_route");
  return 0;
}

// x [rows, K] in the activations' type, w [E, K] float: the router's logits, the choice and the weights.
// How many workgroups had better share a row block's inner dimension (1: none; more need `part`,
// that many * rows * E floats).
// x [rows, K] of dtype (rows ldx apart); w float [E, K]; correction float [E] or null; idx int32 and
// wgt float [rows, top].  n_groups divides E, keep * (E / n_groups) >= top, at most 64 groups.
int lyp_moe_route_grouped(const void* x, int ldx, int dtype, const float* w, const float* correction, int rows, int E,
                          int K, int top, int n_groups, int keep, float scale, int32_t* idx, float* wgt,
                          hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && E > 0 && E <= kMostExperts && K > 0 && ldx >= K && top > 0 && top <= kMostTop,
              "moe_route_grouped: %d rows, %d experts (at most %d), inner size %d, %d chosen (at most %d)", rows, E,
              kMostExperts, K, top, kMostTop);
  LYP_REQUIRE(n_groups >= 1 && n_groups <= 64 && E % n_groups == 0 && keep >= 1 && keep <= n_groups &&
                  keep * (E / n_groups) >= top,
              "moe_route_grouped: %d experts in %d groups of which %d are kept cannot give %d choices", E, n_groups, keep, top);
  if (rows == 0) return 0;
  // few rows: a workgroup's waves share one row's experts, so that the router matrix is pulled through by many
  const int rpb = rows >= 2 * compute_units() ? kGroupedRows : 1;
  const int blocks = (rows + rpb - 1) / rpb;
  const size_t esz = dtype == kF32 ? 4 : 2;
  const int vec_ok = K % 4 == 0 && ldx % 4 == 0 && reinterpret_cast<uintptr_t>(x) % (4 * esz) == 0 &&
                     reinterpret_cast<uintptr_t>(w) % 16 == 0;
  if (dtype == kF32)
    moe_route_grouped_kernel<float><<<blocks, kGroupedRows * kWave, 0, stream>>>(
        static_cast<const float*>(x), ldx, w, correction, rows, E, K, top, n_groups, keep, scale, idx, wgt, rpb, vec_ok);
  else if (dtype == kBF16)
    moe_route_grouped_kernel<bf16_t><<<blocks, kGroupedRows * kWave, 0, stream>>>(
        static_cast<const bf16_t*>(x), ldx, w, correction, rows, E, K, top, n_groups, keep, scale, idx, wgt, rpb, vec_ok);
  else
    LYP_REQUIRE(false, "moe_route_grouped: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("moe_route_grouped");
  return 0;
}

// part float [parts][rows][E]: the router's logits as partial sums; the choice within groups as in lyp_moe_route_grouped.
int lyp_moe_choose_grouped(const float* part, int parts, const float* correction, int rows, int E, int top, int n_groups,
                           int keep, float scale, int32_t* idx, float* wgt, hipStream_t stream) {
  LYP_REQUIRE(part != nullptr && parts >= 1 && rows >= 0 && E > 0 && E <= kMostExperts && top > 0 && top <= kMostTop,
              "moe_choose_grouped: %d parts, %d rows, %d experts (at most %d), %d chosen (at most %d)", parts, rows, E,
              kMostExperts, top, kMostTop);
  LYP_REQUIRE(n_groups >= 1 && n_groups <= 64 && E % n_groups == 0 && keep >= 1 && keep <= n_groups &&
                  keep * (E / n_groups) >= top,
              "moe_choose_grouped: %d experts in %d groups of which %d are kept cannot give %d choices", E, n_groups, keep, top);
  if (rows == 0) return 0;
  moe_choose_grouped_kernel<<<(rows + kGroupedRows - 1) / kGroupedRows, kGroupedRows * kWave, 0, stream>>>(
      part, parts, correction, rows, E, top, n_groups, keep, scale, idx, wgt);
  LYP_LAUNCH_CHECK("moe_choose_grouped");
  return 0;
}

int lyp_moe_route_splits(int rows, int K) {
  const int blocks = (rows + 15) / 16, steps = (K + 15) / 16;
  int ks = compute_units() / std::max(blocks, 1);
  ks = std::min(ks, std::min(16, steps / kRouteWaves));
  return std::max(ks, 1);
}

int lyp_moe_route_fused(const void* x, int ldx, int dtype, const float* w, const float* bias, int rows, int E, int K,
                        int top, int32_t* idx, float* wgt, int always, float* part, int splits, int choose,
                        hipStream_t stream) {
  LYP_REQUIRE(splits >= 1 && (splits == 1 || part != nullptr), "moe_route: %d shares of the inner dimension", splits);
  LYP_REQUIRE(rows >= 0 && E > 0 && E <= kMostExperts && top > 0 && top <= E && top <= kMostTop && K > 0 && ldx >= K,
              "moe_route: %d rows, %d experts (at most %d), %d chosen (at most %d), inner size %d", rows, E,
              kMostExperts, top, kMostTop, K);
  LYP_REQUIRE(top < kMostTop || always < 0, "moe_route: %d chosen and one more", top);
  if (rows == 0) return 0;
  const size_t lds = sizeof(float) * (kRouteWaves * kRouteBlocks * kWave * 4 + 16 * E);
  const dim3 blocks((rows + 15) / 16, splits);
  const int esz = dtype == kF32 ? 4 : 2;
  const int vec_ok = K % 4 == 0 && ldx % 4 == 0 && reinterpret_cast<uintptr_t>(x) % (4 * esz) == 0 &&
                     reinterpret_cast<uintptr_t>(w) % 16 == 0;
  if (dtype == kF32)
    moe_route_fused_kernel<float><<<blocks, kRouteWaves * kWave, lds, stream>>>(
        static_cast<const float*>(x), ldx, w, bias, rows, E, K, top, idx, wgt, always, vec_ok, part);
  else if (dtype == kBF16)
    moe_route_fused_kernel<bf16_t><<<blocks, kRouteWaves * kWave, lds, stream>>>(
        static_cast<const bf16_t*>(x), ldx, w, bias, rows, E, K, top, idx, wgt, always, vec_ok, part);
  else
    LYP_REQUIRE(false, "moe_route: unknown dtype %d", dtype);
  // (choose == 0 with splits > 1: the caller adds the partial sums up and chooses, lyp_moe_route_sort)
  if (splits > 1 && choose)
    moe_route_kernel<<<(rows + 3) / 4, 256, 0, stream>>>(part, bias, rows, E, top, idx, wgt, always, splits);
  LYP_LAUNCH_CHECK("moe_route");
  return 0;
}

// Rows per tile the products had better use for `pairs` pairs over E experts, and the most tiles
// there can then be (the products' grid).
// (from 32 rows an expert on the large tile, half empty as it then is, is ahead of four small ones:
// 512 tokens, 32 experts of 1,536 x 2,048, 4 chosen: 144 / 81 us in tiles of 64 rows, 120 / 73 us so)
int lyp_moe_tile_rows(int pairs, int E) { return pairs >= 32 * E ? 128 : 16; }
int lyp_moe_most_tiles(int pairs, int E, int tile_rows) {
  return (pairs + tile_rows - 1) / tile_rows + std::min(E, pairs);
}

int lyp_moe_sort(const int32_t* idx, int pairs, int E, int tile_rows, int32_t* expert_off, int32_t* sorted_pair,
                 int32_t* place_of, int32_t* tile_expert, int32_t* tile_row0, int32_t* n_tiles, hipStream_t stream) {
  LYP_REQUIRE(pairs >= 0 && E > 0 && E <= kMostExperts && (tile_rows == 16 || tile_rows == 128),
              "moe_sort: %d pairs, %d experts, tiles of %d rows", pairs, E, tile_rows);
  const size_t lds = sizeof(int32_t) * (3 * E + 1 + kSortWaves * E);
  moe_sort_kernel<<<1, kSortThreads, lds, stream>>>(const_cast<int32_t*>(idx), pairs, E, tile_rows, expert_off,
                                                    sorted_pair, place_of, tile_expert, tile_row0, n_tiles,
                                                    RouteFirst{nullptr, nullptr, nullptr, 0, 0, 0, 0, -1});
  LYP_LAUNCH_CHECK("moe_sort");
  return 0;
}

// The same after the choice itself, for few rows: part [parts][rows][experts] are the router's partial
// sums (lyp_moe_route_fused with choose == 0 left them); idx and wgt [rows][top (+ 1)] are written here.
int lyp_moe_route_sort(const float* part, int parts, const float* bias, int rows, int experts, int top, int always,
                       int32_t* idx, float* wgt, int E, int tile_rows, int32_t* expert_off, int32_t* sorted_pair,
                       int32_t* place_of, int32_t* tile_expert, int32_t* tile_row0, int32_t* n_tiles,
                       hipStream_t stream) {
  const int pairs = rows * (top + (always >= 0 ? 1 : 0));
  LYP_REQUIRE(part != nullptr && parts >= 1 && rows > 0 && experts > 0 && experts <= kMostExperts && top > 0 &&
                  top <= experts && top <= kMostTop && (top < kMostTop || always < 0),
              "moe_route_sort: %d rows, %d experts, %d chosen", rows, experts, top);
  LYP_REQUIRE(E >= experts && E <= kMostExperts && (tile_rows == 16 || tile_rows == 128),
              "moe_route_sort: %d matrices, tiles of %d rows", E, tile_rows);
  const size_t lds = sizeof(int32_t) * (3 * E + 1 + kSortWaves * E);
  moe_sort_kernel<<<1, kSortThreads, lds, stream>>>(idx, pairs, E, tile_rows, expert_off, sorted_pair, place_of,
                                                    tile_expert, tile_row0, n_tiles,
                                                    RouteFirst{part, bias, wgt, parts, rows, experts, top, always});
  LYP_LAUNCH_CHECK("moe_route_sort");
  return 0;
}

// gated != 0: a [tokens, K] gathered by token, w [E][2 N rows: gates, then ups][K], out [pairs, N] in the
// operands' type.  gated == 0: a [pairs, K] by place, w [E][N][K], out [pairs, N] in the operands' type;
// flags & 1: a [tokens, K] gathered by token instead; flags & 2: the result's positive part squared.
int lyp_moe_gemm(const void* a, int lda, const void* w, long long w_expert_stride, int ldw, void* out, int ldo,
                 int dtype, int gated, const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* n_tiles,
                 int most_tiles, int tile_rows, const int32_t* expert_off, const int32_t* sorted_pair, int top, int N,
                 int K, float limit, float alpha, int flags, hipStream_t stream) {
  LYP_REQUIRE(N > 0 && K > 0 && lda >= K && ldw >= K && ldo >= N && top > 0 && most_tiles >= 0,
              "moe_gemm: bad sizes N=%d K=%d lda=%d ldw=%d ldo=%d", N, K, lda, ldw, ldo);
  LYP_REQUIRE(tile_rows == 16 || tile_rows == 128, "moe_gemm: tiles of %d rows", tile_rows);
  if (most_tiles == 0) return 0;
  // Tiles of 128 rows take 128 matrix rows (gated: 64 output columns), eight waves a tile.  Measured
  // on 8,192 pairs and 32 experts of 1,536 x 2,048 (gated / down, the kernels alone): four waves a tile
  // 242 / 162 us, eight waves 221 / 146 us, eight waves with rounds of 64 bytes a row 255 / 168 us; a
  // tile of 256 matrix rows with eight waves (one workgroup a compute unit) was slower than either.
  const int tile_cols = gated ? 64 : 128;
  // tiles of 16 rows (few rows an expert: a decode step's, a short portion's) are 16 columns wide, so
  // that the launch has workgroups enough to pull the matrices through (one token that chooses 4 of 32
  // experts of 1,536 x 2,048: 37 / 23 us with tiles of 64 columns through LDS, 15 / 9.5 us so; eight
  // tokens: 64 / 33 us against 53 / 30 us)
  const bool few = tile_rows == 16;
  const int col_tiles = few ? (N + 15) / 16 : (N + tile_cols - 1) / tile_cols;
  LYP_REQUIRE(col_tiles <= 65535, "moe_gemm: too many columns for one launch");
  const int esz = dtype == kF32 ? 4 : 2;
  const int vec = 16 / esz;
  const int vec_ok = lda % vec == 0 && ldw % vec == 0 && w_expert_stride % vec == 0 &&
                     reinterpret_cast<uintptr_t>(a) % 16 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
  dim3 grid(most_tiles, col_tiles);
#define LYP_MOE_WIDE(T, G, NWV)                                                                                 \
  static bool wide_set_##G##NWV = false;   /* the tiles take more LDS than a kernel gets unasked */             \
  if (!wide_set_##G##NWV) {                                                                                     \
    (void)hipFuncSetAttribute(reinterpret_cast<const void*>(moe_gemm_wide_kernel<T, G, NWV>),                   \
                              hipFuncAttributeMaxDynamicSharedMemorySize, MoeWide<T, NWV>::kBytes);             \
    wide_set_##G##NWV = true;                                                                                   \
  }                                                                                                             \
  moe_gemm_wide_kernel<T, G, NWV><<<grid, NWV * 64, MoeWide<T, NWV>::kBytes, stream>>>(                         \
      static_cast<const T*>(a), lda, static_cast<const T*>(w), w_expert_stride, ldw, static_cast<T*>(out), ldo, \
      tile_expert, tile_row0, n_tiles, expert_off, sorted_pair, top, N, K, N, limit, alpha, vec_ok, flags)
#define LYP_MOE_FEW(T, G)                                                                                       \
  moe_gemm_few_kernel<T, G><<<grid, 256, 0, stream>>>(                                                          \
      static_cast<const T*>(a), lda, static_cast<const T*>(w), w_expert_stride, ldw, static_cast<T*>(out), ldo, \
      tile_expert, tile_row0, n_tiles, expert_off, sorted_pair, top, N, K, N, limit, alpha, vec_ok, flags)
#define LYP_MOE_T(T)                                 \
  do {                                               \
    if (few) {                                       \
      if (gated) LYP_MOE_FEW(T, true);               \
      else LYP_MOE_FEW(T, false);                    \
    } else {                                         \
      if (gated) { LYP_MOE_WIDE(T, true, 8); }       \
      else { LYP_MOE_WIDE(T, false, 8); }            \
    }                                                \
  } while (0)
  if (dtype == kF32) LYP_MOE_T(float);
  else if (dtype == kBF16) LYP_MOE_T(bf16_t);
  else LYP_REQUIRE(false, "moe_gemm: unknown dtype %d", dtype);
#undef LYP_MOE_T
#undef LYP_MOE_FEW
#undef LYP_MOE_WIDE
  LYP_LAUNCH_CHECK("moe_gemm");
  return 0;
}

int lyp_glu_clamped(const void* gate_up, void* out, int dtype, int rows, int I, float limit, float alpha,
                    hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && I > 0, "glu_clamped: bad sizes");
  if (rows == 0) return 0;
  const long long total = static_cast<long long>(rows) * I;
  const int blocks = static_cast<int>(std::min<long long>((total + 255) / 256, 8192));
  if (dtype == kF32)
    glu_clamped_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<const float*>(gate_up),
                                                          static_cast<float*>(out), rows, I, limit, alpha);
  else if (dtype == kBF16)
    glu_clamped_kernel<bf16_t><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(gate_up),
                                                           static_cast<bf16_t*>(out), rows, I, limit, alpha);
  else
    LYP_REQUIRE(false, "glu_clamped: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("glu_clamped");
  return 0;
}

int lyp_moe_combine(const void* y, const int32_t* place_of, const float* wgt, int top, const void* addend,
                    const void* shared, float* out, int dtype, int rows, int H, hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && H > 0 && top > 0, "moe_combine: bad sizes");
  if (rows == 0) return 0;
  LYP_REQUIRE(top <= kMostTop, "moe_combine: %d choices a token (at most %d)", top, kMostTop);
  const bool vec = H % 4 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0 && reinterpret_cast<uintptr_t>(addend) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(shared) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const int per = vec ? 4 : 1;
  const int threads = H / per >= 512 ? 256 : (H / per >= 128 ? 128 : 64);
#define LYP_COMBINE(T, V)                                                                                      \
  moe_combine_kernel<T, V><<<rows, threads, 0, stream>>>(static_cast<const T*>(y), place_of, wgt, top,        \
                                                        static_cast<const T*>(addend),                       \
                                                        static_cast<const T*>(shared), out, rows, H)
  if (dtype == kF32) {
    if (vec) LYP_COMBINE(float, 4);
    else LYP_COMBINE(float, 1);
  } else if (dtype == kBF16) {
    if (vec) LYP_COMBINE(bf16_t, 4);
    else LYP_COMBINE(bf16_t, 1);
  } else {
    LYP_REQUIRE(false, "moe_combine: unknown dtype %d", dtype);
  }
#undef LYP_COMBINE
  LYP_LAUNCH_CHECK("moe_combine");
  return 0;
}

}  // extern "C"
