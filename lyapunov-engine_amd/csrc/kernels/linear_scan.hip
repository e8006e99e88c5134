// Linear recurrences with a matrix state per head, for mixers that carry a
// summary S [dim x vdim] instead of keys:
//
//   decayed outer products    S <- diag(g_t) S + k_t v_t^T                     o_t = S^T q_t
//   gated delta rule          S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);
//                             S <- S + k_t u^T                                 o_t = S^T q_t
//
//   bonus for the current token   o_t = (S + diag(u) k_t v_t^T)^T q_t;  S <- diag(g_t) S + k_t v_t^T
//                                 (the output reads the state before the token's decay and write)
//
// with a decay per head and key channel, g = exp(-coef_head * softplus(sign * (z + bias))), which
// covers exp(-A softplus(z + b)) (sign +1, coef A) and sigmoid(z + b)^(1/tau) (sign -1, coef 1/tau);
// sign 0 says that z holds the decays themselves (lowrank_up works them out on its way).  One decay
// per head (z [rows, heads]) is taken for all of the head's key channels; the softplus is then a step
// size that may also multiply the token's key (S <- g S + step k v^T: a discretised state space).
// Queries and keys may be made unit vectors per head first (x / sqrt(sum x^2 + 1e-6)); queries
// take a constant factor.  Decays, unit vectors, gates, sums and the state are 32-bit; q, k, v come
// in the activations' type.
//
//   * linear_scan: the state is kept transposed, [slot][head][vdim][dim], and lives in registers:
//     a column of S (one value of vdim) belongs to L neighbouring lanes (up to 16) that hold DPL key
//     channels each; the two dot products of a token are sums inside a lane and over those L lanes.  The
//     step's tokens of a request are walked in order; what does not depend on the state (decays,
//     the lengths of queries and keys, sigmoid of beta) is worked out for a chunk of tokens at a time,
//     side by side by all threads, into LDS.  A workgroup takes (a block of columns, a head, a request); columns do not depend
//     on each other.  The slot is read unless the request stands at position 0, and written back.
//   * head_norm_gate: every head's o over vdim divided by its root mean square, times a weight
//     shared by the heads, times sigmoid or silu of a gate's pre-activation.
//   * lowrank_up: out = mid W^T (+ bias) in 32-bit for the second half of a low-rank projection
//     (few inner values): eight rows a thread, so a row of W is read once for eight tokens.
#include <algorithm>

#include "common.h"

namespace lyp {

// Tokens staged at a time: what a token needs besides the state (decays, keys, queries, values, beta)
// is worked out for this many tokens side by side, by all threads, so that memory's latency is paid
// once a chunk and not once a token.
__host__ __device__ inline int scan_chunk(int Dp) { return Dp <= 128 ? 32 : (Dp <= 256 ? 16 : 8); }
constexpr int kScanPad = 4;   // floats between the staged rows, so that neighbouring tokens start in other banks

__device__ __forceinline__ float scan_softplus(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }
__device__ __forceinline__ float scan_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

// The sum over a group of L neighbouring lanes (L a power of two up to 16, groups aligned), by
// lane permutations inside a row of 16; every lane of the group gets it.
template <int CTRL>
__device__ __forceinline__ float scan_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float group_sum(float v, int L) {
  // every stage is worked out and taken or not by a select: no branches in the walk over the tokens
  float t = v + scan_dpp<0xB1>(v);    // neighbours: lanes 1 0 3 2 of every four
  v = L > 1 ? t : v;
  t = v + scan_dpp<0x4E>(v);          // lanes 2 3 0 1 of every four
  v = L > 2 ? t : v;
  t = v + scan_dpp<0x141>(v);         // every eight mirrored
  v = L > 4 ? t : v;
  t = v + scan_dpp<0x140>(v);         // every sixteen mirrored
  v = L > 8 ? t : v;
  return v;
}

// With S' = diag(g) S the token's two products with the state are both taken from S' in one pass,
//   r = k . S',  p = q . S';   u = beta (v - r)  (u = v without the delta rule);
//   S = S' + k u^T;  o = q . S = p + (q . k) u,
// and q . k does not depend on the state: it is staged with the lengths.
// STAGE: keys, queries and decays a thread fetches in one round (and half as many values): 16 for steps
// of long portions, 4 for steps of single tokens and short portions, which then need few registers
// and many workgroups fit a compute unit.
// MODE 0: decayed outer products, 1: the delta rule, 2: the bonus form.
template <typename T, int DPL, int MODE, int STAGE>
__global__ __launch_bounds__(256) void linear_scan_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    const float* __restrict__ z, int ldz, const float* __restrict__ zbias, const float* __restrict__ coef, float sign,
    const T* __restrict__ beta, int ldb, float* __restrict__ state, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slots, float* __restrict__ out, int ldo, int H,
    int G, int D, int V, int L, int unit, float q_scale, int chunk, const float* __restrict__ bonus, int z_per_head,
    int key_step) {
  constexpr bool DELTA = MODE == 1, PRE = MODE == 2;
  extern __shared__ __attribute__((aligned(16))) float s_scan[];
  const int Dp = L * DPL;                      // key channels with the padding: a power of two
  const int ld = Dp + kScanPad;
  const int l_shift = __ffs(L) - 1;
  const int cpb = blockDim.x / L;              // columns a workgroup: a power of two
  const int dp_shift = __ffs(Dp) - 1, cpb_shift = __ffs(cpb) - 1;
  float* sk = s_scan;                          // [chunk][ld]   keys as they come
  float* sq = sk + chunk * ld;                 //               queries as they come
  float* sg = sq + chunk * ld;                 //               decays
  float* sv = sg + chunk * ld;                 // [chunk][cpb]  this workgroup's columns of the values
  float* sb = sv + chunk * cpb;                // [chunk]       sigmoid(beta)
  float* sfq = sb + chunk;                     // [chunk]       what a query is multiplied by (unit length, the constant)
  float* sfk = sfq + chunk;                    // [chunk]       what a key is multiplied by
  float* sqk = sfk + chunk;                    // [chunk]       query . key, as they come
  float* so = sqk + chunk;                     // [chunk][cpb]  the tokens' outputs, written out a chunk at a time
  float* sbn = so + chunk * cpb;               // [Dp]          the head's bonus, laid out as a staged key (the bonus form only)
  const int b = blockIdx.z, h = blockIdx.y;
  const int q0 = q_start[b], n = q_start[b + 1] - q0;
  if (n <= 0) return;
  const int tid = threadIdx.x;
  const int l = tid % L, cl = tid / L;
  const int col = blockIdx.x * cpb + cl;
  const int d0 = l * DPL;
  const int kvh = h / (H / G);
  const bool fresh = positions[q0] == 0;
  float* st = state + ((static_cast<size_t>(slots[b]) * H + h) * V + (col < V ? col : 0)) * D;
  float S[DPL];
#pragma unroll
  for (int i = 0; i < DPL; ++i) S[i] = (!fresh && col < V && d0 + i < D) ? st[d0 + i] : 0.f;
  const float a_h = coef[h];

  constexpr int kStage = STAGE, kStageV = STAGE / 2;
  // What a chunk's tokens bring is fetched into registers kStage values a thread at a time, all loads
  // in flight together, and staged in LDS from there.  A workgroup whose threads cover a whole chunk
  // in one such round fetches the next chunk before it walks the current one's tokens, so that
  // memory's latency passes meanwhile.
  T rq[kStage], rk[kStage];
  float rz[kStage];
  T rv[kStageV];
  T rb = from_f32<T>(0.f);
  const int per_round = kStage * blockDim.x;
  const bool ahead = (chunk << dp_shift) <= per_round && (chunk << cpb_shift) <= kStageV * static_cast<int>(blockDim.x);
  auto fetch = [&](int c0, int cn, int base) {
#pragma unroll
    for (int u = 0; u < kStage; ++u) {
      const int idx = base + u * blockDim.x + tid;
      const int j = idx >> dp_shift, d = idx & (Dp - 1);
      rq[u] = rk[u] = from_f32<T>(0.f);
      rz[u] = 0.f;
      if (j < cn && d < D) {
        const size_t row = static_cast<size_t>(q0 + c0 + j);
        rq[u] = q[row * ldq + kvh * D + d];
        rk[u] = k[row * ldk + kvh * D + d];
        rz[u] = z[row * ldz + (z_per_head ? h : h * D + d)];
      }
    }
  };
  auto fetch_values = [&](int c0, int cn) {
#pragma unroll
    for (int u = 0; u < kStageV; ++u) {
      const int idx = u * blockDim.x + tid;
      const int j = idx >> cpb_shift, c = blockIdx.x * cpb + (idx & (cpb - 1));
      rv[u] = (j < cn && c < V) ? v[static_cast<size_t>(q0 + c0 + j) * ldv + h * V + c] : from_f32<T>(0.f);
    }
    if (DELTA && tid < cn) rb = beta[static_cast<size_t>(q0 + c0 + tid) * ldb + h];
  };
  auto stash = [&](int cn, int base) {
#pragma unroll
    for (int u = 0; u < kStage; ++u) {
      const int idx = base + u * blockDim.x + tid;
      const int j = idx >> dp_shift, d = idx & (Dp - 1);
      if (j < cn) {
        float gg = 1.f;
        if (d < D)
          gg = sign == 0.f ? rz[u]
                           : expf(-a_h * scan_softplus(sign * (rz[u] + (zbias != nullptr ? zbias[z_per_head ? h : h * D + d] : 0.f))));
        // a lane's channels four by four in planes, so that a plane's read takes neighbouring lanes to neighbouring words
        const int at = j * ld + ((((d & (DPL - 1)) >> 2) << (l_shift + 2)) | ((d / DPL) << 2) | (d & 3));
        sq[at] = to_f32(rq[u]);
        sk[at] = to_f32(rk[u]);
        sg[at] = gg;
      }
    }
  };
  auto stash_values = [&](int cn) {
#pragma unroll
    for (int u = 0; u < kStageV; ++u) {
      const int idx = u * blockDim.x + tid;
      if (idx < (cn << cpb_shift)) sv[idx] = to_f32(rv[u]);
    }
    if (DELTA && tid < cn) sb[tid] = scan_sigmoid(to_f32(rb));
  };
  if (ahead) {
    fetch(0, min(chunk, n), 0);
    fetch_values(0, min(chunk, n));
  }
  if constexpr (PRE) {
    for (int d = tid; d < Dp; d += blockDim.x)
      sbn[(((d & (DPL - 1)) >> 2) << (l_shift + 2)) | ((d / DPL) << 2) | (d & 3)] = d < D ? bonus[h * D + d] : 0.f;
  }

  for (int c0 = 0; c0 < n; c0 += chunk) {
    const int cn = min(chunk, n - c0);
    if (ahead) {
      stash(cn, 0);
      stash_values(cn);
    } else {
      for (int base = 0; base < (cn << dp_shift); base += per_round) {
        fetch(c0, cn, base);
        stash(cn, base);
      }
      for (int idx = tid; idx < (cn << cpb_shift); idx += blockDim.x) {
        const int j = idx >> cpb_shift, c = blockIdx.x * cpb + (idx & (cpb - 1));
        sv[idx] = c < V ? to_f32(v[static_cast<size_t>(q0 + c0 + j) * ldv + h * V + c]) : 0.f;
      }
      if (DELTA && tid < cn) sb[tid] = scan_sigmoid(to_f32(beta[static_cast<size_t>(q0 + c0 + tid) * ldb + h]));
    }
    __syncthreads();
    // four neighbouring lanes a token: the squares of its query and key and their product, a quarter each
    for (int j = tid / 4; j < cn; j += blockDim.x / 4) {
      float ssq = 0.f, ssk = 0.f, sqkv = 0.f;
      for (int f = tid % 4; f < Dp / 4; f += 4) {
        const f32x4 q4 = *reinterpret_cast<const f32x4*>(sq + j * ld + 4 * f);
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(sk + j * ld + 4 * f);
        ssq += q4[0] * q4[0] + q4[1] * q4[1] + q4[2] * q4[2] + q4[3] * q4[3];
        ssk += k4[0] * k4[0] + k4[1] * k4[1] + k4[2] * k4[2] + k4[3] * k4[3];
        if constexpr (PRE) {
          const f32x4 b4 = *reinterpret_cast<const f32x4*>(sbn + 4 * f);
          sqkv += q4[0] * k4[0] * b4[0] + q4[1] * k4[1] * b4[1] + q4[2] * k4[2] * b4[2] + q4[3] * k4[3] * b4[3];
        } else {
          sqkv += q4[0] * k4[0] + q4[1] * k4[1] + q4[2] * k4[2] + q4[3] * k4[3];
        }
      }
      ssq = group_sum(ssq, 4);
      ssk = group_sum(ssk, 4);
      sqkv = group_sum(sqkv, 4);
      if (tid % 4 == 0) {
        sfq[j] = unit ? q_scale / sqrtf(ssq + 1e-6f) : q_scale;
        float fkey = unit ? 1.0f / sqrtf(ssk + 1e-6f) : 1.f;
        if (key_step)   // the step size: the softplus inside the head's decay
          fkey *= scan_softplus(sign * (z[static_cast<size_t>(q0 + c0 + j) * ldz + h] + (zbias != nullptr ? zbias[h] : 0.f)));
        sfk[j] = fkey;
        sqk[j] = sqkv;
      }
    }
    __syncthreads();
    if (ahead && c0 + chunk < n) {
      fetch(c0 + chunk, min(chunk, n - c0 - chunk), 0);
      fetch_values(c0 + chunk, min(chunk, n - c0 - chunk));
    }
    // a token's operands are read from LDS while the token before it is worked on
    f32x4 g4[DPL / 4], q4[DPL / 4], k4[DPL / 4], ng[DPL / 4], nq[DPL / 4], nk[DPL / 4];
    float fk, fq, qk, u, bt = 1.f, nfk, nfq, nqk, nu, nbt = 1.f;
    auto read = [&](int j, f32x4 (&g_)[DPL / 4], f32x4 (&q_)[DPL / 4], f32x4 (&k_)[DPL / 4], float& fk_, float& fq_, float& qk_,
                    float& u_, float& bt_) {
      const int at = j * ld + 4 * l;
#pragma unroll
      for (int i = 0; i < DPL / 4; ++i) {
        g_[i] = *reinterpret_cast<const f32x4*>(sg + at + ((i << l_shift) << 2));
        q_[i] = *reinterpret_cast<const f32x4*>(sq + at + ((i << l_shift) << 2));
        k_[i] = *reinterpret_cast<const f32x4*>(sk + at + ((i << l_shift) << 2));
      }
      fk_ = sfk[j];
      fq_ = sfq[j];
      qk_ = sqk[j];
      u_ = sv[(j << cpb_shift) + cl];
      if constexpr (DELTA) bt_ = sb[j];
    };
    auto work = [&](int j, const f32x4 (&g_)[DPL / 4], const f32x4 (&q_)[DPL / 4], const f32x4 (&k_)[DPL / 4], float fk_,
                    float fq_, float qk_, float u_, float bt_) {
      float r0 = 0.f, r1 = 0.f, p0 = 0.f, p1 = 0.f;
#pragma unroll
      for (int i = 0; i < DPL / 4; ++i) {
        if constexpr (PRE) {   // the output reads the state as the token found it
          p0 += S[4 * i] * q_[i][0] + S[4 * i + 2] * q_[i][2];
          p1 += S[4 * i + 1] * q_[i][1] + S[4 * i + 3] * q_[i][3];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) S[4 * i + e] *= g_[i][e];
        if constexpr (DELTA) {
          r0 += S[4 * i] * k_[i][0] + S[4 * i + 2] * k_[i][2];
          r1 += S[4 * i + 1] * k_[i][1] + S[4 * i + 3] * k_[i][3];
        }
        if constexpr (!PRE) {
          p0 += S[4 * i] * q_[i][0] + S[4 * i + 2] * q_[i][2];
          p1 += S[4 * i + 1] * q_[i][1] + S[4 * i + 3] * q_[i][3];
        }
      }
      const float p = group_sum(p0 + p1, L);
      if constexpr (DELTA) u_ = bt_ * (u_ - fk_ * group_sum(r0 + r1, L));
      u_ *= fk_;
#pragma unroll
      for (int i = 0; i < DPL / 4; ++i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) S[4 * i + e] += k_[i][e] * u_;
      }
      so[(j << cpb_shift) + cl] = fq_ * (p + qk_ * u_);   // all lanes of the column hold it: no branch
    };
    // two tokens a round, their operands in two sets of registers in turn
    read(0, g4, q4, k4, fk, fq, qk, u, bt);
    for (int j = 0; j < cn; j += 2) {
      read(min(j + 1, cn - 1), ng, nq, nk, nfk, nfq, nqk, nu, nbt);
      work(j, g4, q4, k4, fk, fq, qk, u, bt);
      if (j + 1 < cn) {
        read(min(j + 2, cn - 1), g4, q4, k4, fk, fq, qk, u, bt);
        work(j + 1, ng, nq, nk, nfk, nfq, nqk, nu, nbt);
      }
    }
    __syncthreads();   // the chunk's staging is read to the end before the next overwrites it
    for (int idx = tid; idx < (cn << cpb_shift); idx += blockDim.x) {
      const int j = idx >> cpb_shift, c = blockIdx.x * cpb + (idx & (cpb - 1));
      if (c < V) out[static_cast<size_t>(q0 + c0 + j) * ldo + h * V + c] = so[idx];
    }
  }
  if (col < V) {
#pragma unroll
    for (int i = 0; i < DPL; ++i)
      if (d0 + i < D) st[d0 + i] = S[i];
  }
}

enum GateKind : int { kGateSigmoid = 0, kGateSilu = 1 };

// One wave per (row, head).
template <typename TG, typename T>
__global__ __launch_bounds__(256) void head_norm_gate_kernel(const float* __restrict__ o, const float* __restrict__ w,
                                                             const TG* __restrict__ gate, int ldg, T* __restrict__ out,
                                                             int rows, int H, int V, float eps, int kind, int w_per_head) {
  const int item = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= rows * H) return;
  const int t = item / H, h = item % H, lane = threadIdx.x % kWave;
  const float* orow = o + (static_cast<size_t>(t) * H + h) * V;
  float ss = 0.f;
  for (int c = lane; c < V; c += kWave) ss += orow[c] * orow[c];
  const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(V) + eps);
  const TG* grow = gate + static_cast<size_t>(t) * ldg + h * V;
  T* dst = out + (static_cast<size_t>(t) * H + h) * V;
  if (w_per_head) w += h * V;
  for (int c = lane; c < V; c += kWave) {
    const float g = to_f32(grow[c]);
    const float s = scan_sigmoid(g);
    dst[c] = from_f32<T>(orow[c] * inv * w[c] * (kind == kGateSilu ? g * s : s));
  }
}

constexpr int kLowRows = 8;

template <typename T>
__global__ __launch_bounds__(256) void lowrank_up_kernel(const T* __restrict__ mid, int ldm, const float* __restrict__ w,
                                                         const float* __restrict__ bias, float* __restrict__ out,
                                                         int rows, int N, int R, const float* __restrict__ coef,
                                                         float sign, int per_head, int mid_tanh, int double_exp) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const int t0 = blockIdx.y * kLowRows;
  if (n >= N) return;
  float acc[kLowRows];
  const float b = bias != nullptr ? bias[n] : 0.f;
#pragma unroll
  for (int j = 0; j < kLowRows; ++j) acc[j] = b;
  const float* wr = w + static_cast<size_t>(n) * R;
  for (int r = 0; r < R; ++r) {
    const float x = wr[r];
#pragma unroll
    for (int j = 0; j < kLowRows; ++j)
      if (t0 + j < rows) {
        const float m = to_f32(mid[static_cast<size_t>(t0 + j) * ldm + r]);
        acc[j] += x * (mid_tanh ? tanhf(m) : m);
      }
  }
  const float a = coef != nullptr ? coef[n / per_head] : 0.f;
#pragma unroll
  for (int j = 0; j < kLowRows; ++j)
    if (t0 + j < rows)
      out[static_cast<size_t>(t0 + j) * N + n] = double_exp ? expf(-expf(acc[j]))
                                                 : (coef != nullptr ? expf(-a * scan_softplus(sign * acc[j])) : acc[j]);
}

}  // namespace lyp

using namespace lyp;

extern "C" {

// Key channels a lane holds of its column of the state, for key heads of D values: as few as keep a
// column within the 16 lanes whose sums go by lane permutations (0: D is too large).
static int scan_channels_per_lane(int D) {
  if (D <= 0 || D > 512) return 0;
  return D <= 128 ? 8 : (D <= 256 ? 16 : 32);
}

// Lanes a column of the state is spread over, for key heads of D values (0: D is too large).
int lyp_linear_scan_lanes(int D) {
  const int dpl = scan_channels_per_lane(D);
  if (dpl == 0) return 0;
  int L = 1;
  while (L * dpl < D) L *= 2;
  return L;
}

// q, k [rows, >= G*D] and v [rows, >= H*V] of dtype, rows ldq / ldk / ldv apart; z float [rows, >= H*D] (ldz apart);
// zbias float [H*D] or null (z_per_head: z [rows, >= H], zbias [H]; key_step: the key is multiplied by the softplus);
// bonus float [H*D] or null (the bonus form); coef float [H]; rows: all requests' rows together; beta [rows, >= H] of dtype (ldb apart; the delta rule only: delta != 0);
// state float [slots, H, V, D]; out float [rows, >= H*V] (ldo apart).  Request b owns rows q_start[b] .. q_start[b+1].
int lyp_linear_scan(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, int dtype, const float* z,
                    int ldz, const float* zbias, const float* coef, float sign, const void* beta, int ldb,
                    float* state, const int32_t* q_start, const int32_t* positions, const int32_t* slots, float* out,
                    int ldo, int rows, int B, int H, int G, int D, int V, int delta, int unit, float q_scale,
                    const float* bonus, int z_per_head, int key_step, hipStream_t stream) {
  LYP_REQUIRE(B > 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && V > 0, "linear_scan: B=%d H=%d G=%d D=%d V=%d", B, H, G,
              D, V);
  const int L = lyp_linear_scan_lanes(D);
  LYP_REQUIRE(L > 0 && L <= 16, "linear_scan: key heads of up to 512 values, not %d", D);
  LYP_REQUIRE(!(delta && bonus != nullptr), "linear_scan: the delta rule has no bonus form");
  LYP_REQUIRE(!key_step || (z_per_head && sign != 0.f), "linear_scan: a step size comes with one decay per head, worked out here");
  LYP_REQUIRE(ldq >= G * D && ldk >= G * D && ldv >= H * V && ldz >= (z_per_head ? H : H * D) && ldo >= H * V && (!delta || ldb >= H),
              "linear_scan: rows too short for %d/%d heads of %d/%d", H, G, D, V);
  LYP_REQUIRE(!delta || beta != nullptr, "linear_scan: the delta rule needs beta");
  LYP_REQUIRE(H <= 65535 && B <= 65535, "linear_scan: too many heads or requests for one launch");
  const int dpl = scan_channels_per_lane(D);
  // columns a workgroup: as few as fill a wave when there are few (request, head) pairs, so that
  // the launch has workgroups for the machine; up to four waves otherwise
  // (a request of many rows keeps its waves together all the same: they share the chunk's staging)
  int threads = 256;
  while (threads > 64 && rows < 16LL * B &&
         static_cast<long long>(B) * H * ((V * L + threads - 1) / threads) < 2LL * compute_units())
    threads /= 2;
  while (threads > 64 && threads / 2 >= V * L) threads /= 2;
  const int cpb = threads / L;
  dim3 grid((V + cpb - 1) / cpb, H, B);
  // few rows a request (single tokens, short portions): a short chunk, so that many workgroups fit a compute unit
  const bool brief = rows < 16LL * B;
  int chunk = brief ? (rows <= B ? 2 : std::min(8, scan_chunk(L * dpl))) : scan_chunk(L * dpl);
  const size_t per_token = (3 * (L * dpl + kScanPad) + 2 * cpb + 4) * sizeof(float);
  while (chunk > 1 && chunk * per_token > 65536 - 2048) chunk /= 2;
  const size_t lds = chunk * per_token + (bonus != nullptr ? L * dpl * sizeof(float) : 0);
  const int mode = delta ? 1 : (bonus != nullptr ? 2 : 0);
#define LYP_SCAN_S(T, DPLV, DEL, ST)                                                                                \
  linear_scan_kernel<T, DPLV, DEL, ST><<<grid, threads, lds, stream>>>(                                               \
      static_cast<const T*>(q), ldq, static_cast<const T*>(k), ldk, static_cast<const T*>(v), ldv, z, ldz, zbias,   \
      coef, sign, static_cast<const T*>(beta), ldb, state, q_start, positions, slots, out, ldo, H, G, D, V, L, unit, \
      q_scale, chunk, bonus, z_per_head, key_step)
#define LYP_SCAN(T, DPLV, DEL)              \
  do {                                      \
    if (brief) LYP_SCAN_S(T, DPLV, DEL, 4); \
    else LYP_SCAN_S(T, DPLV, DEL, 16);      \
  } while (0)
#define LYP_SCAN_M(T, DPLV)                    \
  do {                                         \
    if (mode == 1) LYP_SCAN(T, DPLV, 1);       \
    else if (mode == 2) LYP_SCAN(T, DPLV, 2);  \
    else LYP_SCAN(T, DPLV, 0);                 \
  } while (0)
#define LYP_SCAN_T(T)                          \
  do {                                         \
    if (dpl == 8) LYP_SCAN_M(T, 8);            \
    else if (dpl == 16) LYP_SCAN_M(T, 16);     \
    else LYP_SCAN_M(T, 32);                    \
  } while (0)
  if (dtype == kF32) LYP_SCAN_T(float);
  else if (dtype == kBF16) LYP_SCAN_T(bf16_t);
  else LYP_REQUIRE(false, "linear_scan: unknown dtype %d", dtype);
#undef LYP_SCAN_T
#undef LYP_SCAN_M
#undef LYP_SCAN
#undef LYP_SCAN_S
  LYP_LAUNCH_CHECK("linear_scan");
  return 0;
}

// o float [rows, H*V]; w float [V] (w_per_head: [H*V], every head its own); gate [rows, >= H*V] (ldg apart) float (gate_dtype kF32) or of out's type;
// out [rows, H*V] of out_dtype.  kind: 0 sigmoid(gate), 1 silu(gate).
int lyp_head_norm_gate(const float* o, const float* w, const void* gate, int ldg, int gate_dtype, void* out,
                       int out_dtype, int rows, int H, int V, float eps, int kind, int w_per_head, hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && H > 0 && V > 0 && ldg >= H * V && (kind == kGateSigmoid || kind == kGateSilu),
              "head_norm_gate: rows=%d H=%d V=%d ldg=%d kind=%d", rows, H, V, ldg, kind);
  LYP_REQUIRE(gate_dtype == kF32 || gate_dtype == out_dtype, "head_norm_gate: the gate is float or of the output's type");
  if (rows == 0) return 0;
  const long long items = static_cast<long long>(rows) * H;
  const int blocks = static_cast<int>((items + 3) / 4);
#define LYP_HNG(TG, T)                                                                                              \
  head_norm_gate_kernel<TG, T><<<blocks, 256, 0, stream>>>(o, w, static_cast<const TG*>(gate), ldg,                 \
                                                           static_cast<T*>(out), rows, H, V, eps, kind, w_per_head)
  if (out_dtype == kF32) LYP_HNG(float, float);
  else if (out_dtype == kBF16 && gate_dtype == kF32) LYP_HNG(float, bf16_t);
  else if (out_dtype == kBF16) LYP_HNG(bf16_t, bf16_t);
  else LYP_REQUIRE(false, "head_norm_gate: unknown dtype %d", out_dtype);
#undef LYP_HNG
  LYP_LAUNCH_CHECK("head_norm_gate");
  return 0;
}

// mid [rows, >= R] of dtype (ldm apart); w float [N, R]; bias float [N] or null; out float [rows, N].
// coef float [N / per_head] or null: the result y becomes the decay exp(-coef[n / per_head] * softplus(sign * y)).
// mid_tanh: the inner values pass tanh first; double_exp: the result y becomes the decay exp(-exp(y)).
int lyp_lowrank_up(const void* mid, int ldm, int dtype, const float* w, const float* bias, float* out, int rows, int N,
                   int R, const float* coef, float sign, int per_head, int mid_tanh, int double_exp, hipStream_t stream) {
  LYP_REQUIRE(coef == nullptr || (per_head > 0 && N % per_head == 0), "lowrank_up: %d values in heads of %d", N, per_head);
  LYP_REQUIRE(rows >= 0 && N > 0 && R > 0 && ldm >= R, "lowrank_up: rows=%d N=%d R=%d ldm=%d", rows, N, R, ldm);
  if (rows == 0) return 0;
  const int threads = N >= 256 ? 256 : 64 * ((N + 63) / 64);
  dim3 grid((N + threads - 1) / threads, (rows + kLowRows - 1) / kLowRows);
  LYP_REQUIRE(grid.y <= 65535, "lowrank_up: too many rows for one launch");
  if (dtype == kF32)
    lowrank_up_kernel<float><<<grid, threads, 0, stream>>>(static_cast<const float*>(mid), ldm, w, bias, out, rows, N, R, coef, sign, per_head, mid_tanh, double_exp);
  else if (dtype == kBF16)
    lowrank_up_kernel<bf16_t><<<grid, threads, 0, stream>>>(static_cast<const bf16_t*>(mid), ldm, w, bias, out, rows, N, R, coef, sign, per_head, mid_tanh, double_exp);
  else
    LYP_REQUIRE(false, "lowrank_up: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("lowrank_up");
  return 0;
}

}  // extern "C"
