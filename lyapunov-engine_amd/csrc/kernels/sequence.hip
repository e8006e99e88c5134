// Row-wise and time-wise kernels for layers that norm a branch before it joins
// the residual stream, filter a branch's input over time, or carry a
// recurrence: the joining norm, a short causal convolution with its state, the
// minGRU scan, the xIELU / tanh-GELU activations, and what a latent attention
// layer does around its products (norms of the latents, rotation of
// neighbouring pairs, the write of a token's latent into its page slot).
//
// All arithmetic is 32-bit; only loads and stores see the storage type.  Small
// parameter vectors (norm weights, filter taps, biases, sinks) arrive as float.
// Requests are described by the step's tables on the device: request b owns
// rows q_start[b] .. q_start[b+1] of the flat batch, in position order, and a
// request whose first row stands at position 0 starts from an empty state.
#include <algorithm>

#include "common.h"

namespace lyp {

// Request that owns row t: the last b with q_start[b] <= t.
__device__ __forceinline__ int owner_of(const int32_t* __restrict__ q_start, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] <= t) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

// ------------------------------------------------------ a normed branch joins
// h[row] += mult * y[row] / rms(y[row]) * wb (+ shift); optionally the row is
// then normed with w_next into out (out without w_next: the joined row as it is, for a
// consumer that reads the stream itself).  With `rows` the r-th output row is row
// rows[r] and h is left alone (the last norm before the output head).
// y == nullptr: nothing joins (only shift and the following norm).
template <typename TY, typename T>
__global__ void branch_join_kernel(float* __restrict__ h, const TY* __restrict__ y, const float* __restrict__ wb,
                                   float mult, const float* __restrict__ shift, const float* __restrict__ w_next,
                                   T* __restrict__ out, const int32_t* __restrict__ rows, int H, float eps_branch,
                                   float eps_next) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  float* hrow = h + src * H;
  const TY* yrow = y ? y + src * H : nullptr;
  float inv_y = 0.f;
  if (yrow) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < H; i += blockDim.x) {
      const float v = to_f32(yrow[i]);
      ss += v * v;
    }
    ss = block_sum(ss, scratch);
    inv_y = 1.0f / sqrtf(ss / static_cast<float>(H) + eps_branch);
  }
  auto joined = [&](int i) {
    float v = hrow[i];
    if (yrow) v += mult * ((to_f32(yrow[i]) * inv_y) * wb[i]);
    if (shift) v += shift[i];
    return v;
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = joined(i);
    if (!rows) hrow[i] = v;
    ss += v * v;
  }
  if (!out) return;
  T* orow = out + static_cast<size_t>(r) * H;
  if (!w_next) {   // no norm follows: the joined row itself, in the activations' type
    for (int i = threadIdx.x; i < H; i += blockDim.x) orow[i] = from_f32<T>(rows ? joined(i) : hrow[i]);
    return;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(H) + eps_next);
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = rows ? joined(i) : hrow[i];   // a thread reads back what it wrote itself
    orow[i] = from_f32<T>((v * inv) * w_next[i]);
  }
}

// The same with the row in registers (rows of up to 16384 values in steps of 4, 16-byte aligned
// operands): one read of every operand, 16-byte accesses.  CONV: every row is a request of its own
// that brings one token (a decode step), and the short convolution of the normed row with the
// request's state slot follows in the same kernel (see short_conv_kernel): out = x + sum_j w_j *
// (its last inputs), x rounded to the activations' type first as the stand-alone kernel finds it,
// and the slot moves on by one input.
template <typename TY, typename T, bool CONV>
__global__ void branch_join_vec_kernel(float* __restrict__ h, const TY* __restrict__ y, const float* __restrict__ wb,
                                       float mult, const float* __restrict__ shift, const float* __restrict__ w_next,
                                       T* __restrict__ out, const int32_t* __restrict__ rows, int H, float eps_branch,
                                       float eps_next, const float* __restrict__ conv_w, T* __restrict__ state,
                                       const int32_t* __restrict__ slots, const int32_t* __restrict__ positions,
                                       int taps) {
  constexpr int MAXV = 4;
  typedef T Vec4T __attribute__((ext_vector_type(4)));
  typedef TY Vec4Y __attribute__((ext_vector_type(4)));
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  f32x4* hrow = reinterpret_cast<f32x4*>(h + src * H);
  const Vec4Y* yrow = y ? reinterpret_cast<const Vec4Y*>(y + src * H) : nullptr;
  const int nvec = H / 4;
  // every operand is asked for at the start: a step of few rows is as long as its chain of loads
  f32x4 hv[MAXV], yv[MAXV], wbv[MAXV], shv[MAXV], wnv[MAXV];
  float ssy = 0.f;
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int idx = threadIdx.x + v * blockDim.x;
    if (idx < nvec) {
      hv[v] = hrow[idx];
      if (yrow) wbv[v] = reinterpret_cast<const f32x4*>(wb)[idx];
      if (shift) shv[v] = reinterpret_cast<const f32x4*>(shift)[idx];
      if (w_next) wnv[v] = reinterpret_cast<const f32x4*>(w_next)[idx];
      if (yrow) {
        const Vec4Y t = yrow[idx];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          yv[v][i] = to_f32(t[i]);
          ssy += yv[v][i] * yv[v][i];
        }
      }
    }
  }
  float inv_y = 0.f;
  if (yrow) {
    ssy = block_sum(ssy, scratch);
    inv_y = 1.0f / sqrtf(ssy / static_cast<float>(H) + eps_branch);
  }
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int idx = threadIdx.x + v * blockDim.x;
    if (idx < nvec) {
      if (yrow) {
#pragma unroll
        for (int i = 0; i < 4; ++i) hv[v][i] += mult * ((yv[v][i] * inv_y) * wbv[v][i]);
      }
      if (shift) {
#pragma unroll
        for (int i = 0; i < 4; ++i) hv[v][i] += shv[v][i];
      }
      if (!rows && (yrow || shift)) hrow[idx] = hv[v];
#pragma unroll
      for (int i = 0; i < 4; ++i) ss += hv[v][i] * hv[v][i];
    }
  }
  if (!out) return;
  Vec4T* orow = reinterpret_cast<Vec4T*>(out + static_cast<size_t>(r) * H);
  if (!w_next) {   // no norm follows: the joined row itself, in the activations' type
#pragma unroll
    for (int v = 0; v < MAXV; ++v) {
      const int idx = threadIdx.x + v * blockDim.x;
      if (idx < nvec) {
        Vec4T o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = from_f32<T>(hv[v][i]);
        orow[idx] = o;
      }
    }
    return;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(H) + eps_next);
  const int hist = taps - 1;
  bool fresh = true;
  T* st = nullptr;
  if constexpr (CONV) {
    fresh = positions[r] == 0;
    st = state + static_cast<size_t>(slots[r]) * hist * H;
  }
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int idx = threadIdx.x + v * blockDim.x;
    if (idx < nvec) {
      Vec4T o;
#pragma unroll
      for (int i = 0; i < 4; ++i) o[i] = from_f32<T>((hv[v][i] * inv) * wnv[v][i]);
      if constexpr (CONV) {
        float acc[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float x = to_f32(o[i]);
          acc[i] = x + conv_w[(static_cast<size_t>(idx) * 4 + i) * taps + hist] * x;
        }
        for (int j = 0; j < hist; ++j) {
          Vec4T old = *(reinterpret_cast<Vec4T*>(st + static_cast<size_t>(j) * H) + idx);
          if (fresh)
#pragma unroll
            for (int i = 0; i < 4; ++i) old[i] = from_f32<T>(0.f);
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[i] += conv_w[(static_cast<size_t>(idx) * 4 + i) * taps + j] * to_f32(old[i]);
          if (j > 0) *(reinterpret_cast<Vec4T*>(st + static_cast<size_t>(j - 1) * H) + idx) = old;   // the slot moves on
        }
        if (hist > 0) *(reinterpret_cast<Vec4T*>(st + static_cast<size_t>(hist - 1) * H) + idx) = o;
#pragma unroll
        for (int i = 0; i < 4; ++i) o[i] = from_f32<T>(acc[i]);
      }
      orow[idx] = o;
    }
  }
}

// ------------------------------------------- short causal convolution in time
// out[t, c] = x[t, c] + sum_j w[c, j] * x_(t - taps + 1 + j)[c] over the rows of
// t's request; before the step's first row the request's last taps - 1 inputs
// come from its state slot (zeros for a request at position 0), and the slot
// then takes the last taps - 1 inputs including this step's.
// Work items: one per row (rows whose history lies inside the step), then one
// per request, which does the rows that read the slot and then rewrites the
// slot, so that no other thread reads a slot while it changes.
// The input's rows may lie ldx values apart (a column range of a wider tensor);
// act != 0: silu of the result (with residual == 0 a plain convolution and its activation).
__device__ __forceinline__ float conv_silu(float v) { return v / (1.0f + expf(-v)); }

template <typename T>
__global__ void short_conv_kernel(const T* __restrict__ x, const float* __restrict__ w, T* __restrict__ state,
                                  const int32_t* __restrict__ q_start, const int32_t* __restrict__ positions,
                                  const int32_t* __restrict__ slots, T* __restrict__ out, int n_rows, int B, int C,
                                  int taps, int residual, int ldx, int act, const float* __restrict__ bias) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  const int item = blockIdx.x;
  const int hist = taps - 1;
  if (item < n_rows) {
    const int b = owner_of(q_start, B, item);
    const int i = item - q_start[b];
    if (c >= C) return;
    if (item >= q_start[B]) {   // rows past the last request belong to nobody
      out[static_cast<size_t>(item) * C + c] = from_f32<T>(0.f);
      return;
    }
    if (i < hist) return;
    const float* wc = w + static_cast<size_t>(c) * taps;
    float acc = (residual ? to_f32(x[static_cast<size_t>(item) * ldx + c]) : 0.f) + (bias ? bias[c] : 0.f);
    for (int j = 0; j < taps; ++j) acc += wc[j] * to_f32(x[static_cast<size_t>(item - hist + j) * ldx + c]);
    out[static_cast<size_t>(item) * C + c] = from_f32<T>(act ? conv_silu(acc) : acc);
    return;
  }
  const int b = item - n_rows;
  if (c >= C) return;
  const int q0 = q_start[b], n = q_start[b + 1] - q0;
  if (n <= 0) return;
  const bool fresh = positions[q0] == 0;
  T* st = hist > 0 ? state + (static_cast<size_t>(slots[b]) * hist) * C + c : nullptr;
  // input at local index idx (negative: from the slot)
  auto input = [&](int idx) -> float {
    if (idx >= 0) return to_f32(x[static_cast<size_t>(q0 + idx) * ldx + c]);
    return fresh ? 0.f : to_f32(st[static_cast<size_t>(idx + hist) * C]);
  };
  const float* wc = w + static_cast<size_t>(c) * taps;
  const int head = n < hist ? n : hist;
  for (int i = 0; i < head; ++i) {
    float acc = (residual ? input(i) : 0.f) + (bias ? bias[c] : 0.f);
    for (int j = 0; j < taps; ++j) acc += wc[j] * input(i - hist + j);
    out[static_cast<size_t>(q0 + i) * C + c] = from_f32<T>(act ? conv_silu(acc) : acc);
  }
  // slot entry k becomes the input at local index n - hist + k; rising k reads
  // entries k + n > k only, never one already rewritten
  for (int k = 0; k < hist; ++k) st[static_cast<size_t>(k) * C] = from_f32<T>(input(n - hist + k));
}

// The same with 16 bytes of neighbouring channels a thread (C a multiple of the vector's length,
// aligned operands, up to kConvTaps taps): a thread keeps its channels' taps in registers and walks
// kConvRows rows with them (work items: groups of rows, then the requests).
constexpr int kConvRows = 8;
constexpr int kConvTaps = 8;

template <typename T>
__global__ void short_conv_vec_kernel(const T* __restrict__ x, const float* __restrict__ w, T* __restrict__ state,
                                      const int32_t* __restrict__ q_start, const int32_t* __restrict__ positions,
                                      const int32_t* __restrict__ slots, T* __restrict__ out, int n_rows, int B, int C,
                                      int taps, int residual, int ldx, int act, const float* __restrict__ bias) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T VecT __attribute__((ext_vector_type(VEC)));
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * VEC;
  const int groups = (n_rows + kConvRows - 1) / kConvRows;
  const int item = blockIdx.x;
  const int hist = taps - 1;
  if (c >= C) return;
  auto load = [&](const T* p) { return *reinterpret_cast<const VecT*>(p); };
  auto store = [&](T* p, const float (&v)[VEC]) {
    VecT o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) o[e] = from_f32<T>(act ? conv_silu(v[e]) : v[e]);
    *reinterpret_cast<VecT*>(p) = o;
  };
  float wr[VEC][kConvTaps];   // this thread's channels x taps
#pragma unroll
  for (int e = 0; e < VEC; ++e)
#pragma unroll
    for (int j = 0; j < kConvTaps; ++j) wr[e][j] = j < taps ? w[static_cast<size_t>(c + e) * taps + j] : 0.f;
  float br[VEC];
#pragma unroll
  for (int e = 0; e < VEC; ++e) br[e] = bias ? bias[c + e] : 0.f;
  if (item < groups) {
    const int live = q_start[B];
    for (int row = item * kConvRows; row < min(n_rows, (item + 1) * kConvRows); ++row) {
      float acc[VEC];
      if (row >= live) {   // rows past the last request belong to nobody
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
        store(out + static_cast<size_t>(row) * C + c, acc);
        continue;
      }
      const int b = owner_of(q_start, B, row);
      if (row - q_start[b] < hist) continue;   // the request's item does the rows that read its slot
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] = br[e];
#pragma unroll
      for (int j = 0; j < kConvTaps; ++j) {
        if (j < taps) {
          const VecT v = load(x + static_cast<size_t>(row - hist + j) * ldx + c);
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            acc[e] += wr[e][j] * to_f32(v[e]);
            if (residual && j == hist) acc[e] += to_f32(v[e]);
          }
        }
      }
      store(out + static_cast<size_t>(row) * C + c, acc);
    }
    return;
  }
  const int b = item - groups;
  const int q0 = q_start[b], n = q_start[b + 1] - q0;
  if (n <= 0) return;
  const bool fresh = positions[q0] == 0;
  T* st = hist > 0 ? state + (static_cast<size_t>(slots[b]) * hist) * C + c : nullptr;
  auto input = [&](int idx) -> VecT {   // input at local index idx (negative: from the slot)
    if (idx >= 0) return load(x + static_cast<size_t>(q0 + idx) * ldx + c);
    VecT z;
#pragma unroll
    for (int e = 0; e < VEC; ++e) z[e] = from_f32<T>(0.f);
    return fresh ? z : load(st + static_cast<size_t>(idx + hist) * C);
  };
  const int head = n < hist ? n : hist;
  for (int i = 0; i < head; ++i) {
    float acc[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) acc[e] = br[e];
#pragma unroll
    for (int j = 0; j < kConvTaps; ++j) {
      if (j < taps) {
        const VecT v = input(i - hist + j);
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          acc[e] += wr[e][j] * to_f32(v[e]);
          if (residual && j == hist) acc[e] += to_f32(v[e]);
        }
      }
    }
    store(out + static_cast<size_t>(q0 + i) * C + c, acc);
  }
  // slot entry k becomes the input at local index n - hist + k (rising k reads entries k + n > k only)
  for (int k = 0; k < hist; ++k) *reinterpret_cast<VecT*>(st + static_cast<size_t>(k) * C) = input(n - hist + k);
}

// ------------------------------------------------------------- activations
__device__ __forceinline__ float softplus_f(float v) { return v > 20.f ? v : log1pf(expf(v)); }

enum Activation : int { kXielu = 0, kGeluTanh = 1 };

// xIELU with two learned numbers p, q (params[0], params[1]):
//   z > 0:  softplus(p) z^2 + z/2      z <= 0:  (1/2 + softplus(q)) (e^z - 1 - z) + z/2
__device__ __forceinline__ float xielu_f(float z, float ap, float aq) {
  return z > 0.f ? ap * z * z + 0.5f * z : aq * (expm1f(z) - z) + 0.5f * z;
}
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

// vec: 16 bytes a thread and turn; n is then a multiple of the vector's length and the operands are aligned
template <typename T>
__global__ void activation_kernel(const T* __restrict__ in, T* __restrict__ out, size_t n, int kind,
                                  const float* __restrict__ params, int vec) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T VecT __attribute__((ext_vector_type(VEC)));
  float ap = 0.f, aq = 0.f;
  if (kind == kXielu) {
    ap = softplus_f(params[0]);
    aq = 0.5f + softplus_f(params[1]);
  }
  const size_t stride = static_cast<size_t>(gridDim.x) * blockDim.x;
  if (vec) {
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n / VEC; i += stride) {
      VecT v = reinterpret_cast<const VecT*>(in)[i];
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        const float z = to_f32(v[e]);
        v[e] = from_f32<T>(kind == kXielu ? xielu_f(z, ap, aq) : gelu_tanh_f(z));
      }
      reinterpret_cast<VecT*>(out)[i] = v;
    }
    return;
  }
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n; i += stride) {
    const float z = to_f32(in[i]);
    out[i] = from_f32<T>(kind == kXielu ? xielu_f(z, ap, aq) : gelu_tanh_f(z));
  }
}

// ------------------------------------------------------------------- minGRU
// pre [rows, 3 W] float: the z, x and g projections side by side.
//   z = sigmoid(pre_z + bz);  u = pre_x + bx;  c = u + 1/2 (u >= 0) | sigmoid(u);
//   S <- (1 - z) S + z c;     out = S * silu(pre_g)
// One thread per (request, channel) walks the request's rows in order; the
// state slot (float) is read unless the request starts at position 0, and
// written at the end.
__device__ __forceinline__ float sigmoid_f(float v) { return 1.0f / (1.0f + expf(-v)); }

template <typename T>
__global__ void mingru_scan_kernel(const float* __restrict__ pre, const float* __restrict__ bz,
                                   const float* __restrict__ bx, float* __restrict__ state,
                                   const int32_t* __restrict__ q_start, const int32_t* __restrict__ positions,
                                   const int32_t* __restrict__ slots, T* __restrict__ out, int W) {
  const int b = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= W) return;
  const int q0 = q_start[b], q1 = q_start[b + 1];
  if (q1 <= q0) return;
  float* st = state + static_cast<size_t>(slots[b]) * W + c;
  float S = positions[q0] == 0 ? 0.f : *st;
  const float zb = bz[c], xb = bx[c];
  for (int t = q0; t < q1; ++t) {
    const float* row = pre + static_cast<size_t>(t) * 3 * W;
    const float z = sigmoid_f(row[c] + zb);
    const float u = row[W + c] + xb;
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
    S = (1.0f - z) * S + z * cand;
    const float g = row[2 * W + c];
    out[static_cast<size_t>(t) * W + c] = from_f32<T>(S * (g * sigmoid_f(g)));
  }
  *st = S;
}

// The same recurrence for steps with long runs of rows, in two kernels over chunks of kScanChunk
// rows of one request (S_t = a_t S_(t-1) + b_t with a = 1 - z, b = z c is linear in S):
//   summaries: per chunk and channel the product of its a's and its end state from zero; the first
//              chunk of a request also copies the request's incoming state (zero at position 0);
//   outputs:   a chunk folds the summaries of the chunks before it into its incoming state, walks
//              its rows again and writes them; a request's last chunk writes the state slot.
// Chunk c of the launch maps to (request, chunk of the request) by a walk over q_start.
constexpr int kScanChunk = 32;

__device__ __forceinline__ bool scan_chunk_of(const int32_t* __restrict__ q_start, int B, int item, int& b, int& first,
                                              int& r0, int& r1) {
  int rem = item;
  first = 0;
  for (b = 0; b < B; ++b) {
    const int n = q_start[b + 1] - q_start[b];
    const int chunks = (n + kScanChunk - 1) / kScanChunk;
    if (rem < chunks) {
      r0 = q_start[b] + rem * kScanChunk;
      r1 = min(r0 + kScanChunk, q_start[b + 1]);
      first = item - rem;
      return true;
    }
    rem -= chunks;
  }
  return false;
}

__global__ void mingru_chunk_summary_kernel(const float* __restrict__ pre, const float* __restrict__ bz,
                                            const float* __restrict__ bx, const float* __restrict__ state,
                                            const int32_t* __restrict__ q_start,
                                            const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                                            float* __restrict__ prod, float* __restrict__ end, float* __restrict__ init,
                                            int B, int W) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  int b, first, r0, r1;
  if (!scan_chunk_of(q_start, B, blockIdx.x, b, first, r0, r1) || c >= W) return;
  if (r0 == q_start[b])
    init[static_cast<size_t>(b) * W + c] = positions[r0] == 0 ? 0.f : state[static_cast<size_t>(slots[b]) * W + c];
  const float zb = bz[c], xb = bx[c];
  float P = 1.f, S = 0.f;
#pragma unroll 8
  for (int t = r0; t < r1; ++t) {
    const float* row = pre + static_cast<size_t>(t) * 3 * W;
    const float z = sigmoid_f(row[c] + zb);
    const float u = row[W + c] + xb;
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
    S = (1.0f - z) * S + z * cand;
    P *= 1.0f - z;
  }
  prod[static_cast<size_t>(blockIdx.x) * W + c] = P;
  end[static_cast<size_t>(blockIdx.x) * W + c] = S;
}

template <typename T>
__global__ void mingru_chunk_output_kernel(const float* __restrict__ pre, const float* __restrict__ bz,
                                           const float* __restrict__ bx, float* __restrict__ state,
                                           const int32_t* __restrict__ q_start, const int32_t* __restrict__ slots,
                                           const float* __restrict__ prod, const float* __restrict__ end,
                                           const float* __restrict__ init, T* __restrict__ out, int B, int W) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  int b, first, r0, r1;
  if (!scan_chunk_of(q_start, B, blockIdx.x, b, first, r0, r1) || c >= W) return;
  float S = init[static_cast<size_t>(b) * W + c];
  for (int k = first; k < static_cast<int>(blockIdx.x); ++k)
    S = prod[static_cast<size_t>(k) * W + c] * S + end[static_cast<size_t>(k) * W + c];
  const float zb = bz[c], xb = bx[c];
#pragma unroll 8
  for (int t = r0; t < r1; ++t) {
    const float* row = pre + static_cast<size_t>(t) * 3 * W;
    const float z = sigmoid_f(row[c] + zb);
    const float u = row[W + c] + xb;
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_f(u);
    S = (1.0f - z) * S + z * cand;
    const float g = row[2 * W + c];
    out[static_cast<size_t>(t) * W + c] = from_f32<T>(S * (g * sigmoid_f(g)));
  }
  if (r1 == q_start[b + 1]) state[static_cast<size_t>(slots[b]) * W + c] = S;
}

// ------------------------------------------------- around a latent attention
// d [rows, ld]: per token the query latent (q_rank values), the key/value latent
// (kv_rank) and the shared rotated key part (rot_dim), side by side.  Writes the
// RMS-normed query latent to cq [rows, q_rank], and the normed key/value latent
// followed by the key part, rotated by the token's position, into the token's
// page slot: pages [slot][kv_rank + rot_dim].  Pairs (2i, 2i+1) of the first
// `dims` values of the key part turn by the angle of table row `position`
// (dims/2 cosines, then dims/2 sines).
template <typename T>
__global__ void latent_prep_kernel(const T* __restrict__ d, int ld, const float* __restrict__ wq,
                                   const float* __restrict__ wkv, const int32_t* __restrict__ positions,
                                   const float* __restrict__ table, int dims, const int32_t* __restrict__ slot_map,
                                   T* __restrict__ cq, T* __restrict__ pages, int q_rank, int kv_rank, int rot_dim,
                                   float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = d + static_cast<size_t>(t) * ld;
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) {
    const float v = to_f32(row[i]);
    sq += v * v;
  }
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const float v = to_f32(row[q_rank + i]);
    sk += v * v;
  }
  sq = block_sum(sq, scratch);
  sk = block_sum(sk, scratch);
  const float inv_q = 1.0f / sqrtf(sq / static_cast<float>(q_rank) + eps);
  const float inv_k = 1.0f / sqrtf(sk / static_cast<float>(kv_rank) + eps);
  T* cqrow = cq + static_cast<size_t>(t) * q_rank;
  for (int i = threadIdx.x; i < q_rank; i += blockDim.x) cqrow[i] = from_f32<T>((to_f32(row[i]) * inv_q) * wq[i]);
  const int slot = slot_map[t];
  if (slot < 0) return;   // a padded row
  T* prow = pages + static_cast<size_t>(slot) * (kv_rank + rot_dim);
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x)
    prow[i] = from_f32<T>((to_f32(row[q_rank + i]) * inv_k) * wkv[i]);
  const T* kr = row + q_rank + kv_rank;
  const float* cs = table + static_cast<size_t>(positions[t]) * dims;
  const int half = dims / 2;
  for (int i = threadIdx.x; i < rot_dim / 2 + (rot_dim & 1); i += blockDim.x) {
    if (i < half) {
      float y1, y2;
      rotate_pair(to_f32(kr[2 * i]), to_f32(kr[2 * i + 1]), cs[i], cs[half + i], y1, y2);
      prow[kv_rank + 2 * i] = from_f32<T>(y1);
      prow[kv_rank + 2 * i + 1] = from_f32<T>(y2);
    } else {
      prow[kv_rank + 2 * i] = kr[2 * i];
      if (2 * i + 1 < rot_dim) prow[kv_rank + 2 * i + 1] = kr[2 * i + 1];
    }
  }
}

// q [rows, H (dim + rot_dim)]: per head the plain part, then the part to rotate.
// The rotated part goes to qa[row, head, kv_rank ..] of qa [rows, H, kv_rank + rot_dim]
// (the first kv_rank values of every head are written by a product).
template <typename T>
__global__ void latent_query_rotate_kernel(const T* __restrict__ q, const int32_t* __restrict__ positions,
                                           const float* __restrict__ table, int dims, T* __restrict__ qa, int H,
                                           int dim, int rot_dim, int kv_rank) {
  const int t = blockIdx.x;
  const float* cs = table + static_cast<size_t>(positions[t]) * dims;
  const int half = dims / 2;
  const int per = rot_dim / 2 + (rot_dim & 1);
  for (int idx = threadIdx.x; idx < H * per; idx += blockDim.x) {
    const int h = idx / per, i = idx % per;
    const T* src = q + (static_cast<size_t>(t) * H + h) * (dim + rot_dim) + dim;
    T* dst = qa + (static_cast<size_t>(t) * H + h) * (kv_rank + rot_dim) + kv_rank;
    if (i < half) {
      float y1, y2;
      rotate_pair(to_f32(src[2 * i]), to_f32(src[2 * i + 1]), cs[i], cs[half + i], y1, y2);
      dst[2 * i] = from_f32<T>(y1);
      dst[2 * i + 1] = from_f32<T>(y2);
    } else {
      dst[2 * i] = src[2 * i];
      if (2 * i + 1 < rot_dim) dst[2 * i + 1] = src[2 * i + 1];
    }
  }
}

// Attention of every row of the step over its request's latents in the pages,
// one shared key per token for all heads: key = the page row (Dk = kv_rank +
// rot_dim values), value = its first kv_rank values.  One workgroup per (row,
// head); blocks of keys: a thread a key for the scores, a thread a value column
// for the sums.  The softmax's denominator also holds exp(sink[head]).
// Sizes are run-time values; this is the kernel for sizes the matrix-core
// kernel does not take.
constexpr int kLatentBlock = 128;

template <typename T>
__global__ __launch_bounds__(kLatentBlock) void latent_attn_rows_kernel(
    const T* __restrict__ qa, const T* __restrict__ pages, const int32_t* __restrict__ block_tables, int table_width,
    int page_size, const int32_t* __restrict__ q_start, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ ctx_len, int B, const float* __restrict__ sink, float scale, T* __restrict__ out, int H,
    int kv_rank, int rot_dim) {
  extern __shared__ float smem[];
  const int Dk = kv_rank + rot_dim;
  float* qs = smem;                 // Dk
  float* ps = smem + Dk;            // kLatentBlock
  __shared__ float scratch[16];
  const int t = blockIdx.x, h = blockIdx.y;
  T* orow = out + (static_cast<size_t>(t) * H + h) * kv_rank;
  const int b = owner_of(q_start, B, t);
  if (t >= q_start[B] || ctx_len[b] <= 0) {   // a row that belongs to no request, or to a padded one
    for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) orow[i] = from_f32<T>(0.f);
    return;
  }
  const int n_keys = positions[t] + 1;
  const int32_t* table = block_tables + static_cast<size_t>(b) * table_width;
  const T* qrow = qa + (static_cast<size_t>(t) * H + h) * Dk;
  for (int i = threadIdx.x; i < Dk; i += blockDim.x) qs[i] = to_f32(qrow[i]);
  __syncthreads();
  // every thread owns value columns threadIdx.x, + blockDim.x, ... (at most 8 of them here)
  constexpr int kCols = 8;
  float acc[kCols];
#pragma unroll
  for (int v = 0; v < kCols; ++v) acc[v] = 0.f;
  float m = sink[h], l = 1.0f;      // the sink: a score without key or value
  for (int k0 = 0; k0 < n_keys; k0 += kLatentBlock) {
    const int j = k0 + threadIdx.x;
    float s = LYP_NEG_INF;
    if (j < n_keys) {
      const int page = table[j / page_size];
      if (page >= 0) {
        const T* krow = pages + (static_cast<size_t>(page) * page_size + j % page_size) * Dk;
        float dot = 0.f;
        for (int i = 0; i < Dk; ++i) dot += qs[i] * to_f32(krow[i]);
        s = dot * scale;
      }
    }
    const float m_new = fmaxf(m, block_max(s, scratch));
    const float p = s > LYP_NEG_INF ? expf(s - m_new) : 0.f;
    const float rescale = expf(m - m_new);
    const float psum = block_sum(p, scratch);
    l = l * rescale + psum;
    m = m_new;
    __syncthreads();
    ps[threadIdx.x] = p;
    __syncthreads();
    const int live = min(kLatentBlock, n_keys - k0);
#pragma unroll
    for (int v = 0; v < kCols; ++v) {
      const int col = threadIdx.x + v * kLatentBlock;
      if (col < kv_rank) {
        float a = acc[v] * rescale;
        for (int jj = 0; jj < live; ++jj) {
          const int key = k0 + jj;
          const int page = table[key / page_size];
          if (page >= 0)
            a += ps[jj] * to_f32(pages[(static_cast<size_t>(page) * page_size + key % page_size) * Dk + col]);
        }
        acc[v] = a;
      }
    }
  }
  const float inv = 1.0f / l;
#pragma unroll
  for (int v = 0; v < kCols; ++v) {
    const int col = threadIdx.x + v * kLatentBlock;
    if (col < kv_rank) orow[col] = from_f32<T>(acc[v] * inv);
  }
}

// h[row] += v for every row
__global__ void add_row_kernel(float* __restrict__ h, const float* __restrict__ v, int H, size_t total) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x)
    h[i] += v[i % H];
}

static int row_threads(int H) { return H >= 2048 ? 512 : (H >= 512 ? 256 : 128); }

}  // namespace lyp

using namespace lyp;

extern "C" {

// y of y_dtype (the activations' type or float), out of act_dtype; wb, shift, w_next float.
// conv_w (optional; float [H, taps]) with state [slots, taps - 1, H] of act_dtype, slots and positions
// [n_rows]: every row is a request that brings one token, and the short convolution of the normed row
// follows in the same kernel (rows in registers only: H a multiple of 4 up to 16384, aligned operands).
int lyp_branch_join(float* h, const void* y, int y_dtype, const float* wb, float mult, const float* shift,
                    const float* w_next, void* out, int act_dtype, const int32_t* rows, int n_rows, int H,
                    float eps_branch, float eps_next, const float* conv_w, void* state, const int32_t* slots,
                    const int32_t* positions, int taps, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && H > 0, "branch_join: bad sizes rows=%d H=%d", n_rows, H);
  LYP_REQUIRE(y == nullptr || wb != nullptr, "branch_join: a branch without its norm's weights");
  LYP_REQUIRE(w_next == nullptr || out != nullptr, "branch_join: a following norm without an output");
  LYP_REQUIRE(rows == nullptr || out != nullptr, "branch_join: selected rows go to an output");
  if (n_rows == 0) return 0;
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = H % 4 == 0 && H <= 16384 && aligned(h) && aligned(y) && aligned(wb) && aligned(shift) &&
                   aligned(w_next) && aligned(out) && aligned(state);
  const bool conv = conv_w != nullptr;
  if (out == nullptr) act_dtype = kF32;   // nothing is written: any instantiation will do
  LYP_REQUIRE(!conv || (vec && rows == nullptr && w_next != nullptr && taps >= 1 && slots != nullptr &&
                        positions != nullptr && (taps == 1 || state != nullptr)),
              "branch_join: the convolution follows only rows of up to 16384 values in steps of 4 that are all normed");
  const int nv = H / 4;
  const int vthreads = nv <= 64 ? 64 : (nv <= 128 ? 128 : (nv <= 1024 ? 256 : (nv <= 2048 ? 512 : 1024)));
#define LYP_JOIN(TY, T)                                                                                        \
  do {                                                                                                         \
    if (vec && conv)                                                                                           \
      branch_join_vec_kernel<TY, T, true><<<n_rows, vthreads, 0, stream>>>(                                    \
          h, static_cast<const TY*>(y), wb, mult, shift, w_next, static_cast<T*>(out), rows, H, eps_branch,    \
          eps_next, conv_w, static_cast<T*>(state), slots, positions, taps);                                   \
    else if (vec)                                                                                              \
      branch_join_vec_kernel<TY, T, false><<<n_rows, vthreads, 0, stream>>>(                                   \
          h, static_cast<const TY*>(y), wb, mult, shift, w_next, static_cast<T*>(out), rows, H, eps_branch,    \
          eps_next, nullptr, nullptr, nullptr, nullptr, 1);                                                    \
    else                                                                                                       \
      branch_join_kernel<TY, T><<<n_rows, row_threads(H), 0, stream>>>(                                        \
          h, static_cast<const TY*>(y), wb, mult, shift, w_next, static_cast<T*>(out), rows, H, eps_branch,    \
          eps_next);                                                                                           \
  } while (0)
  if (y_dtype == kF32 && act_dtype == kF32) LYP_JOIN(float, float);
  else if (y_dtype == kF32 && act_dtype == kBF16) LYP_JOIN(float, bf16_t);
  else if (y_dtype == kBF16 && act_dtype == kBF16) LYP_JOIN(bf16_t, bf16_t);
  else if (y_dtype == kBF16 && act_dtype == kF32) LYP_JOIN(bf16_t, float);
  else LYP_REQUIRE(false, "branch_join: unknown dtypes y=%d act=%d", y_dtype, act_dtype);
#undef LYP_JOIN
  LYP_LAUNCH_CHECK("branch_join");
  return 0;
}

int lyp_add_row(float* h, const float* v, int n_rows, int H, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && H > 0, "add_row: bad sizes rows=%d H=%d", n_rows, H);
  if (n_rows == 0) return 0;
  const size_t total = static_cast<size_t>(n_rows) * H;
  const int blocks = static_cast<int>(std::min<size_t>((total + 255) / 256, 4096));
  add_row_kernel<<<blocks, 256, 0, stream>>>(h, v, H, total);
  LYP_LAUNCH_CHECK("add_row");
  return 0;
}

// x [n_rows, >= C] (rows ldx apart), out [n_rows, C] and state [slots, taps - 1, C] of dtype; w float [C, taps];
// bias float [C] or null, added before the activation.
int lyp_short_conv(const void* x, const float* w, void* state, const int32_t* q_start, const int32_t* positions,
                   const int32_t* slots, void* out, int dtype, int n_rows, int B, int C, int taps, int residual,
                   int ldx, int act, const float* bias, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && B > 0 && C > 0 && taps >= 1, "short_conv: bad sizes rows=%d B=%d C=%d taps=%d", n_rows, B,
              C, taps);
  LYP_REQUIRE(taps == 1 || state != nullptr, "short_conv: %d taps need a state", taps);
  LYP_REQUIRE(x != out, "short_conv: in place is not possible");
  LYP_REQUIRE(ldx >= C && (act == 0 || act == 1), "short_conv: input rows %d apart for %d channels, activation %d", ldx, C, act);
  if (n_rows == 0) return 0;
  const int vlen = dtype == kF32 ? 4 : 8;
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if ((dtype == kF32 || dtype == kBF16) && C % vlen == 0 && ldx % vlen == 0 && taps <= kConvTaps && aligned(x) && aligned(out) &&
      aligned(state)) {
    const int units = C / vlen;
    const int vt = units >= 256 ? 256 : 64 * ((units + 63) / 64);
    dim3 vgrid((n_rows + kConvRows - 1) / kConvRows + B, (units + vt - 1) / vt);
    if (dtype == kF32)
      short_conv_vec_kernel<float><<<vgrid, vt, 0, stream>>>(static_cast<const float*>(x), w,
                                                             static_cast<float*>(state), q_start, positions, slots,
                                                             static_cast<float*>(out), n_rows, B, C, taps, residual, ldx, act, bias);
    else
      short_conv_vec_kernel<bf16_t><<<vgrid, vt, 0, stream>>>(static_cast<const bf16_t*>(x), w,
                                                              static_cast<bf16_t*>(state), q_start, positions, slots,
                                                              static_cast<bf16_t*>(out), n_rows, B, C, taps, residual, ldx, act, bias);
    LYP_LAUNCH_CHECK("short_conv");
    return 0;
  }
  const int threads = C >= 256 ? 256 : 64 * ((C + 63) / 64);
  dim3 grid(n_rows + B, (C + threads - 1) / threads);
  if (dtype == kF32)
    short_conv_kernel<float><<<grid, threads, 0, stream>>>(static_cast<const float*>(x), w, static_cast<float*>(state),
                                                           q_start, positions, slots, static_cast<float*>(out), n_rows,
                                                           B, C, taps, residual, ldx, act, bias);
  else if (dtype == kBF16)
    short_conv_kernel<bf16_t><<<grid, threads, 0, stream>>>(static_cast<const bf16_t*>(x), w,
                                                            static_cast<bf16_t*>(state), q_start, positions, slots,
                                                            static_cast<bf16_t*>(out), n_rows, B, C, taps, residual, ldx, act, bias);
  else
    LYP_REQUIRE(false, "short_conv: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("short_conv");
  return 0;
}

int lyp_activation(const void* in, void* out, int dtype, long long n, int kind, const float* params,
                   hipStream_t stream) {
  LYP_REQUIRE(n >= 0 && (kind == kXielu || kind == kGeluTanh), "activation: n=%lld kind=%d", n, kind);
  LYP_REQUIRE(kind != kXielu || params != nullptr, "activation: xIELU needs its two numbers");
  if (n == 0) return 0;
  const int per = dtype == kF32 ? 4 : 8;
  const int vec = n % per == 0 && reinterpret_cast<uintptr_t>(in) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0;
  const long long units = vec ? n / per : n;
  const int blocks = static_cast<int>(std::min<long long>((units + 255) / 256, 16384));
  if (dtype == kF32)
    activation_kernel<float><<<blocks, 256, 0, stream>>>(static_cast<const float*>(in), static_cast<float*>(out),
                                                         static_cast<size_t>(n), kind, params, vec);
  else if (dtype == kBF16)
    activation_kernel<bf16_t><<<blocks, 256, 0, stream>>>(static_cast<const bf16_t*>(in), static_cast<bf16_t*>(out),
                                                          static_cast<size_t>(n), kind, params, vec);
  else
    LYP_REQUIRE(false, "activation: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("activation");
  return 0;
}

// pre float [rows, 3 W]; out [rows, W] of out_dtype; state float [slots, W].
int lyp_mingru_scan(const float* pre, const float* bz, const float* bx, float* state, const int32_t* q_start,
                    const int32_t* positions, const int32_t* slots, void* out, int out_dtype, int B, int W,
                    hipStream_t stream) {
  LYP_REQUIRE(B > 0 && W > 0, "mingru_scan: bad sizes B=%d W=%d", B, W);
  const int threads = W >= 256 ? 256 : 64 * ((W + 63) / 64);
  dim3 grid(B, (W + threads - 1) / threads);
  if (out_dtype == kF32)
    mingru_scan_kernel<float><<<grid, threads, 0, stream>>>(pre, bz, bx, state, q_start, positions, slots,
                                                            static_cast<float*>(out), W);
  else if (out_dtype == kBF16)
    mingru_scan_kernel<bf16_t><<<grid, threads, 0, stream>>>(pre, bz, bx, state, q_start, positions, slots,
                                                             static_cast<bf16_t*>(out), W);
  else
    LYP_REQUIRE(false, "mingru_scan: unknown dtype %d", out_dtype);
  LYP_LAUNCH_CHECK("mingru_scan");
  return 0;
}

// The recurrence in chunks (see mingru_chunk_summary_kernel): n_rows rows of B requests; ws holds
// (2 * (n_rows / 32 rounded up + B) + B) * W floats.
int lyp_mingru_scan_chunks(const float* pre, const float* bz, const float* bx, float* state, const int32_t* q_start,
                           const int32_t* positions, const int32_t* slots, void* out, int out_dtype, int n_rows, int B,
                           int W, float* ws, long long ws_floats, hipStream_t stream) {
  LYP_REQUIRE(B > 0 && W > 0 && n_rows > 0, "mingru_scan_chunks: bad sizes rows=%d B=%d W=%d", n_rows, B, W);
  const int chunks = (n_rows + kScanChunk - 1) / kScanChunk + B;
  LYP_REQUIRE(ws != nullptr && ws_floats >= (2LL * chunks + B) * W, "mingru_scan_chunks: workspace of %lld floats",
              ws_floats);
  float* prod = ws;
  float* end = ws + static_cast<size_t>(chunks) * W;
  float* init = end + static_cast<size_t>(chunks) * W;
  const int threads = W >= 256 ? 256 : 64 * ((W + 63) / 64);
  dim3 grid(chunks, (W + threads - 1) / threads);
  mingru_chunk_summary_kernel<<<grid, threads, 0, stream>>>(pre, bz, bx, state, q_start, positions, slots, prod, end,
                                                            init, B, W);
  if (out_dtype == kF32)
    mingru_chunk_output_kernel<float><<<grid, threads, 0, stream>>>(pre, bz, bx, state, q_start, slots, prod, end, init,
                                                                    static_cast<float*>(out), B, W);
  else if (out_dtype == kBF16)
    mingru_chunk_output_kernel<bf16_t><<<grid, threads, 0, stream>>>(pre, bz, bx, state, q_start, slots, prod, end,
                                                                     init, static_cast<bf16_t*>(out), B, W);
  else
    LYP_REQUIRE(false, "mingru_scan_chunks: unknown dtype %d", out_dtype);
  LYP_LAUNCH_CHECK("mingru_scan_chunks");
  return 0;
}

int lyp_latent_prep(const void* d, int ld, const float* wq, const float* wkv, const int32_t* positions,
                    const float* table, int dims, const int32_t* slot_map, void* cq, void* pages, int dtype,
                    int n_rows, int q_rank, int kv_rank, int rot_dim, float eps, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && q_rank > 0 && kv_rank > 0 && rot_dim >= 0 && ld >= q_rank + kv_rank + rot_dim,
              "latent_prep: bad sizes rows=%d q_rank=%d kv_rank=%d rot=%d ld=%d", n_rows, q_rank, kv_rank, rot_dim, ld);
  LYP_REQUIRE(dims >= 0 && dims % 2 == 0 && dims <= rot_dim && (dims == 0 || table != nullptr),
              "latent_prep: %d rotated dimensions of %d", dims, rot_dim);
  if (n_rows == 0) return 0;
  const int threads = row_threads(std::max(q_rank, kv_rank));
#define LYP_PREP(T)                                                                                           \
  latent_prep_kernel<T><<<n_rows, threads, 0, stream>>>(static_cast<const T*>(d), ld, wq, wkv, positions,     \
                                                        table, dims, slot_map, static_cast<T*>(cq),           \
                                                        static_cast<T*>(pages), q_rank, kv_rank, rot_dim, eps)
  if (dtype == kF32) LYP_PREP(float);
  else if (dtype == kBF16) LYP_PREP(bf16_t);
  else LYP_REQUIRE(false, "latent_prep: unknown dtype %d", dtype);
#undef LYP_PREP
  LYP_LAUNCH_CHECK("latent_prep");
  return 0;
}

int lyp_latent_query_rotate(const void* q, const int32_t* positions, const float* table, int dims, void* qa,
                            int dtype, int n_rows, int H, int dim, int rot_dim, int kv_rank, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && H > 0 && dim >= 0 && rot_dim >= 0 && kv_rank > 0, "latent_query_rotate: bad sizes");
  LYP_REQUIRE(dims >= 0 && dims % 2 == 0 && dims <= rot_dim && (dims == 0 || table != nullptr),
              "latent_query_rotate: %d rotated dimensions of %d", dims, rot_dim);
  if (n_rows == 0 || rot_dim == 0) return 0;
  const int threads = 128;
  if (dtype == kF32)
    latent_query_rotate_kernel<float><<<n_rows, threads, 0, stream>>>(static_cast<const float*>(q), positions, table,
                                                                      dims, static_cast<float*>(qa), H, dim, rot_dim,
                                                                      kv_rank);
  else if (dtype == kBF16)
    latent_query_rotate_kernel<bf16_t><<<n_rows, threads, 0, stream>>>(static_cast<const bf16_t*>(q), positions, table,
                                                                       dims, static_cast<bf16_t*>(qa), H, dim, rot_dim,
                                                                       kv_rank);
  else
    LYP_REQUIRE(false, "latent_query_rotate: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("latent_query_rotate");
  return 0;
}

int lyp_latent_attn_rows(const void* qa, const void* pages, const int32_t* block_tables, int table_width,
                         int page_size, const int32_t* q_start, const int32_t* positions, const int32_t* ctx_len,
                         int B, const float* sink, float scale, void* out, int dtype, int n_rows, int H, int kv_rank,
                         int rot_dim, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && B > 0 && H > 0 && kv_rank > 0 && rot_dim >= 0 && page_size > 0 && table_width > 0,
              "latent_attn_rows: bad sizes");
  LYP_REQUIRE(kv_rank <= 8 * kLatentBlock, "latent_attn_rows: latents of up to %d values, not %d", 8 * kLatentBlock,
              kv_rank);
  if (n_rows == 0) return 0;
  const size_t lds = sizeof(float) * (kv_rank + rot_dim + kLatentBlock);
  dim3 grid(n_rows, H);
  if (dtype == kF32)
    latent_attn_rows_kernel<float><<<grid, kLatentBlock, lds, stream>>>(
        static_cast<const float*>(qa), static_cast<const float*>(pages), block_tables, table_width, page_size, q_start,
        positions, ctx_len, B, sink, scale, static_cast<float*>(out), H, kv_rank, rot_dim);
  else if (dtype == kBF16)
    latent_attn_rows_kernel<bf16_t><<<grid, kLatentBlock, lds, stream>>>(
        static_cast<const bf16_t*>(qa), static_cast<const bf16_t*>(pages), block_tables, table_width, page_size,
        q_start, positions, ctx_len, B, sink, scale, static_cast<bf16_t*>(out), H, kv_rank, rot_dim);
  else
    LYP_REQUIRE(false, "latent_attn_rows: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("latent_attn_rows");
  return 0;
}

}  // extern "C"
