// Row-wise kernels around recurrent mixers and token-gated branches:
//
//   * shift_mix: n_mix blends of every row with the row before it in its request,
//     out[s][t] = x[t] + (x[t-1] - x[t]) * mu[s], where x[-1] is the request's last row of the
//     step before (its state slot; zeros for a request at position 0).  The slot then takes the
//     request's last row of this step.
//   * skip_gate_group_norm: y = (o + skip[head] * x) * silu(z), then an RMS norm of y in equal
//     consecutive groups times a weight: what follows a state-space scan.
//   * gather_gelu_mul: out[t] = gelu_tanh(p[t]) * table[token[t]]: a small projection of the stream gated
//     by a row that the token itself picks.
//
// Arithmetic is 32-bit; loads and stores see the storage type.
#include <algorithm>

#include "common.h"

namespace lyp {

__device__ __forceinline__ int rows_owner(const int32_t* __restrict__ q_start, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] <= t) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

// Work items along x: one per row, then one per request.  A request's item does its first row (the
// one that reads the slot) and then rewrites the slot, so that nobody reads a slot while it changes.
template <typename T>
__global__ void shift_mix_kernel(const T* __restrict__ x, int ldx, const float* __restrict__ mu, int n_mix,
                                 T* __restrict__ state, const int32_t* __restrict__ q_start,
                                 const int32_t* __restrict__ positions, const int32_t* __restrict__ slots,
                                 T* __restrict__ out, int n_rows, int B, int C) {
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int item = blockIdx.x;
  const size_t plane = static_cast<size_t>(n_rows) * C;
  int t;
  float cur, prev;
  if (item < n_rows) {
    t = item;
    if (t >= q_start[B]) {   // rows past the last request belong to nobody
      for (int s = 0; s < n_mix; ++s) out[s * plane + static_cast<size_t>(t) * C + c] = from_f32<T>(0.f);
      return;
    }
    const int b = rows_owner(q_start, B, t);
    if (t == q_start[b]) return;   // the request's item does this row
    cur = to_f32(x[static_cast<size_t>(t) * ldx + c]);
    prev = to_f32(x[static_cast<size_t>(t - 1) * ldx + c]);
  } else {
    const int b = item - n_rows;
    const int q0 = q_start[b], n = q_start[b + 1] - q0;
    if (n <= 0) return;
    t = q0;
    T* st = state + static_cast<size_t>(slots[b]) * C + c;
    cur = to_f32(x[static_cast<size_t>(t) * ldx + c]);
    prev = positions[q0] == 0 ? 0.f : to_f32(*st);
    *st = x[static_cast<size_t>(q0 + n - 1) * ldx + c];
  }
  for (int s = 0; s < n_mix; ++s)
    out[s * plane + static_cast<size_t>(t) * C + c] = from_f32<T>(cur + (prev - cur) * mu[static_cast<size_t>(s) * C + c]);
}

// One workgroup per (row, group).
template <typename T>
__global__ __launch_bounds__(256) void skip_gate_group_norm_kernel(
    const float* __restrict__ o, const T* __restrict__ x, int ldx, const float* __restrict__ skip,
    const T* __restrict__ z, int ldz, const float* __restrict__ w, T* __restrict__ out, int N, int V, int groups,
    float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, g = blockIdx.y;
  const int per = N / groups;
  const int base = g * per;
  auto value = [&](int i) {
    const int e = base + i;
    const float zz = to_f32(z[static_cast<size_t>(t) * ldz + e]);
    const float y = o[static_cast<size_t>(t) * N + e] + skip[e / V] * to_f32(x[static_cast<size_t>(t) * ldx + e]);
    return y * (zz / (1.0f + expf(-zz)));
  };
  float ss = 0.f;
  for (int i = threadIdx.x; i < per; i += blockDim.x) {
    const float v = value(i);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / static_cast<float>(per) + eps);
  for (int i = threadIdx.x; i < per; i += blockDim.x)
    out[static_cast<size_t>(t) * N + base + i] = from_f32<T>(value(i) * inv * w[base + i]);
}

template <typename TP, typename T>
__global__ void gather_gelu_mul_kernel(const TP* __restrict__ p, int ldp, const int32_t* __restrict__ tokens,
                                       const T* __restrict__ table, int ldt, int vocab, T* __restrict__ out, int N,
                                       size_t total) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / N;
  const int j = static_cast<int>(idx % N);
  const int tok = tokens[t];
  const float zz = to_f32(p[t * ldp + j]);
  const float act = 0.5f * zz * (1.0f + tanhf(0.7978845608028654f * (zz + 0.044715f * zz * zz * zz)));
  const float e = (tok >= 0 && tok < vocab) ? to_f32(table[static_cast<size_t>(tok) * ldt + j]) : 0.f;
  out[idx] = from_f32<T>(act * e);
}

}  // namespace lyp

using namespace lyp;

extern "C" {

// x [n_rows, >= C] (ldx apart), state [slots, C] and out [n_mix, n_rows, C] of dtype; mu float [n_mix, C].
int lyp_shift_mix(const void* x, int ldx, const float* mu, int n_mix, void* state, const int32_t* q_start,
                  const int32_t* positions, const int32_t* slots, void* out, int dtype, int n_rows, int B, int C,
                  hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && B > 0 && C > 0 && n_mix > 0 && ldx >= C, "shift_mix: rows=%d B=%d C=%d mixes=%d ldx=%d", n_rows, B,
              C, n_mix, ldx);
  LYP_REQUIRE(state != nullptr && x != out, "shift_mix: needs a state and an output of its own");
  if (n_rows == 0) return 0;
  const int threads = C >= 256 ? 256 : 64 * ((C + 63) / 64);
  dim3 grid(n_rows + B, (C + threads - 1) / threads);
  if (dtype == kF32)
    shift_mix_kernel<float><<<grid, threads, 0, stream>>>(static_cast<const float*>(x), ldx, mu, n_mix,
                                                          static_cast<float*>(state), q_start, positions, slots,
                                                          static_cast<float*>(out), n_rows, B, C);
  else if (dtype == kBF16)
    shift_mix_kernel<bf16_t><<<grid, threads, 0, stream>>>(static_cast<const bf16_t*>(x), ldx, mu, n_mix,
                                                           static_cast<bf16_t*>(state), q_start, positions, slots,
                                                           static_cast<bf16_t*>(out), n_rows, B, C);
  else
    LYP_REQUIRE(false, "shift_mix: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("shift_mix");
  return 0;
}

// o float [rows, N]; x and z [rows, >= N] (ldx / ldz apart) and out [rows, N] of dtype; skip float [N / V]; w float [N].
int lyp_skip_gate_group_norm(const float* o, const void* x, int ldx, const float* skip, const void* z, int ldz,
                             const float* w, void* out, int dtype, int rows, int N, int V, int groups, float eps,
                             hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && N > 0 && V > 0 && N % V == 0 && groups > 0 && N % groups == 0 && ldx >= N && ldz >= N,
              "skip_gate_group_norm: rows=%d N=%d V=%d groups=%d", rows, N, V, groups);
  LYP_REQUIRE(groups <= 65535, "skip_gate_group_norm: too many groups for one launch");
  if (rows == 0) return 0;
  const int per = N / groups;
  const int threads = per >= 1024 ? 256 : (per >= 256 ? 128 : 64);
  dim3 grid(rows, groups);
  if (dtype == kF32)
    skip_gate_group_norm_kernel<float><<<grid, threads, 0, stream>>>(o, static_cast<const float*>(x), ldx, skip,
                                                                     static_cast<const float*>(z), ldz, w,
                                                                     static_cast<float*>(out), N, V, groups, eps);
  else if (dtype == kBF16)
    skip_gate_group_norm_kernel<bf16_t><<<grid, threads, 0, stream>>>(o, static_cast<const bf16_t*>(x), ldx, skip,
                                                                      static_cast<const bf16_t*>(z), ldz, w,
                                                                      static_cast<bf16_t*>(out), N, V, groups, eps);
  else
    LYP_REQUIRE(false, "skip_gate_group_norm: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("skip_gate_group_norm");
  return 0;
}

// p [rows, >= N] (ldp apart) float (p_dtype kF32) or of dtype; tokens int32 [rows]; table [vocab, >= N] (ldt apart)
// and out [rows, N] of dtype.
int lyp_gather_gelu_mul(const void* p, int ldp, int p_dtype, const int32_t* tokens, const void* table, int ldt,
                        int vocab, void* out, int dtype, int rows, int N, hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && N > 0 && ldp >= N && ldt >= N && vocab > 0, "gather_gelu_mul: rows=%d N=%d", rows, N);
  LYP_REQUIRE(p_dtype == kF32 || p_dtype == dtype, "gather_gelu_mul: the projection is float or of the output's type");
  if (rows == 0) return 0;
  const size_t total = static_cast<size_t>(rows) * N;
  const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
#define LYP_GGM(TP, T)                                                                                               \
  gather_gelu_mul_kernel<TP, T><<<blocks, 256, 0, stream>>>(static_cast<const TP*>(p), ldp, tokens,                   \
                                                            static_cast<const T*>(table), ldt, vocab,                 \
                                                            static_cast<T*>(out), N, total)
  if (dtype == kF32) LYP_GGM(float, float);
  else if (dtype == kBF16 && p_dtype == kF32) LYP_GGM(float, bf16_t);
  else if (dtype == kBF16) LYP_GGM(bf16_t, bf16_t);
  else LYP_REQUIRE(false, "gather_gelu_mul: unknown dtype %d", dtype);
#undef LYP_GGM
  LYP_LAUNCH_CHECK("gather_gelu_mul");
  return 0;
}

}  // extern "C"
