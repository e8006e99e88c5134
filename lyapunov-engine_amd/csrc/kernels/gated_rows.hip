// Row-wise kernels for layers with grouped norms, scaled branches and gates.
// All arithmetic is 32-bit (angles 64-bit); only loads and stores see the
// storage type.
//
//   * group_rmsnorm: h += scale * delta (a vector times what a branch left to be added, summed
//     over its partial sums), then every one of `groups` equal consecutive parts of the row divided
//     by its own root mean square, the whole times w.  With `rows` only those rows are normed and h
//     is left alone; without an output only the sum is carried out.
//   * add_sinusoid: h[t, 2i] += sin(p_t f_i), h[t, 2i+1] += cos(p_t f_i), f_i = base^(-2i / H); the
//     angle is formed and reduced in 64-bit, so that a far position costs no digits.
//   * glu_act: [rows, 2 I] (gates, then ups) -> act(gate) * up, act = silu or the tanh form of gelu.
//   * gate_mul: x *= sigmoid(gate) or silu(gate), the gate a column range of a wider tensor.
//   * weighted_sum: out = sa * (a + bias) + sb * b as float partial sums for the residual stream.
//   * qkv_bias_temper_kv: from a float projection [q | k | v | ...]: biases added, every query
//     multiplied by 1 + coef * ln(floor((p + 1) / every) + 1), queries out in the activations'
//     type, keys and values into the token's page slot (keys [page][kv head][slot][dim], values
//     [page][kv head][vdim][slot]).
#include <algorithm>

#include "common.h"

namespace lyp {

template <typename TD, typename T>
__global__ __launch_bounds__(256) void group_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                            int n_parts, size_t part_stride,
                                                            const float* __restrict__ scale,
                                                            const float* __restrict__ w, T* __restrict__ out,
                                                            const int32_t* __restrict__ rows, int H, int groups,
                                                            float eps, int stage_w) {
  extern __shared__ float s_group[];   // the row, a float per wave, then (stage_w) the norm's weights
  float* srow = s_group;
  float* scratch = s_group + H;
  float* sw = s_group + H + 16;
  const int r = blockIdx.x;
  const size_t src = rows != nullptr ? static_cast<size_t>(rows[r]) : static_cast<size_t>(r);
  float* hrow = h + src * H;
  // eight values a thread at a time, their loads all issued before the first is used
  constexpr int U = 8;
  for (int i0 = threadIdx.x; i0 < H; i0 += U * blockDim.x) {
    float hv[U], dv[U], sv[U], wv[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * blockDim.x;
      const bool in = i < H;
      hv[u] = in ? hrow[i] : 0.f;
      dv[u] = (in && delta != nullptr) ? to_f32(delta[src * H + i]) : 0.f;
      sv[u] = (in && delta != nullptr && scale != nullptr) ? scale[i] : 1.f;
      wv[u] = (in && stage_w && out != nullptr) ? w[i] : 0.f;
    }
    if (delta != nullptr) {
      for (int p = 1; p < n_parts; ++p) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int i = i0 + u * blockDim.x;
          if (i < H) dv[u] += to_f32(delta[p * part_stride + src * H + i]);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + u * blockDim.x;
      if (i >= H) continue;
      float v = hv[u];
      if (delta != nullptr) {
        v += dv[u] * sv[u];
        if (rows == nullptr) hrow[i] = v;
      }
      srow[i] = v;
      if (stage_w && out != nullptr) sw[i] = wv[u];
    }
  }
  if (out == nullptr) return;
  const float* wn = stage_w ? sw : w;
  const int gs = H / groups;
  T* orow = out + static_cast<size_t>(r) * H;
  const int waves = blockDim.x / kWave;
  if (groups >= waves) {
    // a wave a group at a time: no workgroup-wide sums, and a group's sum does not depend on the others
    __syncthreads();
    const int lane = threadIdx.x % kWave;
    for (int g = threadIdx.x / kWave; g < groups; g += waves) {
      const float* sg = srow + g * gs;
      float ss = 0.f;
      for (int i = lane; i < gs; i += kWave) ss += sg[i] * sg[i];
      const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(gs) + eps);
      for (int i = lane; i < gs; i += kWave) orow[g * gs + i] = from_f32<T>(sg[i] * inv * wn[g * gs + i]);
    }
    return;
  }
  for (int g = 0; g < groups; ++g) {
    float ss = 0.f;
    __syncthreads();
    for (int i = threadIdx.x; i < gs; i += blockDim.x) ss += srow[g * gs + i] * srow[g * gs + i];
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / static_cast<float>(gs) + eps);
    for (int i = threadIdx.x; i < gs; i += blockDim.x)
      orow[g * gs + i] = from_f32<T>(srow[g * gs + i] * inv * wn[g * gs + i]);
  }
}

__global__ void add_sinusoid_kernel(float* __restrict__ h, const int32_t* __restrict__ positions, int H, size_t total,
                                    double log_base) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / H;
  const int c = static_cast<int>(idx % H);
  const double f = exp(-log_base * static_cast<double>(c & ~1) / static_cast<double>(H));
  const double ang = static_cast<double>(positions[t]) * f;
  h[idx] += static_cast<float>((c & 1) ? cos(ang) : sin(ang));
}

enum GluAct : int { kGluSilu = 0, kGluGeluTanh = 1 };

__device__ __forceinline__ float glu_act_f(float g, int act) {
  if (act == kGluSilu) return g / (1.0f + expf(-g));
  return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
}

template <typename T>
__global__ void glu_act_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total, int act) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / I, i = idx % I;
  out[idx] = from_f32<T>(glu_act_f(to_f32(gu[t * 2 * I + i]), act) * to_f32(gu[t * 2 * I + I + i]));
}

// eight outputs a thread with 16-byte accesses: I a multiple of eight, aligned operands
template <typename T>
__global__ void glu_act_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total8, int act) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T VecT __attribute__((ext_vector_type(VEC)));
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total8) return;
  const size_t per_row = I / 8, t = idx / per_row, c = idx % per_row;
  const T* gp = gu + t * 2 * I + c * 8;
  const T* up = gp + I;
  T* op = out + t * I + c * 8;
#pragma unroll
  for (int s = 0; s < 8 / VEC; ++s) {
    const VecT g = *reinterpret_cast<const VecT*>(gp + s * VEC);
    const VecT u = *reinterpret_cast<const VecT*>(up + s * VEC);
    VecT o;
#pragma unroll
    for (int e = 0; e < VEC; ++e) o[e] = from_f32<T>(glu_act_f(to_f32(g[e]), act) * to_f32(u[e]));
    *reinterpret_cast<VecT*>(op + s * VEC) = o;
  }
}

template <typename TG, typename T>
__global__ void gate_mul_kernel(T* __restrict__ x, const TG* __restrict__ gate, int ldg, int N, size_t total,
                                int kind, int per) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / N, c = idx % N;
  const float g = to_f32(gate[t * ldg + c / per]);   // one gate value for `per` neighbours (a head's values)
  const float s = 1.0f / (1.0f + expf(-g));
  x[idx] = from_f32<T>(to_f32(x[idx]) * (kind == 1 ? g * s : s));
}

template <typename TA, typename TB>
__global__ void weighted_sum_kernel(const TA* __restrict__ a, const float* __restrict__ bias, float sa,
                                    const TB* __restrict__ b, float sb, float* __restrict__ out, int H,
                                    size_t total) {
  const size_t idx = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  float x = to_f32(a[idx]);
  if (bias != nullptr) x += bias[idx % H];
  out[idx] = sa * x + sb * to_f32(b[idx]);
}

template <typename T>
__global__ __launch_bounds__(256) void qkv_bias_temper_kv_kernel(
    const float* __restrict__ pre, int ld, const float* __restrict__ bias, const int32_t* __restrict__ positions,
    float coef, int every, const int32_t* __restrict__ slot_map, T* __restrict__ q_out, T* __restrict__ kpool,
    T* __restrict__ vpool, int H, int G, int D, int V, int bs) {
  const int t = blockIdx.x;
  const float* row = pre + static_cast<size_t>(t) * ld;
  const int nq = H * D, nk = G * D, nv = G * V;
  const int p = positions[t];
  const float temper = 1.0f + coef * logf(static_cast<float>((p + 1) / every) + 1.0f);
  for (int i = threadIdx.x; i < nq; i += blockDim.x)
    q_out[static_cast<size_t>(t) * nq + i] = from_f32<T>((row[i] + (bias != nullptr ? bias[i] : 0.f)) * temper);
  const int slot = slot_map[t];
  if (slot < 0) return;   // a padded row
  const int page = slot / bs, off = slot % bs;
  for (int i = threadIdx.x; i < nk; i += blockDim.x) {
    const int g = i / D, d = i % D;
    kpool[((static_cast<size_t>(page) * G + g) * bs + off) * D + d] =
        from_f32<T>(row[nq + i] + (bias != nullptr ? bias[nq + i] : 0.f));
  }
  for (int i = threadIdx.x; i < nv; i += blockDim.x) {
    const int g = i / V, d = i % V;
    vpool[((static_cast<size_t>(page) * G + g) * V + d) * bs + off] =
        from_f32<T>(row[nq + nk + i] + (bias != nullptr ? bias[nq + nk + i] : 0.f));
  }
}

}  // namespace lyp

using namespace lyp;

extern "C" {

// h float [*, H]; delta (optional): one tensor [*, H] of delta_dtype (delta_parts == 0) or delta_parts float
// tensors part_stride elements apart; scale (optional) float [H]; w float [H]; out (optional) [n_rows, H] of
// out_dtype; rows (optional) int32 [n_rows].
int lyp_group_rmsnorm(float* h, const void* delta, int delta_dtype, int delta_parts, long long part_stride,
                      const float* scale, const float* w, void* out, int out_dtype, const int32_t* rows, int n_rows,
                      int H, int groups, float eps, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && H > 0 && groups > 0 && H % groups == 0, "group_rmsnorm: rows=%d H=%d groups=%d", n_rows, H,
              groups);
  LYP_REQUIRE(H <= 15872, "group_rmsnorm: rows of up to 15872 values, not %d", H);
  LYP_REQUIRE(out == nullptr || w != nullptr, "group_rmsnorm: an output needs the norm's weights");
  LYP_REQUIRE(delta_parts == 0 || delta_dtype == kF32, "group_rmsnorm: partial sums are float");
  if (n_rows == 0) return 0;
  const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
  const int stage_w = (2 * static_cast<size_t>(H) + 16) * sizeof(float) <= 65536;
  const size_t lds = (static_cast<size_t>(stage_w ? 2 * H : H) + 16) * sizeof(float);
  const int parts = delta_parts == 0 ? 1 : delta_parts;
#define LYP_GN(TD, T)                                                                                              \
  group_rmsnorm_kernel<TD, T><<<n_rows, threads, lds, stream>>>(h, static_cast<const TD*>(delta), parts,           \
                                                               static_cast<size_t>(part_stride), scale, w,        \
                                                               static_cast<T*>(out), rows, H, groups, eps, stage_w)
  const bool dbf = delta != nullptr && delta_dtype == kBF16;
  if (out_dtype == kBF16 && out != nullptr) {
    if (dbf) LYP_GN(bf16_t, bf16_t);
    else LYP_GN(float, bf16_t);
  } else {
    if (dbf) LYP_GN(bf16_t, float);
    else LYP_GN(float, float);
  }
#undef LYP_GN
  LYP_LAUNCH_CHECK("group_rmsnorm");
  return 0;
}

int lyp_add_sinusoid(float* h, const int32_t* positions, int T, int H, double base, hipStream_t stream) {
  LYP_REQUIRE(T >= 0 && H > 0 && base > 0.0, "add_sinusoid: T=%d H=%d base=%g", T, H, base);
  if (T == 0) return 0;
  const size_t total = static_cast<size_t>(T) * H;
  add_sinusoid_kernel<<<static_cast<unsigned>((total + 255) / 256), 256, 0, stream>>>(h, positions, H, total, log(base));
  LYP_LAUNCH_CHECK("add_sinusoid");
  return 0;
}

int lyp_glu_act(const void* gate_up, void* out, int dtype, int T, int I, int act, hipStream_t stream) {
  LYP_REQUIRE(T >= 0 && I > 0 && (act == kGluSilu || act == kGluGeluTanh), "glu_act: T=%d I=%d act=%d", T, I, act);
  if (T == 0) return 0;
  const int threads = 256;
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (I % 8 == 0 && aligned(gate_up) && aligned(out)) {
    const size_t total8 = static_cast<size_t>(T) * (I / 8);
    const unsigned blocks = static_cast<unsigned>((total8 + threads - 1) / threads);
    if (dtype == kF32)
      glu_act_vec_kernel<float><<<blocks, threads, 0, stream>>>(static_cast<const float*>(gate_up), static_cast<float*>(out), I, total8, act);
    else if (dtype == kBF16)
      glu_act_vec_kernel<bf16_t><<<blocks, threads, 0, stream>>>(static_cast<const bf16_t*>(gate_up), static_cast<bf16_t*>(out), I, total8, act);
    else
      LYP_REQUIRE(false, "glu_act: unknown dtype %d", dtype);
    LYP_LAUNCH_CHECK("glu_act");
    return 0;
  }
  const size_t total = static_cast<size_t>(T) * I;
  const unsigned blocks = static_cast<unsigned>((total + threads - 1) / threads);
  if (dtype == kF32)
    glu_act_kernel<float><<<blocks, threads, 0, stream>>>(static_cast<const float*>(gate_up), static_cast<float*>(out), I, total, act);
  else if (dtype == kBF16)
    glu_act_kernel<bf16_t><<<blocks, threads, 0, stream>>>(static_cast<const bf16_t*>(gate_up), static_cast<bf16_t*>(out), I, total, act);
  else
    LYP_REQUIRE(false, "glu_act: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("glu_act");
  return 0;
}

// x [T, N] of dtype; gate [T, >= N / per] (ldg apart) float (gate_dtype kF32) or of x's type, one value for
// every `per` neighbouring values of x; kind 0 sigmoid, 1 silu.
int lyp_gate_mul(void* x, int dtype, const void* gate, int ldg, int gate_dtype, int T, int N, int kind, int per,
                 hipStream_t stream) {
  LYP_REQUIRE(T >= 0 && N > 0 && per > 0 && N % per == 0 && ldg >= N / per && (kind == 0 || kind == 1),
              "gate_mul: T=%d N=%d ldg=%d kind=%d per=%d", T, N, ldg, kind, per);
  LYP_REQUIRE(gate_dtype == kF32 || gate_dtype == dtype, "gate_mul: the gate is float or of x's type");
  if (T == 0) return 0;
  const size_t total = static_cast<size_t>(T) * N;
  const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
  if (dtype == kF32)
    gate_mul_kernel<float, float><<<blocks, 256, 0, stream>>>(static_cast<float*>(x), static_cast<const float*>(gate), ldg, N, total, kind, per);
  else if (dtype == kBF16 && gate_dtype == kF32)
    gate_mul_kernel<float, bf16_t><<<blocks, 256, 0, stream>>>(static_cast<bf16_t*>(x), static_cast<const float*>(gate), ldg, N, total, kind, per);
  else if (dtype == kBF16)
    gate_mul_kernel<bf16_t, bf16_t><<<blocks, 256, 0, stream>>>(static_cast<bf16_t*>(x), static_cast<const bf16_t*>(gate), ldg, N, total, kind, per);
  else
    LYP_REQUIRE(false, "gate_mul: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("gate_mul");
  return 0;
}

// out float [T, H] = sa * (a + bias) + sb * b; a and b [T, H] float or bfloat16 each; bias float [H] or null.
int lyp_weighted_sum(const void* a, int a_dtype, const float* bias, float sa, const void* b, int b_dtype, float sb,
                     float* out, int T, int H, hipStream_t stream) {
  LYP_REQUIRE(T >= 0 && H > 0, "weighted_sum: T=%d H=%d", T, H);
  if (T == 0) return 0;
  const size_t total = static_cast<size_t>(T) * H;
  const unsigned blocks = static_cast<unsigned>((total + 255) / 256);
#define LYP_WS(TA, TB)                                                                                            \
  weighted_sum_kernel<TA, TB><<<blocks, 256, 0, stream>>>(static_cast<const TA*>(a), bias, sa,                    \
                                                          static_cast<const TB*>(b), sb, out, H, total)
  if (a_dtype == kF32 && b_dtype == kF32) LYP_WS(float, float);
  else if (a_dtype == kF32 && b_dtype == kBF16) LYP_WS(float, bf16_t);
  else if (a_dtype == kBF16 && b_dtype == kF32) LYP_WS(bf16_t, float);
  else if (a_dtype == kBF16 && b_dtype == kBF16) LYP_WS(bf16_t, bf16_t);
  else LYP_REQUIRE(false, "weighted_sum: unknown dtypes %d %d", a_dtype, b_dtype);
#undef LYP_WS
  LYP_LAUNCH_CHECK("weighted_sum");
  return 0;
}

// pre float [T, >= (H + G) D + G V] (ld apart); bias float [(H + G) D + G V] or null; q_out [T, H D] of dtype;
// pools of dtype: keys [pages, G, bs, D], values [pages, G, V, bs]; slot_map int32 [T] (-1: nothing stored).
int lyp_qkv_bias_temper_kv(const float* pre, int ld, const float* bias, const int32_t* positions, float coef,
                           int every, const int32_t* slot_map, void* q_out, void* kpool, void* vpool, int dtype, int T,
                           int H, int G, int D, int V, int bs, hipStream_t stream) {
  LYP_REQUIRE(T >= 0 && H > 0 && G > 0 && D > 0 && V > 0 && bs > 0 && every >= 1 && ld >= (H + G) * D + G * V,
              "qkv_bias_temper_kv: T=%d H=%d G=%d D=%d V=%d bs=%d every=%d ld=%d", T, H, G, D, V, bs, every, ld);
  if (T == 0) return 0;
  const int threads = H * D >= 1024 ? 256 : 128;
  if (dtype == kF32)
    qkv_bias_temper_kv_kernel<float><<<T, threads, 0, stream>>>(pre, ld, bias, positions, coef, every, slot_map,
                                                                static_cast<float*>(q_out), static_cast<float*>(kpool),
                                                                static_cast<float*>(vpool), H, G, D, V, bs);
  else if (dtype == kBF16)
    qkv_bias_temper_kv_kernel<bf16_t><<<T, threads, 0, stream>>>(pre, ld, bias, positions, coef, every, slot_map,
                                                                 static_cast<bf16_t*>(q_out), static_cast<bf16_t*>(kpool),
                                                                 static_cast<bf16_t*>(vpool), H, G, D, V, bs);
  else
    LYP_REQUIRE(false, "qkv_bias_temper_kv: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("qkv_bias_temper_kv");
  return 0;
}

}  // extern "C"
