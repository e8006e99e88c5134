// What an attention layer with normed projections, a rotation of neighbouring
// pairs, a window that keeps a sequence's first tokens and a sink in the
// softmax needs around the matrix products, with every size a run-time value:
//
//   * qk_norm_rope_kv: one RMS norm over a token's whole query projection and one
//     over its whole key projection (all heads' rows at once), rotation of the
//     pairs (2i, 2i+1) of the first `rot` values of every head by the token's
//     position, queries written back in place, keys and values written to the
//     token's page slot (keys [page][kv head][slot][dim], values
//     [page][kv head][vdim][slot]).
//   * attn_rows: attention of every row of the step over its request's pages
//     for any key and value size (the matrix-core kernels take equal sizes in
//     multiples of 16).  A row at position p sees key j when j <= p and
//     (window == 0 or p - j < window or j < keep_first); the softmax's
//     denominator also holds exp(sink[head]) when there is a sink.  Scores may be capped
//     (cap * tanh(s / cap)) and lose slopes[head] * (p - j), a penalty on distance.
//   * stream_add: h += a (+ b) on the 32-bit residual stream.
//
// Norms, angles, scores, weights and sums are 32-bit; only loads and stores see
// the storage type.
#include <algorithm>

#include "common.h"

namespace lyp {

__device__ __forceinline__ int row_owner(const int32_t* __restrict__ q_start, int B, int t) {
  int lo = 0, hi = B - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (q_start[mid] <= t) lo = mid;
    else hi = mid - 1;
  }
  return lo;
}

// qkv [rows, ld]: H*D query values, G*D key values, G*V value values side by side.
// wq / wk: the norms' weights over the whole projections (nullptr: no norm).
template <typename T>
__global__ void qk_norm_rope_kv_kernel(T* __restrict__ qkv, int ld, const float* __restrict__ wq,
                                       const float* __restrict__ wk, float eps,
                                       const int32_t* __restrict__ positions, const float* __restrict__ table,
                                       int rot, const int32_t* __restrict__ slot_map, T* __restrict__ kpool,
                                       T* __restrict__ vpool, int H, int G, int D, int V, int bs) {
  const int t = blockIdx.x;
  T* row = qkv + static_cast<size_t>(t) * ld;
  const int nq = H * D, nk = G * D;
  // both sums of squares in one pass and one reduction (wave by wave, in the waves' order)
  __shared__ float s_sum[2][16];
  float sq = 0.f, sk = 0.f;
  if (wq != nullptr)
    for (int i = threadIdx.x; i < nq; i += blockDim.x) {
      const float v = to_f32(row[i]);
      sq += v * v;
    }
  if (wk != nullptr)
    for (int i = threadIdx.x; i < nk; i += blockDim.x) {
      const float v = to_f32(row[nq + i]);
      sk += v * v;
    }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  if (threadIdx.x % kWave == 0) {
    s_sum[0][threadIdx.x / kWave] = sq;
    s_sum[1][threadIdx.x / kWave] = sk;
  }
  __syncthreads();
  sq = sk = 0.f;
  for (int wv = 0; wv < static_cast<int>(blockDim.x) / kWave; ++wv) {
    sq += s_sum[0][wv];
    sk += s_sum[1][wv];
  }
  const float inv_q = wq != nullptr ? 1.0f / sqrtf(sq / static_cast<float>(nq) + eps) : 1.f;
  const float inv_k = wk != nullptr ? 1.0f / sqrtf(sk / static_cast<float>(nk) + eps) : 1.f;
  __syncthreads();   // every thread has read the row's values it summed before anyone writes queries back
  const float* cs = rot > 0 ? table + static_cast<size_t>(positions[t]) * rot : nullptr;
  const int half = rot / 2;
  const int per = D / 2 + (D & 1);   // pairs of a head (the last one single when D is odd)
  // queries: normed, rotated, back in place
  for (int idx = threadIdx.x; idx < H * per; idx += blockDim.x) {
    const int h = idx / per, i = idx % per;
    const int e = h * D + 2 * i;
    const bool two = 2 * i + 1 < D;
    float a = to_f32(row[e]) * inv_q, b = two ? to_f32(row[e + 1]) * inv_q : 0.f;
    if (wq != nullptr) {
      a *= wq[e];
      if (two) b *= wq[e + 1];
    }
    if (i < half) rotate_pair(a, b, cs[i], cs[half + i], a, b);
    row[e] = from_f32<T>(a);
    if (two) row[e + 1] = from_f32<T>(b);
  }
  const int slot = slot_map != nullptr ? slot_map[t] : -1;
  if (slot < 0) return;   // a padded row, or a layer that stores nothing
  const int page = slot / bs, off = slot % bs;
  for (int idx = threadIdx.x; idx < G * per; idx += blockDim.x) {
    const int g = idx / per, i = idx % per;
    const int e = g * D + 2 * i;
    const bool two = 2 * i + 1 < D;
    float a = to_f32(row[nq + e]) * inv_k, b = two ? to_f32(row[nq + e + 1]) * inv_k : 0.f;
    if (wk != nullptr) {
      a *= wk[e];
      if (two) b *= wk[e + 1];
    }
    if (i < half) rotate_pair(a, b, cs[i], cs[half + i], a, b);
    T* dst = kpool + ((static_cast<size_t>(page) * G + g) * bs + off) * D + 2 * i;
    dst[0] = from_f32<T>(a);
    if (two) dst[1] = from_f32<T>(b);
  }
  const T* vrow = row + nq + nk;
  for (int idx = threadIdx.x; idx < G * V; idx += blockDim.x) {
    const int g = idx / V, d = idx % V;
    vpool[((static_cast<size_t>(page) * G + g) * V + d) * bs + off] = vrow[idx];
  }
}

// The same with 16 bytes a thread and access: head sizes, the rotated width and the row's stride are
// whole multiples of the 16 bytes' values, so a thread's values are whole pairs of one head and
// either all rotate or none.
template <typename T>
__global__ void qk_norm_rope_kv_vec_kernel(T* __restrict__ qkv, int ld, const float* __restrict__ wq,
                                           const float* __restrict__ wk, float eps,
                                           const int32_t* __restrict__ positions, const float* __restrict__ table,
                                           int rot, const int32_t* __restrict__ slot_map, T* __restrict__ kpool,
                                           T* __restrict__ vpool, int H, int G, int D, int V, int bs) {
  constexpr int VEC = 16 / sizeof(T);
  typedef T VecT __attribute__((ext_vector_type(VEC)));
  const int t = blockIdx.x;
  T* row = qkv + static_cast<size_t>(t) * ld;
  const int nq = H * D, nk = G * D;
  __shared__ float s_sum[2][16];
  float sq = 0.f, sk = 0.f;
  for (int i = threadIdx.x * VEC; i < nq + nk; i += blockDim.x * VEC) {
    const VecT x = *reinterpret_cast<const VecT*>(row + i);
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < VEC; ++e) ss += to_f32(x[e]) * to_f32(x[e]);
    if (i < nq) sq += ss;
    else sk += ss;
  }
  sq = wave_sum(sq);
  sk = wave_sum(sk);
  if (threadIdx.x % kWave == 0) {
    s_sum[0][threadIdx.x / kWave] = sq;
    s_sum[1][threadIdx.x / kWave] = sk;
  }
  __syncthreads();
  sq = sk = 0.f;
  for (int wv = 0; wv < static_cast<int>(blockDim.x) / kWave; ++wv) {
    sq += s_sum[0][wv];
    sk += s_sum[1][wv];
  }
  const float inv_q = wq != nullptr ? 1.0f / sqrtf(sq / static_cast<float>(nq) + eps) : 1.f;
  const float inv_k = wk != nullptr ? 1.0f / sqrtf(sk / static_cast<float>(nk) + eps) : 1.f;
  __syncthreads();
  const float* cs = rot > 0 ? table + static_cast<size_t>(positions[t]) * rot : nullptr;
  const int half = rot / 2;
  const int slot = slot_map != nullptr ? slot_map[t] : -1;
  const int page = slot >= 0 ? slot / bs : 0, off = slot >= 0 ? slot % bs : 0;
  for (int i = threadIdx.x * VEC; i < nq + nk; i += blockDim.x * VEC) {
    const bool is_q = i < nq;
    if (!is_q && slot < 0) continue;
    const int e0 = is_q ? i : i - nq;            // place within the projection
    const int d0 = e0 % D;                       // place within the head
    const float* wn = is_q ? wq : wk;
    const float inv = is_q ? inv_q : inv_k;
    const VecT x = *reinterpret_cast<const VecT*>(row + i);
    float v[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) v[e] = to_f32(x[e]) * inv;
    if (wn != nullptr) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] *= wn[e0 + e];
    }
    if (d0 < rot) {
#pragma unroll
      for (int e = 0; e < VEC; e += 2) {
        const int pi = (d0 + e) / 2;
        rotate_pair(v[e], v[e + 1], cs[pi], cs[half + pi], v[e], v[e + 1]);
      }
    }
    VecT y;
#pragma unroll
    for (int e = 0; e < VEC; ++e) y[e] = from_f32<T>(v[e]);
    if (is_q) *reinterpret_cast<VecT*>(row + i) = y;
    else
      *reinterpret_cast<VecT*>(kpool + ((static_cast<size_t>(page) * G + e0 / D) * bs + off) * D + d0) = y;
  }
  if (slot < 0) return;
  const T* vrow = row + nq + nk;
  for (int idx = threadIdx.x; idx < G * V; idx += blockDim.x) {
    const int g = idx / V, d = idx % V;
    vpool[((static_cast<size_t>(page) * G + g) * V + d) * bs + off] = vrow[idx];
  }
}

constexpr int kRowsBlock = 128;
constexpr int kRowsCols = 8;   // value columns a thread may own

// One workgroup per (row, head).  The visible keys of a row are walked as one
// run: the kept first tokens that the window no longer covers, then the window.
template <typename T>
__global__ __launch_bounds__(kRowsBlock) void attn_rows_kernel(
    const T* __restrict__ q, int q_stride, const T* __restrict__ kpool, const T* __restrict__ vpool,
    const int32_t* __restrict__ block_tables, int table_width, int bs, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ ctx_len, int B,
    const float* __restrict__ sink, float scale, int window, int keep_first, T* __restrict__ out, int out_stride,
    int H, int G, int D, int V, float cap, const float* __restrict__ slopes) {
  extern __shared__ float smem[];
  float* qs = smem;              // D
  float* ps = smem + D;          // kRowsBlock
  __shared__ float scratch[16];
  const int t = blockIdx.x, h = blockIdx.y;
  const int g = h / (H / G);
  T* orow = out + static_cast<size_t>(t) * out_stride + static_cast<size_t>(h) * V;
  const int b = row_owner(q_start, B, t);
  if (t >= q_start[B] || ctx_len[b] <= 0) {   // a row that belongs to no request, or to a padded one
    for (int i = threadIdx.x; i < V; i += blockDim.x) orow[i] = from_f32<T>(0.f);
    return;
  }
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int n_kept = window > 0 ? min(keep_first, lo) : 0;
  const int n_vis = n_kept + (pos - lo + 1);
  const int32_t* table = block_tables + static_cast<size_t>(b) * table_width;
  const T* qrow = q + static_cast<size_t>(t) * q_stride + static_cast<size_t>(h) * D;
  for (int i = threadIdx.x; i < D; i += blockDim.x) qs[i] = to_f32(qrow[i]);
  __syncthreads();
  float acc[kRowsCols];
#pragma unroll
  for (int v = 0; v < kRowsCols; ++v) acc[v] = 0.f;
  float m = sink != nullptr ? sink[h] : LYP_NEG_INF;
  float l = sink != nullptr ? 1.0f : 0.f;
  for (int v0 = 0; v0 < n_vis; v0 += kRowsBlock) {
    const int vi = v0 + threadIdx.x;
    float s = LYP_NEG_INF;
    if (vi < n_vis) {
      const int j = vi < n_kept ? vi : lo + (vi - n_kept);
      const int page = table[j / bs];
      if (page >= 0) {
        const T* krow = kpool + ((static_cast<size_t>(page) * G + g) * bs + j % bs) * D;
        float dot = 0.f;
        for (int i = 0; i < D; ++i) dot += qs[i] * to_f32(krow[i]);
        s = dot * scale;
        if (cap > 0.f) s = cap * tanhf(s / cap);
        if (slopes != nullptr) s -= slopes[h] * static_cast<float>(pos - j);
      }
    }
    const float m_new = fmaxf(m, block_max(s, scratch));
    const float p = s > LYP_NEG_INF ? expf(s - m_new) : 0.f;
    const float rescale = m > LYP_NEG_INF ? expf(m - m_new) : 0.f;
    const float psum = block_sum(p, scratch);
    l = l * rescale + psum;
    m = m_new;
    __syncthreads();
    ps[threadIdx.x] = p;
    __syncthreads();
    const int live = min(kRowsBlock, n_vis - v0);
#pragma unroll
    for (int v = 0; v < kRowsCols; ++v) {
      const int col = threadIdx.x + v * kRowsBlock;
      if (col < V) {
        float a = acc[v] * rescale;
        for (int jj = 0; jj < live; ++jj) {
          const int vj = v0 + jj;
          const int key = vj < n_kept ? vj : lo + (vj - n_kept);
          const int page = table[key / bs];
          if (page >= 0)
            a += ps[jj] * to_f32(vpool[((static_cast<size_t>(page) * G + g) * V + col) * bs + key % bs]);
        }
        acc[v] = a;
      }
    }
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
  for (int v = 0; v < kRowsCols; ++v) {
    const int col = threadIdx.x + v * kRowsBlock;
    if (col < V) orow[col] = from_f32<T>(acc[v] * inv);
  }
}

// h += a (+ b): a in TA (partial sums [parts] of n values each when float), b float
template <typename TA>
__global__ void stream_add_kernel(float* __restrict__ h, const TA* __restrict__ a, int parts,
                                  const float* __restrict__ b, size_t n) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < n;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    float v = h[i];
    if (a != nullptr)
      for (int p = 0; p < parts; ++p) v += to_f32(a[static_cast<size_t>(p) * n + i]);
    if (b != nullptr) v += b[i];
    h[i] = v;
  }
}

}  // namespace lyp

using namespace lyp;

extern "C" {

int lyp_qk_norm_rope_kv(void* qkv, int ld, int dtype, const float* wq, const float* wk, float eps,
                        const int32_t* positions, const float* table, int rot, const int32_t* slot_map, void* kpool,
                        void* vpool, int n_rows, int H, int G, int D, int V, int bs, hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && H > 0 && G > 0 && D > 0 && V > 0 && ld >= (H + G) * D + G * V,
              "qk_norm_rope_kv: bad sizes rows=%d H=%d G=%d D=%d V=%d ld=%d", n_rows, H, G, D, V, ld);
  LYP_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D && (rot == 0 || (table != nullptr && positions != nullptr)),
              "qk_norm_rope_kv: %d rotated values of %d", rot, D);
  LYP_REQUIRE(slot_map == nullptr || (kpool != nullptr && vpool != nullptr && bs > 0), "qk_norm_rope_kv: no pools");
  if (n_rows == 0) return 0;
  LYP_REQUIRE(dtype == kF32 || dtype == kBF16, "qk_norm_rope_kv: unknown dtype %d", dtype);
  const int vec = dtype == kF32 ? 4 : 8;
  const bool wide = D % vec == 0 && rot % vec == 0 && ld % vec == 0 && reinterpret_cast<uintptr_t>(qkv) % 16 == 0 &&
                    (kpool == nullptr || reinterpret_cast<uintptr_t>(kpool) % 16 == 0);
  const int work = wide ? (H + G) * D / vec : H * D / 2;
  const int threads = work >= 512 ? 512 : (work >= 256 ? 256 : 128);
#define LYP_QKN(KERNEL, T)                                                                                \
  KERNEL<T><<<n_rows, threads, 0, stream>>>(static_cast<T*>(qkv), ld, wq, wk, eps, positions, table, rot, \
                                            slot_map, static_cast<T*>(kpool), static_cast<T*>(vpool), H, G, D, V, bs)
  if (dtype == kF32) {
    if (wide) LYP_QKN(qk_norm_rope_kv_vec_kernel, float);
    else LYP_QKN(qk_norm_rope_kv_kernel, float);
  } else {
    if (wide) LYP_QKN(qk_norm_rope_kv_vec_kernel, bf16_t);
    else LYP_QKN(qk_norm_rope_kv_kernel, bf16_t);
  }
#undef LYP_QKN
  LYP_LAUNCH_CHECK("qk_norm_rope_kv");
  return 0;
}

int lyp_attn_rows(const void* q, int q_stride, const void* kpool, const void* vpool, const int32_t* block_tables,
                  int table_width, int bs, const int32_t* q_start, const int32_t* positions, const int32_t* ctx_len,
                  int B, const float* sink, float scale, int window, int keep_first, void* out, int out_stride,
                  int dtype, int n_rows, int H, int G, int D, int V, float cap, const float* slopes,
                  hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && B > 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && V > 0 && bs > 0 && table_width > 0,
              "attn_rows: bad sizes");
  LYP_REQUIRE(V <= kRowsCols * kRowsBlock, "attn_rows: values of up to %d, not %d", kRowsCols * kRowsBlock, V);
  LYP_REQUIRE(window >= 0 && keep_first >= 0 && q_stride >= H * D && out_stride >= H * V,
              "attn_rows: window %d, kept %d, strides %d %d", window, keep_first, q_stride, out_stride);
  LYP_REQUIRE(H <= 65535, "attn_rows: too many heads for one launch");
  if (n_rows == 0) return 0;
  const size_t lds = sizeof(float) * (D + kRowsBlock);
  dim3 grid(n_rows, H);
#define LYP_ROWS(T)                                                                                             \
  attn_rows_kernel<T><<<grid, kRowsBlock, lds, stream>>>(                                                       \
      static_cast<const T*>(q), q_stride, static_cast<const T*>(kpool), static_cast<const T*>(vpool),           \
      block_tables, table_width, bs, q_start, positions, ctx_len, B, sink, scale, window, keep_first,           \
      static_cast<T*>(out), out_stride, H, G, D, V, cap, slopes)
  if (dtype == kF32) LYP_ROWS(float);
  else if (dtype == kBF16) LYP_ROWS(bf16_t);
  else LYP_REQUIRE(false, "attn_rows: unknown dtype %d", dtype);
#undef LYP_ROWS
  LYP_LAUNCH_CHECK("attn_rows");
  return 0;
}

int lyp_stream_add(float* h, const void* a, int a_dtype, int parts, const float* b, long long n,
                   hipStream_t stream) {
  LYP_REQUIRE(n >= 0 && parts >= 0 && (a_dtype == kF32 || parts <= 1), "stream_add: bad sizes");
  if (n == 0 || (a == nullptr && b == nullptr)) return 0;
  const int threads = 256;
  const int blocks = static_cast<int>(std::min<long long>((n + threads - 1) / threads, 4096));
  if (a == nullptr || a_dtype == kF32)
    stream_add_kernel<float><<<blocks, threads, 0, stream>>>(h, static_cast<const float*>(a), parts, b,
                                                             static_cast<size_t>(n));
  else if (a_dtype == kBF16)
    stream_add_kernel<bf16_t><<<blocks, threads, 0, stream>>>(h, static_cast<const bf16_t*>(a), parts, b,
                                                              static_cast<size_t>(n));
  else
    LYP_REQUIRE(false, "stream_add: unknown dtype %d", a_dtype);
  LYP_LAUNCH_CHECK("stream_add");
  return 0;
}

}  // extern "C"
