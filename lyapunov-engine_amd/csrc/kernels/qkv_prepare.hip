// What stands between an attention layer's fused projection and its pages, with every choice a
// run-time value, for layers whose projections are biased, normed per head or over the whole
// projection, rotated in either pairing, whose values are their keys, or whose values are blended
// with another layer's:
//
//   pre [rows, ld] float: H*D query values, G*D key values and (unless the values are the keys)
//   G*V value values side by side, as the product's accumulators left them.
//     x <- pre + bias
//     values: the key projection itself (values_from_keys: taken before any norm) or the value
//       projection; blended, v <- (1 - lambda) v + lambda v_other, when another layer's values
//       are given; the unblended values can be kept for a later layer (v_keep)
//     q, k <- x / sqrt(mean(x^2) + eps) (* weight): over each head (norm_mode 1; the weight, if
//       any, is shared by the heads) or over the whole projection (norm_mode 2; weight over all of it)
//     the first `rot` values of every head turn by the token's position: pairs (2i, 2i+1)
//       (pairing 0) or (i, i + rot/2) (pairing 1); angles from a table [positions, rot] of cosines
//       then sines
//     queries to q_out [rows, H*D], keys and values to the token's page slot (keys
//     [page][kv head][slot][D], values [page][kv head][V][slot]).
//
// One workgroup a token.  The token's biased row is staged in LDS once (rows that fit 64 KiB;
// longer ones are read from memory where they are needed), so that the sums and the elements' partners
// cost no further trips to memory.  Everything is 32-bit up to the one rounding at the stores.
#include <algorithm>

#include "common.h"

namespace lyp {

template <typename T>
__global__ __launch_bounds__(512) void qkv_prepare_kernel(
    const float* __restrict__ pre, int ld, const float* __restrict__ bias, int norm_mode, const float* __restrict__ wq,
    const float* __restrict__ wk, float eps, const int32_t* __restrict__ positions, const float* __restrict__ table,
    int rot, int pairing, int values_from_keys, const float* __restrict__ blend, const float* __restrict__ v_other,
    int ld_other, float* __restrict__ v_keep, const int32_t* __restrict__ slot_map, T* __restrict__ q_out,
    T* __restrict__ kpool, T* __restrict__ vpool, int H, int G, int D, int V, int bs, int staged) {
  extern __shared__ __attribute__((aligned(16))) float s_prep[];
  float* s_ss = s_prep;             // H + G sums of squares, then the two whole-projection factors
  float* xs = s_prep + ((H + G + 2 + 3) & ~3);   // the biased row (when staged)
  const int t = blockIdx.x;
  const float* row = pre + static_cast<size_t>(t) * ld;
  const int nq = H * D, nk = G * D;
  const int n_used = nq + nk + (values_from_keys ? 0 : G * V);
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, nwaves = blockDim.x / kWave;
  if (staged) {
    const bool by4 = (ld & 3) == 0 && (n_used & 3) == 0 && (reinterpret_cast<uintptr_t>(pre) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(bias) & 15) == 0;
    if (by4) {
      for (int i = threadIdx.x * 4; i < n_used; i += blockDim.x * 4) {
        f32x4 v = *reinterpret_cast<const f32x4*>(row + i);
        if (bias != nullptr) {
          const f32x4 b = *reinterpret_cast<const f32x4*>(bias + i);
          v[0] += b[0], v[1] += b[1], v[2] += b[2], v[3] += b[3];
        }
        *reinterpret_cast<f32x4*>(xs + i) = v;
      }
    } else {
      for (int i = threadIdx.x; i < n_used; i += blockDim.x) xs[i] = row[i] + (bias != nullptr ? bias[i] : 0.f);
    }
    __syncthreads();
  }
  auto at = [&](int i) { return staged ? xs[i] : row[i] + (bias != nullptr ? bias[i] : 0.f); };
  if (norm_mode != 0) {
    // a wave a head, in the lanes' fixed order; a norm per head needs this workgroup's heads alone
    const int share = (H + G + gridDim.y - 1) / gridDim.y;
    const int s_lo = norm_mode == 2 ? 0 : blockIdx.y * share, s_hi = norm_mode == 2 ? H + G : min(H + G, s_lo + share);
    for (int hh = s_lo + wave; hh < s_hi; hh += nwaves) {
      float ss = 0.f;
      for (int d = lane; d < D; d += kWave) {
        const float v = at(hh * D + d);
        ss += v * v;
      }
      ss = wave_sum(ss);
      if (lane == 0) s_ss[hh] = ss;
    }
    __syncthreads();
    if (norm_mode == 2 && threadIdx.x < 2) {
      float ss = 0.f;
      const int lo = threadIdx.x == 0 ? 0 : H, hi = threadIdx.x == 0 ? H : H + G;
      for (int hh = lo; hh < hi; ++hh) ss += s_ss[hh];
      s_ss[H + G + threadIdx.x] = 1.0f / sqrtf(ss / static_cast<float>(threadIdx.x == 0 ? nq : nk) + eps);
    }
    __syncthreads();
  }
  const float* cs = rot > 0 ? table + static_cast<size_t>(positions[t]) * rot : nullptr;
  const int half = rot / 2;
  const int slot = slot_map != nullptr ? slot_map[t] : -1;
  const int page = slot >= 0 ? slot / bs : 0, off = slot >= 0 ? slot % bs : 0;
  // This workgroup's share of the token's heads (blockIdx.y of gridDim.y shares): a wave a head,
  // a lane a value of it and every 64th after that.
  const int per_block = (H + G + gridDim.y - 1) / gridDim.y;
  const int first = blockIdx.y * per_block, last = min(H + G, first + per_block);
  for (int hh = first + wave; hh < last; hh += nwaves) {
    const bool is_q = hh < H;
    if (!is_q && slot < 0) continue;
    const float* wn = is_q ? wq : wk;
    const int base = is_q ? hh * D : (hh - H) * D;   // the head's place within its projection
    float inv = 1.f;
    if (norm_mode == 1) inv = 1.0f / sqrtf(s_ss[hh] / static_cast<float>(D) + eps);
    else if (norm_mode == 2) inv = s_ss[H + G + (is_q ? 0 : 1)];
    auto normed = [&](int dd) {
      float v = at(hh * D + dd) * inv;
      if (wn != nullptr) v *= norm_mode == 2 ? wn[base + dd] : wn[dd];
      return v;
    };
    T* dst = is_q ? q_out + static_cast<size_t>(t) * nq + base
                  : kpool + ((static_cast<size_t>(page) * G + (hh - H)) * bs + off) * D;
    for (int d = lane; d < D; d += kWave) {
      float y = normed(d);
      if (d < rot) {
        int i, partner;
        bool lead;
        if (pairing == 0) {
          i = d >> 1;
          lead = (d & 1) == 0;
          partner = d ^ 1;
        } else {
          lead = d < half;
          i = lead ? d : d - half;
          partner = lead ? d + half : d - half;
        }
        const float o = normed(partner), c = cs[i], sn = cs[half + i];
        // the roundings of rotate_pair: one product rounded, then a fused multiply-add
        y = lead ? __builtin_fmaf(y, c, -(o * sn)) : __builtin_fmaf(y, c, o * sn);
      }
      dst[d] = from_f32<T>(y);
    }
  }
  // values: the key/value heads of this workgroup's share
  const int voff = values_from_keys ? nq : nq + nk;
  const float lam = blend != nullptr ? blend[0] : 0.f;
  for (int hh = max(first, H) + wave; hh < last; hh += nwaves) {
    const int g = hh - H;
    for (int d = lane; d < V; d += kWave) {
      const int idx = g * V + d;
      float v = at(voff + idx);
      if (v_keep != nullptr) v_keep[static_cast<size_t>(t) * G * V + idx] = v;
      if (blend != nullptr) v = (1.0f - lam) * v + lam * v_other[static_cast<size_t>(t) * ld_other + idx];
      if (slot >= 0) vpool[((static_cast<size_t>(page) * G + g) * V + d) * bs + off] = from_f32<T>(v);
    }
  }
}

}  // namespace lyp

using namespace lyp;

extern "C" {

// pre float [rows, ld]; bias float over pre's used columns or null; wq / wk float or null (norm_mode 1: [D];
// 2: [H*D] / [G*D]); table float [positions, rot] or null; blend: a float on the device, or null; v_other float
// [rows, >= G*V] (ld_other apart); v_keep float [rows, G*V] or null; q_out [rows, H*D] and the pools of dtype.
int lyp_qkv_prepare(const float* pre, int ld, const float* bias, int norm_mode, const float* wq, const float* wk,
                    float eps, const int32_t* positions, const float* table, int rot, int pairing, int values_from_keys,
                    const float* blend, const float* v_other, int ld_other, float* v_keep, const int32_t* slot_map,
                    void* q_out, void* kpool, void* vpool, int dtype, int n_rows, int H, int G, int D, int V, int bs,
                    hipStream_t stream) {
  LYP_REQUIRE(n_rows >= 0 && H > 0 && G > 0 && D > 0 && V > 0 && bs > 0, "qkv_prepare: bad sizes rows=%d H=%d G=%d D=%d V=%d",
              n_rows, H, G, D, V);
  LYP_REQUIRE(ld >= (H + G) * D + (values_from_keys ? 0 : G * V) && (!values_from_keys || V == D),
              "qkv_prepare: rows of %d values for %d+%d heads of %d/%d", ld, H, G, D, V);
  LYP_REQUIRE(norm_mode >= 0 && norm_mode <= 2 && (pairing == 0 || pairing == 1), "qkv_prepare: norm %d, pairing %d",
              norm_mode, pairing);
  LYP_REQUIRE(rot >= 0 && rot % 2 == 0 && rot <= D && (rot == 0 || (table != nullptr && positions != nullptr)),
              "qkv_prepare: %d rotated values of %d", rot, D);
  LYP_REQUIRE(blend == nullptr || (v_other != nullptr && ld_other >= G * V), "qkv_prepare: a blend without the other values");
  LYP_REQUIRE(q_out != nullptr && (slot_map == nullptr || (kpool != nullptr && vpool != nullptr)), "qkv_prepare: no output");
  if (n_rows == 0) return 0;
  const int work = (H + G) * D;
  // few rows (single tokens, short portions): a token's heads are shared out over several workgroups,
  // each of which stages the row and sums its heads' squares for itself
  // (with many rows one workgroup a token: sharing a token out makes every share stage the row again,
  // and the kernel is bound by its bytes then: 2,304 rows of 3,072 values 39 us whole, 56 us in four shares)
  const int shares = n_rows <= 64 ? std::min(H + G, 16) : 1;
  const int heads_each = (H + G + shares - 1) / shares;
  const int threads = std::min(512, std::max(64, 64 * std::min(heads_each, 8)));
  const int n_used = work + (values_from_keys ? 0 : G * V);
  const int head_words = (H + G + 2 + 3) & ~3;
  const int staged = sizeof(float) * (head_words + n_used) <= 64 * 1024 ? 1 : 0;
  const size_t lds = sizeof(float) * (head_words + (staged ? n_used : 0));
#define LYP_PREP(T)                                                                                                  \
  qkv_prepare_kernel<T><<<dim3(n_rows, shares), threads, lds, stream>>>(pre, ld, bias, norm_mode, wq, wk, eps, positions, table, rot, \
                                                          pairing, values_from_keys, blend, v_other, ld_other, v_keep, \
                                                          slot_map, static_cast<T*>(q_out), static_cast<T*>(kpool),    \
                                                          static_cast<T*>(vpool), H, G, D, V, bs, staged)
  if (dtype == kF32) LYP_PREP(float);
  else if (dtype == kBF16) LYP_PREP(bf16_t);
  else LYP_REQUIRE(false, "qkv_prepare: unknown dtype %d", dtype);
#undef LYP_PREP
  LYP_LAUNCH_CHECK("qkv_prepare");
  return 0;
}

}  // extern "C"
