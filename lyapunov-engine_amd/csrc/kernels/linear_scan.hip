// Linear recurrences with a matrix state per head, for mixers that carry a
// summary S [dim x vdim] instead of keys:
//
//   decayed outer products    S <- diag(g_t) S + k_t v_t^T                     o_t = S^T q_t
//   gated delta rule          S <- diag(g_t) S;  u = beta_t (v_t - S^T k_t);
//                             S <- S + k_t u^T                                 o_t = S^T q_t
//
// with a decay per head and key channel, g = exp(-coef_head * softplus(sign * (z + bias))), which
// covers exp(-A softplus(z + b)) (sign +1, coef A) and sigmoid(z + b)^(1/tau) (sign -1, coef 1/tau).
// Queries and keys may be made unit vectors per head first (x / sqrt(sum x^2 + 1e-6)); queries
// take a constant factor.  Decays, unit vectors, gates, sums and the state are 32-bit; q, k, v come
// in the activations' type.
//
//   * linear_scan: the state is kept transposed, [slot][head][vdim][dim], and lives in registers:
//     a column of S (one value of vdim) belongs to L neighbouring lanes that hold DPL key channels
//     each; the two dot products of a token are sums inside a lane and over those L lanes.  The
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
__host__ __device__ inline int scan_chunk(int Dp) { return Dp <= 128 ? 32 : 16; }
constexpr int kScanPad = 4;   // floats between the staged rows, so that neighbouring tokens start in other banks

__device__ __forceinline__ float scan_softplus(float v) { return fmaxf(v, 0.f) + log1pf(expf(-fabsf(v))); }
__device__ __forceinline__ float scan_sigmoid(float v) { return 1.0f / (1.0f + expf(-v)); }

template <typename T, int DPL, bool DELTA>
__global__ __launch_bounds__(256) void linear_scan_kernel(
    const T* __restrict__ q, int ldq, const T* __restrict__ k, int ldk, const T* __restrict__ v, int ldv,
    const float* __restrict__ z, int ldz, const float* __restrict__ zbias, const float* __restrict__ coef, float sign,
    const T* __restrict__ beta, int ldb, float* __restrict__ state, const int32_t* __restrict__ q_start,
    const int32_t* __restrict__ positions, const int32_t* __restrict__ slots, float* __restrict__ out, int ldo, int H,
    int G, int D, int V, int L, int unit, float q_scale) {
  extern __shared__ __attribute__((aligned(16))) float s_scan[];
  const int Dp = L * DPL;                      // key channels with the padding: a power of two
  const int ld = Dp + kScanPad;
  const int chunk = scan_chunk(Dp);
  const int cpb = blockDim.x / L;              // columns a workgroup: a power of two
  const int dp_shift = __ffs(Dp) - 1, cpb_shift = __ffs(cpb) - 1;
  float* sk = s_scan;                          // [chunk][ld]   keys as they come
  float* sq = sk + chunk * ld;                 //               queries as they come
  float* sg = sq + chunk * ld;                 //               decays
  float* sv = sg + chunk * ld;                 // [chunk][cpb]  this workgroup's columns of the values
  float* sb = sv + chunk * cpb;                // [chunk]       sigmoid(beta)
  float* sfq = sb + chunk;                     // [chunk]       what a query is multiplied by (unit length, the constant)
  float* sfk = sfq + chunk;                    // [chunk]       what a key is multiplied by
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

  for (int c0 = 0; c0 < n; c0 += chunk) {
    const int cn = min(chunk, n - c0);
    for (int idx = tid; idx < (cn << dp_shift); idx += blockDim.x) {
      const int j = idx >> dp_shift, d = idx & (Dp - 1);
      const size_t row = static_cast<size_t>(q0 + c0 + j);
      float qq = 0.f, kk = 0.f, gg = 1.f;
      if (d < D) {
        qq = to_f32(q[row * ldq + kvh * D + d]);
        kk = to_f32(k[row * ldk + kvh * D + d]);
        const float zz = z[row * ldz + h * D + d] + (zbias != nullptr ? zbias[h * D + d] : 0.f);
        gg = expf(-a_h * scan_softplus(sign * zz));
      }
      sq[j * ld + d] = qq;
      sk[j * ld + d] = kk;
      sg[j * ld + d] = gg;
    }
    for (int idx = tid; idx < (cn << cpb_shift); idx += blockDim.x) {
      const int j = idx >> cpb_shift, c = blockIdx.x * cpb + (idx & (cpb - 1));
      sv[idx] = c < V ? to_f32(v[static_cast<size_t>(q0 + c0 + j) * ldv + h * V + c]) : 0.f;
    }
    if (tid < cn) {
      if (DELTA) sb[tid] = scan_sigmoid(to_f32(beta[static_cast<size_t>(q0 + c0 + tid) * ldb + h]));
      if (!unit) {
        sfq[tid] = q_scale;
        sfk[tid] = 1.f;
      }
    }
    if (unit) {
      __syncthreads();
      // four neighbouring lanes a token: the squares of its query and key, a quarter each
      for (int j = tid / 4; j < cn; j += blockDim.x / 4) {
        float ssq = 0.f, ssk = 0.f;
        for (int f = tid % 4; f < Dp / 4; f += 4) {
          const f32x4 q4 = *reinterpret_cast<const f32x4*>(sq + j * ld + 4 * f);
          const f32x4 k4 = *reinterpret_cast<const f32x4*>(sk + j * ld + 4 * f);
          ssq += q4[0] * q4[0] + q4[1] * q4[1] + q4[2] * q4[2] + q4[3] * q4[3];
          ssk += k4[0] * k4[0] + k4[1] * k4[1] + k4[2] * k4[2] + k4[3] * k4[3];
        }
        ssq += __shfl_xor(ssq, 1, kWave);
        ssk += __shfl_xor(ssk, 1, kWave);
        ssq += __shfl_xor(ssq, 2, kWave);
        ssk += __shfl_xor(ssk, 2, kWave);
        if (tid % 4 == 0) {
          sfq[j] = q_scale / sqrtf(ssq + 1e-6f);
          sfk[j] = 1.0f / sqrtf(ssk + 1e-6f);
        }
      }
    }
    __syncthreads();
    for (int j = 0; j < cn; ++j) {
      const float* kj = sk + j * ld + d0;
      const float* qj = sq + j * ld + d0;
      const float* gj = sg + j * ld + d0;
      const float fk = sfk[j], fq = sfq[j];
      float u = sv[(j << cpb_shift) + cl];
      float r0 = 0.f, r1 = 0.f;
#pragma unroll
      for (int i = 0; i < DPL; i += 4) {
        const f32x4 g4 = *reinterpret_cast<const f32x4*>(gj + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) S[i + e] *= g4[e];
        if constexpr (DELTA) {
          const f32x4 k4 = *reinterpret_cast<const f32x4*>(kj + i);
          r0 += S[i] * k4[0] + S[i + 2] * k4[2];
          r1 += S[i + 1] * k4[1] + S[i + 3] * k4[3];
        }
      }
      if constexpr (DELTA) {
        float r = r0 + r1;
        for (int off = 1; off < L; off <<= 1) r += __shfl_xor(r, off, kWave);
        u = sb[j] * (u - fk * r);
      }
      u *= fk;
      float o0 = 0.f, o1 = 0.f;
#pragma unroll
      for (int i = 0; i < DPL; i += 4) {
        const f32x4 k4 = *reinterpret_cast<const f32x4*>(kj + i);
        const f32x4 q4 = *reinterpret_cast<const f32x4*>(qj + i);
#pragma unroll
        for (int e = 0; e < 4; ++e) S[i + e] += k4[e] * u;
        o0 += S[i] * q4[0] + S[i + 2] * q4[2];
        o1 += S[i + 1] * q4[1] + S[i + 3] * q4[3];
      }
      float o = o0 + o1;
      for (int off = 1; off < L; off <<= 1) o += __shfl_xor(o, off, kWave);
      if (l == 0 && col < V) out[static_cast<size_t>(q0 + c0 + j) * ldo + h * V + col] = o * fq;
    }
    __syncthreads();   // the chunk's staging is read to the end before the next overwrites it
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
                                                             int rows, int H, int V, float eps, int kind) {
  const int item = blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= rows * H) return;
  const int t = item / H, h = item % H, lane = threadIdx.x % kWave;
  const float* orow = o + (static_cast<size_t>(t) * H + h) * V;
  float ss = 0.f;
  for (int c = lane; c < V; c += kWave) ss += orow[c] * orow[c];
  const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(V) + eps);
  const TG* grow = gate + static_cast<size_t>(t) * ldg + h * V;
  T* dst = out + (static_cast<size_t>(t) * H + h) * V;
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
                                                         int rows, int N, int R) {
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
      if (t0 + j < rows) acc[j] += x * to_f32(mid[static_cast<size_t>(t0 + j) * ldm + r]);
  }
#pragma unroll
  for (int j = 0; j < kLowRows; ++j)
    if (t0 + j < rows) out[static_cast<size_t>(t0 + j) * N + n] = acc[j];
}

}  // namespace lyp

using namespace lyp;

extern "C" {

// Lanes a column of the state is spread over, for key heads of D values (0: D is too large).
int lyp_linear_scan_lanes(int D) {
  if (D <= 0 || D > 256) return 0;
  const int dpl = D <= 64 ? 16 : 32;
  int L = 1;
  while (L * dpl < D) L *= 2;
  return L;
}

// q, k [rows, >= G*D] and v [rows, >= H*V] of dtype, rows ldq / ldk / ldv apart; z float [rows, >= H*D] (ldz apart);
// zbias float [H*D] or null; coef float [H]; rows: all requests' rows together; beta [rows, >= H] of dtype (ldb apart; the delta rule only: delta != 0);
// state float [slots, H, V, D]; out float [rows, >= H*V] (ldo apart).  Request b owns rows q_start[b] .. q_start[b+1].
int lyp_linear_scan(const void* q, int ldq, const void* k, int ldk, const void* v, int ldv, int dtype, const float* z,
                    int ldz, const float* zbias, const float* coef, float sign, const void* beta, int ldb,
                    float* state, const int32_t* q_start, const int32_t* positions, const int32_t* slots, float* out,
                    int ldo, int rows, int B, int H, int G, int D, int V, int delta, int unit, float q_scale,
                    hipStream_t stream) {
  LYP_REQUIRE(B > 0 && H > 0 && G > 0 && H % G == 0 && D > 0 && V > 0, "linear_scan: B=%d H=%d G=%d D=%d V=%d", B, H, G,
              D, V);
  const int L = lyp_linear_scan_lanes(D);
  LYP_REQUIRE(L > 0, "linear_scan: key heads of up to 256 values, not %d", D);
  LYP_REQUIRE(ldq >= G * D && ldk >= G * D && ldv >= H * V && ldz >= H * D && ldo >= H * V && (!delta || ldb >= H),
              "linear_scan: rows too short for %d/%d heads of %d/%d", H, G, D, V);
  LYP_REQUIRE(!delta || beta != nullptr, "linear_scan: the delta rule needs beta");
  LYP_REQUIRE(H <= 65535 && B <= 65535, "linear_scan: too many heads or requests for one launch");
  const int dpl = D <= 64 ? 16 : 32;
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
  const size_t lds = static_cast<size_t>(scan_chunk(L * dpl)) * (3 * (L * dpl + kScanPad) + cpb + 3) * sizeof(float);
#define LYP_SCAN(T, DPLV, DEL)                                                                                      \
  linear_scan_kernel<T, DPLV, DEL><<<grid, threads, lds, stream>>>(                                                 \
      static_cast<const T*>(q), ldq, static_cast<const T*>(k), ldk, static_cast<const T*>(v), ldv, z, ldz, zbias,   \
      coef, sign, static_cast<const T*>(beta), ldb, state, q_start, positions, slots, out, ldo, H, G, D, V, L, unit, \
      q_scale)
#define LYP_SCAN_T(T)                          \
  do {                                         \
    if (dpl == 16) {                           \
      if (delta) LYP_SCAN(T, 16, true);        \
      else LYP_SCAN(T, 16, false);             \
    } else {                                   \
      if (delta) LYP_SCAN(T, 32, true);        \
      else LYP_SCAN(T, 32, false);             \
    }                                          \
  } while (0)
  if (dtype == kF32) LYP_SCAN_T(float);
  else if (dtype == kBF16) LYP_SCAN_T(bf16_t);
  else LYP_REQUIRE(false, "linear_scan: unknown dtype %d", dtype);
#undef LYP_SCAN_T
#undef LYP_SCAN
  LYP_LAUNCH_CHECK("linear_scan");
  return 0;
}

// o float [rows, H*V]; w float [V]; gate [rows, >= H*V] (ldg apart) float (gate_dtype kF32) or of out's type;
// out [rows, H*V] of out_dtype.  kind: 0 sigmoid(gate), 1 silu(gate).
int lyp_head_norm_gate(const float* o, const float* w, const void* gate, int ldg, int gate_dtype, void* out,
                       int out_dtype, int rows, int H, int V, float eps, int kind, hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && H > 0 && V > 0 && ldg >= H * V && (kind == kGateSigmoid || kind == kGateSilu),
              "head_norm_gate: rows=%d H=%d V=%d ldg=%d kind=%d", rows, H, V, ldg, kind);
  LYP_REQUIRE(gate_dtype == kF32 || gate_dtype == out_dtype, "head_norm_gate: the gate is float or of the output's type");
  if (rows == 0) return 0;
  const long long items = static_cast<long long>(rows) * H;
  const int blocks = static_cast<int>((items + 3) / 4);
#define LYP_HNG(TG, T)                                                                                              \
  head_norm_gate_kernel<TG, T><<<blocks, 256, 0, stream>>>(o, w, static_cast<const TG*>(gate), ldg,                 \
                                                           static_cast<T*>(out), rows, H, V, eps, kind)
  if (out_dtype == kF32) LYP_HNG(float, float);
  else if (out_dtype == kBF16 && gate_dtype == kF32) LYP_HNG(float, bf16_t);
  else if (out_dtype == kBF16) LYP_HNG(bf16_t, bf16_t);
  else LYP_REQUIRE(false, "head_norm_gate: unknown dtype %d", out_dtype);
#undef LYP_HNG
  LYP_LAUNCH_CHECK("head_norm_gate");
  return 0;
}

// mid [rows, >= R] of dtype (ldm apart); w float [N, R]; bias float [N] or null; out float [rows, N].
int lyp_lowrank_up(const void* mid, int ldm, int dtype, const float* w, const float* bias, float* out, int rows, int N,
                   int R, hipStream_t stream) {
  LYP_REQUIRE(rows >= 0 && N > 0 && R > 0 && ldm >= R, "lowrank_up: rows=%d N=%d R=%d ldm=%d", rows, N, R, ldm);
  if (rows == 0) return 0;
  const int threads = N >= 256 ? 256 : 64 * ((N + 63) / 64);
  dim3 grid((N + threads - 1) / threads, (rows + kLowRows - 1) / kLowRows);
  LYP_REQUIRE(grid.y <= 65535, "lowrank_up: too many rows for one launch");
  if (dtype == kF32)
    lowrank_up_kernel<float><<<grid, threads, 0, stream>>>(static_cast<const float*>(mid), ldm, w, bias, out, rows, N, R);
  else if (dtype == kBF16)
    lowrank_up_kernel<bf16_t><<<grid, threads, 0, stream>>>(static_cast<const bf16_t*>(mid), ldm, w, bias, out, rows, N, R);
  else
    LYP_REQUIRE(false, "lowrank_up: unknown dtype %d", dtype);
  LYP_LAUNCH_CHECK("lowrank_up");
  return 0;
}

}  // extern "C"
