// Selective state-space recurrence with a scalar decay per head (the "state-space duality" layer),
// carried per sequence slot, and the gated group norm that follows it.
//
//   ssm_scan          per head h (group g = h / (H / G)), state S [N x P] fp32 per (slot, head):
//                       dt_t = softplus(dt_raw_t + dt_bias_h)            (no clamp)
//                       S_t  = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T
//                       y_t  = S_t^T C_t + D_h x_t
//                     x / B / C are columns of one activation row [x (H P) | B (G N) | C (G N)] (already
//                     through their short convolution and activation), dt_raw a column block of another.
//   gated_group_norm  v = y * silu(z);  each of `ng` equal parts of v divided by its own root mean
//                     square, times w: the gate comes BEFORE the norm.
//
// One wave = 16 state columns x 4 row slices: lane (p = lane & 15, qn = lane >> 4) owns rows
// [qn * NI, (qn + 1) * NI) of column p in registers. B / C / x / dt of 16 tokens at a time are
// staged in LDS; the per-token work is 2 FMAs per owned state element plus a 4-lane sum.
#include "mixers_common.h"

namespace xgm {

constexpr int kScanCols = 16;   // state columns per wave
constexpr int kScanTile = 16;   // tokens staged per LDS tile

template <typename T, int NI>
__global__ __launch_bounds__(64) void ssm_scan_kernel(const T* __restrict__ xbc, int64_t ld_x, const T* __restrict__ dt_raw,
                                                      int64_t ld_dt, const float* __restrict__ dt_bias,
                                                      const float* __restrict__ A_log, const float* __restrict__ Dskip,
                                                      float* __restrict__ state, const int32_t* __restrict__ qsl,
                                                      const int32_t* __restrict__ seq_lens,
                                                      const int32_t* __restrict__ slots, float* __restrict__ y, int H, int G,
                                                      int N, int P) {
  constexpr int LDN = 4 * (NI + 4);  // padded row of B or C: slice qn starts at qn * (NI + 4)
  __shared__ __attribute__((aligned(16))) float Bs[kScanTile][LDN];
  __shared__ __attribute__((aligned(16))) float Cs[kScanTile][LDN];
  __shared__ float xs[kScanTile][kScanCols];
  __shared__ float dts[kScanTile], decs[kScanTile];
  const int s = blockIdx.x, h = blockIdx.y;
  const int q0 = qsl[s], q = qsl[s + 1] - q0, slot = slots[s];
  if (slot < 0 || q <= 0) return;
  const int ctx = seq_lens[s] - q;
  const int lane = threadIdx.x, pl = lane & 15, qn = lane >> 4;
  const int p = blockIdx.z * kScanCols + pl;
  const bool pok = p < P;
  const int g = h / (H / G);
  const int inner = H * P;
  const float rate = expf(A_log[h]), bias = dt_bias[h], dsk = Dskip[h];
  float* Sg = state + (((int64_t)slot * H + h) * N) * P;
  float S[NI];
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int n = qn * NI + i;
    S[i] = (ctx > 0 && pok && n < N) ? Sg[(int64_t)n * P + p] : 0.f;
  }
  for (int t0 = 0; t0 < q; t0 += kScanTile) {
    const int nt = min(kScanTile, q - t0);
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const T* row = xbc + (int64_t)(q0 + t0 + tt) * ld_x;
      for (int n = lane; n < 4 * NI; n += 64) {
        const int qq = n / NI, ii = n % NI;
        Bs[tt][qq * (NI + 4) + ii] = n < N ? ldf(row + inner + g * N + n) : 0.f;
        Cs[tt][qq * (NI + 4) + ii] = n < N ? ldf(row + inner + G * N + g * N + n) : 0.f;
      }
      if (lane < kScanCols) xs[tt][lane] = (blockIdx.z * kScanCols + lane < P) ? ldf(row + h * P + blockIdx.z * kScanCols + lane) : 0.f;
    }
    if (lane < nt) {
      const float d = softplusf(ldf(dt_raw + (int64_t)(q0 + t0 + lane) * ld_dt + h) + bias);
      dts[lane] = d;
      decs[lane] = expf(-rate * d);
    }
    __syncthreads();
    for (int tt = 0; tt < nt; ++tt) {
      const float a = decs[tt], xv = xs[tt][pl], dx = dts[tt] * xv;
      const float* Br = &Bs[tt][qn * (NI + 4)];
      const float* Cr = &Cs[tt][qn * (NI + 4)];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < NI; ++i) {
        S[i] = a * S[i] + dx * Br[i];
        acc += S[i] * Cr[i];
      }
      acc += __shfl_xor(acc, 16, 64);
      acc += __shfl_xor(acc, 32, 64);
      if (qn == 0 && pok) y[(int64_t)(q0 + t0 + tt) * inner + h * P + p] = acc + dsk * xv;
    }
  }
  if (pok) {
#pragma unroll
    for (int i = 0; i < NI; ++i) {
      const int n = qn * NI + i;
      if (n < N) Sg[(int64_t)n * P + p] = S[i];
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void gated_group_norm_kernel(const float* __restrict__ y, const T* __restrict__ z,
                                                               int64_t ld_z, const float* __restrict__ w, float eps,
                                                               T* __restrict__ out, int inner, int gs) {
  __shared__ float red[4];
  const int t = blockIdx.x, c0 = blockIdx.y * gs;
  float ss = 0.f;
  for (int c = threadIdx.x; c < gs; c += blockDim.x) {
    const float v = y[(int64_t)t * inner + c0 + c] * siluf(ldf(z + (int64_t)t * ld_z + c0 + c));
    ss += v * v;
  }
  const float r = 1.f / sqrtf(block_sum(ss, red) / (float)gs + eps);
  for (int c = threadIdx.x; c < gs; c += blockDim.x) {
    const float v = y[(int64_t)t * inner + c0 + c] * siluf(ldf(z + (int64_t)t * ld_z + c0 + c));
    stf(out + (int64_t)t * inner + c0 + c, v * r * w[c0 + c]);
  }
}

// ================================================================== host launchers
int ssm_scan(const void* xbc, bool f32, int64_t ld_x, const void* dt_raw, int64_t ld_dt, const float* dt_bias,
             const float* A_log, const float* Dskip, float* state, const int32_t* qsl, const int32_t* seq_lens,
             const int32_t* slots, float* y, int ns, int H, int G, int N, int P, hipStream_t st) {
  if (ns <= 0) return 0;
  if (H <= 0 || G <= 0 || H % G != 0 || N < 1 || N > 256 || P < 1) return -1;
  dim3 grid(ns, H, (P + kScanCols - 1) / kScanCols);
#define XGM_SS(NI)                                                                                                       \
  XGM_DISPATCH_T(f32, ssm_scan_kernel<T, NI><<<grid, 64, 0, st>>>((const T*)xbc, ld_x, (const T*)dt_raw, ld_dt, dt_bias, \
                                                                   A_log, Dskip, state, qsl, seq_lens, slots, y, H, G, N, \
                                                                   P);)                                                   \
  return 0;
  if (N <= 16) { XGM_SS(4) }
  if (N <= 32) { XGM_SS(8) }
  if (N <= 64) { XGM_SS(16) }
  if (N <= 128) { XGM_SS(32) }
  XGM_SS(64)
#undef XGM_SS
}

void gated_group_norm(const float* y, const void* z, bool f32, int64_t ld_z, const float* w, float eps, void* out, int T_,
                      int inner, int ng, hipStream_t st) {
  if (T_ <= 0) return;
  XGM_DISPATCH_T(f32, gated_group_norm_kernel<T><<<dim3(T_, ng), 256, 0, st>>>(y, (const T*)z, ld_z, w, eps, (T*)out, inner,
                                                                                inner / ng);)
}

}  // namespace xgm
