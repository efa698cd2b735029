// Grouped-query softmax attention over a paged K / V cache with a configurable visibility rule,
// per-head temperature and an optional "sink" term in the softmax denominator.
//
//   qk_norm_cache     from a fused projection row [q | k | v]: RMS norm over the WHOLE q vector and the
//                     WHOLE k vector (all heads at once, weights wq / wk; nullptr = no norm), q to a
//                     dense tensor, k and v to the cache rows slot_mapping[t]
//   masked_attention  token at position i of its sequence sees keys j in [lo(i), i]:
//                       kMaskCausal  lo = 0
//                       kMaskWindow  lo = max(0, i - size + 1)
//                       kMaskChunk   lo = floor(i / size) * size   (chunks counted from the sequence's start)
//                     score = (q . k) * scale * temp[h];  p_j = exp(score_j) / (sum_j' exp(score_j') + exp(sink[h]))
//                     (the sink adds to the denominator only: no key, no value, not scaled). Positions do
//                     not enter the scores.
//
// Activations / caches are T = float or bf16; norms, scores, probabilities and the accumulators are fp32.
#include "mixers_common.h"

namespace xgm {

constexpr int kMaskCausal = 0, kMaskWindow = 1, kMaskChunk = 2;

__device__ __forceinline__ int first_visible(int mask, int size, int pos) {
  if (mask == kMaskWindow) return max(0, pos - size + 1);
  if (mask == kMaskChunk) return (pos / size) * size;
  return 0;
}

// ------------------------------------------------------------------ projections -> normed q, cache rows
template <typename T>
__global__ __launch_bounds__(256) void qk_norm_cache_kernel(const T* __restrict__ proj, int64_t ld, int nq, int nk, int nv,
                                                            const float* __restrict__ wq, const float* __restrict__ wk,
                                                            float eps, const int32_t* __restrict__ slot_mapping,
                                                            T* __restrict__ q_out, T* __restrict__ kcache,
                                                            T* __restrict__ vcache) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  const T* row = proj + (int64_t)t * ld;
  float rq = 1.f, rk = 1.f;
  if (wq) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < nq; c += blockDim.x) {
      const float v = ldf(row + c);
      ss += v * v;
    }
    rq = 1.f / sqrtf(block_sum(ss, red) / (float)nq + eps);
  }
  for (int c = threadIdx.x; c < nq; c += blockDim.x)
    stf(q_out + (int64_t)t * nq + c, ldf(row + c) * rq * (wq ? wq[c] : 1.f));
  const int slot = slot_mapping[t];
  if (slot < 0) return;  // padding row: nothing is cached (uniform over the block)
  if (wk) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < nk; c += blockDim.x) {
      const float v = ldf(row + nq + c);
      ss += v * v;
    }
    rk = 1.f / sqrtf(block_sum(ss, red) / (float)nk + eps);
  }
  for (int c = threadIdx.x; c < nk; c += blockDim.x)
    stf(kcache + (int64_t)slot * nk + c, ldf(row + nq + c) * rk * (wk ? wk[c] : 1.f));
  for (int c = threadIdx.x; c < nv; c += blockDim.x) vcache[(int64_t)slot * nv + c] = row[nq + nk + c];
}

// ------------------------------------------------------------------ general kernel (any sizes, float or bf16)
// One workgroup = one token x one key/value head; its query heads (up to 8 per launch row) are spread
// over the 4 waves, 2 per wave. A tile of KT keys (K and V rows) is staged in LDS once for all of them.
constexpr int kQPW = 2;  // query heads per wave

template <typename T, int NR>
__global__ __launch_bounds__(256) void masked_attention_kernel(
    const T* __restrict__ q, const T* __restrict__ kcache, const T* __restrict__ vcache,
    const int32_t* __restrict__ block_tables, int bt_width, int bs, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ token_seq, const float* __restrict__ temp, const float* __restrict__ sink,
    T* __restrict__ out, int H, int G, int dk, int dv, int mask, int size, float scale, int KT) {
  extern __shared__ float smem[];
  const int ldk = dk + 1, ldv = dv + 1;
  float* ktile = smem;                           // [KT][dk + 1]
  float* vtile = ktile + (size_t)KT * ldk;       // [KT][dv + 1]
  float* qs = vtile + (size_t)KT * ldv;          // [4 * kQPW][dk]
  const int t = blockIdx.x, g = blockIdx.y;
  const int rep = H / G;
  const int r0 = blockIdx.z * (4 * kQPW);        // first of this workgroup's query heads within the group
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int s = token_seq[t];
  if (s < 0) {
    for (int a = 0; a < kQPW; ++a) {
      const int r = r0 + wave + 4 * a;
      if (r < rep)
        for (int d = lane; d < dv; d += 64) stf(out + ((int64_t)t * H + g * rep + r) * dv + d, 0.f);
    }
    return;
  }
  const int pos = positions[t];
  const int j0 = first_visible(mask, size, pos);
  float m[kQPW], l[kQPW], acc[kQPW][NR];
#pragma unroll
  for (int a = 0; a < kQPW; ++a) {
    const int r = r0 + wave + 4 * a;
    const int h = g * rep + min(r, rep - 1);
    float* qh = qs + (wave + 4 * a) * dk;
    const float sc = scale * (temp ? temp[h] : 1.f);
    for (int d = lane; d < dk; d += 64) qh[d] = r < rep ? ldf(q + ((int64_t)t * H + h) * dk + d) * sc : 0.f;
    // the sink starts the running softmax: weight exp(sink - m) = 1 with no value behind it
    m[a] = sink ? sink[h] : -INFINITY;
    l[a] = sink ? 1.f : 0.f;
#pragma unroll
    for (int i = 0; i < NR; ++i) acc[a][i] = 0.f;
  }
  const int LPK = 64 / KT;  // lanes per key in the score phase
  const int kj = lane / LPK, part = lane % LPK;
  const int32_t* bt = block_tables + (int64_t)s * bt_width;
  for (int k0 = j0; k0 <= pos; k0 += KT) {
    const int n = min(KT, pos - k0 + 1);
    __syncthreads();  // the previous tile is consumed (and qs is written, on the first pass)
    for (int jj = wave; jj < n; jj += 4) {
      const int key = k0 + jj;
      const int64_t row = (int64_t)bt[key / bs] * bs + key % bs;
      const T* ks = kcache + (row * G + g) * dk;
      const T* vs = vcache + (row * G + g) * dv;
      for (int d = lane; d < dk; d += 64) ktile[jj * ldk + d] = ldf(ks + d);
      for (int d = lane; d < dv; d += 64) vtile[jj * ldv + d] = ldf(vs + d);
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < kQPW; ++a) {
      if (r0 + wave + 4 * a >= rep) continue;
      const float* qh = qs + (wave + 4 * a) * dk;
      float sc = 0.f;
      if (kj < n) {
        const float* kr = ktile + kj * ldk;
        for (int d = part; d < dk; d += LPK) sc += qh[d] * kr[d];
      }
      for (int o = 1; o < LPK; o <<= 1) sc += __shfl_xor(sc, o, 64);
      if (kj >= n) sc = -INFINITY;
      const float mn = fmaxf(m[a], wave_max(sc));
      const float p = kj < n ? expf(sc - mn) : 0.f;
      const float corr = m[a] == -INFINITY ? 0.f : expf(m[a] - mn);
      l[a] = l[a] * corr + wave_sum(part == 0 ? p : 0.f);
      m[a] = mn;
#pragma unroll
      for (int i = 0; i < NR; ++i) acc[a][i] *= corr;
      for (int j = 0; j < n; ++j) {
        const float pj = __shfl(p, j * LPK, 64);
#pragma unroll
        for (int i = 0; i < NR; ++i) {
          const int d = lane + 64 * i;
          if (d < dv) acc[a][i] += pj * vtile[j * ldv + d];
        }
      }
    }
  }
#pragma unroll
  for (int a = 0; a < kQPW; ++a) {
    const int r = r0 + wave + 4 * a;
    if (r >= rep) continue;
    const float inv = 1.f / l[a];
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int d = lane + 64 * i;
      if (d < dv) stf(out + ((int64_t)t * H + g * rep + r) * dv + d, acc[a][i] * inv);
    }
  }
}

// ================================================================== host launchers
void qk_norm_cache(const void* proj, bool f32, int64_t ld, int nq, int nk, int nv, const float* wq, const float* wk,
                   float eps, const int32_t* slot_mapping, void* q_out, void* kcache, void* vcache, int T_,
                   hipStream_t st) {
  if (T_ <= 0) return;
  XGM_DISPATCH_T(f32, qk_norm_cache_kernel<T><<<T_, 256, 0, st>>>((const T*)proj, ld, nq, nk, nv, wq, wk, eps, slot_mapping,
                                                                   (T*)q_out, (T*)kcache, (T*)vcache);)
}

template <typename T, int NR>
static int launch_masked_attention(const void* q, const void* kcache, const void* vcache, const int32_t* block_tables,
                                   int bt_width, int bs, const int32_t* positions, const int32_t* token_seq,
                                   const float* temp, const float* sink, void* out, int T_, int H, int G, int dk, int dv,
                                   int mask, int size, float scale, hipStream_t st) {
  int KT = 64;
  auto bytes = [&](int kt) { return ((size_t)kt * (dk + dv + 2) + (size_t)4 * kQPW * dk) * sizeof(float); };
  while (KT > 4 && bytes(KT) > 60 * 1024) KT >>= 1;
  if (bytes(KT) > 64 * 1024) return -2;
  const int rep = H / G;
  dim3 grid(T_, G, (rep + 4 * kQPW - 1) / (4 * kQPW));
  masked_attention_kernel<T, NR><<<grid, 256, bytes(KT), st>>>((const T*)q, (const T*)kcache, (const T*)vcache,
                                                               block_tables, bt_width, bs, positions, token_seq, temp,
                                                               sink, (T*)out, H, G, dk, dv, mask, size, scale, KT);
  return 0;
}

int masked_attention(const void* q, bool f32, const void* kcache, const void* vcache, const int32_t* block_tables,
                     int bt_width, int bs, const int32_t* positions, const int32_t* token_seq, const float* temp,
                     const float* sink, void* out, int T_, int H, int G, int dk, int dv, int mask, int size, float scale,
                     hipStream_t st) {
  if (T_ <= 0) return 0;
  if (G <= 0 || H % G != 0 || dk <= 0 || dv <= 0 || dv > 512 || mask < 0 || mask > 2 || (mask != kMaskCausal && size < 1))
    return -1;
#define XGM_MA(NR)                                                                                                     \
  XGM_DISPATCH_T(f32, return (launch_masked_attention<T, NR>(q, kcache, vcache, block_tables, bt_width, bs, positions, \
                                                             token_seq, temp, sink, out, T_, H, G, dk, dv, mask, size, \
                                                             scale, st));)
  if (dv <= 64) { XGM_MA(1) }
  if (dv <= 128) { XGM_MA(2) }
  if (dv <= 256) { XGM_MA(4) }
  XGM_MA(8)
#undef XGM_MA
}

}  // namespace xgm
