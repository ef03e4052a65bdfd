// What attention over a cached latent needs around the attention kernel itself.
//
// latent_kv_store: a token's down-projection [kv_rank + rot_dim] (float32 sums) becomes its cache entry: the first
//   kv_rank numbers RMS-normed (the latent c), the last rot_dim position-encoded.  The key row is [c | turned | 0],
//   the value column [c | 0], both padded to P numbers, in the layouts the attention kernels read
//   (keys [pages, 1, page, P], values [pages, 1, P, page]).
// latent_query_rotate: the rotated part of every query head ([T, H, P]: columns kv_rank .. kv_rank + rot_dim), turned in place.
// Rotation: elements 2i and 2i + 1 (or, in the half layout, i and i + n_freq) turn by the angle position * inv_freq[i],
// for i < n_freq; angle, cosine and sine in 32-bit; elements beyond 2 n_freq pass unchanged.
#include "common.hpp"

__device__ __forceinline__ void turn_pair(float u, float v, int pos, float inv_freq, float& ou, float& ov) {
  float sn, cs;
  sincosf((float)pos * inv_freq, &sn, &cs);
  rotate_pair(u, v, cs, sn, ou, ov);
}

template <typename TW, typename TC>
__global__ void __launch_bounds__(256)
latent_kv_store_kernel(const float* __restrict__ sums, long ld, const TW* __restrict__ norm_weight, float eps,
                       const int* __restrict__ positions, const float* __restrict__ inv_freq, int n_freq,
                       TC* __restrict__ k_cache, TC* __restrict__ v_cache, const int* __restrict__ slots, int kv_rank,
                       int rot_dim, int P, int page, const float* __restrict__ q_sums, const TW* __restrict__ q_weight,
                       TC* __restrict__ q_out, int q_rank, int half_layout) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  if (q_out) {                      // the query latent of the same token, normed beside it (one kernel less a layer)
    const float* xq = q_sums + (size_t)t * ld;
    float sq = 0.f;
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x) sq = fmaf(xq[i], xq[i], sq);
    const float rq = 1.0f / sqrtf(block_sum(sq, scratch) / (float)q_rank + eps);
    for (int i = threadIdx.x; i < q_rank; i += blockDim.x)
      q_out[(size_t)t * q_rank + i] = from_float<TC>(xq[i] * rq * to_float(q_weight[i]));
  }
  const float* x = sums + (size_t)t * ld;
  float ss = 0.f;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) ss = fmaf(x[i], x[i], ss);
  const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)kv_rank + eps);
  const int slot = slots[t], pg = slot / page, off = slot % page, pos = positions[t];
  TC* kr = k_cache + ((size_t)pg * page + off) * P;
  TC* vc = v_cache + (size_t)pg * P * page + off;
  for (int i = threadIdx.x; i < kv_rank; i += blockDim.x) {
    const TC c = from_float<TC>(x[i] * rstd * to_float(norm_weight[i]));
    kr[i] = c;
    vc[(size_t)i * page] = c;
  }
  const float* r = x + kv_rank;
  for (int i = threadIdx.x; i < n_freq; i += blockDim.x) {          // the turned pairs
    const int d1 = half_layout ? i : 2 * i, d2 = half_layout ? i + n_freq : 2 * i + 1;
    float u, v;
    turn_pair(r[d1], r[d2], pos, inv_freq[i], u, v);
    kr[kv_rank + d1] = from_float<TC>(u);
    kr[kv_rank + d2] = from_float<TC>(v);
  }
  for (int i = 2 * n_freq + threadIdx.x; i < rot_dim; i += blockDim.x) kr[kv_rank + i] = from_float<TC>(r[i]);
  for (int i = kv_rank + rot_dim + threadIdx.x; i < P; i += blockDim.x) kr[i] = from_float<TC>(0.f);
  for (int i = kv_rank + threadIdx.x; i < P; i += blockDim.x) vc[(size_t)i * page] = from_float<TC>(0.f);
}

MIE_EXPORT const char* latent_attention_last_error() { return g_mie_error; }

// sums points at the first of the kv_rank + rot_dim columns; rows are ld floats apart.  q_out (or null) [tokens, q_rank] of
// the cache's dtype: RMSNorm of the q_rank columns at q_sums (same row stride, same eps) times q_weight (the norm
// weight's dtype).
MIE_EXPORT int mie_latent_kv_store(const float* sums, long ld, const void* norm_weight, int w_dtype, float eps,
                                   const int* positions, const float* inv_freq, int n_freq, void* k_cache, void* v_cache,
                                   int cache_dtype, const int* slots, int tokens, int kv_rank, int rot_dim, int P, int page,
                                   const float* q_sums, const void* q_weight, void* q_out, int q_rank, int half_layout,
                                   hipStream_t s) {
  if (tokens <= 0) return 0;
  if (kv_rank <= 0 || rot_dim < 0 || P < kv_rank + rot_dim || page <= 0 || 2 * n_freq > rot_dim)
    MIE_FAIL("latent_kv_store: kv_rank %d, rot_dim %d, padded %d, page %d, %d turned pairs", kv_rank, rot_dim, P, page, n_freq);
  if (ld < kv_rank + rot_dim || !sums || !norm_weight || !positions || !k_cache || !v_cache || !slots || (n_freq && !inv_freq))
    MIE_FAIL("latent_kv_store: operands");
  if (q_out && (!q_sums || !q_weight || q_rank <= 0 || ld < q_rank)) MIE_FAIL("latent_kv_store: query latent operands");
#define LKV(TW_, TC_)                                                                                                     \
  hipLaunchKernelGGL((latent_kv_store_kernel<TW_, TC_>), dim3(tokens), dim3(256), 0, s, sums, ld, (const TW_*)norm_weight, \
                     eps, positions, inv_freq, n_freq, (TC_*)k_cache, (TC_*)v_cache, slots, kv_rank, rot_dim, P, page, \
                     q_sums, (const TW_*)q_weight, (TC_*)q_out, q_rank, half_layout)
  if (w_dtype == MIE_F32 && cache_dtype == MIE_F32) LKV(float, float);
  else if (w_dtype == MIE_F32 && cache_dtype == MIE_BF16) LKV(float, bf16);
  else if (w_dtype == MIE_BF16 && cache_dtype == MIE_F32) LKV(bf16, float);
  else if (w_dtype == MIE_BF16 && cache_dtype == MIE_BF16) LKV(bf16, bf16);
  else MIE_FAIL("latent_kv_store: dtype codes weight %d, cache %d", w_dtype, cache_dtype);
#undef LKV
  MIE_CHECK_LAUNCH("latent_kv_store");
  return 0;
}

// q [tokens, H, P] (rows ldq apart): the pairs (2i, 2i + 1) (half layout: (i, i + n_freq)), i < n_freq, of columns kv_rank .. of
// every head turn in place.
template <typename T>
__global__ void latent_query_rotate_kernel(T* __restrict__ q, long ldq, const int* __restrict__ positions,
                                           const float* __restrict__ inv_freq, int n_freq, int H, int kv_rank, int P,
                                           int half_layout) {
  const int t = blockIdx.x, pos = positions[t];
  for (int idx = threadIdx.x; idx < H * n_freq; idx += blockDim.x) {
    const int h = idx / n_freq, i = idx - h * n_freq;
    T* part = q + (size_t)t * ldq + (size_t)h * P + kv_rank;
    const int d1 = half_layout ? i : 2 * i, d2 = half_layout ? i + n_freq : 2 * i + 1;
    float u, v;
    turn_pair(to_float(part[d1]), to_float(part[d2]), pos, inv_freq[i], u, v);
    part[d1] = from_float<T>(u);
    part[d2] = from_float<T>(v);
  }
}

MIE_EXPORT int mie_latent_query_rotate(void* q, long ldq, int dtype, const int* positions, const float* inv_freq, int n_freq,
                                       int tokens, int H, int kv_rank, int P, int half_layout, hipStream_t s) {
  if (tokens <= 0 || n_freq <= 0) return 0;
  if (H <= 0 || kv_rank < 0 || P < kv_rank + 2 * n_freq || ldq < (long)H * P)
    MIE_FAIL("latent_query_rotate: %d heads of %d, latent %d, %d turned pairs, row stride %ld", H, P, kv_rank, n_freq, ldq);
  if (!q || !positions || !inv_freq) MIE_FAIL("latent_query_rotate: operands");
  if (dtype == MIE_F32)
    hipLaunchKernelGGL(latent_query_rotate_kernel<float>, dim3(tokens), dim3(128), 0, s, (float*)q, ldq, positions, inv_freq, n_freq,
                       H, kv_rank, P, half_layout);
  else if (dtype == MIE_BF16)
    hipLaunchKernelGGL(latent_query_rotate_kernel<bf16>, dim3(tokens), dim3(128), 0, s, (bf16*)q, ldq, positions, inv_freq, n_freq,
                       H, kv_rank, P, half_layout);
  else
    MIE_FAIL("latent_query_rotate: dtype code %d", dtype);
  MIE_CHECK_LAUNCH("latent_query_rotate");
  return 0;
}
