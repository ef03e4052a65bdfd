// Token embedding into the 32-bit residual stream, and the residual add fused with RMSNorm.
//
// embedding:    stream[t, :] = float(table[ids[t], :]) * scale
// add_rmsnorm:  r = stream[row] (+ float(x[row]));  stream[row] = r (unless rows are gathered);
//               y[row] = r * (1 / sqrt(mean(r^2) + eps)) * weight, rounded once to y's type.
// One workgroup per row; the row's sum of squares is reduced in an order that depends only on
// the row width, so a token's result does not depend on what else is in the batch.
#include "common.hpp"

template <typename TT>
__global__ void embedding_kernel(const int* __restrict__ ids, const TT* __restrict__ table, float* __restrict__ out,
                                 int width, int vocab, const int* __restrict__ taken_from,
                                 const int* __restrict__ earlier_tokens, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (taken_from) {            // a token the host does not know yet: entry taken_from[t] of the tokens chosen last
    const int j = taken_from[t];
    if (j >= 0) id = earlier_tokens[j];
  }
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);   // ids are validated on the host; never read outside
  const TT* src = table + (size_t)id * width;
  float* dst = out + (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_float(src[i]) * scale;
}

#define NORM_THREADS 256
#define NORM_CACHE 16

template <typename TX, typename TW, typename TY>
__global__ void __launch_bounds__(NORM_THREADS)
add_rmsnorm_kernel(const TX* __restrict__ x, float* __restrict__ stream, const TW* __restrict__ weight,
                   TY* __restrict__ y, const int* __restrict__ rows, int width, float eps) {
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int row = rows ? rows[out_row] : out_row;
  float* sr = stream + (size_t)row * width;
  const TX* xr = x ? x + (size_t)row * width : nullptr;
  float cache[NORM_CACHE];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NORM_CACHE; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    float r = 0.f;
    if (i < width) {
      r = sr[i];
      if (xr) r += to_float(xr[i]);
      if (xr && !rows) sr[i] = r;
    }
    cache[k] = r;
    ss += r * r;
  }
  for (int i = threadIdx.x + NORM_CACHE * NORM_THREADS; i < width; i += NORM_THREADS) {
    float r = sr[i];
    if (xr) r += to_float(xr[i]);
    if (xr && !rows) sr[i] = r;
    ss += r * r;
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)width + eps);
  TY* yr = y + (size_t)out_row * width;
#pragma unroll
  for (int k = 0; k < NORM_CACHE; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    if (i < width) yr[i] = from_float<TY>(cache[k] * rstd * to_float(weight[i]));
  }
  for (int i = threadIdx.x + NORM_CACHE * NORM_THREADS; i < width; i += NORM_THREADS) {
    float r = sr[i];
    if (xr && rows) r += to_float(xr[i]);   // gathered rows were not written back
    yr[i] = from_float<TY>(r * rstd * to_float(weight[i]));
  }
}


// Few rows (a decode step): the whole cost is latency, so every load of a row (stream, pending x and
// weight) is issued before anything is reduced, 4 elements a lane at a time.  Same arithmetic and the
// same order of the block reduction inputs as above is not required: the fast path is taken for a row
// whenever width % 4 == 0 and width <= 4 * NORM_FAST_THREADS * NORM_FAST_VEC, whatever the batch is,
// so a row's result still does not depend on the batch.
#define NORM_FAST_THREADS 256
#define NORM_FAST_VEC 8      // float4 groups per thread: widths up to 8192

// four elements as they lie in memory, and as numbers
template <typename T> struct Raw4;
template <> struct Raw4<float> { float4 v; };
template <> struct Raw4<bf16> { uint2 v; };
__device__ __forceinline__ Raw4<float> load_raw(const float* p) { return Raw4<float>{*reinterpret_cast<const float4*>(p)}; }
__device__ __forceinline__ Raw4<bf16> load_raw(const bf16* p) { return Raw4<bf16>{*reinterpret_cast<const uint2*>(p)}; }
__device__ __forceinline__ float4 to_float4(const Raw4<float>& r) { return r.v; }
__device__ __forceinline__ float4 to_float4(const Raw4<bf16>& r) {
  return make_float4(__uint_as_float(r.v.x << 16), __uint_as_float(r.v.x & 0xFFFF0000u), __uint_as_float(r.v.y << 16),
                     __uint_as_float(r.v.y & 0xFFFF0000u));
}
template <typename T> __device__ __forceinline__ float4 load4(const T* p);
template <> __device__ __forceinline__ float4 load4<float>(const float* p) { return *reinterpret_cast<const float4*>(p); }
template <> __device__ __forceinline__ float4 load4<bf16>(const bf16* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xFFFF0000u), __uint_as_float(u.y << 16),
                     __uint_as_float(u.y & 0xFFFF0000u));
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16* p, float4 v) {
  uint2 u;
  u.x = (uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.x)) | ((uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.y)) << 16);
  u.y = (uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.z)) | ((uint32_t)__bfloat16_as_ushort(__float2bfloat16(v.w)) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

// VEC: float4 groups a thread holds (the width is at most 4 * NORM_FAST_THREADS * VEC): as few as the width
// needs, so that narrow rows do not pay in registers, and so in resident workgroups, for wide ones
template <typename TX, typename TW, typename TY, int VEC>
__global__ void __launch_bounds__(NORM_FAST_THREADS)
add_rmsnorm_fast_kernel(const TX* __restrict__ x, float* __restrict__ stream, const TW* __restrict__ weight,
                        TY* __restrict__ y, const int* __restrict__ rows, int width, float eps) {
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int row = rows ? rows[out_row] : out_row;
  float* sr = stream + (size_t)row * width;
  const TX* xr = x ? x + (size_t)row * width : nullptr;
  // first every load, as it comes from memory (a conversion or an add where a value is loaded would make
  // the compiler wait for it there, one memory latency per group of four instead of one in all)
  Raw4<float> r_raw[VEC];
  Raw4<TW> w_raw[VEC];
  Raw4<TX> a_raw[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const int i = (threadIdx.x + k * NORM_FAST_THREADS) * 4;
    r_raw[k] = Raw4<float>{};
    w_raw[k] = Raw4<TW>{};
    a_raw[k] = Raw4<TX>{};
    if (i < width) {
      r_raw[k] = load_raw(sr + i);
      w_raw[k] = load_raw(weight + i);
      if (xr) a_raw[k] = load_raw(xr + i);
    }
  }
  float4 r[VEC], w[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    r[k] = to_float4(r_raw[k]);
    w[k] = to_float4(w_raw[k]);
    const float4 a = to_float4(a_raw[k]);          // zeros where nothing was loaded
    r[k].x += a.x; r[k].y += a.y; r[k].z += a.z; r[k].w += a.w;
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    ss = fmaf(r[k].x, r[k].x, ss); ss = fmaf(r[k].y, r[k].y, ss);
    ss = fmaf(r[k].z, r[k].z, ss); ss = fmaf(r[k].w, r[k].w, ss);
    const int i = (threadIdx.x + k * NORM_FAST_THREADS) * 4;
    if (xr && !rows && i < width) store4(sr + i, r[k]);
  }
  const float total = block_sum(ss, scratch);
  const float rstd = 1.0f / sqrtf(total / (float)width + eps);
  TY* yr = y + (size_t)out_row * width;
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const int i = (threadIdx.x + k * NORM_FAST_THREADS) * 4;
    if (i < width)
      store4(yr + i, make_float4(r[k].x * rstd * w[k].x, r[k].y * rstd * w[k].y, r[k].z * rstd * w[k].z,
                                 r[k].w * rstd * w[k].w));
  }
}

MIE_EXPORT const char* embed_norm_last_error() { return g_mie_error; }

// taken_from (or null) [tokens]: where >= 0, the token is earlier_tokens[taken_from[t]] instead of ids[t]
// (a token chosen by the step before, which the host has not seen yet).
MIE_EXPORT int mie_embedding(const int* ids, const void* table, int table_dtype, float* out, int tokens, int width,
                             int vocab, const int* taken_from, const int* earlier_tokens, float scale,
                             hipStream_t stream) {
  if (tokens <= 0) return 0;
  if (width <= 0 || vocab <= 0) MIE_FAIL("embedding: width %d, vocab %d", width, vocab);
  if (taken_from && !earlier_tokens) MIE_FAIL("embedding: taken_from without the tokens to take from");
  dim3 grid(tokens), block(256);
  if (table_dtype == MIE_F32)
    hipLaunchKernelGGL(embedding_kernel<float>, grid, block, 0, stream, ids, (const float*)table, out, width, vocab,
                       taken_from, earlier_tokens, scale);
  else if (table_dtype == MIE_BF16)
    hipLaunchKernelGGL(embedding_kernel<bf16>, grid, block, 0, stream, ids, (const bf16*)table, out, width, vocab,
                       taken_from, earlier_tokens, scale);
  else
    MIE_FAIL("embedding: table dtype code %d", table_dtype);
  MIE_CHECK_LAUNCH("embedding");
  return 0;
}

template <typename TX, typename TW>
static int launch_norm(const void* x, float* stream, const void* w, void* y, int y_dtype, const int* rows, int n_rows,
                       int width, float eps, hipStream_t s) {
  dim3 grid(n_rows), block(NORM_THREADS);
  // the vector kernel whenever the width allows it (a property of the model, not of the batch)
  const bool fast = width % 4 == 0 && width <= 4 * NORM_FAST_THREADS * NORM_FAST_VEC &&
                    (((uintptr_t)x | (uintptr_t)stream | (uintptr_t)w | (uintptr_t)y) & 15) == 0;
  if (y_dtype != MIE_F32 && y_dtype != MIE_BF16) MIE_FAIL("add_rmsnorm: output dtype code %d", y_dtype);
  if (fast) {
#define NORM_FAST_LAUNCH(TY_, V_)                                                                                     \
  hipLaunchKernelGGL((add_rmsnorm_fast_kernel<TX, TW, TY_, V_>), grid, dim3(NORM_FAST_THREADS), 0, s, (const TX*)x, \
                     stream, (const TW*)w, (TY_*)y, rows, width, eps)
    const int groups = (width / 4 + NORM_FAST_THREADS - 1) / NORM_FAST_THREADS;
    if (y_dtype == MIE_F32) {
      if (groups <= 2) NORM_FAST_LAUNCH(float, 2);
      else if (groups <= 4) NORM_FAST_LAUNCH(float, 4);
      else NORM_FAST_LAUNCH(float, NORM_FAST_VEC);
    } else {
      if (groups <= 2) NORM_FAST_LAUNCH(bf16, 2);
      else if (groups <= 4) NORM_FAST_LAUNCH(bf16, 4);
      else NORM_FAST_LAUNCH(bf16, NORM_FAST_VEC);
    }
#undef NORM_FAST_LAUNCH
  }
  else if (y_dtype == MIE_F32)
    hipLaunchKernelGGL((add_rmsnorm_kernel<TX, TW, float>), grid, block, 0, s, (const TX*)x, stream, (const TW*)w,
                       (float*)y, rows, width, eps);
  else
    hipLaunchKernelGGL((add_rmsnorm_kernel<TX, TW, bf16>), grid, block, 0, s, (const TX*)x, stream, (const TW*)w,
                       (bf16*)y, rows, width, eps);
  MIE_CHECK_LAUNCH("add_rmsnorm");
  return 0;
}

// x may be null (nothing to add).  rows may be null (all n_rows rows, stream updated in place).
MIE_EXPORT int mie_add_rmsnorm(const void* x, int x_dtype, float* stream, const void* weight, int w_dtype, void* y,
                               int y_dtype, const int* rows, int n_rows, int width, float eps, hipStream_t s) {
  if (n_rows <= 0) return 0;
  if (width <= 0) MIE_FAIL("add_rmsnorm: width %d", width);
  if (x_dtype == MIE_F32 && w_dtype == MIE_F32) return launch_norm<float, float>(x, stream, weight, y, y_dtype, rows, n_rows, width, eps, s);
  if (x_dtype == MIE_F32 && w_dtype == MIE_BF16) return launch_norm<float, bf16>(x, stream, weight, y, y_dtype, rows, n_rows, width, eps, s);
  if (x_dtype == MIE_BF16 && w_dtype == MIE_F32) return launch_norm<bf16, float>(x, stream, weight, y, y_dtype, rows, n_rows, width, eps, s);
  if (x_dtype == MIE_BF16 && w_dtype == MIE_BF16) return launch_norm<bf16, bf16>(x, stream, weight, y, y_dtype, rows, n_rows, width, eps, s);
  MIE_FAIL("add_rmsnorm: dtype codes x %d, weight %d", x_dtype, w_dtype);
}


// ---- the norm on a branch's output: stream[row] += y[row] * (1 / sqrt(mean(y[row]^2) + eps)) * weight, in 32-bit,
// and the updated stream once more in the activation dtype (copy; null where that is the stream itself).
// y null: nothing is added, only the copy is made.  One workgroup a row, the same reduction order for every row.
template <typename TY, typename TW, typename TO>
__global__ void __launch_bounds__(NORM_THREADS)
branch_norm_add_kernel(const TY* __restrict__ y, float* __restrict__ stream, const TW* __restrict__ weight,
                       TO* __restrict__ copy, int width, float eps) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  float* sr = stream + (size_t)row * width;
  TO* cr = copy ? copy + (size_t)row * width : nullptr;
  if (!y) {
    if (cr)
      for (int i = threadIdx.x; i < width; i += NORM_THREADS) cr[i] = from_float<TO>(sr[i]);
    return;
  }
  const TY* yr = y + (size_t)row * width;
  float cache[NORM_CACHE];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NORM_CACHE; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    const float v = i < width ? to_float(yr[i]) : 0.f;
    cache[k] = v;
    ss = fmaf(v, v, ss);
  }
  for (int i = threadIdx.x + NORM_CACHE * NORM_THREADS; i < width; i += NORM_THREADS) {
    const float v = to_float(yr[i]);
    ss = fmaf(v, v, ss);
  }
  const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
#pragma unroll
  for (int k = 0; k < NORM_CACHE; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    if (i < width) {
      const float r = sr[i] + cache[k] * rstd * to_float(weight[i]);
      sr[i] = r;
      if (cr) cr[i] = from_float<TO>(r);
    }
  }
  for (int i = threadIdx.x + NORM_CACHE * NORM_THREADS; i < width; i += NORM_THREADS) {
    const float r = sr[i] + to_float(yr[i]) * rstd * to_float(weight[i]);
    sr[i] = r;
    if (cr) cr[i] = from_float<TO>(r);
  }
}

template <typename TY, typename TW>
static int launch_branch_norm(const void* y, float* stream, const void* w, void* copy, int copy_dtype, int rows, int width,
                              float eps, hipStream_t s) {
  if (copy_dtype == MIE_BF16)
    hipLaunchKernelGGL((branch_norm_add_kernel<TY, TW, bf16>), dim3(rows), dim3(NORM_THREADS), 0, s, (const TY*)y, stream,
                       (const TW*)w, (bf16*)copy, width, eps);
  else
    hipLaunchKernelGGL((branch_norm_add_kernel<TY, TW, float>), dim3(rows), dim3(NORM_THREADS), 0, s, (const TY*)y, stream,
                       (const TW*)w, (float*)copy, width, eps);
  MIE_CHECK_LAUNCH("branch_norm_add");
  return 0;
}

// y [rows, width] (or null), weight [width]; copy [rows, width] of copy_dtype, or null.
MIE_EXPORT int mie_branch_norm_add(const void* y, int y_dtype, float* stream, const void* weight, int w_dtype, void* copy,
                                   int copy_dtype, int rows, int width, float eps, hipStream_t s) {
  if (rows <= 0) return 0;
  if (width <= 0 || !stream) MIE_FAIL("branch_norm_add: width %d", width);
  if (y && !weight) MIE_FAIL("branch_norm_add: a branch output without a norm weight");
  if (!y && !copy) return 0;
  if (copy && copy_dtype != MIE_F32 && copy_dtype != MIE_BF16) MIE_FAIL("branch_norm_add: copy dtype code %d", copy_dtype);
  if (y_dtype == MIE_F32 && w_dtype == MIE_F32) return launch_branch_norm<float, float>(y, stream, weight, copy, copy_dtype, rows, width, eps, s);
  if (y_dtype == MIE_F32 && w_dtype == MIE_BF16) return launch_branch_norm<float, bf16>(y, stream, weight, copy, copy_dtype, rows, width, eps, s);
  if (y_dtype == MIE_BF16 && w_dtype == MIE_F32) return launch_branch_norm<bf16, float>(y, stream, weight, copy, copy_dtype, rows, width, eps, s);
  if (y_dtype == MIE_BF16 && w_dtype == MIE_BF16) return launch_branch_norm<bf16, bf16>(y, stream, weight, copy, copy_dtype, rows, width, eps, s);
  MIE_FAIL("branch_norm_add: dtype codes y %d, weight %d", y_dtype, w_dtype);
}

// ---- RMSNorm of a range of columns of a float32 matrix: out[row, i] = x[row, i] * rstd * weight[i], i < n
template <typename TW, typename TO>
__global__ void __launch_bounds__(NORM_THREADS)
rmsnorm_columns_kernel(const float* __restrict__ x, long ldx, const TW* __restrict__ weight, TO* __restrict__ out, int n,
                       float eps) {
  __shared__ float scratch[16];
  const float* xr = x + (size_t)blockIdx.x * ldx;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += NORM_THREADS) ss = fmaf(xr[i], xr[i], ss);
  const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)n + eps);
  TO* o = out + (size_t)blockIdx.x * n;
  for (int i = threadIdx.x; i < n; i += NORM_THREADS) o[i] = from_float<TO>(xr[i] * rstd * to_float(weight[i]));
}

// x points at the first column of the range; rows are ldx floats apart.
MIE_EXPORT int mie_rmsnorm_columns(const float* x, long ldx, const void* weight, int w_dtype, void* out, int out_dtype,
                                   int rows, int n, float eps, hipStream_t s) {
  if (rows <= 0) return 0;
  if (n <= 0 || ldx < n || !x || !weight || !out) MIE_FAIL("rmsnorm_columns: n %d, row stride %ld", n, ldx);
#define RC_LAUNCH(TW_, TO_)                                                                                              \
  hipLaunchKernelGGL((rmsnorm_columns_kernel<TW_, TO_>), dim3(rows), dim3(NORM_THREADS), 0, s, x, ldx, (const TW_*)weight, \
                     (TO_*)out, n, eps)
  if (w_dtype == MIE_F32 && out_dtype == MIE_F32) RC_LAUNCH(float, float);
  else if (w_dtype == MIE_F32 && out_dtype == MIE_BF16) RC_LAUNCH(float, bf16);
  else if (w_dtype == MIE_BF16 && out_dtype == MIE_F32) RC_LAUNCH(bf16, float);
  else if (w_dtype == MIE_BF16 && out_dtype == MIE_BF16) RC_LAUNCH(bf16, bf16);
  else MIE_FAIL("rmsnorm_columns: dtype codes weight %d, out %d", w_dtype, out_dtype);
#undef RC_LAUNCH
  MIE_CHECK_LAUNCH("rmsnorm_columns");
  return 0;
}

// ---- stream[row] += scale * (a * rstd(a) * wa + b * rstd(b) * wb): two branch outputs, each normed over the row, joined
// and added in one pass (b null: one).  One workgroup a row, float32 throughout.
// widths that are a multiple of 4 up to 8192: 16-byte loads, both rows read once and kept in registers
constexpr int NSA_V = 8;
__global__ void __launch_bounds__(NORM_THREADS)
normed_sum_add_vec_kernel(float* __restrict__ stream, const float* __restrict__ a, const float* __restrict__ wa,
                          const float* __restrict__ b, const float* __restrict__ wb, int width, float eps, float scale) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * width;
  const int nv = width / 4;
  float4 va[NSA_V], vb[NSA_V];
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int k = 0; k < NSA_V; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    va[k] = i < nv ? reinterpret_cast<const float4*>(a + base)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    vb[k] = (b && i < nv) ? reinterpret_cast<const float4*>(b + base)[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    sa = fmaf(va[k].x, va[k].x, fmaf(va[k].y, va[k].y, fmaf(va[k].z, va[k].z, fmaf(va[k].w, va[k].w, sa))));
    sb = fmaf(vb[k].x, vb[k].x, fmaf(vb[k].y, vb[k].y, fmaf(vb[k].z, vb[k].z, fmaf(vb[k].w, vb[k].w, sb))));
  }
  const float ra = 1.0f / sqrtf(block_sum(sa, scratch) / (float)width + eps);
  const float rb = b ? 1.0f / sqrtf(block_sum(sb, scratch) / (float)width + eps) : 0.f;
#pragma unroll
  for (int k = 0; k < NSA_V; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    if (i < nv) {
      const float4 ga = reinterpret_cast<const float4*>(wa)[i];
      float4 v = make_float4(va[k].x * ra * ga.x, va[k].y * ra * ga.y, va[k].z * ra * ga.z, va[k].w * ra * ga.w);
      if (b) {
        const float4 gb = reinterpret_cast<const float4*>(wb)[i];
        v.x += vb[k].x * rb * gb.x;
        v.y += vb[k].y * rb * gb.y;
        v.z += vb[k].z * rb * gb.z;
        v.w += vb[k].w * rb * gb.w;
      }
      float4 st = reinterpret_cast<float4*>(stream + base)[i];
      st.x += scale * v.x;
      st.y += scale * v.y;
      st.z += scale * v.z;
      st.w += scale * v.w;
      reinterpret_cast<float4*>(stream + base)[i] = st;
    }
  }
}

__global__ void __launch_bounds__(NORM_THREADS)
normed_sum_add_kernel(float* __restrict__ stream, const float* __restrict__ a, const float* __restrict__ wa,
                      const float* __restrict__ b, const float* __restrict__ wb, int width, float eps, float scale) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * width;
  float sa = 0.f, sb = 0.f;
  for (int i = threadIdx.x; i < width; i += NORM_THREADS) {
    sa = fmaf(a[base + i], a[base + i], sa);
    if (b) sb = fmaf(b[base + i], b[base + i], sb);
  }
  const float ra = 1.0f / sqrtf(block_sum(sa, scratch) / (float)width + eps);
  const float rb = b ? 1.0f / sqrtf(block_sum(sb, scratch) / (float)width + eps) : 0.f;
  for (int i = threadIdx.x; i < width; i += NORM_THREADS) {
    float v = a[base + i] * ra * wa[i];
    if (b) v += b[base + i] * rb * wb[i];
    stream[base + i] += scale * v;
  }
}

MIE_EXPORT int mie_normed_sum_add(float* stream, const float* a, const float* wa, const float* b, const float* wb, int rows,
                                  int width, float eps, float scale, hipStream_t s) {
  if (rows <= 0) return 0;
  if (width <= 0 || !stream || !a || !wa || (b && !wb)) MIE_FAIL("normed_sum_add: width %d or a missing operand", width);
  const bool aligned = !(((uintptr_t)stream | (uintptr_t)a | (uintptr_t)wa | (uintptr_t)b | (uintptr_t)wb) & 15);
  if (width % 4 == 0 && width <= 4 * NSA_V * NORM_THREADS && aligned)
    hipLaunchKernelGGL(normed_sum_add_vec_kernel, dim3(rows), dim3(NORM_THREADS), 0, s, stream, a, wa, b, wb, width, eps, scale);
  else
    hipLaunchKernelGGL(normed_sum_add_kernel, dim3(rows), dim3(NORM_THREADS), 0, s, stream, a, wa, b, wb, width, eps, scale);
  MIE_CHECK_LAUNCH("normed_sum_add");
  return 0;
}

// ---- two norms of the same stream and a short convolution on the first, in one pass:
//   h = x * rstd(x) * w1;  xm[t] = h[t] + sum_k taps[:, k] h[t - (K - 1 - k)]  (a row's earlier tokens; before its first
//   token the K - 1 inputs kept in tail[slot]);  y = x * rstd(x) * w2 (w2 null: none).  One workgroup a token: it
//   takes the root mean square of its own row and of the K - 1 rows before it in the step, and leaves its own in
//   rstd[t] for norm_conv_tail_kernel, which afterwards moves every row's last K - 1 inputs into tail[slot] (a thread
//   a (row, channel), reads ahead of writes).
constexpr int CONV_MAX_TAPS = 8;

template <typename TO>
__global__ void __launch_bounds__(NORM_THREADS)
norm_pair_conv_kernel(const float* __restrict__ stream, const float* __restrict__ w1, const float* __restrict__ w2,
                      const float* __restrict__ taps, const float* __restrict__ tail, const int* __restrict__ token_row,
                      const int* __restrict__ row_start, const int* __restrict__ slots, TO* __restrict__ xm,
                      TO* __restrict__ y, float* __restrict__ rstd_out, int width, int K, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const int r = token_row[t], j = t - row_start[r];
  const int have = j < K - 1 ? j : K - 1;            // rows before this one that are in the step
  float ss[CONV_MAX_TAPS];
#pragma unroll
  for (int b = 0; b < CONV_MAX_TAPS; ++b) ss[b] = 0.f;
  for (int i = threadIdx.x; i < width; i += NORM_THREADS) {
#pragma unroll
    for (int b = 0; b < CONV_MAX_TAPS; ++b)
      if (b <= have) {
        const float v = stream[(size_t)(t - b) * width + i];
        ss[b] = fmaf(v, v, ss[b]);
      }
  }
  float rstd[CONV_MAX_TAPS];
#pragma unroll
  for (int b = 0; b < CONV_MAX_TAPS; ++b)
    rstd[b] = b <= have ? 1.0f / sqrtf(block_sum(ss[b], scratch) / (float)width + eps) : 0.f;    // ``have`` is the workgroup's
  if (threadIdx.x == 0) rstd_out[t] = rstd[0];
  const float* tl = tail + (size_t)slots[r] * (K > 1 ? K - 1 : 1) * width;
  for (int i = threadIdx.x; i < width; i += NORM_THREADS) {
    const float g = w1[i];
    const float own = stream[(size_t)t * width + i];
    float acc = own * rstd[0] * g;
#pragma unroll
    for (int b = 0; b < CONV_MAX_TAPS; ++b)
      if (b < K) {
        const float h = b <= have ? stream[(size_t)(t - b) * width + i] * rstd[b] * g : tl[(size_t)(K - 1 + j - b) * width + i];
        acc = fmaf(taps[(size_t)i * K + (K - 1 - b)], h, acc);
      }
    xm[(size_t)t * width + i] = from_float<TO>(acc);
    if (w2) y[(size_t)t * width + i] = from_float<TO>(own * rstd[0] * w2[i]);
  }
}

// The same for widths that are a multiple of 4 up to 8192, the number of taps known at compile time: 16-byte loads, the
// token's own row read once and kept in registers, four channels' taps as K consecutive 16-byte loads.
constexpr int NPC_V = 8;
__device__ __forceinline__ void store4(float* p, float a, float b, float c, float d) {
  *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
__device__ __forceinline__ void store4(bf16* p, float a, float b, float c, float d) {
  const bf16 v[4] = {__float2bfloat16(a), __float2bfloat16(b), __float2bfloat16(c), __float2bfloat16(d)};
  *reinterpret_cast<uint2*>(p) = *reinterpret_cast<const uint2*>(v);
}

template <typename TO, int K>
__global__ void __launch_bounds__(NORM_THREADS)
norm_pair_conv_vec_kernel(const float* __restrict__ stream, const float* __restrict__ w1, const float* __restrict__ w2,
                          const float* __restrict__ taps, float* __restrict__ tail, const int* __restrict__ token_row,
                          const int* __restrict__ row_start, const int* __restrict__ slots, TO* __restrict__ xm,
                          TO* __restrict__ y, float* __restrict__ rstd_out, int width, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, nv = width / 4;
  const int r = token_row[t], j = t - row_start[r];
  const int have = j < K - 1 ? j : K - 1;            // rows before this one that are in the step
  const float4* own = reinterpret_cast<const float4*>(stream + (size_t)t * width);
  float4 xo[NPC_V];
  float ss[K];
#pragma unroll
  for (int b = 0; b < K; ++b) ss[b] = 0.f;
#pragma unroll
  for (int k = 0; k < NPC_V; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    xo[k] = i < nv ? own[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    ss[0] = fmaf(xo[k].x, xo[k].x, fmaf(xo[k].y, xo[k].y, fmaf(xo[k].z, xo[k].z, fmaf(xo[k].w, xo[k].w, ss[0]))));
#pragma unroll
    for (int b = 1; b < K; ++b)
      if (b <= have && i < nv) {
        const float4 v = (own - (size_t)b * nv)[i];
        ss[b] = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss[b]))));
      }
  }
  float rstd[K];
#pragma unroll
  for (int b = 0; b < K; ++b)
    rstd[b] = b <= have ? 1.0f / sqrtf(block_sum(ss[b], scratch) / (float)width + eps) : 0.f;    // ``have`` is the workgroup's
  if (threadIdx.x == 0) rstd_out[t] = rstd[0];
  float4* tl = reinterpret_cast<float4*>(tail + (size_t)slots[r] * (K > 1 ? K - 1 : 1) * width);
#pragma unroll
  for (int k = 0; k < NPC_V; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    if (i >= nv) continue;
    const float4 g = reinterpret_cast<const float4*>(w1)[i];
    float tp[4 * K];                                  // taps of channels 4 i .. 4 i + 3, K each
#pragma unroll
    for (int q = 0; q < K; ++q) {
      const float4 v = reinterpret_cast<const float4*>(taps + (size_t)i * 4 * K)[q];
      tp[4 * q] = v.x, tp[4 * q + 1] = v.y, tp[4 * q + 2] = v.z, tp[4 * q + 3] = v.w;
    }
    const float h0[4] = {xo[k].x * rstd[0] * g.x, xo[k].y * rstd[0] * g.y, xo[k].z * rstd[0] * g.z, xo[k].w * rstd[0] * g.w};
    float acc[4] = {h0[0], h0[1], h0[2], h0[3]};
#pragma unroll
    for (int b = 0; b < K; ++b) {
      float h[4];
      if (b == 0) {
        h[0] = h0[0], h[1] = h0[1], h[2] = h0[2], h[3] = h0[3];
      } else if (b <= have) {
        const float4 v = (own - (size_t)b * nv)[i];
        h[0] = v.x * rstd[b] * g.x, h[1] = v.y * rstd[b] * g.y, h[2] = v.z * rstd[b] * g.z, h[3] = v.w * rstd[b] * g.w;
      } else {
        const float4 v = tl[(size_t)(K - 1 + j - b) * nv + i];
        h[0] = v.x, h[1] = v.y, h[2] = v.z, h[3] = v.w;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = fmaf(tp[e * K + (K - 1 - b)], h[e], acc[e]);
    }
    store4(xm + (size_t)t * width + 4 * i, acc[0], acc[1], acc[2], acc[3]);
    if (w2) {
      const float4 g2 = reinterpret_cast<const float4*>(w2)[i];
      store4(y + (size_t)t * width + 4 * i, xo[k].x * rstd[0] * g2.x, xo[k].y * rstd[0] * g2.y, xo[k].z * rstd[0] * g2.z,
             xo[k].w * rstd[0] * g2.w);
    }
  }
  // A row of one token is this workgroup's alone: it moves the tail on itself (every thread shifts the channels it has
  // just read, oldest first), and norm_conv_tail_kernel skips such rows.
  if (K > 1 && row_start[r + 1] - row_start[r] == 1) {
    float4* tw = tl;
#pragma unroll
    for (int k = 0; k < NPC_V; ++k) {
      const int i = threadIdx.x + k * NORM_THREADS;
      if (i >= nv) continue;
      const float4 g = reinterpret_cast<const float4*>(w1)[i];
#pragma unroll
      for (int b = 0; b + 2 < K; ++b) tw[(size_t)b * nv + i] = tw[(size_t)(b + 1) * nv + i];
      tw[(size_t)(K - 2) * nv + i] = make_float4(xo[k].x * rstd[0] * g.x, xo[k].y * rstd[0] * g.y, xo[k].z * rstd[0] * g.z,
                                                  xo[k].w * rstd[0] * g.w);
    }
  }
}

__global__ void __launch_bounds__(256)
norm_conv_tail_kernel(const float* __restrict__ stream, const float* __restrict__ w1, const float* __restrict__ rstd,
                      float* __restrict__ tail, const int* __restrict__ row_start, const int* __restrict__ slots, int width,
                      int K, int skip_single) {
  const int r = blockIdx.x, c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= width) return;
  const int a0 = row_start[r], n = row_start[r + 1] - a0, keep = K - 1;
  if (n == 1 && skip_single) return;           // the row's own workgroup has moved its tail on
  float* tl = tail + (size_t)slots[r] * keep * width;
  for (int i = 0; i < keep; ++i) {
    const int src = n + i;                     // place in the joined sequence of keep + n inputs
    const int tok = a0 + src - keep;
    tl[(size_t)i * width + c] = src < keep ? tl[(size_t)src * width + c] : stream[(size_t)tok * width + c] * rstd[tok] * w1[c];
  }
}

// stream [tokens, width] float32; w1, w2 (or null), taps [width, K] float32; tail [slots, max(1, K - 1), width] float32;
// xm, y [tokens, width] of out_dtype; rstd: scratch of tokens floats.
MIE_EXPORT int mie_norm_pair_conv(const float* stream, const float* w1, const float* w2, const float* taps, float* tail,
                                  const int* token_row, const int* row_start, const int* slots, void* xm, void* y, int out_dtype,
                                  float* rstd, int tokens, int rows, int width, int K, float eps, hipStream_t s) {
  if (tokens <= 0 || rows <= 0) return 0;
  if (width <= 0 || K < 1 || K > CONV_MAX_TAPS) MIE_FAIL("norm_pair_conv: width %d, %d taps (1 to %d)", width, K, CONV_MAX_TAPS);
  if (!stream || !w1 || !taps || !tail || !xm || !rstd || (w2 && !y)) MIE_FAIL("norm_pair_conv: a missing operand");
  if (out_dtype != MIE_F32 && out_dtype != MIE_BF16) MIE_FAIL("norm_pair_conv: out dtype code %d", out_dtype);
  const bool aligned = !(((uintptr_t)stream | (uintptr_t)w1 | (uintptr_t)w2 | (uintptr_t)taps | (uintptr_t)tail | (uintptr_t)xm |
                          (uintptr_t)y) & 15);
  const bool vec = width % 4 == 0 && width <= 4 * NPC_V * NORM_THREADS && aligned;    // that kernel moves single-token rows' tails itself
  if (vec) {
#define NPC_LAUNCH(TO_, K_)                                                                                                   \
  hipLaunchKernelGGL((norm_pair_conv_vec_kernel<TO_, K_>), dim3(tokens), dim3(NORM_THREADS), 0, s, stream, w1, w2, taps, tail, \
                     token_row, row_start, slots, (TO_*)xm, (TO_*)y, rstd, width, eps)
#define NPC_TAPS(TO_)                                                                                           \
  switch (K) {                                                                                                  \
    case 1: NPC_LAUNCH(TO_, 1); break; case 2: NPC_LAUNCH(TO_, 2); break; case 3: NPC_LAUNCH(TO_, 3); break;     \
    case 4: NPC_LAUNCH(TO_, 4); break; case 5: NPC_LAUNCH(TO_, 5); break; case 6: NPC_LAUNCH(TO_, 6); break;     \
    case 7: NPC_LAUNCH(TO_, 7); break; default: NPC_LAUNCH(TO_, 8); break;                                       \
  }
    if (out_dtype == MIE_F32) { NPC_TAPS(float) } else { NPC_TAPS(bf16) }
#undef NPC_TAPS
#undef NPC_LAUNCH
  } else if (out_dtype == MIE_F32)
    hipLaunchKernelGGL(norm_pair_conv_kernel<float>, dim3(tokens), dim3(NORM_THREADS), 0, s, stream, w1, w2, taps, tail, token_row,
                       row_start, slots, (float*)xm, (float*)y, rstd, width, K, eps);
  else
    hipLaunchKernelGGL(norm_pair_conv_kernel<bf16>, dim3(tokens), dim3(NORM_THREADS), 0, s, stream, w1, w2, taps, tail, token_row,
                       row_start, slots, (bf16*)xm, (bf16*)y, rstd, width, K, eps);
  MIE_CHECK_LAUNCH("norm_pair_conv");
  if (K > 1 && !(vec && tokens == rows)) {
    hipLaunchKernelGGL(norm_conv_tail_kernel, dim3(rows, (width + 255) / 256), dim3(256), 0, s, stream, w1, rstd, tail, row_start,
                       slots, width, K, (int)vec);
    MIE_CHECK_LAUNCH("norm_pair_conv (tail)");
  }
  return 0;
}

// ---- a normed branch output added to the stream, and the next sublayer's normed, convolved input, for steps whose rows
// are single tokens (every input before a row's token comes from its tail):
//   stream[t] += y[t] * rstd(y[t]) * wb;  h = stream[t] * rstd(stream[t]) * w1;
//   xm[t] = h + sum_k taps[:, k] * (k == K - 1 ? h : tail[slot][k]);  tail[slot] moves on by h.
// One workgroup a token; widths that are a multiple of 4 up to 8192; the sums in the order of the two kernels it replaces.
template <typename TO, int K>
__global__ void __launch_bounds__(NORM_THREADS)
branch_norm_conv_single_kernel(const float* __restrict__ y, float* __restrict__ stream, const float* __restrict__ wb, float eps_b,
                               const float* __restrict__ w1, const float* __restrict__ taps, float* __restrict__ tail,
                               const int* __restrict__ slots, TO* __restrict__ xm, int width, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, nv = width / 4;
  const float4* yr = reinterpret_cast<const float4*>(y + (size_t)t * width);
  float4* sr = reinterpret_cast<float4*>(stream + (size_t)t * width);
  float4 xo[NPC_V];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NPC_V; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    xo[k] = i < nv ? yr[i] : make_float4(0.f, 0.f, 0.f, 0.f);
    ss = fmaf(xo[k].x, xo[k].x, fmaf(xo[k].y, xo[k].y, fmaf(xo[k].z, xo[k].z, fmaf(xo[k].w, xo[k].w, ss))));
  }
  const float rb = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps_b);
  ss = 0.f;
#pragma unroll
  for (int k = 0; k < NPC_V; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    if (i >= nv) continue;
    const float4 s = sr[i], g = reinterpret_cast<const float4*>(wb)[i];
    xo[k] = make_float4(s.x + xo[k].x * rb * g.x, s.y + xo[k].y * rb * g.y, s.z + xo[k].z * rb * g.z, s.w + xo[k].w * rb * g.w);
    sr[i] = xo[k];
    ss = fmaf(xo[k].x, xo[k].x, fmaf(xo[k].y, xo[k].y, fmaf(xo[k].z, xo[k].z, fmaf(xo[k].w, xo[k].w, ss))));
  }
  const float rstd = 1.0f / sqrtf(block_sum(ss, scratch) / (float)width + eps);
  float4* tl = reinterpret_cast<float4*>(tail + (size_t)slots[t] * (K > 1 ? K - 1 : 1) * width);
#pragma unroll
  for (int k = 0; k < NPC_V; ++k) {
    const int i = threadIdx.x + k * NORM_THREADS;
    if (i >= nv) continue;
    const float4 g = reinterpret_cast<const float4*>(w1)[i];
    float tp[4 * K];                                  // taps of channels 4 i .. 4 i + 3, K each
#pragma unroll
    for (int q = 0; q < K; ++q) {
      const float4 v = reinterpret_cast<const float4*>(taps + (size_t)i * 4 * K)[q];
      tp[4 * q] = v.x, tp[4 * q + 1] = v.y, tp[4 * q + 2] = v.z, tp[4 * q + 3] = v.w;
    }
    const float h0[4] = {xo[k].x * rstd * g.x, xo[k].y * rstd * g.y, xo[k].z * rstd * g.z, xo[k].w * rstd * g.w};
    float acc[4] = {h0[0], h0[1], h0[2], h0[3]};
    float4 old[K > 1 ? K - 1 : 1];
#pragma unroll
    for (int b = 0; b < K; ++b) {
      float h[4];
      if (b == 0) {
        h[0] = h0[0], h[1] = h0[1], h[2] = h0[2], h[3] = h0[3];
      } else {
        const float4 v = tl[(size_t)(K - 1 - b) * nv + i];
        old[K - 1 - b] = v;
        h[0] = v.x, h[1] = v.y, h[2] = v.z, h[3] = v.w;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = fmaf(tp[e * K + (K - 1 - b)], h[e], acc[e]);
    }
    store4(xm + (size_t)t * width + 4 * i, acc[0], acc[1], acc[2], acc[3]);
    if (K > 1) {
#pragma unroll
      for (int b = 0; b + 2 < K; ++b) tl[(size_t)b * nv + i] = old[b + 1];
      tl[(size_t)(K - 2) * nv + i] = make_float4(h0[0], h0[1], h0[2], h0[3]);
    }
  }
}

// y, stream [tokens, width] float32 (every token a row of its own, in slots[token]); wb, w1 [width] and taps [width, K]
// float32; tail [slots, max(1, K - 1), width] float32; xm [tokens, width] of out_dtype.  Width a multiple of 4 up to
// 8192, operands 16-byte aligned.
MIE_EXPORT int mie_branch_norm_conv_single(const float* y, float* stream, const float* wb, float eps_b, const float* w1,
                                           const float* taps, float* tail, const int* slots, void* xm, int out_dtype, int tokens,
                                           int width, int K, float eps, hipStream_t s) {
  if (tokens <= 0) return 0;
  if (K < 1 || K > CONV_MAX_TAPS) MIE_FAIL("branch_norm_conv_single: %d taps (1 to %d)", K, CONV_MAX_TAPS);
  if (!y || !stream || !wb || !w1 || !taps || !tail || !slots || !xm) MIE_FAIL("branch_norm_conv_single: a missing operand");
  if (out_dtype != MIE_F32 && out_dtype != MIE_BF16) MIE_FAIL("branch_norm_conv_single: out dtype code %d", out_dtype);
  const bool aligned = !(((uintptr_t)y | (uintptr_t)stream | (uintptr_t)wb | (uintptr_t)w1 | (uintptr_t)taps | (uintptr_t)tail |
                          (uintptr_t)xm) & 15);
  if (width <= 0 || width % 4 || width > 4 * NPC_V * NORM_THREADS || !aligned)
    MIE_FAIL("branch_norm_conv_single: width %d (a multiple of 4 up to %d) or an operand that is not 16-byte aligned", width,
             4 * NPC_V * NORM_THREADS);
#define BNC_LAUNCH(TO_, K_)                                                                                                   \
  hipLaunchKernelGGL((branch_norm_conv_single_kernel<TO_, K_>), dim3(tokens), dim3(NORM_THREADS), 0, s, y, stream, wb, eps_b, w1, \
                     taps, tail, slots, (TO_*)xm, width, eps)
#define BNC_TAPS(TO_)                                                                                           \
  switch (K) {                                                                                                  \
    case 1: BNC_LAUNCH(TO_, 1); break; case 2: BNC_LAUNCH(TO_, 2); break; case 3: BNC_LAUNCH(TO_, 3); break;     \
    case 4: BNC_LAUNCH(TO_, 4); break; case 5: BNC_LAUNCH(TO_, 5); break; case 6: BNC_LAUNCH(TO_, 6); break;     \
    case 7: BNC_LAUNCH(TO_, 7); break; default: BNC_LAUNCH(TO_, 8); break;                                       \
  }
  if (out_dtype == MIE_F32) { BNC_TAPS(float) } else { BNC_TAPS(bf16) }
#undef BNC_TAPS
#undef BNC_LAUNCH
  MIE_CHECK_LAUNCH("branch_norm_conv_single");
  return 0;
}

// ---- t *= factor
__global__ void scale_kernel(float* __restrict__ t, size_t n, float factor) {
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) t[i] *= factor;
}

MIE_EXPORT int mie_scale(float* t, long n, float factor, hipStream_t s) {
  if (n <= 0) return 0;
  long blocks = (n + 255) / 256;
  hipLaunchKernelGGL(scale_kernel, dim3((unsigned)(blocks > 4096 ? 4096 : blocks)), dim3(256), 0, s, t, (size_t)n, factor);
  MIE_CHECK_LAUNCH("scale");
  return 0;
}
