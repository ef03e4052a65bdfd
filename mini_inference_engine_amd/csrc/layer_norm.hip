// Layer norm with weight and bias on the 32-bit residual stream, and what follows the last product of a model.
//
// ln(r)[i] = (r[i] - mean) / sqrt(var + eps) * w[i] + b[i], mean and var (the mean of the squared deviations) of the
// row, two passes over values kept in registers, all in 32-bit.  Weights and biases are float32.
//
// add_layernorm:        r = stream[row] (+ x[row]); stream[row] = r (unless rows are gathered); y = ln(r)
// branch_layernorm_add: stream[row] += ln_out(y[row]); and, if a next norm is named, x[row] = ln_next(stream[row]):
//                       the step between two sublayers of a block with a norm before and after each, as one kernel
// scale_softcap:        t = cap * tanh(t * scale / cap) (cap <= 0: t * scale)
// One workgroup a row; every reduction's order depends on the width alone.
#include "common.hpp"

#define LN_THREADS 256
#define LN_CACHE 16          // numbers of a row a thread keeps: widths up to 4096 stay in registers

// mean and 1 / sqrt(var + eps) of a row whose first LN_CACHE * LN_THREADS numbers are in ``cache`` (zeros beyond the
// width) and the rest in ``rest`` (global or LDS memory, read again)
template <typename F>
__device__ __forceinline__ void row_moments(const float (&cache)[LN_CACHE], F rest, int width, float eps, float* scratch,
                                            float& mean, float& rstd) {
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < LN_CACHE; ++k) sum += cache[k];
  for (int i = threadIdx.x + LN_CACHE * LN_THREADS; i < width; i += LN_THREADS) sum += rest(i);
  mean = block_sum(sum, scratch) / (float)width;
  float dev = 0.f;
#pragma unroll
  for (int k = 0; k < LN_CACHE; ++k) {
    const int i = threadIdx.x + k * LN_THREADS;
    const float d = i < width ? cache[k] - mean : 0.f;
    dev = fmaf(d, d, dev);
  }
  for (int i = threadIdx.x + LN_CACHE * LN_THREADS; i < width; i += LN_THREADS) {
    const float d = rest(i) - mean;
    dev = fmaf(d, d, dev);
  }
  rstd = 1.0f / sqrtf(block_sum(dev, scratch) / (float)width + eps);
}

template <typename TX, typename TY>
__global__ void __launch_bounds__(LN_THREADS)
add_layernorm_kernel(const TX* __restrict__ x, float* __restrict__ stream, const float* __restrict__ weight,
                     const float* __restrict__ bias, TY* __restrict__ y, const int* __restrict__ rows, int width, float eps) {
  __shared__ float scratch[16];
  const int out_row = blockIdx.x;
  const int row = rows ? rows[out_row] : out_row;
  float* sr = stream + (size_t)row * width;
  const TX* xr = x ? x + (size_t)row * width : nullptr;
  const bool write_back = xr && !rows;
  float cache[LN_CACHE];
#pragma unroll
  for (int k = 0; k < LN_CACHE; ++k) {
    const int i = threadIdx.x + k * LN_THREADS;
    float r = 0.f;
    if (i < width) {
      r = sr[i];
      if (xr) r += to_float(xr[i]);
      if (write_back) sr[i] = r;
    }
    cache[k] = r;
  }
  // beyond the registers a thread reads its own numbers again (what it wrote back itself, or stream + x)
  auto rest = [&](int i) {
    float r = sr[i];
    if (xr && !write_back) r += to_float(xr[i]);
    return r;
  };
  if (write_back)
    for (int i = threadIdx.x + LN_CACHE * LN_THREADS; i < width; i += LN_THREADS) sr[i] += to_float(xr[i]);
  float mean, rstd;
  row_moments(cache, rest, width, eps, scratch, mean, rstd);
  TY* yr = y + (size_t)out_row * width;
#pragma unroll
  for (int k = 0; k < LN_CACHE; ++k) {
    const int i = threadIdx.x + k * LN_THREADS;
    if (i < width) yr[i] = from_float<TY>(fmaf((cache[k] - mean) * rstd, weight[i], bias[i]));
  }
  for (int i = threadIdx.x + LN_CACHE * LN_THREADS; i < width; i += LN_THREADS)
    yr[i] = from_float<TY>(fmaf((rest(i) - mean) * rstd, weight[i], bias[i]));
}

// x [rows, width] of x_dtype or null; weight, bias float32 [width]; y [n_rows, width] of y_dtype; rows int32 [n_rows] or null
MIE_EXPORT int mie_add_layernorm(const void* x, int x_dtype, float* stream, const float* weight, const float* bias, void* y,
                                 int y_dtype, const int* rows, int n_rows, int width, float eps, hipStream_t s) {
  if (n_rows <= 0) return 0;
  if (width <= 0 || !stream || !weight || !bias || !y) MIE_FAIL("add_layernorm: width %d or a null operand", width);
#define LN_LAUNCH(TX, TY)                                                                                              \
  hipLaunchKernelGGL((add_layernorm_kernel<TX, TY>), dim3(n_rows), dim3(LN_THREADS), 0, s, (const TX*)x, stream, weight, \
                     bias, (TY*)y, rows, width, eps)
  if (x_dtype == MIE_F32 && y_dtype == MIE_F32) LN_LAUNCH(float, float);
  else if (x_dtype == MIE_F32 && y_dtype == MIE_BF16) LN_LAUNCH(float, bf16);
  else if (x_dtype == MIE_BF16 && y_dtype == MIE_F32) LN_LAUNCH(bf16, float);
  else if (x_dtype == MIE_BF16 && y_dtype == MIE_BF16) LN_LAUNCH(bf16, bf16);
  else MIE_FAIL("add_layernorm: dtype codes x %d, y %d", x_dtype, y_dtype);
#undef LN_LAUNCH
  MIE_CHECK_LAUNCH("add_layernorm");
  return 0;
}

template <typename TY, typename TO>
__global__ void __launch_bounds__(LN_THREADS)
branch_layernorm_add_kernel(const TY* __restrict__ y, float* __restrict__ stream, const float* __restrict__ w_out,
                            const float* __restrict__ b_out, float eps_out, const float* __restrict__ w_next,
                            const float* __restrict__ b_next, float eps_next, TO* __restrict__ x, int width) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  float* sr = stream + (size_t)row * width;
  const TY* yr = y + (size_t)row * width;
  float cache[LN_CACHE];
#pragma unroll
  for (int k = 0; k < LN_CACHE; ++k) {
    const int i = threadIdx.x + k * LN_THREADS;
    cache[k] = i < width ? to_float(yr[i]) : 0.f;
  }
  float mean, rstd;
  row_moments(cache, [&](int i) { return to_float(yr[i]); }, width, eps_out, scratch, mean, rstd);
  // the updated stream takes the branch output's place in the registers
#pragma unroll
  for (int k = 0; k < LN_CACHE; ++k) {
    const int i = threadIdx.x + k * LN_THREADS;
    if (i < width) {
      const float r = sr[i] + fmaf((cache[k] - mean) * rstd, w_out[i], b_out[i]);
      sr[i] = r;
      cache[k] = r;
    }
  }
  for (int i = threadIdx.x + LN_CACHE * LN_THREADS; i < width; i += LN_THREADS)
    sr[i] += fmaf((to_float(yr[i]) - mean) * rstd, w_out[i], b_out[i]);
  if (!w_next) return;
  auto rest = [&](int i) { return sr[i]; };      // a thread reads what it wrote itself
  row_moments(cache, rest, width, eps_next, scratch, mean, rstd);
  TO* xr = x + (size_t)row * width;
#pragma unroll
  for (int k = 0; k < LN_CACHE; ++k) {
    const int i = threadIdx.x + k * LN_THREADS;
    if (i < width) xr[i] = from_float<TO>(fmaf((cache[k] - mean) * rstd, w_next[i], b_next[i]));
  }
  for (int i = threadIdx.x + LN_CACHE * LN_THREADS; i < width; i += LN_THREADS)
    xr[i] = from_float<TO>(fmaf((rest(i) - mean) * rstd, w_next[i], b_next[i]));
}


// The same for widths that are a multiple of 4 up to 4 * LN_THREADS * VEC: four numbers a load, every load of a row
// (branch output, stream, weights, biases) issued before anything is reduced.  Few rows (a decode step) cost latency
// alone, and the waits of one load after the other were most of it.  A row takes this path whenever its width allows,
// whatever the batch is, so a row's result does not depend on the batch.
__device__ __forceinline__ float4 ln_load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ln_load4(const bf16* p) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xFFFF0000u), __uint_as_float(r.y << 16),
                     __uint_as_float(r.y & 0xFFFF0000u));
}
__device__ __forceinline__ void ln_store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void ln_store4(bf16* p, float4 v) {
  union { bf16 h[4]; uint2 u; } o;
  o.h[0] = __float2bfloat16(v.x); o.h[1] = __float2bfloat16(v.y); o.h[2] = __float2bfloat16(v.z); o.h[3] = __float2bfloat16(v.w);
  *reinterpret_cast<uint2*>(p) = o.u;
}

template <int VEC>
__device__ __forceinline__ void row_moments4(const float4 (&v)[VEC], int groups, int width, float eps, float* scratch,
                                             float& mean, float& rstd) {
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < VEC; ++k) sum += (v[k].x + v[k].y) + (v[k].z + v[k].w);      // zeros beyond the width
  mean = block_sum(sum, scratch) / (float)width;
  float dev = 0.f;
#pragma unroll
  for (int k = 0; k < VEC; ++k)
    if ((int)threadIdx.x + k * LN_THREADS < groups) {
      const float a = v[k].x - mean, b = v[k].y - mean, c = v[k].z - mean, d = v[k].w - mean;
      dev += (a * a + b * b) + (c * c + d * d);
    }
  rstd = 1.0f / sqrtf(block_sum(dev, scratch) / (float)width + eps);
}

template <typename TY, typename TO, int VEC>
__global__ void __launch_bounds__(LN_THREADS)
branch_layernorm_add_fast_kernel(const TY* __restrict__ y, float* __restrict__ stream, const float* __restrict__ w_out,
                                 const float* __restrict__ b_out, float eps_out, const float* __restrict__ w_next,
                                 const float* __restrict__ b_next, float eps_next, TO* __restrict__ x, int width) {
  __shared__ float scratch[16];
  const int row = blockIdx.x, groups = width >> 2;
  float* sr = stream + (size_t)row * width;
  const TY* yr = y + (size_t)row * width;
  float4 v[VEC], s[VEC], w[VEC], b[VEC];
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const int i = 4 * ((int)threadIdx.x + k * LN_THREADS);
    const bool in = i < width;
    v[k] = in ? ln_load4(yr + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    s[k] = in ? ln_load4(sr + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    w[k] = in ? ln_load4(w_out + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    b[k] = in ? ln_load4(b_out + i) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  float4 w2[VEC], b2[VEC];
  if (w_next) {
#pragma unroll
    for (int k = 0; k < VEC; ++k) {
      const int i = 4 * ((int)threadIdx.x + k * LN_THREADS);
      const bool in = i < width;
      w2[k] = in ? ln_load4(w_next + i) : make_float4(0.f, 0.f, 0.f, 0.f);
      b2[k] = in ? ln_load4(b_next + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
  float mean, rstd;
  row_moments4<VEC>(v, groups, width, eps_out, scratch, mean, rstd);
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const int i = 4 * ((int)threadIdx.x + k * LN_THREADS);
    s[k].x += fmaf((v[k].x - mean) * rstd, w[k].x, b[k].x);
    s[k].y += fmaf((v[k].y - mean) * rstd, w[k].y, b[k].y);
    s[k].z += fmaf((v[k].z - mean) * rstd, w[k].z, b[k].z);
    s[k].w += fmaf((v[k].w - mean) * rstd, w[k].w, b[k].w);
    if (i < width) ln_store4(sr + i, s[k]);
    else s[k] = make_float4(0.f, 0.f, 0.f, 0.f);
  }
  if (!w_next) return;
  row_moments4<VEC>(s, groups, width, eps_next, scratch, mean, rstd);
  TO* xr = x + (size_t)row * width;
#pragma unroll
  for (int k = 0; k < VEC; ++k) {
    const int i = 4 * ((int)threadIdx.x + k * LN_THREADS);
    if (i < width)
      ln_store4(xr + i, make_float4(fmaf((s[k].x - mean) * rstd, w2[k].x, b2[k].x), fmaf((s[k].y - mean) * rstd, w2[k].y, b2[k].y),
                                    fmaf((s[k].z - mean) * rstd, w2[k].z, b2[k].z), fmaf((s[k].w - mean) * rstd, w2[k].w, b2[k].w)));
  }
}

template <typename TY, typename TO>
static bool branch_layernorm_add_fast(const void* y, float* stream, const float* w_out, const float* b_out, float eps_out,
                                      const float* w_next, const float* b_next, float eps_next, void* x, int rows, int width,
                                      hipStream_t s) {
  auto aligned = [](const void* p, size_t a) { return ((uintptr_t)p % a) == 0; };
  if (width % 4 || width > 4 * LN_THREADS * 8 || !aligned(y, sizeof(TY) * 4) || !aligned(stream, 16) || !aligned(w_out, 16) ||
      !aligned(b_out, 16) || !aligned(w_next, 16) || !aligned(b_next, 16) || !aligned(x, sizeof(TO) * 4))
    return false;
  const int per = (width / 4 + LN_THREADS - 1) / LN_THREADS;
#define BLNF(V)                                                                                                          \
  hipLaunchKernelGGL((branch_layernorm_add_fast_kernel<TY, TO, V>), dim3(rows), dim3(LN_THREADS), 0, s, (const TY*)y, stream, \
                     w_out, b_out, eps_out, w_next, b_next, eps_next, (TO*)x, width)
  if (per <= 1) BLNF(1); else if (per <= 2) BLNF(2); else if (per <= 4) BLNF(4); else BLNF(8);
#undef BLNF
  return true;
}

// y [rows, width] of y_dtype; w_out, b_out float32 [width]; w_next, b_next float32 [width] or both null (then x is not written);
// x [rows, width] of x_dtype
MIE_EXPORT int mie_branch_layernorm_add(const void* y, int y_dtype, float* stream, const float* w_out, const float* b_out,
                                        float eps_out, const float* w_next, const float* b_next, float eps_next, void* x,
                                        int x_dtype, int rows, int width, hipStream_t s) {
  if (rows <= 0) return 0;
  if (width <= 0 || !y || !stream || !w_out || !b_out) MIE_FAIL("branch_layernorm_add: width %d or a null operand", width);
  if ((w_next == nullptr) != (b_next == nullptr) || (w_next && !x))
    MIE_FAIL("branch_layernorm_add: the next norm needs weight, bias and an output");
#define BLN_LAUNCH(TY, TO)                                                                                                 \
  do {                                                                                                                     \
    if (!branch_layernorm_add_fast<TY, TO>(y, stream, w_out, b_out, eps_out, w_next, b_next, eps_next, x, rows, width, s)) \
      BLN_SLOW(TY, TO);                                                                                                    \
  } while (0)
#define BLN_SLOW(TY, TO)                                                                                            \
  hipLaunchKernelGGL((branch_layernorm_add_kernel<TY, TO>), dim3(rows), dim3(LN_THREADS), 0, s, (const TY*)y, stream, \
                     w_out, b_out, eps_out, w_next, b_next, eps_next, (TO*)x, width)
  if (y_dtype == MIE_F32 && x_dtype == MIE_F32) BLN_LAUNCH(float, float);
  else if (y_dtype == MIE_F32 && x_dtype == MIE_BF16) BLN_LAUNCH(float, bf16);
  else if (y_dtype == MIE_BF16 && x_dtype == MIE_F32) BLN_LAUNCH(bf16, float);
  else if (y_dtype == MIE_BF16 && x_dtype == MIE_BF16) BLN_LAUNCH(bf16, bf16);
  else MIE_FAIL("branch_layernorm_add: dtype codes y %d, x %d", y_dtype, x_dtype);
#undef BLN_LAUNCH
#undef BLN_SLOW
  MIE_CHECK_LAUNCH("branch_layernorm_add");
  return 0;
}

// ---- t = cap * tanh(t * scale / cap), or t * scale where cap <= 0
__global__ void scale_softcap_kernel(float* __restrict__ t, size_t n, float scale, float cap) {
  const float inv = cap > 0.f ? 1.0f / cap : 0.f;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) {
    const float v = t[i] * scale;
    t[i] = cap > 0.f ? cap * tanhf(v * inv) : v;
  }
}

MIE_EXPORT int mie_scale_softcap(float* t, long n, float scale, float cap, hipStream_t s) {
  if (n <= 0) return 0;
  long blocks = (n + 255) / 256;
  hipLaunchKernelGGL(scale_softcap_kernel, dim3((unsigned)(blocks > 4096 ? 4096 : blocks)), dim3(256), 0, s, t, (size_t)n,
                     scale, cap);
  MIE_CHECK_LAUNCH("scale_softcap");
  return 0;
}

MIE_EXPORT const char* layer_norm_last_error() { return g_mie_error; }
