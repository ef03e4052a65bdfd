// Between a q/k/v projection's float32 sums and attention, for mixers that want more than a rotation there:
// an RMS norm over a token's whole query (key) projection (or head by head, with one weight of a head's size for all
// heads), the rotation of the first numbers of every head by
// angles computed here in 32-bit (adjacent pairs or the two halves of the turned part), a temperature a query
// head, the projection's biases, a query temperature that grows with the logarithm of the position, values that are the keys as projected, and heads kept in the cache at a padded size.
//
// qkv_finish: one workgroup a token.  Queries go out as [T, Hq, P], keys to k_cache [pages, Hkv, page, P], values
// to v_cache [pages, Hkv, P, page] (transposed within a page), zeros beyond dim / vdim.  Everything is computed in
// 32-bit from the sums and rounded once on the way out.
// head_gate:  o[t, h, :] *= sigmoid(gate[t, h]).
#include "common.hpp"

enum { LAYOUT_INTERLEAVED = 0, LAYOUT_HALF = 1 };

struct FinishArgs {
  const float* sums; long ld; int q_col, k_col, v_col;      // v_col < 0: the values are the keys as projected
  const float* q_norm; const float* k_norm; float eps;
  int norm_per_head;            // the norms are taken head by head; q_norm and k_norm hold dim numbers each
  const float* inv_freq; int nf, layout;
  const float* q_head_scale;
  const float* col_bias;        // one number a column of the sums, added to queries, keys and values first (or null)
  float temp_coef; int temp_every;   // queries times 1 + temp_coef * ln(floor((p + 1) / temp_every) + 1) at position p (temp_every 0: not)
  const int* positions; const int* slots;
  void* q_out; void* k_cache; void* v_cache;
  int Hq, Hkv, dim, vdim, P, page;
};

template <typename TO>
__global__ void __launch_bounds__(256)
qkv_finish_kernel(FinishArgs a) {
  __shared__ float scratch[16];
  // blockIdx.y: which share of the token's heads this workgroup makes (every one takes the norms' sums itself)
  const int t = blockIdx.x;
  const float* __restrict__ row = a.sums + (size_t)t * a.ld;
  const float* __restrict__ q = row + a.q_col;
  const float* __restrict__ k = row + a.k_col;
  const float* __restrict__ qb = a.col_bias ? a.col_bias + a.q_col : nullptr;
  const float* __restrict__ kb = a.col_bias ? a.col_bias + a.k_col : nullptr;
  const float* __restrict__ vb = a.col_bias ? a.col_bias + (a.v_col < 0 ? a.k_col : a.v_col) : nullptr;
  const int nq = a.Hq * a.dim, nk = a.Hkv * a.dim;
  float rq = 1.f, rk = 1.f;
  if (a.q_norm && !a.norm_per_head) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nq; i += blockDim.x) {
      const float v = qb ? q[i] + qb[i] : q[i];
      ss = fmaf(v, v, ss);
    }
    rq = 1.0f / sqrtf(block_sum(ss, scratch) / (float)nq + a.eps);
  }
  if (a.k_norm && !a.norm_per_head) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nk; i += blockDim.x) {
      const float v = kb ? k[i] + kb[i] : k[i];
      ss = fmaf(v, v, ss);
    }
    rk = 1.0f / sqrtf(block_sum(ss, scratch) / (float)nk + a.eps);
  }
  // the angles' cosines and sines once a token: every head turns by the same ones
  extern __shared__ float cs[];                 // cos [nf], sin [nf]
  const float pos = (float)a.positions[t];
  const float temperature = a.temp_every > 0 ? 1.0f + a.temp_coef * logf((float)((a.positions[t] + 1) / a.temp_every) + 1.0f) : 1.0f;
  for (int i = threadIdx.x; i < a.nf; i += blockDim.x) sincosf(pos * a.inv_freq[i], &cs[a.nf + i], &cs[i]);
  __syncthreads();
  // A wave a head (query heads first, then key heads with their values), lanes over the head's pairs and then over what
  // does not turn: both members of a pair come from one lane, which reads each of its numbers once.
  const int turned = 2 * a.nf, lane = threadIdx.x & 63;
  const int wave = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6), waves = gridDim.y * (blockDim.x >> 6);
  const int slot = a.slots[t];
  const size_t pg = slot / a.page, off = slot % a.page;
  TO* __restrict__ qo = (TO*)a.q_out + (size_t)t * a.Hq * a.P;
  TO* __restrict__ kc = (TO*)a.k_cache;
  TO* __restrict__ vc = (TO*)a.v_cache;
  const float* __restrict__ vals = a.v_col < 0 ? k : row + a.v_col;
  for (int job = wave; job < a.Hq + a.Hkv; job += waves) {
    const bool is_q = job < a.Hq;
    const int h = is_q ? job : job - a.Hq;
    const float* __restrict__ x = (is_q ? q : k) + (size_t)h * a.dim;
    const float* __restrict__ xb = (is_q ? qb : kb) ? (is_q ? qb : kb) + (size_t)h * a.dim : nullptr;
    const float* __restrict__ w = is_q ? a.q_norm : a.k_norm;
    if (w && !a.norm_per_head) w += (size_t)h * a.dim;
    float r = is_q ? rq : rk;
    if (w && a.norm_per_head) {       // the wave owns the head: its root mean square by a sum over the lanes
      float ss = 0.f;
      for (int d = lane; d < a.dim; d += 64) {
        const float v = xb ? x[d] + xb[d] : x[d];
        ss = fmaf(v, v, ss);
      }
      r = 1.0f / sqrtf(wave_sum(ss) / (float)a.dim + a.eps);
    }
    const float mult = is_q ? (a.q_head_scale ? a.q_head_scale[h] * temperature : temperature) : 1.f;
    TO* __restrict__ dst = is_q ? qo + (size_t)h * a.P : kc + ((pg * a.Hkv + h) * a.page + off) * a.P;
    for (int i = lane; i < a.nf; i += 64) {
      const int d1 = a.layout == LAYOUT_INTERLEAVED ? 2 * i : i, d2 = a.layout == LAYOUT_INTERLEAVED ? 2 * i + 1 : i + a.nf;
      const float y1 = xb ? x[d1] + xb[d1] : x[d1], y2 = xb ? x[d2] + xb[d2] : x[d2];
      const float x1 = w ? y1 * r * w[d1] : y1, x2 = w ? y2 * r * w[d2] : y2;
      float o1, o2;
      rotate_pair(x1, x2, cs[i], cs[a.nf + i], o1, o2);
      dst[d1] = from_float<TO>(o1 * mult);
      dst[d2] = from_float<TO>(o2 * mult);
    }
    for (int d = turned + lane; d < a.P; d += 64) {
      const float y = d < a.dim ? (xb ? x[d] + xb[d] : x[d]) : 0.f;
      const float v = d < a.dim ? (w ? y * r * w[d] : y) * mult : 0.f;
      dst[d] = from_float<TO>(v);
    }
    if (!is_q) {
      const float* __restrict__ vh = vals + (size_t)h * a.vdim;
      const float* __restrict__ vhb = vb ? vb + (size_t)h * a.vdim : nullptr;
      TO* __restrict__ vd = vc + (pg * a.Hkv + h) * a.P * a.page + off;
      for (int d = lane; d < a.P; d += 64) vd[(size_t)d * a.page] = from_float<TO>(d < a.vdim ? (vhb ? vh[d] + vhb[d] : vh[d]) : 0.f);
    }
  }
}

MIE_EXPORT const char* attention_prep_last_error() { return g_mie_error; }

MIE_EXPORT int mie_qkv_finish(const float* sums, long ld, int q_col, int k_col, int v_col, const float* q_norm,
                              const float* k_norm, float eps, int norm_per_head, const float* inv_freq, int nf, int layout,
                              const float* q_head_scale, const int* positions, const int* slots, void* q_out, void* k_cache,
                              void* v_cache, int dtype, int tokens, int Hq, int Hkv, int dim, int vdim, int P, int page,
                              const float* col_bias, float temp_coef, int temp_every, hipStream_t s) {
  if (tokens <= 0) return 0;
  if (Hq <= 0 || Hkv <= 0 || dim <= 0 || vdim <= 0 || P < dim || P < vdim || page <= 0)
    MIE_FAIL("qkv_finish: %d / %d heads of %d (values %d) in %d, page %d", Hq, Hkv, dim, vdim, P, page);
  if (2 * nf > dim || nf < 0 || (nf > 0 && !inv_freq)) MIE_FAIL("qkv_finish: %d turned pairs in heads of %d", nf, dim);
  if (layout != LAYOUT_INTERLEAVED && layout != LAYOUT_HALF) MIE_FAIL("qkv_finish: layout code %d", layout);
  if (v_col < 0 && vdim != dim) MIE_FAIL("qkv_finish: values that are the keys have their size");
  if (temp_every < 0) MIE_FAIL("qkv_finish: a query temperature every %d positions", temp_every);
  FinishArgs a{sums, ld, q_col, k_col, v_col, q_norm, k_norm, eps, norm_per_head, inv_freq, nf, layout, q_head_scale, col_bias, temp_coef, temp_every,
               positions, slots, q_out, k_cache, v_cache, Hq, Hkv, dim, vdim, P, page};
  const size_t lds = (size_t)2 * (nf > 0 ? nf : 1) * sizeof(float);
  // few tokens: several workgroups a token, so that a decode step's few rows are spread over the GPU
  int parts = tokens >= 256 ? 1 : (Hq + Hkv + 3) / 4;
  parts = parts < 1 ? 1 : parts > 8 ? 8 : parts;
  if (dtype == MIE_F32) hipLaunchKernelGGL(qkv_finish_kernel<float>, dim3(tokens, parts), dim3(256), lds, s, a);
  else if (dtype == MIE_BF16) hipLaunchKernelGGL(qkv_finish_kernel<bf16>, dim3(tokens, parts), dim3(256), lds, s, a);
  else MIE_FAIL("qkv_finish: dtype code %d", dtype);
  MIE_CHECK_LAUNCH("qkv_finish");
  return 0;
}

template <typename T>
__global__ void __launch_bounds__(256)
head_gate_kernel(T* __restrict__ o, const float* __restrict__ gate, long ldg, int H, int D) {
  const int t = blockIdx.x;
  T* row = o + (size_t)t * H * D;
  for (int e = threadIdx.x; e < H * D; e += blockDim.x)
    row[e] = from_float<T>(to_float(row[e]) * mie_sigmoid(gate[(size_t)t * ldg + e / D]));
}

// gate points at the first gate column; rows are ldg floats apart
MIE_EXPORT int mie_head_gate(void* o, int dtype, const float* gate, long ldg, int tokens, int H, int D, hipStream_t s) {
  if (tokens <= 0) return 0;
  if (H <= 0 || D <= 0 || ldg < H) MIE_FAIL("head_gate: %d heads of %d, gate rows %ld apart", H, D, ldg);
  if (dtype == MIE_F32) hipLaunchKernelGGL(head_gate_kernel<float>, dim3(tokens), dim3(256), 0, s, (float*)o, gate, ldg, H, D);
  else if (dtype == MIE_BF16) hipLaunchKernelGGL(head_gate_kernel<bf16>, dim3(tokens), dim3(256), 0, s, (bf16*)o, gate, ldg, H, D);
  else MIE_FAIL("head_gate: dtype code %d", dtype);
  MIE_CHECK_LAUNCH("head_gate");
  return 0;
}
