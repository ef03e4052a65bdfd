// Gated linear attention over a step's rows, with the request's state in its slot; everything is 32-bit.
//
// Per head a state S [d, dv] (key channel i, value channel j):
//     S <- diag(alpha) S + k v^T,   o = S^T q,   alpha = sigmoid(z)^(1 / tau),  z = W2 a + b
// with q, k [d], v [dv] and the decay's inner activations a [rank] a token from one product's float32 sums.
// gla_prepare: a thread a (token, key channel): z in FMAs over the inner size, ascending; alpha = exp(logsigmoid(z) / tau),
//     the logarithm in the form that neither overflows nor cancels (min(z, 0) - log1p(exp(-|z|))).  -> decay [T, H d]
// gla_scan: a workgroup a (row, chunk, head); thread j owns column j of S in registers (the update of column j reads
//     that column only), tokens in order.  What all columns share (q * q_scale, k, alpha of a token) comes in through the
//     LDS, GLA_TB tokens at a time, the next batch on its way meanwhile.  The head's output is divided by its root mean
//     square, times the weight and silu of the output gate, and rounded once.
//
// Rows run whole (one chunk: S from state[slot], left there afterwards), or, long rows, in chunks of L tokens side by
// side in three passes, since a chunk acts on the state it starts from as S_end = diag(A) S_start + B, A the product of
// the chunk's decays and B the recurrence on zero:  (1) every chunk but a row's last computes A and B;  (2) per row and
// head, chunk after chunk, S_start(c + 1) = diag(A_c) S_start(c) + B_c from S_start(0) = state[slot];  (3) every chunk runs its tokens
// from its S_start and writes the outputs, a row's last chunk leaves state[slot].  The two ways differ by the rounding of
// pass 2 alone.
#include "common.hpp"

#define GLA_TB 8            // tokens staged in the LDS at a time

__global__ void __launch_bounds__(256)
gla_prepare_kernel(const float* __restrict__ sums, long ld, int a_col, const float* __restrict__ w2, int rank,
                   const float* __restrict__ bias, float inv_tau, float* __restrict__ decay, int tokens, int n) {
  extern __shared__ float inner[];          // [rank] of this token
  const int t = blockIdx.x;
  for (int r = threadIdx.x; r < rank; r += blockDim.x) inner[r] = sums[(size_t)t * ld + a_col + r];
  __syncthreads();
  for (int c = threadIdx.x; c < n; c += blockDim.x) {
    const float* w = w2 + (size_t)c * rank;
    float z = bias ? bias[c] : 0.f;
    float acc = 0.f;
    for (int r = 0; r < rank; ++r) acc = fmaf(w[r], inner[r], acc);
    z += acc;
    const float ls = fminf(z, 0.f) - log1pf(expf(-fabsf(z)));
    decay[(size_t)t * n + c] = expf(ls * inv_tau);
  }
}

struct GlaArgs {
  const float* sums; long ld; int q_col, k_col, v_col, g_col;
  const float* decay;            // [T, H d]
  const float* norm_weight; float eps, q_scale;
  float* state;                  // [slots, H, d, dv]
  const int* row_start; const int* slots;
  void* out;                     // [T, H dv]
  int H, d, dv;
  int chunk_tokens, max_chunks;  // 0: rows run whole
  int pass;                      // 0 whole rows; 1 summaries; 3 chunks from their starts
  float* sum_a;                  // [rows * max_chunks * H, d]
  float* sum_b;                  // [rows * max_chunks * H, d, dv]
  float* starts;                 // [rows * max_chunks * H, d, dv]
};

template <int DK, typename TO>
__global__ void __launch_bounds__(256)
gla_scan_kernel(GlaArgs a) {
  extern __shared__ __align__(16) float lds[];
  const int d = a.d, dv = a.dv, H = a.H;
  float* sq = lds;                       // [GLA_TB][DK]
  float* sk = sq + GLA_TB * DK;
  float* sa = sk + GLA_TB * DK;
  float* so = sa + GLA_TB * DK;          // [GLA_TB][dv]
  const int h = blockIdx.y, j = threadIdx.x, nthreads = blockDim.x;
  const int chunks = a.chunk_tokens > 0 ? a.max_chunks : 1;
  const int row = blockIdx.x / chunks, c = blockIdx.x % chunks;
  int t_begin = a.row_start[row], t_end = a.row_start[row + 1];
  int n_chunks = 1;
  if (a.chunk_tokens > 0) {
    n_chunks = (t_end - t_begin + a.chunk_tokens - 1) / a.chunk_tokens;
    if (c >= n_chunks) return;
    t_begin += c * a.chunk_tokens;
    if (t_begin + a.chunk_tokens < t_end) t_end = t_begin + a.chunk_tokens;
  }
  const bool last = c == n_chunks - 1;
  if (a.pass == 1 && last) return;          // nobody starts from the end of a row's last chunk
  const bool active = j < dv;
  const size_t unit = (size_t)blockIdx.x * H + h;       // this (row, chunk, head) in the scratch arrays
  float S[DK];
  float* st = a.state + ((size_t)a.slots[row] * H + h) * d * dv;
  const float* from = a.pass == 3 ? a.starts + unit * d * dv : st;      // pass 3 never reads the slot, which a row's last chunk writes
#pragma unroll
  for (int i = 0; i < DK; ++i) S[i] = (a.pass != 1 && active && i < d) ? from[(size_t)i * dv + j] : 0.f;
  float prod[(DK + 63) / 64];               // pass 1: the product of the decays of channels j, j + nthreads, ...
#pragma unroll
  for (int i = 0; i < (DK + 63) / 64; ++i) prod[i] = 1.f;
  const int waves = nthreads >> 6, wave = j >> 6, lane = j & 63;

  // What a batch of GLA_TB tokens brings in: q, k and the decays of the head (to the LDS) and this thread's values.  Up to
  // key sizes of 128 the next batch's numbers are asked for into registers before the current batch is computed (loads
  // from clamped addresses, never predicated: the compiler would wait for each where it is issued), so that memory's
  // latency hides behind the recurrence; wider heads have no registers to spare and load where they need.
  constexpr bool AHEAD = DK <= 128;
  constexpr int R = AHEAD ? (GLA_TB * DK + 63) / 64 : 1;      // numbers a thread carries when a workgroup is one wave
  float pq[R], pk[R], pa[R], pv[GLA_TB];
  auto fetch = [&](int t0) {
    const int nt = t_end - t0 < GLA_TB ? t_end - t0 : GLA_TB;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      int e = j + r * nthreads;
      e = e < nt * DK ? e : nt * DK - 1;
      const int tt = e / DK, i = e - tt * DK, ic = i < d ? i : d - 1;
      const size_t at = (size_t)(t0 + tt) * a.ld + (size_t)h * d + ic;
      pq[r] = a.sums[at + a.q_col];
      pk[r] = a.sums[at + a.k_col];
      pa[r] = a.decay[((size_t)(t0 + tt) * H + h) * d + ic];
    }
#pragma unroll
    for (int tt = 0; tt < GLA_TB; ++tt)
      pv[tt] = a.sums[(size_t)(t0 + (tt < nt ? tt : nt - 1)) * a.ld + a.v_col + (size_t)h * dv + (active ? j : 0)];
  };
  if (AHEAD && t_begin < t_end) fetch(t_begin);

  for (int t0 = t_begin; t0 < t_end; t0 += GLA_TB) {
    const int nt = t_end - t0 < GLA_TB ? t_end - t0 : GLA_TB;
    __syncthreads();
    float v[GLA_TB];
    if constexpr (AHEAD) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int e = j + r * nthreads;
        if (e < nt * DK) {
          const bool in = e % DK < d;
          sq[e] = in ? pq[r] * a.q_scale : 0.f;
          sk[e] = in ? pk[r] : 0.f;
          sa[e] = in ? pa[r] : 1.f;
        }
      }
#pragma unroll
      for (int tt = 0; tt < GLA_TB; ++tt) v[tt] = (active && tt < nt) ? pv[tt] : 0.f;
    } else {
      for (int e = j; e < nt * DK; e += nthreads) {
        const int tt = e / DK, i = e - tt * DK;
        const size_t r = (size_t)(t0 + tt) * a.ld + (size_t)h * d + i;
        const bool in = i < d;
        sq[e] = in ? a.sums[r + a.q_col] * a.q_scale : 0.f;
        sk[e] = in ? a.sums[r + a.k_col] : 0.f;
        sa[e] = in ? a.decay[((size_t)(t0 + tt) * H + h) * d + i] : 1.f;
      }
#pragma unroll
      for (int tt = 0; tt < GLA_TB; ++tt)
        v[tt] = (active && tt < nt) ? a.sums[(size_t)(t0 + tt) * a.ld + a.v_col + (size_t)h * dv + j] : 0.f;
    }
    __syncthreads();
    if (AHEAD && t0 + GLA_TB < t_end) fetch(t0 + GLA_TB);          // on its way while this batch is computed
#pragma unroll
    for (int tt = 0; tt < GLA_TB; ++tt) {
      if (tt < nt) {
        float o = 0.f;
        const float4* q4 = reinterpret_cast<const float4*>(sq + tt * DK);
        const float4* k4 = reinterpret_cast<const float4*>(sk + tt * DK);
        const float4* a4 = reinterpret_cast<const float4*>(sa + tt * DK);
#pragma unroll
        for (int i4 = 0; i4 < DK / 4; ++i4) {
          const float4 qq = q4[i4], kk = k4[i4], aa = a4[i4];
          S[4 * i4 + 0] = fmaf(aa.x, S[4 * i4 + 0], kk.x * v[tt]); o = fmaf(S[4 * i4 + 0], qq.x, o);
          S[4 * i4 + 1] = fmaf(aa.y, S[4 * i4 + 1], kk.y * v[tt]); o = fmaf(S[4 * i4 + 1], qq.y, o);
          S[4 * i4 + 2] = fmaf(aa.z, S[4 * i4 + 2], kk.z * v[tt]); o = fmaf(S[4 * i4 + 2], qq.z, o);
          S[4 * i4 + 3] = fmaf(aa.w, S[4 * i4 + 3], kk.w * v[tt]); o = fmaf(S[4 * i4 + 3], qq.w, o);
        }
        if (a.pass != 1 && active) so[tt * dv + j] = o;
        if (a.pass == 1) {
#pragma unroll
          for (int i = 0; i < (DK + 63) / 64; ++i)
            if (j + i * nthreads < DK) prod[i] *= sa[tt * DK + j + i * nthreads];
        }
      }
    }
    if (a.pass == 1) continue;
    __syncthreads();
    // the norm over the head's output, a wave a token: sums in lane order, the same whatever the step holds
    for (int tt = wave; tt < nt; tt += waves) {
      float ss = 0.f;
      for (int e = lane; e < dv; e += 64) ss = fmaf(so[tt * dv + e], so[tt * dv + e], ss);
      const float rstd = 1.0f / sqrtf(wave_sum(ss) / (float)dv + a.eps);
      const size_t r = (size_t)(t0 + tt);
      for (int e = lane; e < dv; e += 64) {
        const float g = a.sums[r * a.ld + a.g_col + (size_t)h * dv + e];
        const float y = so[tt * dv + e] * rstd * a.norm_weight[e] * (g / (1.0f + expf(-g)));
        ((TO*)a.out)[(r * H + h) * dv + e] = from_float<TO>(y);
      }
    }
  }
  if (a.pass == 1) {
    float* B = a.sum_b + unit * d * dv;
    if (active)
#pragma unroll
      for (int i = 0; i < DK; ++i)
        if (i < d) B[(size_t)i * dv + j] = S[i];
#pragma unroll
    for (int i = 0; i < (DK + 63) / 64; ++i)
      if (j + i * nthreads < d) a.sum_a[unit * d + j + i * nthreads] = prod[i];
  } else if (last && active) {
#pragma unroll
    for (int i = 0; i < DK; ++i)
      if (i < d) st[(size_t)i * dv + j] = S[i];
  }
}

// pass 2: S_start(0) = state[slot]; S_start(c + 1) = diag(A_c) S_start(c) + B_c, chunk after chunk; a thread an entry
__global__ void __launch_bounds__(256)
gla_fold_kernel(GlaArgs a) {
  const int row = blockIdx.x, h = blockIdx.y, d = a.d, dv = a.dv, H = a.H;
  const int n = a.row_start[row + 1] - a.row_start[row];
  const int n_chunks = (n + a.chunk_tokens - 1) / a.chunk_tokens;
  const float* st = a.state + ((size_t)a.slots[row] * H + h) * d * dv;
  for (int e = blockIdx.z * blockDim.x + threadIdx.x; e < d * dv; e += gridDim.z * blockDim.x) {
    const int i = e / dv;
    float s = st[e];
    a.starts[((size_t)row * a.max_chunks * H + h) * d * dv + e] = s;
    for (int c = 0; c + 1 < n_chunks; ++c) {
      const size_t unit = ((size_t)row * a.max_chunks + c) * H + h;
      s = fmaf(a.sum_a[unit * d + i], s, a.sum_b[unit * d * dv + e]);
      a.starts[(unit + H) * d * dv + e] = s;          // the start of chunk c + 1
    }
  }
}

MIE_EXPORT const char* gla_last_error() { return g_mie_error; }

template <int DK>
static void gla_launch_scan(const GlaArgs& a, int out_dtype, int units, int threads, hipStream_t s) {
  const size_t lds = (size_t)(3 * GLA_TB * DK + GLA_TB * a.dv) * sizeof(float);
  if (out_dtype == MIE_F32) hipLaunchKernelGGL((gla_scan_kernel<DK, float>), dim3(units, a.H), dim3(threads), lds, s, a);
  else hipLaunchKernelGGL((gla_scan_kernel<DK, bf16>), dim3(units, a.H), dim3(threads), lds, s, a);
}

static int gla_scan_any(const GlaArgs& a, int out_dtype, int units, hipStream_t s) {
  const int threads = (a.dv + 63) / 64 * 64;
  const int dk = (a.d + 15) / 16 * 16;
  switch (dk) {
#define GLA_CASE(N) case N: gla_launch_scan<N>(a, out_dtype, units, threads, s); break
    GLA_CASE(16); GLA_CASE(32); GLA_CASE(48); GLA_CASE(64); GLA_CASE(80); GLA_CASE(96); GLA_CASE(112); GLA_CASE(128);
#undef GLA_CASE
    default:
      if (dk <= 192) gla_launch_scan<192>(a, out_dtype, units, threads, s);
      else gla_launch_scan<256>(a, out_dtype, units, threads, s);
  }
  MIE_CHECK_LAUNCH("gla_scan");
  return 0;
}

// decay: scratch of tokens * H * d floats.  chunk_tokens 0: rows run whole.  Else rows run in chunks of that many tokens, at most
// max_chunks a row, with scratch sum_a [rows * max_chunks * H * d], sum_b and starts [rows * max_chunks * H * d * dv] floats.
MIE_EXPORT int mie_gla(const float* sums, long ld, int q_col, int k_col, int v_col, int g_col, int a_col, const float* w2,
                       int rank, const float* bias, float tau, float q_scale, const float* norm_weight, float eps, float* state,
                       const int* row_start, const int* slots, float* decay, void* out, int out_dtype, int tokens, int rows,
                       int H, int d, int dv, int chunk_tokens, int max_chunks, float* sum_a, float* sum_b, float* starts,
                       hipStream_t s) {
  if (tokens <= 0 || rows <= 0) return 0;
  if (H <= 0 || d <= 0 || dv <= 0 || d > 256 || dv > 256 || rank <= 0)
    MIE_FAIL("gla: %d heads of %d x %d, inner size %d (heads up to 256 x 256)", H, d, dv, rank);
  if (H > 65535) MIE_FAIL("gla: %d heads is beyond the grid", H);
  if (!(tau > 0.f)) MIE_FAIL("gla: tau %g", (double)tau);
  if (out_dtype != MIE_F32 && out_dtype != MIE_BF16) MIE_FAIL("gla: dtype code %d", out_dtype);
  if (chunk_tokens < 0 || (chunk_tokens > 0 && (max_chunks < 1 || !sum_a || !sum_b || !starts)))
    MIE_FAIL("gla: chunks of %d tokens, %d a row, need their scratch", chunk_tokens, max_chunks);
  if (!sums || !w2 || !norm_weight || !state || !row_start || !slots || !decay || !out) MIE_FAIL("gla: a null operand");
  hipLaunchKernelGGL(gla_prepare_kernel, dim3(tokens), dim3(256), (size_t)rank * sizeof(float), s, sums, ld, a_col, w2, rank,
                     bias, 1.0f / tau, decay, tokens, H * d);
  MIE_CHECK_LAUNCH("gla_prepare");
  GlaArgs a{sums, ld, q_col, k_col, v_col, g_col, decay, norm_weight, eps, q_scale, state, row_start, slots, out, H, d, dv,
            chunk_tokens, max_chunks, 0, sum_a, sum_b, starts};
  if (chunk_tokens == 0) return gla_scan_any(a, out_dtype, rows, s);
  const int units = rows * max_chunks;
  a.pass = 1;
  if (gla_scan_any(a, out_dtype, units, s)) return -1;
  const int per = (d * dv + 255) / 256;
  hipLaunchKernelGGL(gla_fold_kernel, dim3(rows, H, per < 8 ? per : 8), dim3(256), 0, s, a);
  MIE_CHECK_LAUNCH("gla_fold");
  a.pass = 3;
  return gla_scan_any(a, out_dtype, units, s);
}
