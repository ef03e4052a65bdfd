// Many small products in one launch, and the kernels around routed experts.
//
// grouped_linear: group g of G computes C_g = A_g W_g^T (+ bias_g), A_g [M_g, K], W_g [N, K], in one of two shapes:
//   columns   every group takes all M rows; its operands are column blocks: A + (g % a_mod) * a_group, W + g * w_group,
//             C + g * c_group (heads of an attention layer, the diagonal blocks of a block-diagonal matrix);
//   rows      group g takes rows offs[g] .. offs[g + 1] of a list sorted by group (experts): row r of the list reads
//             A row gather[r] / gather_div (or r) and writes C row r; offs lives on the device, so nothing waits for
//             the host to learn how many rows a group got.
// Epilogues: bias, an activation, or times sigmoid(gate[m, g N + n]).  Accumulation is one 32-bit FMA chain per
// output in increasing k whatever the tile, so a row's result does not depend on the rows beside it.
//
// route_topk, moe_align, moe_combine: choose a token's experts and their shares, sort (token, choice) pairs by
// expert, and add a token's expert outputs back together in the order of its choices.
#include "common.hpp"

#define GG_T 64
#define GG_K 16
#define GG_PAD 4

struct GroupedArgs {
  const void* A; long lda; long a_group; int a_mod;
  const void* W; long ldw; long w_group;
  void* C; long ldc; long c_group;
  const float* bias;            // [G, N] or null
  const float* gate; long ldg;  // gate[m * ldg + g * N + n] before its sigmoid, or null
  const int* offs;              // rows shape: [G + 1]; null: columns shape
  const int* gather; int gather_div;
  int M, N, K, G, act;
  const void* zeros;            // 64 bytes of zeros in device memory: what a load beyond a tile's rows or beyond K reads
  // glu != 0 (matrix-core kernel only): W's rows alternate in blocks of 16 gate rows and 16 up rows, and C [.., N / 2]
  // receives g * sigmoid(glu_alpha g) * (u + glu_shift), g = min(gate sum, glu_limit), u = clamp(up sum, -glu_limit, glu_limit)
  int glu; float glu_limit, glu_alpha, glu_shift;
};

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
grouped_gemm_kernel(GroupedArgs p) {
  __shared__ float As[GG_K][GG_T + GG_PAD];
  __shared__ float Ws[GG_K][GG_T + GG_PAD];
  __shared__ int a_rows[GG_T];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int n0 = blockIdx.x * GG_T;
  int g, m0, m_end, c_row0;
  if (p.offs) {
    int tile = blockIdx.y, start = 0, cnt = 0;
    for (g = 0; g < p.G; ++g) {
      start = p.offs[g];
      cnt = p.offs[g + 1] - start;
      const int nt = (cnt + GG_T - 1) / GG_T;
      if (tile < nt) break;
      tile -= nt;
    }
    if (g == p.G) return;
    m0 = tile * GG_T;
    m_end = cnt;
    c_row0 = start;
    if (tid < GG_T) {
      const int r = m0 + tid;
      a_rows[tid] = r < cnt ? (p.gather ? p.gather[start + r] / p.gather_div : start + r) : -1;
    }
  } else {
    g = blockIdx.z;
    m0 = blockIdx.y * GG_T;
    m_end = p.M;
    c_row0 = 0;
    if (tid < GG_T) a_rows[tid] = m0 + tid < p.M ? m0 + tid : -1;
  }
  __syncthreads();
  const TA* A = (const TA*)p.A + (size_t)(g % p.a_mod) * p.a_group;
  const TW* W = (const TW*)p.W + (size_t)g * p.w_group;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;
  for (int k0 = 0; k0 < p.K; k0 += GG_K) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int idx = tid + i * 256;
      const int r = idx >> 4, c = idx & 15, k = k0 + c;
      float a = 0.f, w = 0.f;
      if (k < p.K) {
        const int ar = a_rows[r];
        if (ar >= 0) a = to_float(A[(size_t)ar * p.lda + k]);
        if (n0 + r < p.N) w = to_float(W[(size_t)(n0 + r) * p.ldw + k]);
      }
      As[c][r] = a;
      Ws[c][r] = w;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GG_K; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
  TC* C = (TC*)p.C + (size_t)g * p.c_group;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= m_end) continue;
    const size_t crow = (size_t)(c_row0 + m);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= p.N) continue;
      float v = acc[i][j];
      if (p.bias) v += p.bias[(size_t)g * p.N + n];
      v = mie_act(v, p.act);
      if (p.gate) v *= mie_sigmoid(p.gate[crow * p.ldg + (size_t)g * p.N + n]);
      C[crow * p.ldc + n] = from_float<TC>(v);
    }
  }
}

// Few rows (a decode step) in the columns shape, any operand types, 32-bit FMAs: one wave an output column, the lanes
// spread over k (a weight row is read once, 64 consecutive numbers at a time), every lane one partial sum a row, then
// the wave's sum.  The order of a sum depends on K alone.
#define GV_ROWS 16
template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
grouped_gemv_kernel(GroupedArgs p) {
  const int lane = threadIdx.x & 63;
  const int n = blockIdx.x * 4 + (threadIdx.x >> 6), g = blockIdx.z;
  if (n >= p.N) return;
  const TA* A = (const TA*)p.A + (size_t)(g % p.a_mod) * p.a_group;
  const TW* w = (const TW*)p.W + (size_t)g * p.w_group + (size_t)n * p.ldw;
  float acc[GV_ROWS];
#pragma unroll
  for (int m = 0; m < GV_ROWS; ++m) acc[m] = 0.f;
  for (int k = lane; k < p.K; k += 64) {
    const float wv = to_float(w[k]);
#pragma unroll
    for (int m = 0; m < GV_ROWS; ++m)
      if (m < p.M) acc[m] = fmaf(to_float(A[(size_t)m * p.lda + k]), wv, acc[m]);
  }
  TC* C = (TC*)p.C + (size_t)g * p.c_group;
  const float bias = p.bias ? p.bias[(size_t)g * p.N + n] : 0.f;
#pragma unroll
  for (int m = 0; m < GV_ROWS; ++m) {
    if (m >= p.M) break;
    float v = wave_sum(acc[m]);
    if (lane == 0) {
      v = mie_act(v + bias, p.act);
      if (p.gate) v *= mie_sigmoid(p.gate[(size_t)m * p.ldg + (size_t)g * p.N + n]);
      C[(size_t)m * p.ldc + n] = from_float<TC>(v);
    }
  }
}

// The same product for bfloat16 operands on the matrix cores (v_mfma_f32_16x16x32_bf16).
typedef __bf16 gg_bf16x8 __attribute__((ext_vector_type(8)));
typedef float gg_f32x4 __attribute__((ext_vector_type(4)));
union GGFrag {
  gg_bf16x8 v;
  uint4 q;
};

// A workgroup of four waves (2 x 2) owns TM x 128 of C.  The k-steps of 32 come into a ring of LDS stages by loads that
// write the LDS directly (no registers in between; all stages but one are on their way while one is multiplied),
// 1 KB a fragment of 16 rows x 32 k: lane l brings k-block (l % 4) ^ (l / 16) % 4 of row l / 4, so that the piece of
// row r, k-block b sits at slot 4 r + (b ^ (r / 4) % 4) and the fragment reads spread over all banks.  A lane whose row
// or k-block does not exist reads from a block of zeros instead, so every wave issues the same loads a stage and one
// count tells when a stage has landed.  The fragments are read back in one piece of assembly with its own wait: the
// compiler does not know of the loads that write the LDS.  TM = 128 with three stages for steps of many rows (four were measured: no faster); TM = 64
// with five stages for few rows (decode steps: the weights stream, and what counts is the bytes on their way).
// Every output is the same chain of matrix instructions in increasing k wherever its tile lies, so a row's result
// does not depend on the rows beside it.  K, the row strides and the group offsets are multiples of 8 and the
// operands 16-byte aligned (checked by the caller).
#define GG_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))
typedef uint32_t gg_u32x4 __attribute__((ext_vector_type(4)));

template <int N> struct GGRead;
template <> struct GGRead<4> {
  static __device__ __forceinline__ void run(uint32_t base, gg_u32x4 (&f)[4]) {
    asm volatile(
      "ds_read_b128 %0, %4\n\t"
      "ds_read_b128 %1, %4 offset:1024\n\t"
      "ds_read_b128 %2, %4 offset:2048\n\t"
      "ds_read_b128 %3, %4 offset:3072\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(f[0]), "=&v"(f[1]), "=&v"(f[2]), "=&v"(f[3])
      : "v"(base)
      : "memory");
  }
};
template <> struct GGRead<2> {
  static __device__ __forceinline__ void run(uint32_t base, gg_u32x4 (&f)[2]) {
    asm volatile(
      "ds_read_b128 %0, %2\n\t"
      "ds_read_b128 %1, %2 offset:1024\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&v"(f[0]), "=&v"(f[1])
      : "v"(base)
      : "memory");
  }
};

template <int TM, int STAGES, typename TC>
__global__ void __launch_bounds__(256)
grouped_gemm_ring_kernel(GroupedArgs p) {
  constexpr int TN = 128, FA = TM / 16, FW = TN / 16, LPW = (FA + FW) / 4, MT = TM / 32, NT = 4;
  constexpr int STAGE_BYTES = (FA + FW) * 1024;
  static_assert((FA + FW) % 4 == 0, "the fragments of a stage must divide over the waves");
  static_assert(STAGES * STAGE_BYTES <= 65536, "LDS");
  static_assert(LPW * (STAGES - 2) <= 63, "more loads in flight than the counter holds");
  __shared__ __align__(16) char lds[STAGES * STAGE_BYTES];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * TN;
  int g, m0, m_end, c_row0;
  if (p.offs) {
    int tile = blockIdx.y, start = 0, cnt = 0;
    for (g = 0; g < p.G; ++g) {
      start = p.offs[g];
      cnt = p.offs[g + 1] - start;
      const int nt = (cnt + TM - 1) / TM;
      if (tile < nt) break;
      tile -= nt;
    }
    if (g == p.G) return;
    m0 = tile * TM;
    m_end = cnt;
    c_row0 = start;
  } else {
    g = blockIdx.z;
    m0 = blockIdx.y * TM;
    m_end = p.M;
    c_row0 = 0;
  }
  const bf16* A = (const bf16*)p.A + (size_t)(g % p.a_mod) * p.a_group;
  const bf16* W = (const bf16*)p.W + (size_t)g * p.w_group;
  // what this lane brings in: row lane / 4 of the fragments wave * LPW .. (A's fragments come first in a stage)
  const int lrow = lane >> 2, lkb = (lane & 3) ^ ((lane >> 4) & 3);
  const bf16* zero_lane = (const bf16*)p.zeros + lkb * 8;
  const bf16* src[LPW];
#pragma unroll
  for (int j = 0; j < LPW; ++j) {
    const int f = wave * LPW + j;
    if (f < FA) {
      const int r = m0 + f * 16 + lrow;          // the row of the tile this lane brings in, and the row of A behind it
      const int ar = r >= m_end ? -1 : (p.offs ? (p.gather ? p.gather[c_row0 + r] / p.gather_div : c_row0 + r) : r);
      src[j] = ar >= 0 ? A + (size_t)ar * p.lda + lkb * 8 : nullptr;
    } else {
      const int n = n0 + (f - FA) * 16 + lrow;
      src[j] = n < p.N ? W + (size_t)n * p.ldw + lkb * 8 : nullptr;
    }
  }
  auto issue = [&](int s) {
    char* base = lds + (s % STAGES) * STAGE_BYTES + wave * LPW * 1024;
    const int k0 = s * 32;
    const bool kok = k0 + lkb * 8 < p.K;
#pragma unroll
    for (int j = 0; j < LPW; ++j) {
      const bf16* from = src[j] && kok ? src[j] + k0 : zero_lane;
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)from,
                                       (__attribute__((address_space(3))) void*)(base + j * 1024), 16, 0, 0);
    }
  };
  const int col = lane & 15, kb = lane >> 4;
  const int rslot = col * 4 + (kb ^ ((col >> 2) & 3));
  const uint32_t lds0 = (uint32_t)(size_t)(__attribute__((address_space(3))) char*)lds;
  const uint32_t a_off = (wave >> 1) * MT * 1024 + rslot * 16, b_off = FA * 1024 + (wave & 1) * NT * 1024 + rslot * 16;
  gg_f32x4 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int j = 0; j < NT; ++j) acc[i][j] = gg_f32x4{0.f, 0.f, 0.f, 0.f};
  const int nk = (p.K + 31) / 32;
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) issue(s);
  for (int it = 0; it < nk; ++it) {
    GG_VMCNT(LPW * (STAGES - 2));      // this wave's loads of stage `it` have landed
    __builtin_amdgcn_s_barrier();      // and everybody else's; everybody is done reading stage it - 1
    issue(it + STAGES - 1);            // into the buffer stage it - 1 used (zeros beyond K)
    const uint32_t base = lds0 + (it % STAGES) * STAGE_BYTES;
    gg_u32x4 fa[MT], fb[NT];
    GGRead<MT>::run(base + a_off, fa);
    GGRead<NT>::run(base + b_off, fb);
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int j = 0; j < NT; ++j) {
        GGFrag a, b;
        a.q = *reinterpret_cast<uint4*>(&fa[i]);
        b.q = *reinterpret_cast<uint4*>(&fb[j]);
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[i][j], 0, 0, 0);
      }
  }
  GG_VMCNT(0);                         // nothing of this wave may still be writing the LDS when it ends
  const int wm = (wave >> 1) * (TM / 2), wn = (wave & 1) * (TN / 2);
  TC* C = (TC*)p.C + (size_t)g * p.c_group;
  if (p.glu) {
    // tiles 2 jj and 2 jj + 1 of a lane are the gate and the up sums of the same 16 inner channels
#pragma unroll
    for (int jj = 0; jj < NT / 2; ++jj) {
      if (n0 + wn + (2 * jj + 1) * 16 + col >= p.N) continue;
      const int n = (n0 + wn) / 2 + jj * 16 + col;
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int m = m0 + wm + i * 16 + kb * 4 + e;
          if (m >= m_end) continue;
          const float gt = fminf(acc[i][2 * jj][e], p.glu_limit);
          const float up = fminf(fmaxf(acc[i][2 * jj + 1][e], -p.glu_limit), p.glu_limit);
          C[(size_t)(c_row0 + m) * p.ldc + n] = from_float<TC>(gt * mie_sigmoid(p.glu_alpha * gt) * (up + p.glu_shift));
        }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int n = n0 + wn + j * 16 + col;
    if (n >= p.N) continue;
    const float bias = p.bias ? p.bias[(size_t)g * p.N + n] : 0.f;
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = m0 + wm + i * 16 + kb * 4 + e;
        if (m >= m_end) continue;
        const size_t crow = (size_t)(c_row0 + m);
        float v = mie_act(acc[i][j][e] + bias, p.act);
        if (p.gate) v *= mie_sigmoid(p.gate[crow * p.ldg + (size_t)g * p.N + n]);
        C[crow * p.ldc + n] = from_float<TC>(v);
      }
  }
}

MIE_EXPORT const char* grouped_gemm_last_error() { return g_mie_error; }

template <typename TA, typename TW>
static int launch_grouped(const GroupedArgs& p, int c_dtype, dim3 grid, hipStream_t s) {
  if (!p.offs && p.M <= GV_ROWS && (c_dtype == MIE_F32 || c_dtype == MIE_BF16)) {     // few rows: a wave a column
    dim3 vgrid((p.N + 3) / 4, 1, p.G);
    if (c_dtype == MIE_F32)
      hipLaunchKernelGGL((grouped_gemv_kernel<TA, TW, float>), vgrid, dim3(256), 0, s, p);
    else
      hipLaunchKernelGGL((grouped_gemv_kernel<TA, TW, bf16>), vgrid, dim3(256), 0, s, p);
    MIE_CHECK_LAUNCH("grouped_linear");
    return 0;
  }
  if (c_dtype == MIE_F32)
    hipLaunchKernelGGL((grouped_gemm_kernel<TA, TW, float>), grid, dim3(256), 0, s, p);
  else if (c_dtype == MIE_BF16)
    hipLaunchKernelGGL((grouped_gemm_kernel<TA, TW, bf16>), grid, dim3(256), 0, s, p);
  else
    MIE_FAIL("grouped_linear: output dtype code %d", c_dtype);
  MIE_CHECK_LAUNCH("grouped_linear");
  return 0;
}

// Strides and group offsets are in elements.  zeros: 64 bytes of zeros in device memory (or null: the kernels that
// need them are not used).  Rows shape: offs non-null, M = the length of the sorted list (an upper
// bound of any group's rows), a_group / c_group / a_mod unused.
static int grouped_linear_run(const void* A, int a_dtype, long lda, long a_group, int a_mod, const void* W, int w_dtype,
                              long ldw, long w_group, void* C, int c_dtype, long ldc, long c_group, const float* bias,
                              const float* gate, long ldg, const int* offs, const int* gather, int gather_div, int M,
                              int N, int K, int G, int act, const void* zeros, int glu, float glu_limit, float glu_alpha,
                              float glu_shift, hipStream_t s) {
  if (M <= 0 || N <= 0 || G <= 0) return 0;
  if (K <= 0 || !A || !W || !C) MIE_FAIL("grouped_linear: K %d or a null operand", K);
  if (lda < K && !offs && a_group == 0) MIE_FAIL("grouped_linear: A row stride %ld < K %d", lda, K);
  if (ldw < K || ldc < (glu ? N / 2 : N)) MIE_FAIL("grouped_linear: strides %ld, %ld for K %d, N %d", ldw, ldc, K, N);
  if (glu && (N % 32 || bias || gate || !(glu_limit > 0.f)))
    MIE_FAIL("grouped_linear: the gated epilogue takes N %d in blocks of 16 gate and 16 up rows, no bias, limit %g", N, (double)glu_limit);
  if (a_mod <= 0) a_mod = G;
  if (gather && gather_div <= 0) MIE_FAIL("grouped_linear: gather divisor %d", gather_div);
  if (act < MIE_ACT_NONE || act > MIE_ACT_RELU2) MIE_FAIL("grouped_linear: activation code %d", act);
  GroupedArgs p = {A, lda, offs ? 0 : a_group, offs ? 1 : a_mod, W, ldw, w_group, C, ldc, offs ? 0 : c_group, bias, gate, ldg,
                   offs, gather, gather_div, M, N, K, G, act, zeros, glu, glu_limit, glu_alpha, glu_shift};
  const long mt = (M + GG_T - 1) / GG_T + (offs ? G : 0);
  if (mt > 65535 || G > 65535) MIE_FAIL("grouped_linear: %ld row tiles, %d groups are beyond the grid", mt, G);
  dim3 grid((N + GG_T - 1) / GG_T, (unsigned)mt, offs ? 1 : G);
  // bfloat16 operands that the matrix-core kernel's 16-byte loads can take: row tiles of 128 where there are rows
  // enough to fill them (a function of the step's size, not of a row's place in it), of 64 otherwise
  if (zeros && a_dtype == MIE_BF16 && w_dtype == MIE_BF16 && (c_dtype == MIE_BF16 || c_dtype == MIE_F32) && K % 8 == 0 &&
      lda % 8 == 0 && ldw % 8 == 0 && p.a_group % 8 == 0 && w_group % 8 == 0 && (((uintptr_t)A | (uintptr_t)W) & 15) == 0) {
    const bool big = offs ? M >= 128L * G : M >= 256;
    const int T = big ? 128 : 64;
    const long mtiles = (M + T - 1) / T + (offs ? G : 0);
    if (mtiles > 65535) MIE_FAIL("grouped_linear: %ld row tiles are beyond the grid", mtiles);
    dim3 mgrid((N + 127) / 128, (unsigned)mtiles, offs ? 1 : G);
#define GG_RING(TM_, ST_, TC_) hipLaunchKernelGGL((grouped_gemm_ring_kernel<TM_, ST_, TC_>), mgrid, dim3(256), 0, s, p)
    if (big && c_dtype == MIE_BF16) GG_RING(128, 3, bf16);
    else if (big) GG_RING(128, 3, float);
    else if (c_dtype == MIE_BF16) GG_RING(64, 5, bf16);
    else GG_RING(64, 5, float);
#undef GG_RING
    MIE_CHECK_LAUNCH("grouped_linear");
    return 0;
  }
  if (glu) MIE_FAIL("grouped_linear: the gated epilogue needs bfloat16 operands with K %d, strides %ld, %ld multiples of 8", K, lda, ldw);
  if (a_dtype == MIE_F32 && w_dtype == MIE_F32) return launch_grouped<float, float>(p, c_dtype, grid, s);
  if (a_dtype == MIE_F32 && w_dtype == MIE_BF16) return launch_grouped<float, bf16>(p, c_dtype, grid, s);
  if (a_dtype == MIE_BF16 && w_dtype == MIE_F32) return launch_grouped<bf16, float>(p, c_dtype, grid, s);
  if (a_dtype == MIE_BF16 && w_dtype == MIE_BF16) return launch_grouped<bf16, bf16>(p, c_dtype, grid, s);
  MIE_FAIL("grouped_linear: dtype codes A %d, W %d", a_dtype, w_dtype);
}

MIE_EXPORT int mie_grouped_linear(const void* A, int a_dtype, long lda, long a_group, int a_mod, const void* W, int w_dtype,
                                  long ldw, long w_group, void* C, int c_dtype, long ldc, long c_group, const float* bias,
                                  const float* gate, long ldg, const int* offs, const int* gather, int gather_div, int M,
                                  int N, int K, int G, int act, const void* zeros, hipStream_t s) {
  return grouped_linear_run(A, a_dtype, lda, a_group, a_mod, W, w_dtype, ldw, w_group, C, c_dtype, ldc, c_group, bias, gate, ldg,
                            offs, gather, gather_div, M, N, K, G, act, zeros, 0, 0.f, 0.f, 0.f, s);
}

// The same in the rows shape for gated experts, on the matrix cores only (bfloat16 A and W, K and the strides multiples
// of 8): W's N rows alternate in blocks of 16 gate rows and 16 up rows, C [rows, N / 2] receives
// g * sigmoid(alpha g) * (u + shift) with g = min(gate sum, limit), u = clamp(up sum, -limit, limit) (an infinite limit
// clamps nothing).
MIE_EXPORT int mie_grouped_glu(const void* A, int a_dtype, long lda, const void* W, int w_dtype, long ldw, long w_group, void* C,
                               int c_dtype, long ldc, const int* offs, const int* gather, int gather_div, int M, int N, int K,
                               int G, float limit, float alpha, float shift, const void* zeros, hipStream_t s) {
  if (!offs || !zeros) MIE_FAIL("grouped_glu: group offsets and the block of zeros are needed");
  return grouped_linear_run(A, a_dtype, lda, 0, 1, W, w_dtype, ldw, w_group, C, c_dtype, ldc, 0, nullptr, nullptr, 0, offs, gather,
                            gather_div, M, N, K, G, MIE_ACT_NONE, zeros, 1, limit, alpha, shift, s);
}

// ---- router, one thread a token.  over_all == 0: the `top` largest of logits[t, :] + bias (lowest index first among
// equals), in falling order, and the softmax over those alone.  over_all != 0: scores = softmax of logits + bias over
// all E; chosen are the `top` largest of scores + choice_bias (same order rules); the shares are the chosen ones'
// scores as they are (over_all == 1) or divided by their sum + 1e-20 (over_all == 2).
#define ROUTE_MAX_TOP 16
__global__ void route_topk_kernel(const float* __restrict__ logits, long ld, const float* __restrict__ bias,
                                  const float* __restrict__ choice_bias, int over_all, int* __restrict__ experts,
                                  float* __restrict__ shares, int T, int E, int top) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= T) return;
  const float* z = logits + (size_t)t * ld;
  float largest = 0.f, total = 1.f;
  if (over_all) {
    largest = -INFINITY;
    for (int e = 0; e < E; ++e) largest = fmaxf(largest, z[e] + (bias ? bias[e] : 0.f));
    total = 0.f;
    for (int e = 0; e < E; ++e) total += expf(z[e] + (bias ? bias[e] : 0.f) - largest);
  }
  int chosen[ROUTE_MAX_TOP];
  float val[ROUTE_MAX_TOP];
  for (int j = 0; j < top; ++j) {
    int best = -1;
    float bv = 0.f, bs = 0.f;
    for (int e = 0; e < E; ++e) {
      bool taken = false;
      for (int i = 0; i < j; ++i) taken |= chosen[i] == e;
      if (taken) continue;
      float v = z[e] + (bias ? bias[e] : 0.f), sc = v;
      if (over_all) {
        sc = expf(v - largest) / total;
        v = sc + (choice_bias ? choice_bias[e] : 0.f);
      }
      if (best < 0 || v > bv) { best = e; bv = v; bs = sc; }
    }
    chosen[j] = best;
    val[j] = bs;
  }
  if (!over_all) {
    float sum = 0.f;
    const float first = val[0];
    for (int j = 0; j < top; ++j) { val[j] = expf(val[j] - first); sum += val[j]; }
    for (int j = 0; j < top; ++j) val[j] /= sum;
  } else if (over_all == 2) {
    float sum = 0.f;
    for (int j = 0; j < top; ++j) sum += val[j];
    for (int j = 0; j < top; ++j) val[j] /= sum + 1e-20f;
  }
  for (int j = 0; j < top; ++j) {
    experts[(size_t)t * top + j] = chosen[j];
    shares[(size_t)t * top + j] = val[j];
  }
}

// The same with a wave a token (up to ROUTE_WAVE_E router outputs, two a lane): maximum, sum and every choice are
// reductions over the wave instead of loops of one thread (which wait for each value in turn: 12 us at 18 outputs).
// A chosen output is struck out in its lane.  The order of a token's sums depends on E alone.
#define ROUTE_WAVE_E 128
__global__ void __launch_bounds__(256)
route_topk_wave_kernel(const float* __restrict__ logits, long ld, const float* __restrict__ bias,
                       const float* __restrict__ choice_bias, int over_all, int* __restrict__ experts,
                       float* __restrict__ shares, int T, int E, int top) {
  const int lane = threadIdx.x & 63, t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;                        // the whole wave
  const float* z = logits + (size_t)t * ld;
  float v[2], c[2];                          // values and choice biases of outputs lane and lane + 64
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int e = lane + 64 * i;
    v[i] = e < E ? z[e] + (bias ? bias[e] : 0.f) : -INFINITY;
    c[i] = e < E && over_all && choice_bias ? choice_bias[e] : 0.f;
  }
  if (over_all) {
    const float largest = wave_max(fmaxf(v[0], v[1]));
    const float x0 = lane < E ? expf(v[0] - largest) : 0.f, x1 = lane + 64 < E ? expf(v[1] - largest) : 0.f;
    const float total = wave_sum(x0 + x1);
    v[0] = lane < E ? x0 / total : -INFINITY;
    v[1] = lane + 64 < E ? x1 / total : -INFINITY;
  }
  float mine = 0.f;                          // lane j keeps the value of choice j
  for (int j = 0; j < top; ++j) {
    const float k0 = v[0] + c[0], k1 = v[1] + c[1];          // a struck or missing output stays -inf
    const float m = wave_max(fmaxf(k0, k1));
    int best = k0 == m ? lane : (k1 == m ? lane + 64 : 1 << 30);   // lowest index first among equals
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const int other = __shfl_xor(best, o, MIE_WAVE);
      best = other < best ? other : best;
    }
    if (best >= E) best = 0;                 // every value left is -inf or a NaN: cannot happen with finite logits
    const float s = __shfl(best < 64 ? v[0] : v[1], best & 63, MIE_WAVE);
    if (lane == (best & 63)) v[best >> 6] = -INFINITY;
    if (lane == j) mine = s;
    if (lane == 0) experts[(size_t)t * top + j] = best;
  }
  if (!over_all) {
    const float first = __shfl(mine, 0, MIE_WAVE);
    mine = lane < top ? expf(mine - first) : 0.f;
    mine /= wave_sum(mine);
  } else if (over_all == 2) {
    mine = lane < top ? mine : 0.f;
    mine /= wave_sum(mine) + 1e-20f;
  }
  if (lane < top) shares[(size_t)t * top + lane] = mine;
}

static int route_topk_launch(const float* logits, long ld, const float* bias, const float* choice_bias, int over_all,
                             int* experts, float* shares, int T, int E, int top, hipStream_t s) {
  if (T <= 0) return 0;
  if (E <= 0 || top <= 0 || top > E || top > ROUTE_MAX_TOP) MIE_FAIL("route_topk: top %d of %d experts (at most %d)", top, E, ROUTE_MAX_TOP);
  if (ld < E) MIE_FAIL("route_topk: row stride %ld < %d", ld, E);
  if (E <= ROUTE_WAVE_E)
    hipLaunchKernelGGL(route_topk_wave_kernel, dim3((T + 3) / 4), dim3(256), 0, s, logits, ld, bias, choice_bias, over_all,
                       experts, shares, T, E, top);
  else
    hipLaunchKernelGGL(route_topk_kernel, dim3((T + 63) / 64), dim3(64), 0, s, logits, ld, bias, choice_bias, over_all, experts,
                       shares, T, E, top);
  MIE_CHECK_LAUNCH("route_topk");
  return 0;
}

MIE_EXPORT int mie_route_topk(const float* logits, long ld, const float* bias, int* experts, float* shares, int T, int E,
                              int top, hipStream_t s) {
  return route_topk_launch(logits, ld, bias, nullptr, 0, experts, shares, T, E, top, s);
}

MIE_EXPORT int mie_route_topk_all(const float* logits, long ld, const float* bias, const float* choice_bias, int* experts,
                                  float* shares, int T, int E, int top, int renormalise, hipStream_t s) {
  return route_topk_launch(logits, ld, bias, choice_bias, renormalise ? 2 : 1, experts, shares, T, E, top, s);
}

// ---- sort the n = T * top (token, choice) pairs by expert: offs [E + 1] (where each expert's pairs start in the
// sorted list), sorted [n] (the pair at each place), place [n] (the place of each pair).  One workgroup; the order
// of pairs inside an expert is whatever the counters gave, which no result depends on.
#define ALIGN_THREADS 1024
#define ALIGN_MAX_EXPERTS 1024
__global__ void __launch_bounds__(ALIGN_THREADS)
moe_align_kernel(const int* __restrict__ experts, int n, int E, int* __restrict__ offs, int* __restrict__ sorted,
                 int* __restrict__ place) {
  __shared__ int count[ALIGN_MAX_EXPERTS];
  __shared__ int start[ALIGN_MAX_EXPERTS + 1];
  for (int e = threadIdx.x; e < E; e += ALIGN_THREADS) count[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += ALIGN_THREADS) {
    int e = experts[i];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    place[i] = atomicAdd(&count[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) { start[e] = run; run += count[e]; }
    start[E] = run;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += ALIGN_THREADS) offs[e] = start[e];
  for (int i = threadIdx.x; i < n; i += ALIGN_THREADS) {
    int e = experts[i];
    e = e < 0 ? 0 : (e >= E ? E - 1 : e);
    const int at = start[e] + place[i];
    place[i] = at;
    sorted[at] = i;
  }
}

MIE_EXPORT int mie_moe_align(const int* experts, int n, int E, int* offs, int* sorted, int* place, hipStream_t s) {
  if (n <= 0) return 0;
  if (E <= 0 || E > ALIGN_MAX_EXPERTS) MIE_FAIL("moe_align: %d experts (at most %d)", E, ALIGN_MAX_EXPERTS);
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(ALIGN_THREADS), 0, s, experts, n, E, offs, sorted, place);
  MIE_CHECK_LAUNCH("moe_align");
  return 0;
}

// ---- out[t, :] = sum over a token's choices j, in order, of shares[t, j] * y[place[t * top + j], :].  With x given,
// a choice of an expert >= identity_from stands for the token's own input: its term is shares[t, j] * x[t, :] and its
// row of y is not read.
template <typename TX>
__global__ void moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ place, const float* __restrict__ shares,
                                   float* __restrict__ out, int width, int top, const int* __restrict__ experts,
                                   int identity_from, const TX* __restrict__ x, long ldx) {
  const int t = blockIdx.x;
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < width; c += gridDim.y * blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < top; ++j) {
      const size_t at = (size_t)t * top + j;
      const bool same = x != nullptr && experts[at] >= identity_from;
      const float v = same ? to_float(x[(size_t)t * ldx + c]) : y[(size_t)place[at] * width + c];
      acc = fmaf(shares[at], v, acc);
    }
    out[(size_t)t * width + c] = acc;
  }
}

MIE_EXPORT int mie_moe_combine(const float* y, const int* place, const float* shares, float* out, int T, int width, int top,
                               hipStream_t s) {
  if (T <= 0 || width <= 0) return 0;
  if (top <= 0) MIE_FAIL("moe_combine: top %d", top);
  int by = (width + 255) / 256;
  hipLaunchKernelGGL(moe_combine_kernel<float>, dim3(T, by > 16 ? 16 : by), dim3(256), 0, s, y, place, shares, out, width, top,
                     (const int*)nullptr, 0, (const float*)nullptr, 0L);
  MIE_CHECK_LAUNCH("moe_combine");
  return 0;
}

MIE_EXPORT int mie_moe_combine_identity(const float* y, const int* place, const float* shares, float* out, int T, int width,
                                        int top, const int* experts, int identity_from, const void* x, int x_dtype, long ldx,
                                        hipStream_t s) {
  if (T <= 0 || width <= 0) return 0;
  if (top <= 0 || !experts || !x || ldx < width || identity_from < 0)
    MIE_FAIL("moe_combine: top %d, identity experts from %d, input rows %ld apart", top, identity_from, ldx);
  if (identity_from > 0 && !y) MIE_FAIL("moe_combine: experts without outputs");
  int by = (width + 255) / 256;
  dim3 grid(T, by > 16 ? 16 : by);
  if (x_dtype == MIE_F32)
    hipLaunchKernelGGL(moe_combine_kernel<float>, grid, dim3(256), 0, s, y, place, shares, out, width, top, experts,
                       identity_from, (const float*)x, ldx);
  else if (x_dtype == MIE_BF16)
    hipLaunchKernelGGL(moe_combine_kernel<bf16>, grid, dim3(256), 0, s, y, place, shares, out, width, top, experts,
                       identity_from, (const bf16*)x, ldx);
  else
    MIE_FAIL("moe_combine: dtype code %d", x_dtype);
  MIE_CHECK_LAUNCH("moe_combine");
  return 0;
}
