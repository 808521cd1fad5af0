// Weight-streaming matrix product for few rows (decode): C[M,N] = A[M,K] * W[N,K]^T,
// bfloat16 in and out, float32 accumulate on the matrix cores, M <= 16.
//
// At these sizes the product is bound by reading W once from HBM.  A block owns 16
// output features and all of K: its 8 waves each stream one eighth of every one of
// the 16 weight rows (16 contiguous bytes per lane and k-step, MFMA 16x16x32 with
// the weights as the A operand and the activations, transposed, as the B operand),
// then add their partial tiles through LDS in a fixed order, so the result does not
// depend on timing.  Activations are small and come from the cache hierarchy.
//
// This stands where the reference's engine calls the vendor BLAS
// (distributed/linear.py:167); that library's kernels reach about half of the HBM
// rate at these shapes.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define SK_WAVES 8

// NT = 16-feature tiles per block (the activations a wave loads are used NT times),
// U = k-steps whose loads are issued together before their products run.  Register
// use is kept low on purpose: many resident waves, each with U*(NT+1) loads in
// flight, hide the memory latency better than a deeper pipeline in fewer waves.
template <int NT, int U>
__global__ __launch_bounds__(64 * SK_WAVES) void gemm_skinny_bf16_kernel(
    const bf16_t* __restrict__ a, int64_t lda, const bf16_t* __restrict__ w, int64_t ldw,
    bf16_t* __restrict__ c, int64_t ldc, int m, int n, int k) {
  __shared__ float red[SK_WAVES][NT][256];

  const int wave = threadIdx.x / MI_WAVE;
  const int lane = threadIdx.x % MI_WAVE;
  const int col = lane % 16;
  const int quad = lane / 16;
  const int n0 = blockIdx.x * 16 * NT;

  const int ksteps = k / 32;
  const int per_wave = (ksteps + SK_WAVES - 1) / SK_WAVES;
  const int s_begin = min(wave * per_wave, ksteps);
  const int s_end = min(s_begin + per_wave, ksteps);

  // weights: lane reads feature n0 + 16*nt + col, 8 consecutive k; rows past N repeat the last one
  const bf16_t* wp[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) wp[nt] = w + (int64_t)min(n0 + nt * 16 + col, n - 1) * ldw + quad * 8;
  // activations: lane reads token `col`; lanes past M re-read the last token (the same
  // cache lines as its own lane, so no extra traffic) and their columns are never stored
  const bf16_t* ap = a + (int64_t)min(col, m - 1) * lda + quad * 8;

  f32x4_t acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  int s = s_begin;
  for (; s + U <= s_end; s += U) {
    bf16x8_t w_reg[U][NT];
    bf16x8_t a_reg[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        w_reg[u][nt] = *reinterpret_cast<const bf16x8_t*>(wp[nt] + (int64_t)(s + u) * 32);
      a_reg[u] = *reinterpret_cast<const bf16x8_t*>(ap + (int64_t)(s + u) * 32);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_reg[u][nt], a_reg[u], acc[nt], 0, 0, 0);
  }
  for (; s < s_end; ++s) {  // fewer than U k-steps left
    const bf16x8_t a_tail = *reinterpret_cast<const bf16x8_t*>(ap + (int64_t)s * 32);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const bf16x8_t w_tail = *reinterpret_cast<const bf16x8_t*>(wp[nt] + (int64_t)s * 32);
      acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_tail, a_tail, acc[nt], 0, 0, 0);
    }
  }

  // acc[nt][r] = C^T[feature n0 + 16*nt + 4*quad + r][token col]; add the 8 waves in order
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][nt][(quad * 4 + r) * 16 + col] = acc[nt][r];
  }
  __syncthreads();
  // 256*NT sums of 8: a thread takes 4 consecutive features of one token
  for (int item = threadIdx.x; item < NT * 64; item += 64 * SK_WAVES) {
    const int nt = item / 64;
    const int token = (item % 64) % 16;
    const int fq = (item % 64) / 16;
    if (token >= m) continue;
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int wv = 0; wv < SK_WAVES; ++wv)
#pragma unroll
      for (int r = 0; r < 4; ++r) sum[r] += red[wv][nt][(fq * 4 + r) * 16 + token];
    const int feature = n0 + nt * 16 + fq * 4;
    bf16_t* dst = c + (int64_t)token * ldc + feature;
    if (feature + 3 < n && (ldc % 4 == 0)) {
      bf16x4_t packed;
#pragma unroll
      for (int r = 0; r < 4; ++r) packed[r] = (bf16_t)sum[r];
      *reinterpret_cast<bf16x4_t*>(dst) = packed;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (feature + r < n) dst[r] = (bf16_t)sum[r];
    }
  }
}

#define SK_MAX_ROWS 16

extern "C" int mi_gemm_skinny_bf16_supported(int m, int n, int k, int64_t lda, int64_t ldw) {
  return (m >= 1 && m <= SK_MAX_ROWS && n >= 1 && k >= 32 && k % 32 == 0 && lda % 8 == 0 && ldw % 8 == 0) ? 1 : 0;
}

extern "C" int mi_gemm_skinny_bf16(const void* a, int64_t lda, const void* w, int64_t ldw, void* c,
                                   int64_t ldc, int m, int n, int k, hipStream_t stream) {
  MI_REQUIRE(mi_gemm_skinny_bf16_supported(m, n, k, lda, ldw),
             "gemm_skinny_bf16: takes 1 <= m <= 16, k a multiple of 32, rows aligned to 16 bytes; "
             "got m=%d n=%d k=%d lda=%lld ldw=%lld", m, n, k, (long long)lda, (long long)ldw);
  MI_REQUIRE(lda >= k && ldw >= k && ldc >= n, "gemm_skinny_bf16: a row stride is shorter than its row");
  const bf16_t* ap = (const bf16_t*)a;
  const bf16_t* wp = (const bf16_t*)w;
  bf16_t* cp = (bf16_t*)c;
  // Block shapes measured on MI355X at Llama-8B sizes: wide blocks (each activation
  // load used for 4 weight tiles) once there are blocks to spare, narrow ones when
  // the output is so small that every block is needed to fill the 256 CUs.
  const int tiles = ceil_div(n, 16);
  if (tiles >= 1024) {
    gemm_skinny_bf16_kernel<4, 2><<<ceil_div(tiles, 4), 64 * SK_WAVES, 0, stream>>>(ap, lda, wp, ldw, cp, ldc, m, n, k);
  } else if (tiles >= 320) {
    gemm_skinny_bf16_kernel<2, 8><<<ceil_div(tiles, 2), 64 * SK_WAVES, 0, stream>>>(ap, lda, wp, ldw, cp, ldc, m, n, k);
  } else {
    gemm_skinny_bf16_kernel<1, 8><<<tiles, 64 * SK_WAVES, 0, stream>>>(ap, lda, wp, ldw, cp, ldc, m, n, k);
  }
  MI_CHECK_LAUNCH("gemm_skinny_bf16");
  return MI_OK;
}

// Tuning hook: the same product with the block shape chosen by the caller.
extern "C" int mi_gemm_skinny_bf16_variant(const void* a, int64_t lda, const void* w, int64_t ldw, void* c,
                                           int64_t ldc, int m, int n, int k, int nt, int u, hipStream_t stream) {
  const bf16_t* ap = (const bf16_t*)a;
  const bf16_t* wp = (const bf16_t*)w;
  bf16_t* cp = (bf16_t*)c;
  const int tiles = ceil_div(n, 16);
#define V(NT_, U_) if (nt == NT_ && u == U_) { gemm_skinny_bf16_kernel<NT_, U_><<<ceil_div(tiles, NT_), 64 * SK_WAVES, 0, stream>>>(ap, lda, wp, ldw, cp, ldc, m, n, k); return 0; }
  V(1, 16) V(1, 8) V(2, 8) V(2, 4) V(4, 2)
#undef V
  return -1;
}
