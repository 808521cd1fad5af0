// True float32 matrix product for the 32-bit path: C[M,N] = A[M,K] * W[N,K]^T.
// Plain FMA, no reduced-precision matrix mode.  Each output element is summed by
// one thread in the order of k, so a row's result does not depend on how many other
// rows are in the batch or on where its tile lies.  The sum is carried in 64-bit and
// rounded to float32 once, when it is written: an output differs from the exact product
// of its float32 operands by that one rounding (relative 2.5e-8 on average), whatever K
// is.  (Float32 sums in 16-deep slices added up with compensation measured 8e-8 at K =
// 4,096, a plain float32 sum 2.7e-6; over 32 layers such errors are what the logits show.)
//
// 64x64 output tile per 256-thread block, 16-deep K slices staged in LDS, 4x4
// outputs per thread.  Any M, N, K; rows of A and W may have strides.
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ a, int64_t lda,
                                                       const float* __restrict__ w, int64_t ldw,
                                                       float* __restrict__ c, int64_t ldc, int m,
                                                       int n, int k) {
  __shared__ float a_s[BK][BM + 4];
  __shared__ float w_s[BK][BN + 4];

  const int tid = threadIdx.x;
  const int row0 = blockIdx.y * BM;
  const int col0 = blockIdx.x * BN;
  const int ty = tid / 16, tx = tid % 16;

  // loader mapping: thread loads 4 consecutive k of one row
  const int l_row = tid / 4;
  const int l_k = (tid % 4) * 4;

  double acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0;

  for (int k0 = 0; k0 < k; k0 += BK) {
    {
      const int r = row0 + l_row;
      const float* src = a + (int64_t)r * lda + k0 + l_k;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        a_s[l_k + i][l_row] = (r < m && k0 + l_k + i < k) ? src[i] : 0.f;
    }
    {
      const int r = col0 + l_row;
      const float* src = w + (int64_t)r * ldw + k0 + l_k;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        w_s[l_k + i][l_row] = (r < n && k0 + l_k + i < k) ? src[i] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      double av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = (double)a_s[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = (double)w_s[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fma(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + ty * 4 + i;
    if (r >= m) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = col0 + tx * 4 + j;
      if (col < n) c[(int64_t)r * ldc + col] = (float)acc[i][j];
    }
  }
}

// The same product for at most 16 rows (decode): a 64x64 tile would be three quarters empty and
// its 16-byte loads per thread leave most of the memory system idle.  A block owns all rows
// and 32 or 64 features; W is staged 64 deep (256 contiguous bytes of a row by a few threads),
// and a thread sums one row x two or four features.  Every output is summed EXACTLY as above (in
// the order of k, in 64-bit, rounded once); so a row gives the same bits whichever of the two
// kernels its step takes.
#define RM 16
#define RK 64

// TN = features per thread (the block owns 16 * TN): the more, the less is read from LDS per
// product, the fewer blocks.
template <int TN>
__global__ __launch_bounds__(256) void gemm_f32_rows_kernel(const float* __restrict__ a, int64_t lda,
                                                            const float* __restrict__ w, int64_t ldw,
                                                            float* __restrict__ c, int64_t ldc, int m,
                                                            int n, int k, int aligned) {
  constexpr int RN = 16 * TN;
  constexpr int W_PER = RN * RK / 256;  // consecutive k of one feature a thread stages: 8 or 16
  __shared__ float a_s[RK][RM + 1];
  __shared__ __attribute__((aligned(16))) float w_s[RK][RN + 4];
  const int tid = threadIdx.x;
  const int col0 = blockIdx.x * RN;
  const int row = tid / 16, tx = tid % 16;  // this thread's outputs: row, features col0 + TN*tx ..
  // loaders: W: W_PER consecutive k of one feature; A: 4 consecutive k of row tid / 16
  const int w_feature = tid / (RK / W_PER), w_k = (tid % (RK / W_PER)) * W_PER;
  const int w_row = col0 + w_feature;
  const int a_row = tid / 16, a_k = (tid % 16) * 4;
  double acc[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) acc[j] = 0.0;
  for (int k0 = 0; k0 < k; k0 += RK) {
    {
      const float* src = w + (int64_t)w_row * ldw + k0 + w_k;
      float v[W_PER];
      if (aligned && w_row < n && k0 + w_k + W_PER <= k) {
#pragma unroll
        for (int i = 0; i < W_PER; i += 4) {
          const float4 q = *reinterpret_cast<const float4*>(src + i);
          v[i] = q.x; v[i + 1] = q.y; v[i + 2] = q.z; v[i + 3] = q.w;
        }
      } else {
#pragma unroll
        for (int i = 0; i < W_PER; ++i) v[i] = (w_row < n && k0 + w_k + i < k) ? src[i] : 0.f;
      }
#pragma unroll
      for (int i = 0; i < W_PER; ++i) w_s[w_k + i][w_feature] = v[i];
    }
    {
      const float* src = a + (int64_t)a_row * lda + k0 + a_k;
#pragma unroll
      for (int i = 0; i < 4; ++i) a_s[a_k + i][a_row] = (a_row < m && k0 + a_k + i < k) ? src[i] : 0.f;
    }
    __syncthreads();
    // (staged values past K are zeros: they add nothing, exactly)
#pragma unroll
    for (int kk = 0; kk < RK; ++kk) {
      const double av = (double)a_s[kk][row];
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[j] = fma(av, (double)w_s[kk][TN * tx + j], acc[j]);
    }
    __syncthreads();
  }
  if (row < m) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = col0 + TN * tx + j;
      if (col < n) c[(int64_t)row * ldc + col] = (float)acc[j];
    }
  }
}

extern "C" int mi_gemm_f32(const float* a, int64_t lda, const float* w, int64_t ldw, float* c,
                           int64_t ldc, int m, int n, int k, hipStream_t stream) {
  MI_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm_f32: bad sizes m=%d n=%d k=%d", m, n, k);
  MI_REQUIRE(lda >= k && ldw >= k && ldc >= n, "gemm_f32: a row stride is shorter than its row");
  MI_REQUIRE(ceil_div(m, BM) <= 65535, "gemm_f32: m=%d is too large for one call", m);
  if (m == 0) return MI_OK;
  if (m <= RM) {
    const int aligned = ldw % 4 == 0 && ((uintptr_t)w % 16 == 0) ? 1 : 0;
    // (four features a thread where that still leaves a block for every CU; measured at 8B sizes,
    // 8 rows: 34.7 ms a step this way, 45.5 with four or eight everywhere, 36.5 with two everywhere)
    if (n >= 8192) gemm_f32_rows_kernel<4><<<ceil_div(n, 64), 256, 0, stream>>>(a, lda, w, ldw, c, ldc, m, n, k, aligned);
    else gemm_f32_rows_kernel<2><<<ceil_div(n, 32), 256, 0, stream>>>(a, lda, w, ldw, c, ldc, m, n, k, aligned);
    MI_CHECK_LAUNCH("gemm_f32 (few rows)");
    return MI_OK;
  }
  dim3 grid(ceil_div(n, BN), ceil_div(m, BM));
  gemm_f32_kernel<<<grid, 256, 0, stream>>>(a, lda, w, ldw, c, ldc, m, n, k);
  MI_CHECK_LAUNCH("gemm_f32");
  return MI_OK;
}
