// Weight-streaming matrix product for up to 128 rows, left as float32 sums over ranges of K:
// part[s][M][N] = sum over the s-th range of K of A[M, k] * W[N, k], bfloat16 in.
//
// The product is bound by reading W once, but the activations do not come for free: a
// block that owns few features and all of K (the shape of gemm_skinny_bf16) reads all rows
// of them, and with one block per 16 features and a long K, or many rows, that costs as
// much as the weights.  Here a block owns 128 features (8 waves x 16) and ONE range of K;
// its waves share the activations of that range through LDS (loaded once per block, 256
// columns at a time, the next piece in flight in registers while this one is used), and
// every wave streams its own 16 weight rows straight from memory into registers, one piece
// ahead.  Cutting K across blocks is what fills the GPU when N is small; the pieces are
// added up, in order, by the kernel that consumes the product (add_rmsnorm).  Measured on
// MI355X: 4096 x 14336 in 24.5 us at 1 to 16 rows (gemm_skinny_bf16: 27 / 31 / 37 us at
// 1 / 8 / 16 rows), 25 / 29 / 39 us at 32 / 64 / 128 rows (vendor library: 34 / 41 / 75 us).
//
// This stands where the reference's engine calls the vendor BLAS (distributed/linear.py:167).
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define MID_WAVES 8
#define MID_KC 8  // k-steps of 32 per piece
#define MID_AROW (MID_KC * 32 + 8)  // elements: rows 16 bytes apart in the banks, so 16 rows read side by side

// LINES: the weights are read in whole cache lines (lines_to_operands in common.h), where the
// matrix lies so that they can be.  Measured against half lines, microseconds at 16 / 64 / 128
// rows: 4096 x 14336 23.4 / 28.0 / 41.5 against 23.7 / 28.3 / 39.6, 3072 x 8192 16.2 / 20.6 /
// 31.6 against 18.5 / 22.3 / 30.7, 8192 x 28672 78 / 91 / 133 against 86 / 101 / 132: so up to
// 64 rows.
template <int MT, bool LINES>
__global__ __launch_bounds__(64 * MID_WAVES) void gemm_mid_partial_kernel(
    const bf16_t* __restrict__ a, int64_t lda, const bf16_t* __restrict__ w, int64_t ldw,
    float* __restrict__ part, int m, int n, int k, int pieces_per_range) {
  constexpr int THREADS = 64 * MID_WAVES;
  constexpr int ROWS = 16 * MT;
  constexpr int A_IDS = ROWS * MID_KC * 4;  // 16-byte chunks of one piece of the activations
  constexpr int A_PER = A_IDS / THREADS;
  static_assert(A_IDS % THREADS == 0, "the activations' piece is shared out evenly");
  __shared__ __attribute__((aligned(16))) bf16_t a_lds[2][ROWS * MID_AROW];

  // (with LINES made uniform for the compiler, so that the base address of the weight loads is scalar)
  const int wave = LINES ? __builtin_amdgcn_readfirstlane(threadIdx.x / MI_WAVE) : threadIdx.x / MI_WAVE;
  const int lane = threadIdx.x % MI_WAVE;
  const int col = lane % 16, quad = lane / 16;
  const int n0 = blockIdx.x * (16 * MID_WAVES) + wave * 16;
  const int ksteps = k / 32;
  const int s_begin = min((int)blockIdx.y * pieces_per_range * MID_KC, ksteps);
  const int s_end = min(s_begin + pieces_per_range * MID_KC, ksteps);
  const int pieces = (s_end - s_begin + MID_KC - 1) / MID_KC;

  // weights: this lane reads feature n0 + col (past N: the last one, never stored), 8 consecutive k
  const bf16_t* wp = w + (int64_t)min(n0 + col, n - 1) * ldw + quad * 8;
  // LINES: byte offsets of this lane's 16 bytes in the lower and upper 8 of the wave's rows
  const uint32_t line_lo = (uint32_t)min(n0 + line_row_of_lane(lane), n - 1) * (uint32_t)(ldw * 2) + line_chunk_of_lane(lane);
  const uint32_t line_hi = (uint32_t)min(n0 + 8 + line_row_of_lane(lane), n - 1) * (uint32_t)(ldw * 2) + line_chunk_of_lane(lane);
  // activations: chunk id -> (row, 16-byte part of the piece); rows past M repeat the last one
  const bf16_t* a_src[A_PER];
  int a_dst[A_PER];
#pragma unroll
  for (int j = 0; j < A_PER; ++j) {
    const int id = threadIdx.x + j * THREADS;
    const int row = id / (MID_KC * 4), chunk = id % (MID_KC * 4);
    a_src[j] = a + (int64_t)min(row, m - 1) * lda + chunk * 8;
    a_dst[j] = row * MID_AROW + chunk * 8;
  }
  auto request_a = [&](int s0, bf16x8_t* stage) {
    // (k-steps past the end of K re-read the last one; their products are not made)
#pragma unroll
    for (int j = 0; j < A_PER; ++j) {
      const int id = threadIdx.x + j * THREADS;
      const int in_piece = (id % (MID_KC * 4)) / 4;
      const int kstep = min(s0 + in_piece, ksteps - 1);
      stage[j] = *reinterpret_cast<const bf16x8_t*>(a_src[j] + (int64_t)(kstep - in_piece) * 32);
    }
  };
  auto store_a = [&](int buf, const bf16x8_t* stage) {
#pragma unroll
    for (int j = 0; j < A_PER; ++j) *reinterpret_cast<bf16x8_t*>(&a_lds[buf][a_dst[j]]) = stage[j];
  };
  auto request_w = [&](int s0, bf16x8_t* regs) {
    if constexpr (LINES) {  // (K holds an even number of k-steps and s0 is even)
#pragma unroll
      for (int u = 0; u < MID_KC; u += 2) load_line_pair(w, min(s0 + u, ksteps - 2), line_lo, line_hi, regs[u], regs[u + 1]);
    } else {
#pragma unroll
      for (int u = 0; u < MID_KC; ++u) regs[u] = *reinterpret_cast<const bf16x8_t*>(wp + (int64_t)min(s0 + u, ksteps - 1) * 32);
    }
  };

  f32x4_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  if (pieces > 0) {
    bf16x8_t a_stage[A_PER];
    bf16x8_t w_now[MID_KC], w_next[MID_KC];
    request_a(s_begin, a_stage);
    request_w(s_begin, w_now);
    store_a(0, a_stage);
    __syncthreads();
    for (int p = 0; p < pieces; ++p) {
      const int s0 = s_begin + p * MID_KC;
      const int buf = p & 1;
      // the next piece is requested before this one is used (past the end: the last one again)
      request_a(min(s0 + MID_KC, s_end - 1), a_stage);
      request_w(min(s0 + MID_KC, s_end - 1), w_next);
      const int steps = min(MID_KC, s_end - s0);
      if constexpr (LINES) {  // what was requested a turn ago, as the operands of its k-steps
#pragma unroll
        for (int u = 0; u < MID_KC; u += 2) lines_to_operands(w_now[u], w_now[u + 1]);
      }
#pragma unroll
      for (int u = 0; u < MID_KC; ++u) {
        if (u < steps) {
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            const bf16x8_t act = *reinterpret_cast<const bf16x8_t*>(&a_lds[buf][(mt * 16 + col) * MID_AROW + u * 32 + quad * 8]);
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_now[u], act, acc[mt], 0, 0, 0);
          }
        }
      }
      store_a(buf ^ 1, a_stage);
#pragma unroll
      for (int u = 0; u < MID_KC; ++u) w_now[u] = w_next[u];
      __syncthreads();
    }
  }

  // acc[mt][r] = C^T[feature n0 + 4*quad + r][row 16*mt + col] over this block's range of K
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int row = mt * 16 + col;
    const int feature = n0 + quad * 4;
    if (row >= m || feature >= n) continue;
    float* dst = part + ((int64_t)blockIdx.y * m + row) * n + feature;
    if (feature + 3 < n && n % 4 == 0) {
      *reinterpret_cast<f32x4_t*>(dst) = acc[mt];
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (feature + r < n) dst[r] = acc[mt][r];
    }
  }
}

extern "C" int mi_gemm_mid_bf16_supported(int m, int n, int k, int64_t lda, int64_t ldw) {
  return (m >= 1 && m <= 128 && n >= 1 && k >= 32 && k % 32 == 0 && lda % 8 == 0 && ldw % 8 == 0) ? 1 : 0;
}

// How many ranges K is cut into for these sizes on the current device (the caller sizes
// `part` with it): enough blocks for one per compute unit (measured best: 8 ranges for 4096
// features, against 4 and 16), whole pieces of 256 columns each.
extern "C" int mi_gemm_mid_bf16_ranges(int n, int k) {
  int device = 0, cus = 0;
  if (hipGetDevice(&device) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || cus <= 0)
    return 0;
  const int feature_blocks = ceil_div(n, 16 * MID_WAVES);
  const int pieces = ceil_div(k / 32, MID_KC);
  int ranges = (cus + feature_blocks - 1) / feature_blocks;
  if (ranges > 16) ranges = 16;
  if (ranges > pieces) ranges = pieces;
  if (ranges < 1) ranges = 1;
  const int per_range = ceil_div(pieces, ranges);
  return ceil_div(pieces, per_range);
}

// part[s][m][n] (float32, contiguous), s < mi_gemm_mid_bf16_ranges(n, k).
extern "C" int mi_gemm_mid_partial_bf16(const void* a, int64_t lda, const void* w, int64_t ldw, float* part,
                                        int m, int n, int k, hipStream_t stream) {
  MI_REQUIRE(mi_gemm_mid_bf16_supported(m, n, k, lda, ldw),
             "gemm_mid_partial_bf16: takes 1 <= m <= 128, k a multiple of 32, rows aligned to 16 bytes; "
             "got m=%d n=%d k=%d lda=%lld ldw=%lld", m, n, k, (long long)lda, (long long)ldw);
  MI_REQUIRE(lda >= k && ldw >= k, "gemm_mid_partial_bf16: a row stride is shorter than its row");
  const int ranges = mi_gemm_mid_bf16_ranges(n, k);
  MI_REQUIRE(ranges >= 1, "gemm_mid_partial_bf16: cannot read the device's compute unit count");
  const int pieces = ceil_div(k / 32, MID_KC);
  const int per_range = ceil_div(pieces, ranges);
  const dim3 grid(ceil_div(n, 16 * MID_WAVES), ranges);
  // whole cache lines: rows of the matrix on 128-byte boundaries, an even number of k-steps,
  // byte offsets into it that fit 32 bits
  const bool lines = (uintptr_t)w % 128 == 0 && ldw % 64 == 0 && k % 64 == 0 && (int64_t)n * ldw * 2 < ((int64_t)1 << 32);
#define MID_GO(MT_)                                                                                          \
  if (lines)                                                                                                 \
    gemm_mid_partial_kernel<MT_, true><<<grid, 64 * MID_WAVES, 0, stream>>>((const bf16_t*)a, lda, (const bf16_t*)w, ldw, \
                                                                           part, m, n, k, per_range);         \
  else                                                                                                       \
    gemm_mid_partial_kernel<MT_, false><<<grid, 64 * MID_WAVES, 0, stream>>>((const bf16_t*)a, lda, (const bf16_t*)w, ldw, \
                                                                            part, m, n, k, per_range)
  if (m <= 16) { MID_GO(1); }
  else if (m <= 32) { MID_GO(2); }
  else if (m <= 64) { MID_GO(4); }
  else gemm_mid_partial_kernel<8, false><<<grid, 64 * MID_WAVES, 0, stream>>>((const bf16_t*)a, lda, (const bf16_t*)w, ldw, part, m, n, k, per_range);
#undef MID_GO
  MI_CHECK_LAUNCH("gemm_mid_partial_bf16");
  return MI_OK;
}
