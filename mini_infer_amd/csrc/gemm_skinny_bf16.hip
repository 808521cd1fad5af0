// Weight-streaming matrix product for few rows (decode): C[M,N] = A[M,K] * W[N,K]^T,
// bfloat16 in and out, float32 accumulate on the matrix cores, M <= 16 (<= 32 for the
// gated and the rotary product).
//
// At these sizes the product is bound by reading W once from HBM.  A block owns 8 to 64
// output features and all of K: its 8 waves each stream one eighth of every one of its
// weight rows (MFMA 16x16x32 with the weights as the A operand and the activations,
// transposed, as the B operand), then add their partial tiles through LDS in a fixed order,
// so the result does not depend on timing.  Activations are small and come from the cache
// hierarchy.  How the weight rows are read decides the kernel's speed: in whole cache lines
// with non-temporal loads where the matrix lies so that they can be (LINES; common.h says
// how and what was measured), else 16 contiguous bytes per lane and k-step.
//
// What follows a product in a decoder layer is folded into its last step where that saves a
// launch: the SiLU-gated product, the rotary encoding with the cache write, the residual
// add with the beginning of the norm (EPI_*).
//
// This stands where the reference's engine calls the vendor BLAS
// (distributed/linear.py:167); that library's kernels reach about half of the HBM
// rate at these shapes.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define SK_WAVES 8

// LINES: the weights are read in whole cache lines (lines_to_operands in common.h), where
// the matrix lies so that they can be.  RT = tiles of 16 rows (tokens) a wave keeps sums for.
// NT = 16-feature tiles of the OUTPUT per block (the activations a wave loads are used
// for every weight tile of the block), U = k-steps whose loads are issued together
// before their products run.  Register use is kept low on purpose: many resident waves,
// each with U*(tiles+1) loads in flight, hide the memory latency better than a deeper
// pipeline in fewer waves.
//
// What the last step does with the products (each folds a neighbouring launch of a
// decoder layer into this one):
//   EPI_STORE  c = bf16(product).
//   EPI_STORE_F32  c (float32) = float(bf16(product)): the output head's logits, which are
//              wanted in float32 (no cast launch after the product).  Rounded to bfloat16 on the
//              way like every product of this path, so that a position's logits are the same
//              numbers whether its step had few rows (this kernel) or many (the vendor
//              library's bfloat16 product, widened afterwards).
//   EPI_GATED  W holds two stacked matrices [gate; up] of n rows each and the output is
//              silu(gate . a) * (up . a): a block computes both halves of its features,
//              so the [m, 2n] intermediate is never written.
//   EPI_ROPE   W is the stacked q|k|v projection of an attention layer with half-paired
//              rotary encoding over the whole head: a block computes some dims of a
//              head's first half and their partners, rotates them, and writes queries
//              to c[m, q_heads*head_dim] and keys and values straight into their cache
//              slots.
//   EPI_ADDNORM  the product is a layer's contribution to the residual stream and the next
//              thing to happen is an RMS norm: residual += bf16(product) (float32, stored), and
//              c = bf16(residual * norm_weight), the norm's output but for the row's factor
//              rsqrt(mean(residual^2) + eps).  That factor needs the whole row, which no block
//              has: every block leaves the sum of squares of its features per row in
//              sumsq[block][row], and the product that consumes c (PRO_SCALED) adds them up
//              and multiplies its own sums with the factor, which commutes with the product.
//              The norm's launch between two products is saved.
// In every case the sums are rounded to bfloat16 before the activation or rotation,
// exactly as when the product and the second step run as two kernels.
enum { EPI_STORE = 0, EPI_GATED = 1, EPI_ROPE = 2, EPI_ADDNORM = 3, EPI_STORE_F32 = 4 };
// Where the activations come from: a matrix in memory, or (PRO_ATTN, few rows) the
// uncombined key ranges of attn_mfma: each wave first combines its own columns of the
// attention output (what attn_reduce would have written) into LDS, so the combining launch
// between the attention and its output projection is saved at the smallest batches.
// PRO_SCALED: rows whose norm factor is still apart (what EPI_ADDNORM leaves): the sums are
// multiplied with rsqrt(sum of the pieces' squares / width + eps) of their row before rounding.
enum { PRO_NONE = 0, PRO_ATTN = 1, PRO_SCALED = 2 };
#define SK_SCALE_PARTS 32  // threads per row that add up the pieces of a row's sum of squares
#define SK_SCALE_PIECES 8  // pieces per such thread: 256 pieces at most
#define SK_PRO_VALUES 4096  // activations a wave makes and holds: rows * (K / 8 waves) at most

struct FoldArgs {  // what the folded neighbours of a product need
  // EPI_ROPE:
  const float* cos_t;  // [m, head_dim/2]
  const float* sin_t;
  const int* slot_mapping;  // [m]: page * page_size + offset, negative: write nothing
  bf16_t* k_pages;  // [pages][kv_heads][page_size][head_dim]
  bf16_t* v_pages;  // the same, or [pages][kv_heads][head_dim][page_size] if v_transposed
  int q_heads, kv_heads, head_dim, page_size, v_transposed;
  // PRO_ATTN: partial accumulators [row][head][split][head_dim], (max in natural-log units,
  // sum) pairs [row][head][split][2], as attn_mfma leaves them; K = attn_heads * attn_head_dim
  const float* part_acc;
  const float* part_ml;
  int num_splits, attn_heads, attn_head_dim;
  // EPI_ADDNORM: the float32 residual rows [m, n] the product is added to, the norm's weight [n],
  // where the block's sums of squares go ([blocks][m])
  float* residual;
  int64_t ld_residual;
  const bf16_t* norm_weight;
  float* sumsq_out;
  // PRO_SCALED: the pieces of the rows' sums of squares [pieces][m], the norm's eps and width
  const float* sumsq_in;
  int sumsq_pieces;
  float norm_eps;
  int norm_width;
};

template <int NT, int U, int EPI, int PRO = PRO_NONE, bool LINES = false, int RT = 1>
__global__ __launch_bounds__(64 * SK_WAVES) void gemm_skinny_bf16_kernel(
    const bf16_t* __restrict__ a, int64_t lda, const bf16_t* __restrict__ w, int64_t ldw,
    bf16_t* __restrict__ c, int64_t ldc, int m, int n, int k, int features_per_block, const FoldArgs fold) {
  constexpr bool GATED = EPI == EPI_GATED;
  constexpr bool ROPE = EPI == EPI_ROPE;
  constexpr bool ADDNORM = EPI == EPI_ADDNORM;
  constexpr bool SCALED = PRO == PRO_SCALED;
  static_assert(!ROPE || NT == 1, "the rotary epilogue takes one tile of dims and its partner tile");
  static_assert(!LINES || U % 2 == 0, "whole lines are read for pairs of k-steps");
  // RT = tiles of 16 ROWS (tokens): a weight operand once in registers is used for every row tile
  static_assert(RT == 1 || (PRO == PRO_NONE && !ADDNORM), "more than 16 rows: plain activations, no folded norm");
  constexpr int WT = (GATED || ROPE) ? 2 * NT : NT;  // weight tiles per block
  __shared__ float red[SK_WAVES][WT][256];

  // (with LINES made uniform for the compiler: the wave's range of K and with it the loop and
  // the base address of every load are scalar)
  const int wave = LINES ? __builtin_amdgcn_readfirstlane(threadIdx.x / MI_WAVE) : threadIdx.x / MI_WAVE;
  const int lane = threadIdx.x % MI_WAVE;
  const int col = lane % 16;
  const int quad = lane / 16;
  // the block's features [n0, n_end): up to 16*NT, a multiple of 4 chosen by the host so
  // that the blocks spread evenly over the CUs (rows past n_end repeat the last one)
  // Rotary epilogue: the unit of work is a PAIR (a dim of a head's first half and its
  // partner half a head further on); pairs are numbered through all heads and a block
  // takes `features_per_block` (a multiple of 4, at most 16) consecutive ones, which may
  // lie in two heads: tile 0 holds the pairs' first dims, tile 1 their partners.
  const int half = ROPE ? fold.head_dim / 2 : 0;
  const int total_pairs = ROPE ? (fold.q_heads + 2 * fold.kv_heads) * half : 0;
  const int pair0 = ROPE ? blockIdx.x * features_per_block : 0;
  const int pair_end = ROPE ? min(pair0 + features_per_block, total_pairs) : 0;
  const int n0 = blockIdx.x * features_per_block;
  const int n_end = min(n0 + features_per_block, n);

  const int ksteps = k / 32;
  const int per_wave = (ksteps + SK_WAVES - 1) / SK_WAVES;
  const int s_begin = min(wave * per_wave, ksteps);
  const int s_end = min(s_begin + per_wave, ksteps);

  // weights: lane reads feature n0 + 16*nt + col (and its twin n rows further down when
  // gated), 8 consecutive k
  auto weight_row = [&](int t, int c) -> int {  // the matrix row behind row c of weight tile t
    if (ROPE) {
      const int pair = min(pair0 + c, pair_end - 1);
      return (pair / half) * fold.head_dim + pair % half + t * half;
    }
    return min(n0 + (t % NT) * 16 + c, n_end - 1) + (t / NT) * n;
  };
  const bf16_t* wp[LINES ? 1 : WT];
  // LINES: byte offsets of this lane's 16 bytes in the tile's lower and upper 8 rows
  uint32_t line_lo[LINES ? WT : 1], line_hi[LINES ? WT : 1];
#pragma unroll
  for (int t = 0; t < WT; ++t) {
    if constexpr (LINES) {
      const uint32_t chunk = line_chunk_of_lane(lane);
      line_lo[t] = (uint32_t)weight_row(t, line_row_of_lane(lane)) * (uint32_t)(ldw * 2) + chunk;
      line_hi[t] = (uint32_t)weight_row(t, 8 + line_row_of_lane(lane)) * (uint32_t)(ldw * 2) + chunk;
    } else {
      wp[t] = w + (int64_t)weight_row(t, col) * ldw + quad * 8;
    }
  }
  // the lane's operands of the k-steps first, first + 1 of weight tile t (LINES)
  auto load_lines = [&](int t, int first, bf16x8_t& even_step, bf16x8_t& odd_step) {
    load_line_pair(w, first, line_lo[LINES ? t : 0], line_hi[LINES ? t : 0], even_step, odd_step);
  };
  // activations: lane reads token `col`; lanes past M re-read the last token (the same
  // cache lines as its own lane, so no extra traffic) and their columns are never stored
  const bf16_t* ap[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) ap[rt] = a + (int64_t)min(rt * 16 + col, m - 1) * lda + quad * 8;
  __shared__ __attribute__((aligned(16))) bf16_t a_own[PRO == PRO_ATTN ? SK_WAVES : 1][PRO == PRO_ATTN ? SK_PRO_VALUES : 8];
  const int own_stride = per_wave * 32;  // elements from one row of this wave's columns to the next
  // PRO_ATTN: the weights of the first U k-steps are requested before the activations are
  // made, so that the trips to the key ranges' results hide behind the first trip to memory
  bf16x8_t w_first[PRO == PRO_ATTN ? U : 1][WT];
  const bool first_ahead = PRO == PRO_ATTN && s_begin + U <= s_end;
  if constexpr (PRO == PRO_ATTN) {
    if (first_ahead) {
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < WT; ++t) {
          if constexpr (LINES) {
            if (u % 2 == 0) load_lines(t, s_begin + u, w_first[u][t], w_first[u + 1][t]);
          } else {
            w_first[u][t] = *reinterpret_cast<const bf16x8_t*>(wp[LINES ? 0 : t] + (int64_t)(s_begin + u) * 32);
          }
        }
    }
  }
  if constexpr (PRO == PRO_ATTN) {
    // this wave's columns [32*s_begin, 32*s_end) of the attention output, 8 at a time per
    // lane: the key ranges' accumulators weighted by exp(max - overall max), added in range
    // order, divided by the weighted sum of their sums (the arithmetic of attn_reduce_kernel)
    const int chunks = (s_end - s_begin) * 4;
    const int head_dim = fold.attn_head_dim, splits = fold.num_splits;
    for (int idx = lane; idx < m * chunks; idx += MI_WAVE) {
      const int row = idx / chunks, chunk = idx % chunks;
      const int k0 = s_begin * 32 + chunk * 8;
      const int head = k0 / head_dim, dim = k0 % head_dim;
      const int64_t base = ((int64_t)row * fold.attn_heads + head) * splits;
      const float* ml = fold.part_ml + base * 2;
      const float* pa = fold.part_acc + base * head_dim + dim;
      // (requesting every range's values before the first use measured slower than this loop)
      float m_all = -INFINITY;
#pragma unroll 8
      for (int sp = 0; sp < splits; ++sp) m_all = fmaxf(m_all, ml[sp * 2]);
      float o[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      float l_all = 0.f;
#pragma unroll 4
      for (int sp = 0; sp < splits; ++sp) {
        const float weight = expf(ml[sp * 2] - m_all);
        l_all += ml[sp * 2 + 1] * weight;
        const f32x4_t lo = *reinterpret_cast<const f32x4_t*>(pa + (int64_t)sp * head_dim);
        const f32x4_t hi = *reinterpret_cast<const f32x4_t*>(pa + (int64_t)sp * head_dim + 4);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          o[j] += lo[j] * weight;
          o[4 + j] += hi[j] * weight;
        }
      }
      const float inv = 1.f / l_all;
      bf16x8_t packed;
#pragma unroll
      for (int j = 0; j < 8; ++j) packed[j] = (bf16_t)(o[j] * inv);
      *reinterpret_cast<bf16x8_t*>(&a_own[wave][row * own_stride + chunk * 8]) = packed;
    }
    __syncthreads();
  }
  const bf16_t* own = &a_own[PRO == PRO_ATTN ? wave : 0][(PRO == PRO_ATTN ? min(col, m - 1) * own_stride : 0) + quad * 8];

  __shared__ float scale_part[SCALED ? SK_SCALE_PARTS : 1][16];
  // EPI_ADDNORM: the residual values and norm weights of the thread's four outputs, asked for
  // now, so that the last step does not begin with a trip to memory
  f32x4_t res_old = {0.f, 0.f, 0.f, 0.f};
  float norm_w4[4] = {0.f, 0.f, 0.f, 0.f};
  if constexpr (ADDNORM) {
    const int item = threadIdx.x;
    const int token = (item % 64) % 16, feature = n0 + (item / 64) * 16 + ((item % 64) / 16) * 4;
    if (item < NT * 64 && token < m) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (feature + r < n_end) {
          res_old[r] = fold.residual[(int64_t)token * fold.ld_residual + feature + r];
          norm_w4[r] = (float)fold.norm_weight[feature + r];
        }
      }
    }
  }

  // PRO_SCALED: SK_SCALE_PARTS threads per row each add up every SK_SCALE_PARTS-th piece of the
  // row's sum of squares, in a fixed order.  Where the loop below leaves registers to spare the
  // pieces are asked for before it, so that the trip to them is over when it ends (whole decode
  // steps 0.9-1.3 % faster); with four weight tiles they would cost the registers of a resident
  // block per CU (measured: 16 % slower), and are asked for after it.  (Capping the registers
  // of the variants just above 80 at 80 measured 0.8-1.4 % slower.)
  constexpr bool SCALE_EARLY = SCALED && WT <= 2;
  float scale_piece[SCALED ? SK_SCALE_PIECES : 1];
  auto load_scale_pieces = [&]() {
    const int row = threadIdx.x % 16, part = threadIdx.x / 16;
#pragma unroll
    for (int i = 0; i < SK_SCALE_PIECES; ++i) {
      const int piece = part + i * SK_SCALE_PARTS;
      scale_piece[SCALED ? i : 0] = (row < m && piece < fold.sumsq_pieces) ? fold.sumsq_in[(int64_t)piece * m + row] : 0.f;
    }
  };
  if constexpr (SCALE_EARLY) load_scale_pieces();

  f32x4_t acc[RT][WT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int t = 0; t < WT; ++t) acc[rt][t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  int s = s_begin;
  for (; s + U <= s_end; s += U) {
    bf16x8_t w_reg[U][WT];
    bf16x8_t a_reg[RT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < WT; ++t) {
        if constexpr (LINES) {
          if (u % 2 == 0) {
            if (PRO == PRO_ATTN && first_ahead && s == s_begin) {
              w_reg[u][t] = w_first[PRO == PRO_ATTN ? u : 0][t];
              w_reg[u + 1][t] = w_first[PRO == PRO_ATTN ? u + 1 : 0][t];
            } else {
              load_lines(t, s + u, w_reg[u][t], w_reg[u + 1][t]);
            }
          }
        } else {
          if (PRO == PRO_ATTN && first_ahead && s == s_begin) w_reg[u][t] = w_first[PRO == PRO_ATTN ? u : 0][t];
          else w_reg[u][t] = *reinterpret_cast<const bf16x8_t*>(wp[LINES ? 0 : t] + (int64_t)(s + u) * 32);
        }
      }
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        if constexpr (PRO == PRO_ATTN) a_reg[rt][u] = *reinterpret_cast<const bf16x8_t*>(own + (s + u - s_begin) * 32);
        else a_reg[rt][u] = *reinterpret_cast<const bf16x8_t*>(ap[rt] + (int64_t)(s + u) * 32);
      }
    }
    if constexpr (LINES) {
#pragma unroll
      for (int u = 0; u < U; u += 2)
#pragma unroll
        for (int t = 0; t < WT; ++t) lines_to_operands(w_reg[u][t], w_reg[u + 1][t]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < WT; ++t)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_reg[u][t], a_reg[rt][u], acc[rt][t], 0, 0, 0);
  }
  if constexpr (LINES) {
    for (; s + 2 <= s_end; s += 2) {  // fewer than U k-steps left: pair by pair (their number is even)
      bf16x8_t a_even[RT], a_odd[RT];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        a_even[rt] = PRO == PRO_ATTN ? *reinterpret_cast<const bf16x8_t*>(own + (s - s_begin) * 32)
                                     : *reinterpret_cast<const bf16x8_t*>(ap[rt] + (int64_t)s * 32);
        a_odd[rt] = PRO == PRO_ATTN ? *reinterpret_cast<const bf16x8_t*>(own + (s + 1 - s_begin) * 32)
                                    : *reinterpret_cast<const bf16x8_t*>(ap[rt] + (int64_t)(s + 1) * 32);
      }
#pragma unroll
      for (int t = 0; t < WT; ++t) {
        bf16x8_t w_even, w_odd;
        load_lines(t, s, w_even, w_odd);
        lines_to_operands(w_even, w_odd);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_even, a_even[rt], acc[rt][t], 0, 0, 0);
          acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_odd, a_odd[rt], acc[rt][t], 0, 0, 0);
        }
      }
    }
  }
  for (; !LINES && s < s_end; ++s) {  // fewer than U k-steps left
    bf16x8_t a_tail[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
      a_tail[rt] = PRO == PRO_ATTN ? *reinterpret_cast<const bf16x8_t*>(own + (s - s_begin) * 32)
                                   : *reinterpret_cast<const bf16x8_t*>(ap[rt] + (int64_t)s * 32);
#pragma unroll
    for (int t = 0; t < WT; ++t) {
      const bf16x8_t w_tail = *reinterpret_cast<const bf16x8_t*>(wp[LINES ? 0 : t] + (int64_t)s * 32);
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
        acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_tail, a_tail[rt], acc[rt][t], 0, 0, 0);
    }
  }

  if constexpr (SCALED && !SCALE_EARLY) load_scale_pieces();
  __shared__ float squares[ADDNORM ? NT * 4 : 1][16];  // EPI_ADDNORM: per (4 features, row) of the block
  // acc[rt][t][r] = C^T[feature n0 + 16*(t % NT) + 4*quad + r][token 16*rt + col]; add the 8 waves
  // in order, one row tile after the other through the same LDS
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
  if (rt > 0) __syncthreads();
#pragma unroll
  for (int t = 0; t < WT; ++t) {
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][t][(quad * 4 + r) * 16 + col] = acc[rt][t][r];
  }
  if constexpr (SCALED) {
    float scale_mine = 0.f;
#pragma unroll
    for (int i = 0; i < SK_SCALE_PIECES; ++i) scale_mine += scale_piece[i];
    scale_part[threadIdx.x / 16][threadIdx.x % 16] = scale_mine;
  }
  __syncthreads();
  // 256*NT outputs, each a sum of 8 (two such when gated): a thread takes 4 consecutive
  // features of one token
  for (int item = threadIdx.x; item < NT * 64; item += 64 * SK_WAVES) {
    const int nt = item / 64;
    const int token_in_tile = (item % 64) % 16;
    const int token = rt * 16 + token_in_tile;
    const int fq = (item % 64) / 16;
    if (token >= m) continue;
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int wv = 0; wv < SK_WAVES; ++wv)
#pragma unroll
      for (int r = 0; r < 4; ++r) sum[r] += red[wv][nt][(fq * 4 + r) * 16 + token_in_tile];
    float up[4] = {0.f, 0.f, 0.f, 0.f};  // the twin tile's sums: the up half (gated), the partner dims (rotary)
    if (GATED || ROPE) {
#pragma unroll
      for (int wv = 0; wv < SK_WAVES; ++wv)
#pragma unroll
        for (int r = 0; r < 4; ++r) up[r] += red[wv][NT + nt][(fq * 4 + r) * 16 + token_in_tile];
    }
    if constexpr (SCALED) {
      float total = 0.f;
#pragma unroll
      for (int part = 0; part < SK_SCALE_PARTS; ++part) total += scale_part[part][token];
      const float inv = rsqrtf(total / (float)fold.norm_width + fold.norm_eps);
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        sum[r] *= inv;
        up[r] *= inv;
      }
    }
    if (GATED) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float g = (float)(bf16_t)sum[r];
        sum[r] = g / (1.f + expf(-g)) * (float)(bf16_t)up[r];
      }
    }
    if constexpr (ADDNORM) {
      const int feature = n0 + nt * 16 + fq * 4;
      float* res = fold.residual + (int64_t)token * fold.ld_residual + feature;
      bf16_t* dst = c + (int64_t)token * ldc + feature;
      float sq = 0.f;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        if (feature + r < n_end) {  // (rows past n_end repeat the last feature: not counted twice)
          const float x = res_old[r] + (float)(bf16_t)sum[r];
          res[r] = x;
          dst[r] = (bf16_t)(x * norm_w4[r]);
          sq += x * x;
        }
      }
      squares[nt * 4 + fq][token] = sq;
      continue;
    }
    if (ROPE) {
      // this thread: four consecutive pairs (never across a head: half is a multiple of 4), one token
      const int pair = pair0 + fq * 4;
      if (pair >= pair_end) continue;
      const int rope_head = pair / half, j = pair % half;
      const int q_heads = fold.q_heads, kv_heads = fold.kv_heads, hd = fold.head_dim;
      float lo[4], hi[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        lo[r] = (float)(bf16_t)sum[r];
        hi[r] = (float)(bf16_t)up[r];
      }
      if (rope_head < q_heads + kv_heads) {  // queries and keys are rotated (formula: models/blocks/fold.py:411-431)
        const f32x4_t cs = *reinterpret_cast<const f32x4_t*>(fold.cos_t + (int64_t)token * half + j);
        const f32x4_t sn = *reinterpret_cast<const f32x4_t*>(fold.sin_t + (int64_t)token * half + j);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float x0 = lo[r], x1 = hi[r];
          lo[r] = x0 * cs[r] - x1 * sn[r];
          hi[r] = x1 * cs[r] + x0 * sn[r];
        }
      }
      bf16x4_t lo_b, hi_b;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        lo_b[r] = (bf16_t)lo[r];
        hi_b[r] = (bf16_t)hi[r];
      }
      if (rope_head < q_heads) {
        bf16_t* dst = c + (int64_t)token * ldc + (int64_t)rope_head * hd + j;
        *reinterpret_cast<bf16x4_t*>(dst) = lo_b;
        *reinterpret_cast<bf16x4_t*>(dst + half) = hi_b;
      } else {
        const int slot = fold.slot_mapping[token];
        if (slot >= 0) {  // padding rows of a replayed step write nothing
          const int page = slot / fold.page_size, off = slot % fold.page_size;
          const bool is_key = rope_head < q_heads + kv_heads;
          const int h = rope_head - q_heads - (is_key ? 0 : kv_heads);
          const int64_t chunk = ((int64_t)page * kv_heads + h) * fold.page_size * hd;
          if (is_key || !fold.v_transposed) {
            bf16_t* dst = (is_key ? fold.k_pages : fold.v_pages) + chunk + (int64_t)off * hd + j;
            *reinterpret_cast<bf16x4_t*>(dst) = lo_b;
            *reinterpret_cast<bf16x4_t*>(dst + half) = hi_b;
          } else {
            bf16_t* dst = fold.v_pages + chunk + off;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              dst[(int64_t)(j + r) * fold.page_size] = lo_b[r];
              dst[(int64_t)(half + j + r) * fold.page_size] = hi_b[r];
            }
          }
        }
      }
      continue;
    }
    const int feature = n0 + nt * 16 + fq * 4;
    if constexpr (EPI == EPI_STORE_F32) {
      float* dst32 = reinterpret_cast<float*>(c) + (int64_t)token * ldc + feature;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (feature + r < n_end) dst32[r] = (float)(bf16_t)sum[r];
      continue;
    }
    bf16_t* dst = c + (int64_t)token * ldc + feature;
    if (feature + 3 < n_end && (ldc % 4 == 0)) {
      bf16x4_t packed;
#pragma unroll
      for (int r = 0; r < 4; ++r) packed[r] = (bf16_t)sum[r];
      *reinterpret_cast<bf16x4_t*>(dst) = packed;
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (feature + r < n_end) dst[r] = (bf16_t)sum[r];
    }
  }
  }  // row tiles
  if constexpr (ADDNORM) {
    __syncthreads();
    if ((int)threadIdx.x < m) {
      float total = 0.f;
#pragma unroll
      for (int i = 0; i < NT * 4; ++i) total += squares[i][threadIdx.x];
      fold.sumsq_out[(int64_t)blockIdx.x * m + threadIdx.x] = total;
    }
  }
}

// Rows.  The gated and the rotary product take two row tiles (17-32 rows: measured against the
// vendor product followed by silu_mul / rope_kv_write, microseconds at 24 / 32 rows: gate|up
// 2x14336x4096 42.9 / 46.2 against 54.6 / 54.6, q|k|v 6144x4096 17.0 / 17.2 against 20.2 / 19.5,
// gate|up 2x8192x3072 22.4 / 23.3 against 23.8 / 23.9, q|k|v 5120x3072 13.9 / 14.6 against
// 17.8 / 16.4; with four row tiles, 48 / 64 rows, they are level or slower: every block reads
// all the rows' activations).  Everything else takes one.
#define SK_MAX_ROWS 16
#define SK_WIDE_MAX_ROWS 32

// Compute units of the current device (asked once per device).
static int compute_units() {
  static int cached[64] = {0};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 0;
  if (cached[device] == 0) {
    int count = 0;
    if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
    cached[device] = count;
  }
  return cached[device];
}

static bool skinny_takes(int m, int n, int k, int64_t lda, int64_t ldw, int max_rows) {
  return m >= 1 && m <= max_rows && n >= 1 && k >= 32 && k % 32 == 0 && lda % 8 == 0 && ldw % 8 == 0;
}

extern "C" int mi_gemm_skinny_bf16_supported(int m, int n, int k, int64_t lda, int64_t ldw) {
  return skinny_takes(m, n, k, lda, ldw, SK_MAX_ROWS) ? 1 : 0;
}

// the gated and the rotary product (mi_gemm_skinny_swiglu_bf16, mi_gemm_skinny_rope_bf16)
extern "C" int mi_gemm_skinny_wide_bf16_supported(int m, int n, int k, int64_t lda, int64_t ldw) {
  return skinny_takes(m, n, k, lda, ldw, SK_WIDE_MAX_ROWS) ? 1 : 0;
}

// Features per block: as even a share of the output as a multiple of 4 allows, in
// whole rounds over the CUs (an HBM-bound kernel ends when its most loaded CU does),
// at most 16*max_tiles.  Measured on MI355X at Llama-8B sizes, batch 8: 6144 features
// run 10% faster as 256 blocks of 24 than as 192 of 32; 28672 as 512 blocks of 56
// rather than 448 of 64.
static int features_per_block_for(int n, int cus, int max_tiles) {
  const int rounds = ceil_div(n, cus * 16 * max_tiles);
  const int fpb = ceil_div(ceil_div(n, cus * rounds), 4) * 4;
  return fpb < 8 ? 8 : fpb;
}

// Whether a weight matrix of `rows` rows can be read in whole cache lines (LINES): its rows
// begin on 128-byte boundaries, every wave gets an even number of k-steps, and byte offsets
// into it fit 32 bits.
static bool whole_lines(const void* w, int64_t ldw, int64_t rows, int k) {
  return (uintptr_t)w % 128 == 0 && ldw % 64 == 0 && (k / 32) % (2 * SK_WAVES) == 0 &&
         rows * ldw * 2 < ((int64_t)1 << 32);
}

// `out_f32`: c is float32 [m, ldc] (EPI_STORE_F32).
static int skinny_plain(const void* a, int64_t lda, const void* w, int64_t ldw, void* c, int64_t ldc, int m, int n,
                        int k, bool out_f32, hipStream_t stream) {
  MI_REQUIRE(mi_gemm_skinny_bf16_supported(m, n, k, lda, ldw),
             "gemm_skinny_bf16: takes 1 <= m <= 16, k a multiple of 32, rows aligned to 16 bytes; "
             "got m=%d n=%d k=%d lda=%lld ldw=%lld", m, n, k, (long long)lda, (long long)ldw);
  MI_REQUIRE(lda >= k && ldw >= k && ldc >= n, "gemm_skinny_bf16: a row stride is shorter than its row");
  const bf16_t* ap = (const bf16_t*)a;
  const bf16_t* wp = (const bf16_t*)w;
  bf16_t* cp = (bf16_t*)c;
  const FoldArgs nothing_folded = {};
  const int cus = compute_units();
  MI_REQUIRE(cus > 0, "gemm_skinny_bf16: cannot read the device's compute unit count");
  const int fpb = features_per_block_for(n, cus, 4);
  const int blocks = ceil_div(n, fpb);
  const int threads = 64 * SK_WAVES;
  const bool lines = whole_lines(w, ldw, n, k);
#define SK_PLAIN_AS(NT_, U_, EPI_)                                                                                 \
  if (lines)                                                                                                       \
    gemm_skinny_bf16_kernel<NT_, U_, EPI_, PRO_NONE, true><<<blocks, threads, 0, stream>>>(ap, lda, wp, ldw, cp, ldc, m, n, k, fpb, nothing_folded); \
  else                                                                                                             \
    gemm_skinny_bf16_kernel<NT_, U_, EPI_><<<blocks, threads, 0, stream>>>(ap, lda, wp, ldw, cp, ldc, m, n, k, fpb, nothing_folded)
#define SK_PLAIN(NT_, U_)                                \
  if (out_f32) { SK_PLAIN_AS(NT_, U_, EPI_STORE_F32); } \
  else { SK_PLAIN_AS(NT_, U_, EPI_STORE); }
  switch (ceil_div(fpb, 16)) {
    case 1: SK_PLAIN(1, 8); break;
    case 2: SK_PLAIN(2, 8); break;
    case 3: SK_PLAIN(3, 4); break;
    default: SK_PLAIN(4, 2); break;
  }
#undef SK_PLAIN
#undef SK_PLAIN_AS
  MI_CHECK_LAUNCH("gemm_skinny_bf16");
  return MI_OK;
}

extern "C" int mi_gemm_skinny_bf16(const void* a, int64_t lda, const void* w, int64_t ldw, void* c,
                                   int64_t ldc, int m, int n, int k, hipStream_t stream) {
  return skinny_plain(a, lda, w, ldw, c, ldc, m, n, k, false, stream);
}

// The same product, the same values, written as float32 [m, ldc].
extern "C" int mi_gemm_skinny_f32out_bf16(const void* a, int64_t lda, const void* w, int64_t ldw, float* c,
                                          int64_t ldc, int m, int n, int k, hipStream_t stream) {
  return skinny_plain(a, lda, w, ldw, c, ldc, m, n, k, true, stream);
}

// c[m, n] = attention output [m, heads*head_dim] . w^T, the attention output still lying in
// attn_mfma's uncombined key ranges (part_acc, part_ml as that kernel leaves them, rows
// 0..m-1): few rows, m * heads*head_dim at most 32768 (8 rows of 4096; see
// mi_gemm_skinny_attn_bf16_supported).
extern "C" int mi_gemm_skinny_attn_bf16_supported(int m, int heads, int head_dim) {
  if (m < 1 || m > SK_MAX_ROWS || heads < 1 || head_dim < 32 || head_dim % 32 != 0) return 0;
  const int k = heads * head_dim;
  return m * ceil_div(k / 32, SK_WAVES) * 32 <= SK_PRO_VALUES ? 1 : 0;
}

extern "C" int mi_gemm_skinny_attn_bf16(const float* part_acc, const float* part_ml, int num_splits, int heads,
                                        int head_dim, const void* w, int64_t ldw, void* c, int64_t ldc, int m,
                                        int n, hipStream_t stream) {
  MI_REQUIRE(part_acc && part_ml && num_splits >= 1 && num_splits <= 64,
             "gemm_skinny_attn_bf16: needs the partial buffers of 1..64 key ranges, got %d", num_splits);
  MI_REQUIRE(heads >= 1 && head_dim >= 32 && head_dim % 32 == 0,
             "gemm_skinny_attn_bf16: takes head_dim a multiple of 32; got heads=%d head_dim=%d", heads, head_dim);
  const int k = heads * head_dim;
  MI_REQUIRE(n >= 1 && ldw % 8 == 0 && ldw >= k && ldc >= n,
             "gemm_skinny_attn_bf16: weight rows must be aligned to 16 bytes; got n=%d k=%d ldw=%lld", n, k,
             (long long)ldw);
  MI_REQUIRE(mi_gemm_skinny_attn_bf16_supported(m, heads, head_dim),
             "gemm_skinny_attn_bf16: rows x (heads*head_dim / 8) must be at most %d; got m=%d k=%d", SK_PRO_VALUES, m, k);
  const bf16_t* ap = (const bf16_t*)w;  // never read: the activations are made in the kernel
  const int64_t lda = ldw;
  const bf16_t* wp = (const bf16_t*)w;
  bf16_t* cp = (bf16_t*)c;
  FoldArgs args = {};
  args.part_acc = part_acc;
  args.part_ml = part_ml;
  args.num_splits = num_splits;
  args.attn_heads = heads;
  args.attn_head_dim = head_dim;
  const int cus = compute_units();
  MI_REQUIRE(cus > 0, "gemm_skinny_attn_bf16: cannot read the device's compute unit count");
  const int fpb = features_per_block_for(n, cus, 4);
  const int blocks = ceil_div(n, fpb);
  const int threads = 64 * SK_WAVES;
  const bool lines = whole_lines(w, ldw, n, k);
#define SK_ATTN(NT_, U_)                                                                                          \
  if (lines)                                                                                                      \
    gemm_skinny_bf16_kernel<NT_, U_, EPI_STORE, PRO_ATTN, true><<<blocks, threads, 0, stream>>>(ap, lda, wp, ldw, cp, ldc, m, n, k, fpb, args); \
  else                                                                                                            \
    gemm_skinny_bf16_kernel<NT_, U_, EPI_STORE, PRO_ATTN><<<blocks, threads, 0, stream>>>(ap, lda, wp, ldw, cp, ldc, m, n, k, fpb, args)
  switch (ceil_div(fpb, 16)) {
    case 1: SK_ATTN(1, 8); break;
    case 2: SK_ATTN(2, 8); break;
    case 3: SK_ATTN(3, 4); break;
    default: SK_ATTN(4, 2); break;
  }
#undef SK_ATTN
  MI_CHECK_LAUNCH("gemm_skinny_attn_bf16");
  return MI_OK;
}

// The product as a layer's contribution to the residual stream, with the following RMS norm but
// for its row factor (EPI_ADDNORM): residual[m, n] += bf16(a . w^T); values[m, n] =
// bf16(residual * norm_weight); sumsq[pieces][m] = each block's sums of squares, where
// pieces = mi_gemm_skinny_addnorm_pieces(n).  With part_acc the activations are the
// uncombined key ranges of attn_mfma (as in mi_gemm_skinny_attn_bf16; a, lda unused).
extern "C" int mi_gemm_skinny_addnorm_pieces(int n) {
  const int cus = compute_units();
  if (cus <= 0 || n < 1) return 0;
  return ceil_div(n, features_per_block_for(n, cus, 4));
}

extern "C" int mi_gemm_skinny_addnorm_bf16(const void* a, int64_t lda, const float* part_acc, const float* part_ml,
                                           int num_splits, int heads, int head_dim, const void* w, int64_t ldw,
                                           float* residual, int64_t ld_residual, const void* norm_weight,
                                           void* values, int64_t ldv, float* sumsq, int m, int n, int k,
                                           hipStream_t stream) {
  const bool from_attention = part_acc != nullptr;
  if (from_attention) {
    MI_REQUIRE(part_ml && num_splits >= 1 && num_splits <= 64 && heads * head_dim == k,
               "gemm_skinny_addnorm_bf16: needs the partial buffers of 1..64 key ranges over k = heads*head_dim; "
               "got splits=%d heads=%d head_dim=%d k=%d", num_splits, heads, head_dim, k);
    MI_REQUIRE(mi_gemm_skinny_attn_bf16_supported(m, heads, head_dim) && ldw % 8 == 0,
               "gemm_skinny_addnorm_bf16: rows x (heads*head_dim / 8) must be at most %d, head_dim a multiple of 32; "
               "got m=%d heads=%d head_dim=%d", SK_PRO_VALUES, m, heads, head_dim);
  } else {
    MI_REQUIRE(mi_gemm_skinny_bf16_supported(m, n, k, lda, ldw) && lda >= k,
               "gemm_skinny_addnorm_bf16: takes 1 <= m <= 16, k a multiple of 32, rows aligned to 16 bytes; "
               "got m=%d n=%d k=%d lda=%lld ldw=%lld", m, n, k, (long long)lda, (long long)ldw);
  }
  MI_REQUIRE(n >= 1 && ldw >= k && ldv >= n && ld_residual >= n, "gemm_skinny_addnorm_bf16: a row stride is shorter than its row");
  MI_REQUIRE(residual && norm_weight && values && sumsq, "gemm_skinny_addnorm_bf16: needs residual, norm weight and both outputs");
  FoldArgs args = {};
  args.part_acc = part_acc;
  args.part_ml = part_ml;
  args.num_splits = num_splits;
  args.attn_heads = heads;
  args.attn_head_dim = head_dim;
  args.residual = residual;
  args.ld_residual = ld_residual;
  args.norm_weight = (const bf16_t*)norm_weight;
  args.sumsq_out = sumsq;
  const bf16_t* wp = (const bf16_t*)w;
  const bf16_t* ap = from_attention ? wp : (const bf16_t*)a;  // (never read when the activations are made in the kernel)
  if (from_attention) lda = ldw;
  bf16_t* cp = (bf16_t*)values;
  const int cus = compute_units();
  MI_REQUIRE(cus > 0, "gemm_skinny_addnorm_bf16: cannot read the device's compute unit count");
  const int fpb = features_per_block_for(n, cus, 4);
  const int blocks = ceil_div(n, fpb);
  const int threads = 64 * SK_WAVES;
  const bool lines = whole_lines(w, ldw, n, k);
#define SK_ADDNORM(NT_, U_)                                                                                        \
  if (from_attention && lines)                                                                                     \
    gemm_skinny_bf16_kernel<NT_, U_, EPI_ADDNORM, PRO_ATTN, true><<<blocks, threads, 0, stream>>>(ap, lda, wp, ldw, cp, ldv, m, n, k, fpb, args); \
  else if (from_attention)                                                                                         \
    gemm_skinny_bf16_kernel<NT_, U_, EPI_ADDNORM, PRO_ATTN><<<blocks, threads, 0, stream>>>(ap, lda, wp, ldw, cp, ldv, m, n, k, fpb, args); \
  else if (lines)                                                                                                  \
    gemm_skinny_bf16_kernel<NT_, U_, EPI_ADDNORM, PRO_NONE, true><<<blocks, threads, 0, stream>>>(ap, lda, wp, ldw, cp, ldv, m, n, k, fpb, args); \
  else                                                                                                             \
    gemm_skinny_bf16_kernel<NT_, U_, EPI_ADDNORM><<<blocks, threads, 0, stream>>>(ap, lda, wp, ldw, cp, ldv, m, n, k, fpb, args)
  switch (ceil_div(fpb, 16)) {
    case 1: SK_ADDNORM(1, 8); break;
    case 2: SK_ADDNORM(2, 8); break;
    case 3: SK_ADDNORM(3, 4); break;
    default: SK_ADDNORM(4, 2); break;
  }
#undef SK_ADDNORM
  MI_CHECK_LAUNCH("gemm_skinny_addnorm_bf16");
  return MI_OK;
}

// The gated product on rows whose norm factor is still apart (PRO_SCALED): a = the values of
// mi_gemm_skinny_addnorm_bf16, sumsq[pieces][m] its sums of squares; out[m, n] =
// silu(f * a . gate^T) * (f * a . up^T) with f = rsqrt(sum of the row's pieces / k + eps).
extern "C" int mi_gemm_skinny_swiglu_scaled_bf16(const void* a, int64_t lda, const float* sumsq, int pieces, float eps,
                                                 const void* w, int64_t ldw, void* out, int64_t ldo, int m, int n,
                                                 int k, hipStream_t stream) {
  MI_REQUIRE(mi_gemm_skinny_bf16_supported(m, n, k, lda, ldw),
             "gemm_skinny_swiglu_scaled_bf16: takes 1 <= m <= 16, k a multiple of 32, rows aligned to 16 bytes; "
             "got m=%d n=%d k=%d lda=%lld ldw=%lld", m, n, k, (long long)lda, (long long)ldw);
  MI_REQUIRE(lda >= k && ldw >= k && ldo >= n, "gemm_skinny_swiglu_scaled_bf16: a row stride is shorter than its row");
  MI_REQUIRE(sumsq && pieces >= 1 && pieces <= SK_SCALE_PARTS * SK_SCALE_PIECES && eps >= 0.f,
             "gemm_skinny_swiglu_scaled_bf16: needs the rows' sums of squares in 1..%d pieces, got %d",
             SK_SCALE_PARTS * SK_SCALE_PIECES, pieces);
  FoldArgs args = {};
  args.sumsq_in = sumsq;
  args.sumsq_pieces = pieces;
  args.norm_eps = eps;
  args.norm_width = k;
  const int cus = compute_units();
  MI_REQUIRE(cus > 0, "gemm_skinny_swiglu_scaled_bf16: cannot read the device's compute unit count");
  const int fpb = features_per_block_for(n, cus, 2);
  const int blocks = ceil_div(n, fpb);
  const int threads = 64 * SK_WAVES;
  const bool lines = whole_lines(w, ldw, 2 * (int64_t)n, k);
#define SK_SCALED(NT_, U_, LINES_)                                                          \
  gemm_skinny_bf16_kernel<NT_, U_, EPI_GATED, PRO_SCALED, LINES_><<<blocks, threads, 0, stream>>>( \
      (const bf16_t*)a, lda, (const bf16_t*)w, ldw, (bf16_t*)out, ldo, m, n, k, fpb, args)
  if (fpb <= 16) {
    if (lines) SK_SCALED(1, 4, true); else SK_SCALED(1, 4, false);
  } else {
    if (lines) SK_SCALED(2, 4, true); else SK_SCALED(2, 2, false);
  }
#undef SK_SCALED
  MI_CHECK_LAUNCH("gemm_skinny_swiglu_scaled_bf16");
  return MI_OK;
}

// out[m, n] = silu(a . gate^T) * (a . up^T) with w = [gate; up] stacked, [2n, k].
extern "C" int mi_gemm_skinny_swiglu_bf16(const void* a, int64_t lda, const void* w, int64_t ldw, void* out,
                                          int64_t ldo, int m, int n, int k, hipStream_t stream) {
  MI_REQUIRE(mi_gemm_skinny_wide_bf16_supported(m, n, k, lda, ldw),
             "gemm_skinny_swiglu_bf16: takes 1 <= m <= 32, k a multiple of 32, rows aligned to 16 bytes; "
             "got m=%d n=%d k=%d lda=%lld ldw=%lld", m, n, k, (long long)lda, (long long)ldw);
  MI_REQUIRE(lda >= k && ldw >= k && ldo >= n, "gemm_skinny_swiglu_bf16: a row stride is shorter than its row");
  const bf16_t* ap = (const bf16_t*)a;
  const bf16_t* wp = (const bf16_t*)w;
  bf16_t* cp = (bf16_t*)out;
  const FoldArgs nothing_folded = {};
  const int cus = compute_units();
  MI_REQUIRE(cus > 0, "gemm_skinny_swiglu_bf16: cannot read the device's compute unit count");
  const int fpb = features_per_block_for(n, cus, 2);  // two output tiles = four weight tiles
  const int blocks = ceil_div(n, fpb);
  const int threads = 64 * SK_WAVES;
  const bool lines = whole_lines(w, ldw, 2 * (int64_t)n, k);
#define SK_GATED(NT_, U_, LINES_, RT_) \
  gemm_skinny_bf16_kernel<NT_, U_, EPI_GATED, PRO_NONE, LINES_, RT_><<<blocks, threads, 0, stream>>>(ap, lda, wp, ldw, cp, ldo, m, n, k, fpb, nothing_folded)
  if (m <= 16) {
    if (fpb <= 16) {
      if (lines) SK_GATED(1, 4, true, 1); else SK_GATED(1, 4, false, 1);
    } else {
      if (lines) SK_GATED(2, 4, true, 1); else SK_GATED(2, 2, false, 1);
    }
  } else {  // (two row tiles: fewer k-steps in flight, the registers hold both tiles' sums)
    if (fpb <= 16) {
      if (lines) SK_GATED(1, 4, true, 2); else SK_GATED(1, 4, false, 2);
    } else {
      if (lines) SK_GATED(2, 2, true, 2); else SK_GATED(2, 2, false, 2);
    }
  }
#undef SK_GATED
  MI_CHECK_LAUNCH("gemm_skinny_swiglu_bf16");
  return MI_OK;
}

// The stacked q|k|v projection of an attention layer with the rotary encoding and the
// cache write in its last step: q_out[m, q_heads*head_dim] gets the rotated queries, the
// rotated keys and the values go to their slots (slot_mapping[m]; kv_heads = 0: queries only,
// w then holds the query rows alone).  Half-paired rotation over the whole head,
// cos/sin [m, head_dim/2] float32.  With `sumsq` the rows are a norm's output but for the
// rows' factors (PRO_SCALED, as in mi_gemm_skinny_swiglu_scaled_bf16).
static int rope_product(const char* name, const void* a, int64_t lda, const float* sumsq, int pieces, float eps,
                        const void* w, int64_t ldw, void* q_out, int64_t ldq, const float* cos_t,
                        const float* sin_t, const int* slot_mapping, void* k_pages, void* v_pages, int m, int k,
                        int q_heads, int kv_heads, int head_dim, int page_size, int num_pages, int v_transposed,
                        hipStream_t stream) {
  MI_REQUIRE(q_heads >= 1 && kv_heads >= 0 && head_dim >= 32 && head_dim % 32 == 0,
             "%s: takes head_dim a multiple of 32; got q_heads=%d kv_heads=%d head_dim=%d", name, q_heads, kv_heads,
             head_dim);
  const int n = (q_heads + 2 * kv_heads) * head_dim;
  MI_REQUIRE(mi_gemm_skinny_wide_bf16_supported(m, n, k, lda, ldw),
             "%s: takes 1 <= m <= 32, k a multiple of 32, rows aligned to 16 bytes; "
             "got m=%d n=%d k=%d lda=%lld ldw=%lld", name, m, n, k, (long long)lda, (long long)ldw);
  MI_REQUIRE(lda >= k && ldw >= k && ldq >= (int64_t)q_heads * head_dim && ldq % 4 == 0,
             "%s: a row stride is shorter than its row or not 8-byte aligned", name);
  MI_REQUIRE(cos_t && sin_t, "%s: needs the rotation tables", name);
  MI_REQUIRE(kv_heads == 0 || (slot_mapping && k_pages && v_pages && page_size > 0 && num_pages > 0),
             "%s: pages and slots are needed to write keys and values", name);
  MI_REQUIRE(!sumsq || (pieces >= 1 && pieces <= SK_SCALE_PARTS * SK_SCALE_PIECES && eps >= 0.f),
             "%s: needs the rows' sums of squares in 1..%d pieces, got %d", name, SK_SCALE_PARTS * SK_SCALE_PIECES,
             pieces);
  FoldArgs fold = {};
  fold.cos_t = cos_t;
  fold.sin_t = sin_t;
  fold.slot_mapping = slot_mapping;
  fold.k_pages = (bf16_t*)k_pages;
  fold.v_pages = (bf16_t*)v_pages;
  fold.q_heads = q_heads;
  fold.kv_heads = kv_heads;
  fold.head_dim = head_dim;
  fold.page_size = page_size;
  fold.v_transposed = v_transposed;
  fold.sumsq_in = sumsq;
  fold.sumsq_pieces = pieces;
  fold.norm_eps = eps;
  fold.norm_width = k;
  // pairs per block: an even share over the CUs in whole rounds, as for the plain product
  const int cus = compute_units();
  MI_REQUIRE(cus > 0, "%s: cannot read the device's compute unit count", name);
  const int total_pairs = n / 2;
  const int rounds = ceil_div(total_pairs, cus * 16);
  int pairs_per_block = ceil_div(ceil_div(total_pairs, cus * rounds), 4) * 4;
  if (pairs_per_block > 16) pairs_per_block = 16;
  const int blocks = ceil_div(total_pairs, pairs_per_block);
  const bool lines = whole_lines(w, ldw, n, k);
#define SK_ROPE(U_, PRO_, LINES_, RT_)                                                                \
  gemm_skinny_bf16_kernel<1, U_, EPI_ROPE, PRO_, LINES_, RT_><<<blocks, 64 * SK_WAVES, 0, stream>>>( \
      (const bf16_t*)a, lda, (const bf16_t*)w, ldw, (bf16_t*)q_out, ldq, m, n, k, pairs_per_block, fold)
  if (sumsq) {
    MI_REQUIRE(m <= SK_MAX_ROWS, "%s: rows with their norm factor apart come 16 at most, got %d", name, m);
    if (lines) SK_ROPE(8, PRO_SCALED, true, 1); else SK_ROPE(8, PRO_SCALED, false, 1);
  } else if (m <= 16) {
    if (lines) SK_ROPE(8, PRO_NONE, true, 1); else SK_ROPE(8, PRO_NONE, false, 1);
  } else {
    if (lines) SK_ROPE(4, PRO_NONE, true, 2); else SK_ROPE(4, PRO_NONE, false, 2);
  }
#undef SK_ROPE
  MI_CHECK_LAUNCH(name);
  return MI_OK;
}

extern "C" int mi_gemm_skinny_rope_bf16(const void* a, int64_t lda, const void* w, int64_t ldw, void* q_out,
                                        int64_t ldq, const float* cos_t, const float* sin_t,
                                        const int* slot_mapping, void* k_pages, void* v_pages, int m, int k,
                                        int q_heads, int kv_heads, int head_dim, int page_size, int num_pages,
                                        int v_transposed, hipStream_t stream) {
  return rope_product("gemm_skinny_rope_bf16", a, lda, nullptr, 0, 0.f, w, ldw, q_out, ldq, cos_t, sin_t, slot_mapping,
                      k_pages, v_pages, m, k, q_heads, kv_heads, head_dim, page_size, num_pages, v_transposed, stream);
}

// The same on rows whose norm factor is still apart: a = the values of mi_gemm_skinny_addnorm_bf16,
// sumsq[pieces][m] its sums of squares; the products are multiplied with
// rsqrt(sum of the row's pieces / k + eps) before they are rounded and rotated.
extern "C" int mi_gemm_skinny_rope_scaled_bf16(const void* a, int64_t lda, const float* sumsq, int pieces, float eps,
                                               const void* w, int64_t ldw, void* q_out, int64_t ldq,
                                               const float* cos_t, const float* sin_t, const int* slot_mapping,
                                               void* k_pages, void* v_pages, int m, int k, int q_heads,
                                               int kv_heads, int head_dim, int page_size, int num_pages,
                                               int v_transposed, hipStream_t stream) {
  MI_REQUIRE(sumsq, "gemm_skinny_rope_scaled_bf16: needs the rows' sums of squares");
  return rope_product("gemm_skinny_rope_scaled_bf16", a, lda, sumsq, pieces, eps, w, ldw, q_out, ldq, cos_t, sin_t,
                      slot_mapping, k_pages, v_pages, m, k, q_heads, kv_heads, head_dim, page_size, num_pages,
                      v_transposed, stream);
}
