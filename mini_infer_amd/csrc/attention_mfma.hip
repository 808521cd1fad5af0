// Paged causal attention on the matrix cores (bfloat16 in, float32 accumulate), for
// prefill portions and decode tokens alike.  gfx950 MFMA 16x16x32.
//
// Rows of work are (query token, query head of one key/value group) pairs, so the
// heads that share a key/value head share its loads.  A wave owns 16 such rows and
// walks the keys 32 at a time, computing the TRANSPOSED score block
//     S^T[key, row] = K[key, :] . Q[row, :]
// with K as the A operand (each lane reads 16 contiguous bytes of a key row straight
// from the cache page) and Q^T as the B operand (kept in registers).  The MFMA
// result leaves every lane with 8 scores of ONE row (lane % 16), so the online
// softmax needs two cross-lane steps, and the probabilities are already laid out
// as the B operand of the second product
//     O^T[dim, row] += V^T[dim, key] . P^T[key, row]
// whose A operand wants, per lane, consecutive keys of one dim: the cache stores
// values transposed inside each page ([page][head][dim][slot]) to make that a
// contiguous load.
//
// Two shapes of block:
//  * decode (one token per request): 16 rows = one row group; `KW` waves share the rows,
//    each taking every KW-th block of 32 keys straight from the pages into registers
//    (two register sets: the next block's loads are in flight while this one is
//    computed), and merge through LDS.  Keys may also be cut into `num_splits` ranges
//    across blocks; those partial (max, sum, accumulator) triples are combined by
//    attn_reduce_kernel (attention_generic.hip).
//  * prefill: `WAVES` waves x `RG` row groups = 128 rows = one tile of consecutive
//    tokens of one request, times `heads_per_block` heads of one key/value group.  The
//    waves load each 32-key tile of keys and values TOGETHER into LDS (SHARED), two
//    tiles deep, and read their matrix operands from there; two blocks run per CU.
//
// Semantics as in the reference's oracle (cache/packed_attention.py:296-338):
// row at absolute position p sees keys 0..p, or p-window+1..p with a window.
// Requires head_dim % 32 == 0 and page_size % 16 == 0; other sizes use the plain kernel.
#include "common.h"

#include <math.h>

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;

#define RESCALE_SLACK 8.0f
#define LOG2E 1.4426950408889634f
#define LN2 0.6931471805599453f

// Reductions over the 4 lanes that hold one row's scores (lane, lane^16, lane^32, lane^48)
// with the gfx950 lane-swap instructions: no trip through the LDS crossbar.
__device__ __forceinline__ float quad_max(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(a[0]), __uint_as_float(a[1]));
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(b[0]), __uint_as_float(b[1]));
}
__device__ __forceinline__ float quad_sum(float v) {
  auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

// OCC: waves per SIMD the registers are budgeted for.  SHARED: the block's waves load key
// and value tiles together through LDS (prefill); else every wave loads its own operands
// through two register sets (decode), the values at the start of the block that uses them.
template <int D, int WAVES, int KW, int RG, int OCC, bool SHARED, int PS>
__global__ __launch_bounds__(64 * WAVES * KW, OCC) void attn_mfma_kernel(
    const bf16_t* __restrict__ q, int64_t q_row_stride, const bf16_t* __restrict__ k_pages,
    const bf16_t* __restrict__ vt_pages, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ cu_seqlens_q, const int* __restrict__ positions, int num_requests,
    bf16_t* __restrict__ out, int64_t out_row_stride, float* __restrict__ part_acc,
    float* __restrict__ part_ml, int q_heads, int kv_heads, int page_size_arg, unsigned page_magic, float scale_log2,
    int window, int num_splits, int heads_per_block, int tokens_per_tile, int one_tile_per_request,
    int pair_group, int first_token) {
  constexpr int KSTEPS = D / 32;  // MFMA k-steps over the head dim for S^T
  // PS != 0: the page size is this constant (divisions become shifts, value offsets
  // immediates); PS == 0: any multiple of 16, divided by multiplying with
  // page_magic = floor(2^32 / page_size) + 1 (exact for keys below 2^32 / page_size).
  const int page_size = PS ? PS : page_size_arg;
  auto page_index = [&](int key) -> int {  // (keys are never negative: unsigned division is a shift)
    return PS ? (int)((unsigned)key / (unsigned)(PS ? PS : 1)) : (int)__umulhi((unsigned)key, page_magic);
  };
  constexpr int DBLOCKS = D / 16;  // 16-dim blocks of the output

  // ---- which tile of which request ----------------------------------------
  // Every wave finds it on its own.  With at most one tile per request (decode, short
  // portions) the tile IS the request; otherwise the lanes share the search: each takes
  // a request, a prefix sum over the requests' tile counts locates the tile.
  // The grid is one-dimensional in (tile, head block) with the HEAD BLOCK running
  // fastest: consecutive workgroups go to different XCDs (8, each with an L2 of its
  // own), so with a multiple of 8 head blocks every XCD sees the keys and values of
  // only its share of the heads, whatever the number of tiles, and they stay in its L2
  // for all the tiles of a prompt.
  const int group = q_heads / kv_heads;
  const int head_blocks = (group + heads_per_block - 1) / heads_per_block;
  const int head_slots = kv_heads * head_blocks;
  const int grid_tile = (int)(blockIdx.x / (unsigned)head_slots);
  const int grid_head = (int)(blockIdx.x % (unsigned)head_slots);
  const int grid_tiles = (int)(gridDim.x / (unsigned)head_slots);
  int req = -1, t0 = 0, n_tok = 0;
  if (one_tile_per_request == 2) {
    // every request brings exactly one token (a decode step): request b's token is the
    // b-th after first_token, and nothing has to be read to know it
    if (grid_tile < num_requests) {
      req = grid_tile;
      t0 = first_token + req;
      n_tok = 1;
    }
  } else if (one_tile_per_request) {
    if (grid_tile < num_requests) {
      req = grid_tile;
      t0 = cu_seqlens_q[req];
      n_tok = cu_seqlens_q[req + 1] - t0;
    }
  } else {
    // Tiles are handed out last first: under the causal mask a request's later tiles
    // have more keys, and starting the long ones first keeps the GPU's tail short.
    // With two blocks resident per CU the first 2*pair_group tiles an XCD receives start at
    // once, CU i taking the i-th and the (pair_group+i)-th: the longest pair_group tiles
    // are followed by the SHORTEST ones in rising order, so that every CU's pair has the
    // same sum; the rest follow longest first as CUs come free.  (pair_group 0: plain
    // longest-first order.  Only the running time depends on this guess at the dispatcher.)
    int tile_index = grid_tiles - 1 - grid_tile;
    if (pair_group > 0 && grid_tiles >= 2 * pair_group) {
      if (grid_tile >= pair_group && grid_tile < 2 * pair_group) tile_index = grid_tile - pair_group;
      else if (grid_tile >= 2 * pair_group) tile_index = grid_tiles - 1 - (grid_tile - pair_group);
    }
    const int search_lane = threadIdx.x % MI_WAVE;
    int tiles_before = 0;
    for (int b0 = 0; b0 < num_requests && req < 0; b0 += MI_WAVE) {
      const int b = b0 + search_lane;
      const int start = (b < num_requests) ? cu_seqlens_q[b] : 0;
      const int q_len = (b < num_requests) ? cu_seqlens_q[b + 1] - start : 0;
      const int n_tiles = (q_len + tokens_per_tile - 1) / tokens_per_tile;
      int inclusive = n_tiles;
#pragma unroll
      for (int off = 1; off < MI_WAVE; off <<= 1) {
        const int up = __shfl_up(inclusive, off, MI_WAVE);
        if (search_lane >= off) inclusive += up;
      }
      const int first = tiles_before + inclusive - n_tiles;
      const bool mine = n_tiles > 0 && tile_index >= first && tile_index < first + n_tiles;
      const unsigned long long owners = __ballot(mine);
      if (owners) {
        const int src = __ffsll((long long)owners) - 1;
        const int ti = tile_index - __shfl(first, src, MI_WAVE);
        req = b0 + src;
        t0 = __shfl(start, src, MI_WAVE) + ti * tokens_per_tile;
        n_tok = min(tokens_per_tile, __shfl(q_len, src, MI_WAVE) - ti * tokens_per_tile);
      }
      tiles_before += __shfl(inclusive, MI_WAVE - 1, MI_WAVE);
    }
  }
  if (req < 0 || n_tok <= 0) return;
  req = __builtin_amdgcn_readfirstlane(req);
  t0 = __builtin_amdgcn_readfirstlane(t0);
  n_tok = __builtin_amdgcn_readfirstlane(n_tok);

  const int kvh = grid_head / head_blocks;
  const int g0 = (grid_head % head_blocks) * heads_per_block;
  const int n_heads = min(heads_per_block, group - g0);
  const int split = blockIdx.z;

  static_assert(WAVES == 1 || KW == 1, "key-splitting waves are for single-row-group blocks");
  // WAVES wave slots of RG row groups (16 rows each); KW waves share a slot's rows and
  // take every KW-th key block.  (Wave numbers are made uniform for the compiler, so
  // that key block numbers and with them the block-table reads are scalar and do not
  // wait on the vector loads in flight.)
  const int wave_id = __builtin_amdgcn_readfirstlane(threadIdx.x / MI_WAVE);
  const int wave = wave_id / KW;
  const int key_wave = wave_id % KW;
  const int lane = threadIdx.x % MI_WAVE;
  const int col = lane % 16;  // this lane's row of work within a row group
  const int quad = lane / 16;  // 0..3

  // a wave whose rows are all padding has nothing to do (unless the block's waves load
  // the keys and values together: then it stays for the loads and the barriers)
  if (KW == 1 && !SHARED && wave * 16 * RG >= n_tok * heads_per_block) return;

  const int pos0 = positions[t0];  // tokens of a tile sit at consecutive positions
  int token[RG], head[RG], pos[RG], lo_row[RG];
  bool row_valid[RG];
#pragma unroll
  for (int rg = 0; rg < RG; ++rg) {
    const int row = (wave * RG + rg) * 16 + col;
    int tok_in_tile = row / heads_per_block;
    int head_in_block = row % heads_per_block;
    row_valid[rg] = tok_in_tile < n_tok && head_in_block < n_heads;
    tok_in_tile = min(tok_in_tile, n_tok - 1);  // padded rows repeat a real row and store nothing
    head_in_block = min(head_in_block, n_heads - 1);
    token[rg] = t0 + tok_in_tile;
    head[rg] = kvh * group + g0 + head_in_block;
    pos[rg] = pos0 + tok_in_tile;
    lo_row[rg] = (window > 0) ? max(0, pos[rg] - window + 1) : 0;
  }

  // smallest position and largest window start among this wave's rows (for the mask-free test)
  int wave_pos_min = pos[0], wave_lo_max = lo_row[0];
#pragma unroll
  for (int rg = 1; rg < RG; ++rg) {
    wave_pos_min = min(wave_pos_min, pos[rg]);
    wave_lo_max = max(wave_lo_max, lo_row[rg]);
  }
#pragma unroll
  for (int off = 1; off < 16; off <<= 1) {
    wave_pos_min = min(wave_pos_min, __shfl_xor(wave_pos_min, off, MI_WAVE));
    wave_lo_max = max(wave_lo_max, __shfl_xor(wave_lo_max, off, MI_WAVE));
  }
  wave_pos_min = __builtin_amdgcn_readfirstlane(wave_pos_min);
  wave_lo_max = __builtin_amdgcn_readfirstlane(wave_lo_max);

  // ---- key range of this block ------------------------------------------------
  const int tile_lo = (window > 0) ? max(0, pos0 - window + 1) : 0;
  const int tile_hi = pos0 + n_tok;  // exclusive
  int chunk = (tile_hi - tile_lo + num_splits - 1) / num_splits;
  chunk = (chunk + 31) / 32 * 32;
  const int k_begin = tile_lo + split * chunk;
  const int k_end = min(k_begin + chunk, tile_hi);
  const int* bt = block_table + (int64_t)req * max_blocks;
  // 32-key blocks starting in [interior_first, interior_last] are seen whole by every row of this wave
  const int interior_first = max(wave_lo_max, k_begin);
  const int interior_last = min(wave_pos_min - 31, k_end - 32);

  // ---- Q^T operands: this lane's rows, 8 consecutive dims per k-step --------------
  bf16x8_t q_reg[RG][KSTEPS];
#pragma unroll
  for (int rg = 0; rg < RG; ++rg) {
    const bf16_t* q_row = q + (int64_t)token[rg] * q_row_stride + (int64_t)head[rg] * D + quad * 8;
#pragma unroll
    for (int s = 0; s < KSTEPS; ++s) q_reg[rg][s] = *reinterpret_cast<const bf16x8_t*>(q_row + s * 32);
  }

  // Where the sum of a row's probabilities is kept.  Prefill shape (SHARED): in one more
  // block of the value product, o_acc[rg][DBLOCKS], whose value rows are all ones: the matrix
  // pipe adds up the probabilities (as rounded to bfloat16, the very numbers the values are
  // weighted with), every lane finds its row's sum in all four values it holds of that
  // block, and the vector pipe is spared an addition per score and a reduction per block.
  // Decode shape: in l_run, added up by the vector pipe (which idles there anyway).
  constexpr bool SUM_ON_MATRIX_PIPE = SHARED;
  constexpr int ACC_BLOCKS = DBLOCKS + (SUM_ON_MATRIX_PIPE ? 1 : 0);
  f32x4_t o_acc[RG][ACC_BLOCKS];
  float m_run[RG], l_run[RG];  // reference point of the exponentials (log2 units); sum of exp2(score - reference)
  // Two values that follow m_run and change only when it does, so that a block whose maximum
  // stays below the reference spends nothing on them: the addend of the exponentials'
  // arguments (-m_run, or 0 while the row has seen nothing), and the RAW score (before the
  // scale) above which the reference has to move.
  float neg_ref[RG], raw_limit[RG];
  const float inv_scale_log2 = 1.f / scale_log2;
#pragma unroll
  for (int rg = 0; rg < RG; ++rg) {
#pragma unroll
    for (int db = 0; db < ACC_BLOCKS; ++db) o_acc[rg][db] = (f32x4_t){0.f, 0.f, 0.f, 0.f};
    m_run[rg] = -INFINITY;
    l_run[rg] = 0.f;
    neg_ref[rg] = 0.f;
    raw_limit[rg] = -INFINITY;
  }
  bf16x8_t ones;
#pragma unroll
  for (int i = 0; i < 8; ++i) ones[i] = (bf16_t)1.0f;
  asm volatile("" : "+v"(ones));  // registers of its own for the whole kernel, not a constant made anew in every turn

  // One 32-key block: the K operands of its two 16-key halves and where its V^T operands
  // start.  A half never straddles a page; K rows of a (page, head) chunk are
  // [slot][D], V^T rows are [D][slot].  Released or unallocated pages read page 0:
  // every key of them is masked in the compute step.
  struct KVBlock {
    bf16x8_t k[2][KSTEPS];
    const bf16_t* v_base[2];
  };
  // Addresses are a wave-uniform base (page, head, first slot: scalar registers) plus a
  // per-lane 32-bit offset that never changes, so a load costs no vector arithmetic.
  // Page ids are read with SCALAR loads (the key block number is wave-uniform and the
  // block table is not written while the kernel runs) one block ahead of their use: they
  // are counted apart from the vector loads, so waiting for a page id never waits for the
  // keys and values in flight.
  struct PageIds {
    int page[2];  // of the two 16-key halves of a block
  };
  auto fetch_pages = [&](int kb) -> PageIds {
    PageIds ids;
#pragma unroll
    for (int hlf = 0; hlf < 2; ++hlf) {
      // (past the table only for keys past the request's end, which are masked)
      const unsigned entry = (unsigned)min(page_index(kb + 16 * hlf), max_blocks - 1);
      ids.page[hlf] = *reinterpret_cast<const int*>(reinterpret_cast<const char*>(bt) + entry * 4u);
    }
    return ids;
  };
  const int page_stride = kv_heads * page_size * D;  // elements from one page to the next
  const int head_off = kvh * page_size * D;
  const unsigned k_lane_off = (unsigned)(col * D + quad * 8);
  const unsigned v_lane_off = (unsigned)(col * page_size + 4 * quad);
  // Decode shape with 16-slot pages and key rows of whole cache lines: keys and values are read
  // once, so with non-temporal loads, and the keys in whole lines (lines_to_operands in
  // common.h; the values' 16 rows of 32 bytes per load are whole lines as they are).
  constexpr bool STREAM_KV = !SHARED && PS == 16 && D % 64 == 0;
  const uint32_t k_line_lo = (uint32_t)(line_row_of_lane(lane) * D * 2) + line_chunk_of_lane(lane);
  const uint32_t k_line_hi = k_line_lo + 8u * D * 2u;
  auto load_values = [&](const bf16_t* const v_base[2], bf16x8_t* v) {
#pragma unroll
    for (int db = 0; db < DBLOCKS; ++db) {
      const unsigned off = v_lane_off + (unsigned)(db * 16) * (unsigned)page_size;
      const bf16x4_t* from0 = reinterpret_cast<const bf16x4_t*>(v_base[0] + off);
      const bf16x4_t* from1 = reinterpret_cast<const bf16x4_t*>(v_base[1] + off);
      const bf16x4_t v0 = STREAM_KV ? __builtin_nontemporal_load(from0) : *from0;
      const bf16x4_t v1 = STREAM_KV ? __builtin_nontemporal_load(from1) : *from1;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[db][i] = v0[i];
        v[db][4 + i] = v1[i];
      }
    }
  };
  auto load_block = [&](int kb, const PageIds& ids, KVBlock& blk) {
    const bf16_t* k_base[2];
#pragma unroll
    for (int hlf = 0; hlf < 2; ++hlf) {
      const int key0 = kb + 16 * hlf;
      const int page = max(ids.page[hlf], 0);
      const int64_t chunk_off = (int64_t)page * page_stride + head_off;
      const int slot0 = key0 - page_index(key0) * page_size;
      k_base[hlf] = k_pages + chunk_off + (int64_t)slot0 * D;
      blk.v_base[hlf] = vt_pages + chunk_off + slot0;
    }
#pragma unroll
    for (int hlf = 0; hlf < 2; ++hlf) {
      if constexpr (STREAM_KV) {
#pragma unroll
        for (int s = 0; s < KSTEPS; s += 2)
          load_line_pair(k_base[hlf], s, k_line_lo, k_line_hi, blk.k[hlf][s], blk.k[hlf][s + 1]);
      } else {
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
          blk.k[hlf][s] = *reinterpret_cast<const bf16x8_t*>(k_base[hlf] + (k_lane_off + s * 32));
      }
    }
  };

  // The three phases run over all row groups of the wave in turn (scores for every
  // group, then every group's softmax, then every group's value product): the groups
  // are independent, so one group's vector work overlaps another's matrix work.
  // ---- S^T = K . Q^T for 32 keys ------------------------------------------------
  auto block_scores = [&](const KVBlock& blk, f32x4_t (&s_acc)[RG][2]) {
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
#pragma unroll
      for (int hlf = 0; hlf < 2; ++hlf) {
        f32x4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(blk.k[hlf][s], q_reg[rg][s], acc, 0, 0, 0);
        s_acc[rg][hlf] = acc;
      }
    }
  };
  // ---- scale, mask, online softmax (lane holds keys kb + 16*hlf + 4*quad + r) -----
  // Leaves the probabilities in p_reg (already the B operand of the value product) and
  // the factor the old accumulator must be multiplied with in alpha; returns whether any
  // row of the wave needs that multiplication (alpha != 1 somewhere).
  auto block_softmax = [&](int kb, f32x4_t (&s_acc)[RG][2], bf16x8_t (&p_reg)[RG], float (&alpha)[RG]) -> bool {
    // a block every row of this wave sees whole needs no mask (most blocks of a long prompt);
    // elsewhere hidden scores become -inf where they lie, before anything reads them (one
    // branch for all row groups, and no second copy of the scores for the two ways to merge in)
    const bool interior = kb >= interior_first && kb <= interior_last;
    if (!interior) {
#pragma unroll
      for (int rg = 0; rg < RG; ++rg)
#pragma unroll
        for (int hlf = 0; hlf < 2; ++hlf)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int key = kb + 16 * hlf + 4 * quad + r;
            const bool visible = key >= lo_row[rg] && key <= pos[rg] && key >= k_begin && key < k_end;
            s_acc[rg][hlf][r] = visible ? s_acc[rg][hlf][r] : -INFINITY;
          }
    }
    bool moved = false;
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
      // raw scores; the scale (positive) is applied to their maximum once and to each
      // score inside the exponential's argument, as one multiply-add
      float sc[8];
      float mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        sc[i] = s_acc[rg][i / 4][i % 4];
        mx = fmaxf(mx, sc[i]);
      }
      if constexpr (SUM_ON_MATRIX_PIPE) {
        // The reference point of the exponentials follows the running maximum lazily: it
        // moves only when the maximum grows by more than RESCALE_SLACK (in log2 units), so
        // probabilities stay below 2^RESCALE_SLACK and the accumulator is rarely rescaled.
        // Each lane looks at its own 8 raw scores first; only if some lane of the wave finds
        // one that far above the reference do the 4 lanes of a row agree on a maximum.
        alpha[rg] = 1.f;
        if (__ballot(mx > raw_limit[rg]) != 0ull) {
          mx = quad_max(mx) * scale_log2;
          const float m_new = (mx > m_run[rg] + RESCALE_SLACK) ? mx : m_run[rg];
          // A row's first visible block moves the reference from -inf; its sums are still
          // zero, so nothing is to be rescaled (alpha 1, not exp2(-inf)).
          alpha[rg] = (m_run[rg] == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_run[rg] - m_new);
          m_run[rg] = m_new;
          neg_ref[rg] = (m_new == -INFINITY) ? 0.f : -m_new;  // (0: a row that has seen nothing yet)
          raw_limit[rg] = (m_new + RESCALE_SLACK) * inv_scale_log2;
          moved = moved || (__ballot(alpha[rg] != 1.f) != 0ull);
        }
        // arguments are bounded above: the hardware exp2 is exact enough, tiny results flush to 0
#pragma unroll
        for (int i = 0; i < 8; i += 2) {  // (pairs: one conversion instruction for two)
          const f32x2_t e = {__builtin_amdgcn_exp2f(__builtin_fmaf(sc[i], scale_log2, neg_ref[rg])),
                             __builtin_amdgcn_exp2f(__builtin_fmaf(sc[i + 1], scale_log2, neg_ref[rg]))};
          const bf16x2_t b = __builtin_convertvector(e, bf16x2_t);
          p_reg[rg][i] = b[0];
          p_reg[rg][i + 1] = b[1];
        }
      } else {
        mx = quad_max(mx) * scale_log2;
        // (the same lazy reference point; here every block agrees on the row's maximum)
        const float m_new = (mx > m_run[rg] + RESCALE_SLACK) ? mx : m_run[rg];
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;  // a row that has seen nothing yet
        alpha[rg] = (m_run[rg] == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_run[rg] - m_safe);
        float sum = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(sc[i], scale_log2, -m_safe));
          sum += p;
          p_reg[rg][i] = (bf16_t)p;
        }
        sum = quad_sum(sum);
        l_run[rg] = l_run[rg] * alpha[rg] + sum;
        m_run[rg] = m_new;
        moved = moved || (__ballot(alpha[rg] != 1.f) != 0ull);
      }
    }
    return moved;
  };
  // ---- O^T *= alpha (only where block_softmax said so) ---------------------------------
  auto rescale = [&](const float (&alpha)[RG]) {
#pragma unroll
    for (int rg = 0; rg < RG; ++rg)
#pragma unroll
      for (int db = 0; db < ACC_BLOCKS; ++db)
#pragma unroll
        for (int r = 0; r < 4; ++r) o_acc[rg][db][r] *= alpha[rg];
  };
  // ---- O^T += V^T . P^T ------------------------------------------------------------------
  auto block_values = [&](const bf16x8_t* v_op, const bf16x8_t (&p_reg)[RG]) {
#pragma unroll
    for (int rg = 0; rg < RG; ++rg) {
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db)
        o_acc[rg][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_op[db], p_reg[rg], o_acc[rg][db], 0, 0, 0);
      if constexpr (SUM_ON_MATRIX_PIPE)
        o_acc[rg][DBLOCKS] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, p_reg[rg], o_acc[rg][DBLOCKS], 0, 0, 0);
    }
  };
  auto compute_block = [&](int kb, KVBlock& blk) {
    bf16x8_t v_late[DBLOCKS];
    load_values(blk.v_base, v_late);  // in flight during the scores and the softmax
    if constexpr (STREAM_KV) {
#pragma unroll
      for (int hlf = 0; hlf < 2; ++hlf)
#pragma unroll
        for (int s = 0; s < KSTEPS; s += 2) lines_to_operands(blk.k[hlf][s], blk.k[hlf][s + 1]);
    }
    f32x4_t s_acc[RG][2];
    block_scores(blk, s_acc);
    bf16x8_t p_reg[RG];
    float alpha[RG];
    // (one branch around the whole rescale, so that it is not turned into selects)
    if (block_softmax(kb, s_acc, p_reg, alpha)) rescale(alpha);
    block_values(v_late, p_reg);
  };

  // Software pipeline: the loads of the next block are in flight while this one is
  // computed (two register sets, the loop advances two blocks a turn).
  constexpr int STEP = 32 * KW;
  if constexpr (SHARED) {
    // The block's waves load each 32-key tile TOGETHER (every byte leaves the cache
    // hierarchy once per block instead of once per wave: with 4 waves a quarter of the
    // vector-memory traffic) into LDS, two tiles deep: while a tile is computed from one
    // buffer, the next one's global loads are in flight in a few staging registers and
    // are written to the other buffer at the end of the turn; one barrier per turn.
    // Key rows are padded by 16 bytes and value rows by 8 so that the operand reads of
    // 16 lanes fall into different banks.
    static_assert(KW == 1, "shared tiles are for blocks whose waves walk the same keys");
    constexpr int THREADS = 64 * WAVES;
    constexpr int CPR = D / 8;  // 16-byte chunks per key row
    constexpr int KROW = D + 8;  // elements
    constexpr int VROW = 32 + 4;
    constexpr int K_CHUNKS = 32 * CPR, V_CHUNKS = 4 * D;
    constexpr int K_PER = (K_CHUNKS + THREADS - 1) / THREADS, V_PER = (V_CHUNKS + THREADS - 1) / THREADS;
    __shared__ __attribute__((aligned(16))) bf16_t k_lds[2][32 * KROW];
    __shared__ __attribute__((aligned(16))) bf16_t v_lds[2][D * VROW];
    const int tid = threadIdx.x;
    bf16x8_t k_stage[K_PER], v_stage[V_PER];
    // Which half of the tile (16 keys of one page) and which 16 bytes of it a thread fetches
    // never changes: the byte offsets inside the half are made once, and the half is the same
    // for all lanes of a wave (a half's chunks are a multiple of 64), so the address of
    // a load is a 64-bit scalar base (pages + page * bytes per page + head + first slot) plus
    // a fixed 32-bit lane offset: the form a global load takes as it is, with no vector
    // arithmetic, and with a handful of scalar instructions per tile.
    // (Bases are made from the kernel's own pointer arguments, not picked from an array of
    // pointers: those lose their address space, become flat loads, and flat loads are
    // counted with the LDS reads, so that every wait for an operand read would wait for them.)
    static_assert((16 * CPR) % 64 == 0 && (2 * D) % 64 == 0, "a half's chunks fill whole waves");
    constexpr bool K_HALF_KNOWN = (16 * CPR) % THREADS == 0;  // then (tid + j * THREADS) / (16 * CPR) is j's alone
    constexpr bool V_HALF_KNOWN = (2 * D) % THREADS == 0;
    int k_half[K_PER], v_half[V_PER];
    unsigned k_lane_byte[K_PER], v_lane_byte[V_PER];
#pragma unroll
    for (int j = 0; j < K_PER; ++j) {
      const int id = tid + j * THREADS;
      k_half[j] = K_HALF_KNOWN ? (j * THREADS) / (16 * CPR) : __builtin_amdgcn_readfirstlane(id / (16 * CPR));
      k_lane_byte[j] = (unsigned)(id % (16 * CPR)) * 16u;  // a half's 16 key rows are contiguous
    }
#pragma unroll
    for (int j = 0; j < V_PER; ++j) {
      const int id = tid + j * THREADS;
      v_half[j] = V_HALF_KNOWN ? (j * THREADS) / (2 * D) : __builtin_amdgcn_readfirstlane(id / (2 * D));
      const int dim = (id % (2 * D)) / 2, part = id % 2;
      v_lane_byte[j] = (unsigned)(dim * page_size + part * 8) * 2u;
    }
    const unsigned page_bytes = (unsigned)page_stride * 2u;
    const char* const k_head = reinterpret_cast<const char*>(k_pages + head_off);
    const char* const v_head = reinterpret_cast<const char*>(vt_pages + head_off);
    auto request_tile = [&](int kb, const PageIds& ids) {
      uint64_t k_base[2], v_base[2];
#pragma unroll
      for (int hlf = 0; hlf < 2; ++hlf) {
        const int key0 = kb + 16 * hlf;
        const unsigned page = (unsigned)max(ids.page[hlf], 0);
        // (tiles start at multiples of 32 keys: with pages of 16 a half is a whole page)
        const unsigned slot0 = PS == 16 ? 0u : (unsigned)(key0 - page_index(key0) * page_size);
        const uint64_t chunk = (uint64_t)page * page_bytes;
        k_base[hlf] = reinterpret_cast<uint64_t>(k_head) + chunk + slot0 * (unsigned)(D * 2);
        v_base[hlf] = reinterpret_cast<uint64_t>(v_head) + chunk + slot0 * 2u;
        // (kept in scalar registers as they are: otherwise the lane offset is added to the
        // heads once and the page product is redone per load on the vector pipe, in 64 bits)
        asm("" : "+s"(k_base[hlf]));
        asm("" : "+s"(v_base[hlf]));
      }
      using global_bytes = const __attribute__((address_space(1))) char;
      using global_chunk = const __attribute__((address_space(1))) bf16x8_t;
#pragma unroll
      for (int j = 0; j < K_PER; ++j) {
        if (K_CHUNKS % THREADS == 0 || tid + j * THREADS < K_CHUNKS) {
          global_bytes* base = reinterpret_cast<global_bytes*>(k_half[j] ? k_base[1] : k_base[0]);
          k_stage[j] = *reinterpret_cast<global_chunk*>(base + k_lane_byte[j]);
        }
      }
#pragma unroll
      for (int j = 0; j < V_PER; ++j) {
        if (V_CHUNKS % THREADS == 0 || tid + j * THREADS < V_CHUNKS) {
          global_bytes* base = reinterpret_cast<global_bytes*>(v_half[j] ? v_base[1] : v_base[0]);
          v_stage[j] = *reinterpret_cast<global_chunk*>(base + v_lane_byte[j]);
        }
      }
    };
    auto store_tile = [&](int buf) {
#pragma unroll
      for (int j = 0; j < K_PER; ++j) {
        const int id = tid + j * THREADS;
        if (K_CHUNKS % THREADS == 0 || id < K_CHUNKS) {
          const int key = id / CPR, part = id % CPR;
          *reinterpret_cast<bf16x8_t*>(&k_lds[buf][key * KROW + part * 8]) = k_stage[j];
        }
      }
#pragma unroll
      for (int j = 0; j < V_PER; ++j) {
        const int id = tid + j * THREADS;
        if (V_CHUNKS % THREADS == 0 || id < V_CHUNKS) {
          const int hlf = id / (2 * D), dim = (id % (2 * D)) / 2, part = id % 2;
          bf16x4_t lo, hi;  // rows are 8-byte aligned only: two 8-byte stores
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            lo[i] = v_stage[j][i];
            hi[i] = v_stage[j][4 + i];
          }
          bf16_t* dst = &v_lds[buf][dim * VROW + hlf * 16 + part * 8];
          *reinterpret_cast<bf16x4_t*>(dst) = lo;
          *reinterpret_cast<bf16x4_t*>(dst + 4) = hi;
        }
      }
    };
    auto read_operands = [&](int buf, KVBlock& blk, bf16x8_t* v) {
#pragma unroll
      for (int hlf = 0; hlf < 2; ++hlf)
#pragma unroll
        for (int s = 0; s < KSTEPS; ++s)
          blk.k[hlf][s] = *reinterpret_cast<const bf16x8_t*>(&k_lds[buf][(16 * hlf + col) * KROW + quad * 8 + s * 32]);
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) {
        const bf16_t* src = &v_lds[buf][(db * 16 + col) * VROW + 4 * quad];
        const bf16x4_t v0 = *reinterpret_cast<const bf16x4_t*>(src);
        const bf16x4_t v1 = *reinterpret_cast<const bf16x4_t*>(src + 16);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          v[db][i] = v0[i];
          v[db][4 + i] = v1[i];
        }
      }
    };
    KVBlock blk;
    int kb = (k_begin / 32) * 32;
    if (kb < k_end) {  // the same for every wave of the block
      const int kb_last = kb + (k_end - 1 - kb) / 32 * 32;
      request_tile(kb, fetch_pages(kb));
      PageIds ids_next = fetch_pages(min(kb + 32, kb_last));
      store_tile(0);
      __syncthreads();
      int buf = 0;
      bf16x8_t v_now[DBLOCKS];
      bf16x8_t p_reg[RG];
      float alpha[RG];
      bool more = true;
      // Two loops in each other: the inner one runs while no row's reference point moves and
      // touches the accumulator with matrix instructions only, so the compiler keeps it in
      // place; a block that moves a reference leaves the inner loop, has the accumulator
      // rescaled out here, and the inner loop is entered again.
      while (more) {
        bool moved = false;
        while (true) {
          request_tile(min(kb + 32, kb_last), ids_next);  // past the end: re-reads the last tile
          ids_next = fetch_pages(min(kb + 64, kb_last));
          read_operands(buf, blk, v_now);
          f32x4_t s_acc[RG][2];
          block_scores(blk, s_acc);
          moved = block_softmax(kb, s_acc, p_reg, alpha);
          if (moved) break;
          block_values(v_now, p_reg);
          store_tile(buf ^ 1);
          __syncthreads();
          buf ^= 1;
          kb += 32;
          if (kb >= k_end) {
            more = false;
            break;
          }
        }
        if (moved) {
          rescale(alpha);
          block_values(v_now, p_reg);
          store_tile(buf ^ 1);
          __syncthreads();
          buf ^= 1;
          kb += 32;
          more = kb < k_end;
        }
      }
    }
  } else {
    // The prefetch is unconditional (past the end it re-reads this wave's last block),
    // so the compiler can count outstanding loads exactly instead of draining them all.
    KVBlock blk_a, blk_b;
    int kb = (k_begin / 32) * 32 + 32 * key_wave;
    if (kb < k_end) {
      const int kb_last = kb + (k_end - 1 - kb) / STEP * STEP;
      load_block(kb, fetch_pages(kb), blk_a);
      PageIds ids_next = fetch_pages(min(kb + STEP, kb_last));
      while (true) {
        load_block(min(kb + STEP, kb_last), ids_next, blk_b);
        ids_next = fetch_pages(min(kb + 2 * STEP, kb_last));
        __builtin_amdgcn_sched_barrier(0);
        compute_block(kb, blk_a);
        __builtin_amdgcn_sched_barrier(0);
        kb += STEP;
        if (kb >= k_end) break;
        load_block(min(kb + STEP, kb_last), ids_next, blk_a);
        ids_next = fetch_pages(min(kb + 2 * STEP, kb_last));
        __builtin_amdgcn_sched_barrier(0);
        compute_block(kb, blk_b);
        __builtin_amdgcn_sched_barrier(0);
        kb += STEP;
        if (kb >= k_end) break;
      }
    }
  }

  // ---- waves that shared the rows merge their (max, sum, accumulator) in a fixed order ----
  if (KW > 1) {
    __shared__ float merge_o[KW > 1 ? KW - 1 : 1][RG * DBLOCKS * 4][MI_WAVE];
    __shared__ float merge_ml[KW > 1 ? KW - 1 : 1][RG * 2][MI_WAVE];
    if (key_wave > 0) {
#pragma unroll
      for (int rg = 0; rg < RG; ++rg) {
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
          for (int r = 0; r < 4; ++r) merge_o[key_wave - 1][(rg * DBLOCKS + db) * 4 + r][lane] = o_acc[rg][db][r];
        merge_ml[key_wave - 1][rg * 2][lane] = m_run[rg];
        merge_ml[key_wave - 1][rg * 2 + 1][lane] = l_run[rg];
      }
    }
    __syncthreads();
    if (key_wave > 0) return;
    for (int other = 0; other < KW - 1; ++other) {
#pragma unroll
      for (int rg = 0; rg < RG; ++rg) {
        const float m_o = merge_ml[other][rg * 2][lane];
        const float l_o = merge_ml[other][rg * 2 + 1][lane];
        const float m_new = fmaxf(m_run[rg], m_o);
        const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
        const float a = exp2f(m_run[rg] - m_safe), b = exp2f(m_o - m_safe);
#pragma unroll
        for (int db = 0; db < DBLOCKS; ++db)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            o_acc[rg][db][r] = o_acc[rg][db][r] * a + merge_o[other][(rg * DBLOCKS + db) * 4 + r][lane] * b;
        l_run[rg] = l_run[rg] * a + l_o * b;
        m_run[rg] = m_new;
      }
    }
  }

  // ---- write: lane holds O^T[dim = 16*db + 4*quad + r][its row] ------------------------
#pragma unroll
  for (int rg = 0; rg < RG; ++rg) {
    if (!row_valid[rg]) continue;
    if constexpr (SUM_ON_MATRIX_PIPE) {
      // the four values are equal; 4x/4 is exact, and reading all four leaves no dead
      // lane in a register tuple that lives across the key loop
      const f32x4_t s4 = o_acc[rg][ACC_BLOCKS - 1];
      l_run[rg] = 0.25f * ((s4[0] + s4[1]) + (s4[2] + s4[3]));
    }
    if (num_splits == 1) {
      const float inv = 1.f / l_run[rg];
      bf16_t* o = out + (int64_t)token[rg] * out_row_stride + (int64_t)head[rg] * D + quad * 4;
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) {
        bf16x4_t packed;
#pragma unroll
        for (int r = 0; r < 4; ++r) packed[r] = (bf16_t)(o_acc[rg][db][r] * inv);
        *reinterpret_cast<bf16x4_t*>(o + db * 16) = packed;
      }
    } else {
      const int64_t slot = ((int64_t)token[rg] * q_heads + head[rg]) * num_splits + split;
      float* pa = part_acc + slot * D + quad * 4;
#pragma unroll
      for (int db = 0; db < DBLOCKS; ++db) {
        *reinterpret_cast<f32x4_t*>(pa + db * 16) = o_acc[rg][db];
      }
      if (quad == 0) {
        part_ml[slot * 2] = m_run[rg] * LN2;  // natural-log units, as the combining kernel expects
        part_ml[slot * 2 + 1] = l_run[rg];
      }
    }
  }
}

extern "C" int mi_attn_reduce_bf16(const float* part_acc, const float* part_ml, void* out,
                                   int64_t out_row_stride, int num_tokens, int q_heads,
                                   int head_dim, int num_splits, hipStream_t stream);

static int heads_per_block_for(int group, int rows) { return group < rows ? group : rows; }

// Tiling the Python side needs to size the grid: tokens per tile for a group size.
#define MI_DECODE_KW 4  // waves that share a decode block's rows, each taking every KW-th key block
// prefill blocks per CU: two where a wave's state fits 256 registers without spilling
#define MI_PREFILL_OCC(DD) ((DD) <= 128 ? 2 : 1)
#define MI_PREFILL_WAVES 4  // waves per block in the prefill shape
#define MI_PREFILL_RG 2  // row groups (of 16 rows) per wave in the prefill shape
#define MI_PREFILL_ROWS (16 * MI_PREFILL_WAVES * MI_PREFILL_RG)
// The shape of a launch: prefill (128 rows a block, two blocks a CU), decode (16 rows, waves
// split the keys), or wide prefill (8 waves, 256 rows a block, one block a CU: every key and
// value tile is fetched half as often; measured on one prompt of 8,192 / 32,768 / 131,072
// tokens 666-679 us / 8.17 ms / 130 ms against 715 us / 8.75 ms / 140 ms, but 73 against 61 us
// for 2,048 tokens, whose 256 blocks of unequal length fill the GPU badly; the caller chooses).
#define MI_SHAPE_PREFILL 0
#define MI_SHAPE_DECODE 1
#define MI_SHAPE_PREFILL_WIDE 2
#define MI_WIDE_WAVES 8
static int rows_of_shape(int shape) {
  return shape == MI_SHAPE_DECODE ? 16 : shape == MI_SHAPE_PREFILL_WIDE ? 16 * MI_WIDE_WAVES * MI_PREFILL_RG : MI_PREFILL_ROWS;
}

extern "C" int mi_attn_mfma_tokens_per_tile(int q_heads, int kv_heads, int shape) {
  if (q_heads <= 0 || kv_heads <= 0 || q_heads % kv_heads != 0) return 0;
  const int rows = rows_of_shape(shape);
  const int hb = heads_per_block_for(q_heads / kv_heads, rows);
  const int t = rows / hb;
  return t < 1 ? 1 : t;
}

extern "C" int mi_attn_mfma_supported(int head_dim, int page_size) {
  const bool d_ok = head_dim == 32 || head_dim == 64 || head_dim == 96 || head_dim == 128 ||
                    head_dim == 192 || head_dim == 256;
  return (d_ok && page_size > 0 && page_size % 16 == 0) ? 1 : 0;
}

// `num_tiles` = sum over requests of ceil(q_len / tokens_per_tile), computed by the
// caller from the host copy of cu_seqlens_q (a larger number is harmless).
// `one_tile_per_request` = 1 promises that no request has more than tokens_per_tile
// tokens in this step, 2 that every request has exactly one (then cu_seqlens_q is not
// read); in both cases num_tiles must be num_requests.
// The requests may be a run out of a larger step: cu_seqlens_q and block_table then point
// at the run's first request, while q, out, positions and the partial buffers stay
// those of the whole step (cu_seqlens_q holds token numbers of the whole step);
// `first_token` is the run's first token and `num_tokens` the run's token count.
// With num_splits > 1, part_acc holds (first_token+num_tokens)*q_heads*num_splits*head_dim
// floats and part_ml (first_token+num_tokens)*q_heads*num_splits*2; `combine` = 0 leaves the
// key ranges' results there for the caller's next kernel to combine (`out` is not written).
extern "C" int mi_attn_mfma(const void* q, int64_t q_row_stride, const void* k_pages,
                            const void* vt_pages, const int* block_table, int max_blocks,
                            const int* cu_seqlens_q, const int* positions, int num_requests,
                            int num_tokens, int num_tiles, void* out, int64_t out_row_stride,
                            float* part_acc, float* part_ml, int q_heads, int kv_heads,
                            int head_dim, int page_size, int num_pages, float scale, int window,
                            int num_splits, int shape, int one_tile_per_request,
                            int first_token, int combine, hipStream_t stream) {
  MI_REQUIRE(first_token >= 0, "attn_mfma: first_token=%d is negative", first_token);
  MI_REQUIRE(num_tokens >= 0 && num_requests >= 0 && num_tiles >= 0,
             "attn_mfma: bad sizes tokens=%d requests=%d tiles=%d", num_tokens, num_requests, num_tiles);
  MI_REQUIRE(q_heads > 0 && kv_heads > 0 && q_heads % kv_heads == 0,
             "attn_mfma: q_heads=%d is not a multiple of kv_heads=%d", q_heads, kv_heads);
  MI_REQUIRE(mi_attn_mfma_supported(head_dim, page_size),
             "attn_mfma: head_dim=%d (32, 64, 96, 128, 192 or 256) or page_size=%d (multiple of 16) not taken",
             head_dim, page_size);
  MI_REQUIRE(num_pages > 0 && max_blocks > 0, "attn_mfma: bad page counts num_pages=%d max_blocks=%d",
             num_pages, max_blocks);
  MI_REQUIRE((uintptr_t)k_pages % 128 == 0 && (uintptr_t)vt_pages % 128 == 0,
             "attn_mfma: the pages must begin on a 128-byte boundary (they are read in whole cache lines)");
  MI_REQUIRE(window >= 0, "attn_mfma: window=%d must be 0 (none) or positive", window);
  MI_REQUIRE(scale > 0.f, "attn_mfma: the score scale must be positive, got %g", (double)scale);
  MI_REQUIRE(num_splits >= 1 && num_splits <= 64, "attn_mfma: num_splits=%d must be 1..64", num_splits);
  MI_REQUIRE(num_splits == 1 || (part_acc && part_ml), "attn_mfma: split keys need partial buffers");
  MI_REQUIRE(q_row_stride >= (int64_t)q_heads * head_dim && out_row_stride >= (int64_t)q_heads * head_dim,
             "attn_mfma: row strides shorter than q_heads*head_dim");
  MI_REQUIRE(q_row_stride % 8 == 0 && out_row_stride % 4 == 0,
             "attn_mfma: row strides must keep 16-byte (q) and 8-byte (out) alignment");
  MI_REQUIRE(one_tile_per_request >= 0 && one_tile_per_request <= 2, "attn_mfma: one_tile_per_request is 0, 1 or 2");
  MI_REQUIRE(one_tile_per_request != 2 || num_tokens == num_requests,
             "attn_mfma: one token per request needs num_tokens == num_requests");
  MI_REQUIRE(!one_tile_per_request || num_tiles == num_requests,
             "attn_mfma: one tile per request needs num_tiles == num_requests");
  if (num_tokens == 0 || num_tiles == 0) return MI_OK;

  MI_REQUIRE(shape == MI_SHAPE_PREFILL || shape == MI_SHAPE_DECODE || (shape == MI_SHAPE_PREFILL_WIDE && head_dim <= 128),
             "attn_mfma: shape %d (0 prefill, 1 decode, 2 wide prefill for head sizes up to 128)", shape);
  const bool decode_only = shape == MI_SHAPE_DECODE;
  const int group = q_heads / kv_heads;
  const int rows = rows_of_shape(shape);
  const int hb = heads_per_block_for(group, rows);
  const int tq = mi_attn_mfma_tokens_per_tile(q_heads, kv_heads, shape);
  const int head_blocks = ceil_div(group, hb);
  MI_REQUIRE((int64_t)num_tiles * kv_heads * head_blocks < (1ll << 31), "attn_mfma: too many tiles x heads");
  MI_REQUIRE(num_splits <= 65535, "attn_mfma: too many splits");
  dim3 grid((unsigned)(num_tiles * kv_heads * head_blocks), 1, num_splits);
  const float scale_log2 = scale * LOG2E;
  // prefill blocks run two to a CU: see the tile order in the kernel (8 XCDs share the CUs evenly)
  int pair_group = 0;
  if (shape == MI_SHAPE_PREFILL && MI_PREFILL_OCC(head_dim) == 2) {
    int device = 0, cus = 0;
    if (hipGetDevice(&device) == hipSuccess &&
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) == hipSuccess)
      pair_group = cus / 8;
  }
  // keys reach max_blocks*page_size + 32 at most; the multiply-high division is exact below 2^32/page_size
  MI_REQUIRE(((int64_t)max_blocks * page_size + 64) * page_size < (1ll << 32),
             "attn_mfma: block table of %d pages of %d is too long for this kernel", max_blocks, page_size);
  const unsigned page_magic = (unsigned)((1ull << 32) / (unsigned)page_size) + 1u;

#define MI_LAUNCH(DD, WW, KK, RR, OO, SS, PP)                                                 \
  attn_mfma_kernel<DD, WW, KK, RR, OO, SS, PP><<<grid, 64 * WW * KK, 0, stream>>>(                    \
      (const bf16_t*)q, q_row_stride, (const bf16_t*)k_pages, (const bf16_t*)vt_pages,            \
      block_table, max_blocks, cu_seqlens_q, positions, num_requests, (bf16_t*)out,               \
      out_row_stride, part_acc, part_ml, q_heads, kv_heads, page_size, page_magic, scale_log2,    \
      window,                                                                                     \
      num_splits, hb, tq, one_tile_per_request, pair_group, first_token)
// (head sizes above 128 have no wide shape and were refused above: their cases name the 128 kernel,
// so that nothing is compiled for them)
#define MI_LAUNCH_P(DD, PP)                                                                       \
  if (decode_only) MI_LAUNCH(DD, 1, MI_DECODE_KW, 1, 2, false, PP);                               \
  else if (shape == MI_SHAPE_PREFILL_WIDE) MI_LAUNCH((DD <= 128 ? DD : 128), MI_WIDE_WAVES, 1, MI_PREFILL_RG, 2, true, PP); \
  else MI_LAUNCH(DD, MI_PREFILL_WAVES, 1, MI_PREFILL_RG, MI_PREFILL_OCC(DD), true, PP)
#define MI_LAUNCH_D(DD)                 \
  if (page_size == 16) {                \
    MI_LAUNCH_P(DD, 16);                \
  } else {                              \
    MI_LAUNCH_P(DD, 0);                 \
  }
  switch (head_dim) {
    case 32: MI_LAUNCH_D(32); break;
    case 64: MI_LAUNCH_D(64); break;
    case 96: MI_LAUNCH_D(96); break;
    case 128: MI_LAUNCH_D(128); break;
    case 192: MI_LAUNCH_D(192); break;
    default: MI_LAUNCH_D(256); break;
  }
#undef MI_LAUNCH_D
#undef MI_LAUNCH_P
#undef MI_LAUNCH
  MI_CHECK_LAUNCH("attn_mfma");
  if (num_splits > 1 && combine) {
    const int64_t first_slot = (int64_t)first_token * q_heads * num_splits;
    return mi_attn_reduce_bf16(part_acc + first_slot * head_dim, part_ml + first_slot * 2,
                               (bf16_t*)out + (int64_t)first_token * out_row_stride, out_row_stride,
                               num_tokens, q_heads, head_dim, num_splits, stream);
  }
  return MI_OK;
}
