// Next-token choice on the device: one 1024-thread block per row of logits.
//
// Meaning of the options follows the reference (engine/sampler.py:24-110):
//   temperature 0      first index of the maximum
//   temperature > 0    logits / temperature, then
//   top_k in (0, V)    values below the k-th largest value are dropped (ties stay)
//   top_p < 1          a token is dropped when the probability mass of the tokens
//                      above it exceeds top_p (the boundary token stays)
//   draw               argmax of p_i / q_i with q_i ~ Exp(1), here in log form
//                      x_i - log(q_i)
// Unlike the reference's global generator, the random numbers come from a
// counter-based generator (Philox 4x32-10) keyed by the request's seed and the
// index of the draw, so a request's tokens do not depend on what else is in the
// batch.  Thresholds are found without sorting, by descending over the bytes of
// an order-preserving integer image of the values; probability mass is summed in
// 64-bit fixed point so the result does not depend on the order of the sum.
#include "common.h"

#include <math.h>

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / MI_WAVE)
#define SAMPLE_BATCH 16  // loads a thread has in flight
#define MASS_ONE 1099511627776.0f  // 2^40

// A request's row in the table of state slots (int32 words), as the cache manager lays it out.
#define SLOT_WORDS 8
#define SLOT_POSITION 0
#define SLOT_SEED_LO 1
#define SLOT_SEED_HI 2
#define SLOT_DRAW 3
#define SLOT_TEMPERATURE 4  // float bits
#define SLOT_TOP_K 5
#define SLOT_TOP_P 6  // float bits

__device__ __forceinline__ uint32_t order_key(float x) {
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ void philox4x32_10(uint32_t c[4], uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c[0];
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c[2];
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c[1] ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c[3] ^ k1;
    const uint32_t n3 = (uint32_t)p0;
    c[0] = n0; c[1] = n1; c[2] = n2; c[3] = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
}

// -log(-log(u)) for u uniform in (0, 1), from 24 random bits
__device__ __forceinline__ float gumbel_from_bits(uint32_t bits) {
  const float u = ((float)(bits >> 8) + 0.5f) * (1.0f / 16777216.0f);
  return -logf(-logf(u));
}

struct ArgBest {
  float val;
  int idx;
};

__device__ __forceinline__ ArgBest better(ArgBest a, ArgBest b) {
  // larger value wins; equal values: smaller index wins
  if (b.val > a.val || (b.val == a.val && b.idx < a.idx)) return b;
  return a;
}

__device__ ArgBest block_argbest(ArgBest mine, ArgBest* scratch) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) {
    ArgBest other;
    other.val = __shfl_xor(mine.val, off, MI_WAVE);
    other.idx = __shfl_xor(mine.idx, off, MI_WAVE);
    mine = better(mine, other);
  }
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = mine;
  __syncthreads();
  ArgBest best = scratch[0];
  for (int w = 1; w < SAMPLE_WAVES; ++w) best = better(best, scratch[w]);
  return best;
}

// Calls fn(i, x[i]) for this thread's elements i = tid, tid + THREADS, ... in rising order.
// The elements are read in batches of independent loads: a loop with one load per turn
// costs a memory latency per element.
template <typename T, typename F>
__device__ __forceinline__ void scan_row(const T* __restrict__ x, int vocab, int tid, F&& fn) {
  for (int i0 = tid; i0 < vocab; i0 += SAMPLE_THREADS * SAMPLE_BATCH) {
    float v[SAMPLE_BATCH];
#pragma unroll
    for (int u = 0; u < SAMPLE_BATCH; ++u) {
      const int i = i0 + u * SAMPLE_THREADS;
      v[u] = (i < vocab) ? to_f32(x[i]) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < SAMPLE_BATCH; ++u) {
      const int i = i0 + u * SAMPLE_THREADS;
      if (i < vocab) fn(i, v[u]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const T* __restrict__ logits, int64_t row_stride, int vocab,
    const float* __restrict__ temperature, const int* __restrict__ top_k,
    const float* __restrict__ top_p, const uint32_t* __restrict__ seed_lo,
    const uint32_t* __restrict__ seed_hi, const uint32_t* __restrict__ draw_index,
    int* __restrict__ out, const int* __restrict__ slots, int* __restrict__ slot_table, int num_slots) {
  __shared__ ArgBest best_scratch[SAMPLE_WAVES];
  __shared__ uint32_t cnt[256];
  __shared__ unsigned long long mass[256];
  __shared__ uint32_t sh_prefix;
  __shared__ unsigned long long sh_above;
  __shared__ unsigned long long sh_limit;

  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const T* x = logits + (int64_t)row * row_stride;
  // the row's settings: from the request's state slot, or from one array per setting
  // (a slot id outside the table, such as the -1 of a padding row, belongs to no request: the
  // row is sampled greedily and nothing is written back)
  const bool by_slot = slot_table != nullptr;
  const int slot_id = by_slot ? slots[row] : -1;
  int* slot = (by_slot && slot_id >= 0 && slot_id < num_slots) ? slot_table + (int64_t)slot_id * SLOT_WORDS : nullptr;
  const float temp = slot ? __int_as_float(slot[SLOT_TEMPERATURE]) : (by_slot ? 0.f : temperature[row]);
  const int k = slot ? slot[SLOT_TOP_K] : (by_slot ? 0 : top_k[row]);
  const float p = slot ? __int_as_float(slot[SLOT_TOP_P]) : (by_slot ? 1.f : top_p[row]);
  const uint32_t k0 = slot ? (uint32_t)slot[SLOT_SEED_LO] : (by_slot ? 0u : seed_lo[row]);
  const uint32_t k1 = slot ? (uint32_t)slot[SLOT_SEED_HI] : (by_slot ? 0u : seed_hi[row]);
  const uint32_t draw = slot ? (uint32_t)slot[SLOT_DRAW] : (by_slot ? 0u : draw_index[row]);
  // every thread has read the draw index before thread 0 may advance it at the end
  __syncthreads();

  if (temp == 0.f) {
    ArgBest mine = {-INFINITY, 0x7fffffff};  // rising index order: ties go to the first
    scan_row(x, vocab, tid, [&](int i, float v) {
      if (v > mine.val || mine.idx == 0x7fffffff) { mine.val = v; mine.idx = i; }
    });
    const ArgBest best = block_argbest(mine, best_scratch);
    if (tid == 0) {
      out[row] = best.idx;
      if (slot) slot[SLOT_DRAW] = (int)(draw + 1u);
    }
    return;
  }

  // maximum of the scaled logits
  ArgBest top = {-INFINITY, 0x7fffffff};
  scan_row(x, vocab, tid, [&](int i, float raw) {
    const float v = raw / temp;
    if (v > top.val) { top.val = v; top.idx = i; }
  });
  const float v_max = block_argbest(top, best_scratch).val;

  uint32_t key_floor = 0;  // tokens whose key is below this are dropped

  // ---- top-k: the key of the k-th largest value ---------------------------
  if (k > 0 && k < vocab) {
    uint32_t prefix = 0, mask = 0;
    uint32_t remaining = (uint32_t)k;
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      if (tid < 256) cnt[tid] = 0;
      __syncthreads();
      int run_bin = -1;
      uint32_t run_cnt = 0;
      scan_row(x, vocab, tid, [&](int, float raw) {
        const uint32_t key = order_key(raw / temp);
        if ((key & mask) != prefix) return;
        const int bin = (key >> shift) & 255;
        if (bin != run_bin) {
          if (run_cnt) atomicAdd(&cnt[run_bin], run_cnt);
          run_bin = bin;
          run_cnt = 0;
        }
        ++run_cnt;
      });
      if (run_cnt) atomicAdd(&cnt[run_bin], run_cnt);
      __syncthreads();
      if (tid == 0) {
        int bin = 255;
        for (; bin > 0; --bin) {
          if (remaining <= cnt[bin]) break;
          remaining -= cnt[bin];
        }
        sh_prefix = prefix | ((uint32_t)bin << shift);
        sh_above = remaining;
      }
      __syncthreads();
      prefix = sh_prefix;
      remaining = (uint32_t)sh_above;
      mask |= 255u << shift;
      __syncthreads();
    }
    key_floor = prefix;
  }

  // ---- top-p: the smallest key whose mass-above is within top_p ------------
  if (p < 1.f) {
    uint32_t prefix = 0, mask = 0;
    unsigned long long above = 0;
    for (int pass = 0; pass < 4; ++pass) {
      const int shift = 24 - 8 * pass;
      if (tid < 256) { cnt[tid] = 0; mass[tid] = 0; }
      __syncthreads();
      int run_bin = -1;
      uint32_t run_cnt = 0;
      unsigned long long run_mass = 0;
      scan_row(x, vocab, tid, [&](int, float raw) {
        const float v = raw / temp;
        const uint32_t key = order_key(v);
        if (key < key_floor || (key & mask) != prefix) return;
        const int bin = (key >> shift) & 255;
        if (bin != run_bin) {
          if (run_cnt) { atomicAdd(&cnt[run_bin], run_cnt); atomicAdd(&mass[run_bin], run_mass); }
          run_bin = bin;
          run_cnt = 0;
          run_mass = 0;
        }
        ++run_cnt;
        run_mass += (unsigned long long)(expf(v - v_max) * MASS_ONE);
      });
      if (run_cnt) { atomicAdd(&cnt[run_bin], run_cnt); atomicAdd(&mass[run_bin], run_mass); }
      __syncthreads();
      if (tid == 0) {
        if (pass == 0) {
          unsigned long long total = 0;
          for (int b = 0; b < 256; ++b) total += mass[b];
          sh_limit = (unsigned long long)((double)p * (double)total);
        }
        const unsigned long long limit = sh_limit;
        unsigned long long run = above, chosen_above = above;
        int chosen = -1;
        for (int b = 255; b >= 0; --b) {
          if (cnt[b] > 0) {
            if (run <= limit || chosen < 0) { chosen = b; chosen_above = run; }
            else break;
          }
          run += mass[b];
        }
        sh_prefix = prefix | ((uint32_t)chosen << shift);
        sh_above = chosen_above;
      }
      __syncthreads();
      prefix = sh_prefix;
      above = sh_above;
      mask |= 255u << shift;
      __syncthreads();
    }
    if (prefix > key_floor) key_floor = prefix;
  }

  // ---- draw -----------------------------------------------------------------
  ArgBest mine = {-INFINITY, 0x7fffffff};
  const int n_quads = (vocab + 3) / 4;
  constexpr int QUADS = 4;  // quads whose 16 loads are issued together
  for (int quad0 = tid; quad0 < n_quads; quad0 += SAMPLE_THREADS * QUADS) {
    float raw[QUADS][4];
#pragma unroll
    for (int u = 0; u < QUADS; ++u) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = (quad0 + u * SAMPLE_THREADS) * 4 + e;
        raw[u][e] = (i < vocab) ? to_f32(x[i]) : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < QUADS; ++u) {
      const int quad = quad0 + u * SAMPLE_THREADS;
      if (quad >= n_quads) break;
      uint32_t c[4] = {(uint32_t)quad, draw, 0u, 0u};
      philox4x32_10(c, k0, k1);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = quad * 4 + e;
        if (i >= vocab) break;
        const float v = raw[u][e] / temp;
        if (order_key(v) < key_floor) continue;
        const float score = v + gumbel_from_bits(c[e]);
        if (score > mine.val || mine.idx == 0x7fffffff) { mine.val = score; mine.idx = i; }
      }
    }
  }
  const ArgBest best = block_argbest(mine, best_scratch);
  if (tid == 0) {
    out[row] = best.idx;
    if (slot) slot[SLOT_DRAW] = (int)(draw + 1u);
  }
}

extern "C" int mi_sample(int dtype, const void* logits, int64_t row_stride, int num_rows, int vocab,
                         const float* temperature, const int* top_k, const float* top_p,
                         const uint32_t* seed_lo, const uint32_t* seed_hi,
                         const uint32_t* draw_index, int* out, hipStream_t stream) {
  MI_REQUIRE(num_rows >= 0 && vocab > 0, "sample: bad sizes rows=%d vocab=%d", num_rows, vocab);
  MI_REQUIRE(row_stride >= vocab, "sample: row stride %lld is shorter than the vocabulary %d",
             (long long)row_stride, vocab);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "sample: unknown dtype %d", dtype);
  if (num_rows == 0) return MI_OK;
  if (dtype == MI_F32) {
    sample_kernel<float><<<num_rows, SAMPLE_THREADS, 0, stream>>>(
        (const float*)logits, row_stride, vocab, temperature, top_k, top_p, seed_lo, seed_hi,
        draw_index, out, nullptr, nullptr, 0);
  } else {
    sample_kernel<bf16_t><<<num_rows, SAMPLE_THREADS, 0, stream>>>(
        (const bf16_t*)logits, row_stride, vocab, temperature, top_k, top_p, seed_lo, seed_hi,
        draw_index, out, nullptr, nullptr, 0);
  }
  MI_CHECK_LAUNCH("sample");
  return MI_OK;
}

// The same choice with every row's settings read from its request's state slot:
// `slots[row]` indexes `slot_table` [num_slots][8] (position, seed low, seed high, draw
// index, temperature bits, top_k, top_p bits, unused).  The draw index of each sampled
// slot is advanced by one, so the next call draws the request's next number without
// the host sending anything.  A request appears in at most one row.  A slot id outside
// 0..num_slots-1 (the -1 of a padding row) is sampled greedily and nothing is written for it.
extern "C" int mi_sample_slots(int dtype, const void* logits, int64_t row_stride, int num_rows, int vocab,
                               const int* slots, int* slot_table, int num_slots, int* out, hipStream_t stream) {
  MI_REQUIRE(num_rows >= 0 && vocab > 0, "sample_slots: bad sizes rows=%d vocab=%d", num_rows, vocab);
  MI_REQUIRE(row_stride >= vocab, "sample_slots: row stride %lld is shorter than the vocabulary %d",
             (long long)row_stride, vocab);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "sample_slots: unknown dtype %d", dtype);
  MI_REQUIRE(slots && slot_table && num_slots > 0, "sample_slots: needs the slot ids and the slot table");
  if (num_rows == 0) return MI_OK;
  if (dtype == MI_F32) {
    sample_kernel<float><<<num_rows, SAMPLE_THREADS, 0, stream>>>(
        (const float*)logits, row_stride, vocab, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, out,
        slots, slot_table, num_slots);
  } else {
    sample_kernel<bf16_t><<<num_rows, SAMPLE_THREADS, 0, stream>>>(
        (const bf16_t*)logits, row_stride, vocab, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, out,
        slots, slot_table, num_slots);
  }
  MI_CHECK_LAUNCH("sample_slots");
  return MI_OK;
}
