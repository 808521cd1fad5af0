// Per-token kernels: embedding lookup, residual add + RMSNorm, rotation tables,
// rotary position encoding fused with the write of keys and values into cache
// pages, and SiLU(gate) * up.  Storage is float32 or bfloat16; arithmetic on bfloat16
// elements is float32, on float32 elements (the 32-bit path) the norm and the activation
// are evaluated in 64-bit and rounded once.  The residual stream is float32 in both modes.
//
// Formulas follow the reference (JonathanBerhe/mini-infer, src/mini_infer/):
//   RMSNorm           models/blocks/rmsnorm.py:81-93, rms_norm_kernel.py:98-144
//   rotation          models/blocks/rope.py:392-431, rope_write_kernel.py:119-152
//   SiLU * up         models/blocks/silu_mul_kernel.py:86-90
// but round once at the end instead of after every operation.
#include "common.h"

#include <math.h>

typedef bf16_t bf16x4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ void load4(const float* p, float v[4]) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
__device__ __forceinline__ void load4(const bf16_t* p, float v[4]) {
  const bf16x4_t x = *reinterpret_cast<const bf16x4_t*>(p);
  v[0] = (float)x[0]; v[1] = (float)x[1]; v[2] = (float)x[2]; v[3] = (float)x[3];
}
__device__ __forceinline__ void store4(float* p, const float v[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}
__device__ __forceinline__ void store4(bf16_t* p, const float v[4]) {
  bf16x4_t x;
  x[0] = (bf16_t)v[0]; x[1] = (bf16_t)v[1]; x[2] = (bf16_t)v[2]; x[3] = (bf16_t)v[3];
  *reinterpret_cast<bf16x4_t*>(p) = x;
}

// ---------------------------------------------------------------------------
// embedding: residual[t, :] = float(table[ids[t], :])
// ---------------------------------------------------------------------------

template <typename T, int VEC>
__global__ void embed_gather_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ residual, int hidden) {
  const int t = blockIdx.x;
  const T* row = table + (int64_t)ids[t] * hidden;
  float* out = residual + (int64_t)t * hidden;
  if (VEC == 4) {
    for (int i = threadIdx.x * 4; i < hidden; i += blockDim.x * 4) {
      float v[4];
      load4(row + i, v);
      store4(out + i, v);
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[i] = to_f32(row[i]);
  }
}

template <typename T>
static int embed_gather_launch(const void* table, const int* ids, float* residual, int num_tokens,
                               int hidden, hipStream_t stream) {
  if (num_tokens == 0) return MI_OK;
  if (hidden % 4 == 0) {
    embed_gather_kernel<T, 4><<<num_tokens, 256, 0, stream>>>((const T*)table, ids, residual, hidden);
  } else {
    embed_gather_kernel<T, 1><<<num_tokens, 256, 0, stream>>>((const T*)table, ids, residual, hidden);
  }
  MI_CHECK_LAUNCH("embed_gather");
  return MI_OK;
}

extern "C" int mi_embed_gather(int dtype, const void* table, const int* ids, float* residual,
                               int num_tokens, int hidden, int vocab, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && hidden > 0 && vocab > 0,
             "embed_gather: bad sizes tokens=%d hidden=%d vocab=%d", num_tokens, hidden, vocab);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "embed_gather: unknown dtype %d", dtype);
  if (dtype == MI_F32) return embed_gather_launch<float>(table, ids, residual, num_tokens, hidden, stream);
  return embed_gather_launch<bf16_t>(table, ids, residual, num_tokens, hidden, stream);
}

// ---------------------------------------------------------------------------
// Token ids that are still on the device: ids[i] = source[from_rows[i]] where
// from_rows[i] >= 0 (the token a previous step sampled, not yet read by the host), else
// ids[i] stays what the host sent.  Values are clamped into the vocabulary.
// ---------------------------------------------------------------------------

__global__ void take_device_tokens_kernel(int* __restrict__ ids, const int* __restrict__ from_rows,
                                          const int* __restrict__ source, int n, int source_len, int vocab) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int row = from_rows[i];
  if (row < 0) return;
  const int token = source[min(row, source_len - 1)];
  ids[i] = min(max(token, 0), vocab - 1);
}

extern "C" int mi_take_device_tokens(int* ids, const int* from_rows, const int* source, int n, int source_len,
                                     int vocab, hipStream_t stream) {
  MI_REQUIRE(n >= 0 && source_len >= 1 && vocab >= 1, "take_device_tokens: bad sizes n=%d source=%d vocab=%d", n,
             source_len, vocab);
  if (n == 0) return MI_OK;
  take_device_tokens_kernel<<<ceil_div(n, 256), 256, 0, stream>>>(ids, from_rows, source, n, source_len, vocab);
  MI_CHECK_LAUNCH("take_device_tokens");
  return MI_OK;
}

// ---------------------------------------------------------------------------
// The first kernel of a step: what `take_device_tokens` does (if `from_rows` is given), and
// the position word of every request's state slot set to the request's length after the
// step: slot_table[state_slots[b]][0] = seq_lens[b].  A negative slot (a padding row of a
// recorded step) is skipped.  Slot rows are 8 int32 words.
// ---------------------------------------------------------------------------

__global__ void begin_step_kernel(int* __restrict__ ids, const int* __restrict__ from_rows,
                                  const int* __restrict__ source, int n, int source_len, int vocab,
                                  int* __restrict__ slot_table, const int* __restrict__ state_slots,
                                  const int* __restrict__ seq_lens, int num_requests, int num_slots) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (from_rows != nullptr && i < n) {
    const int row = from_rows[i];
    if (row >= 0) {
      const int token = source[min(row, source_len - 1)];
      ids[i] = min(max(token, 0), vocab - 1);
    }
  }
  if (slot_table != nullptr && i < num_requests) {
    const int slot = state_slots[i];
    if (slot >= 0 && slot < num_slots) slot_table[(int64_t)slot * 8] = seq_lens[i];
  }
}

extern "C" int mi_begin_step(int* ids, const int* from_rows, const int* source, int n, int source_len, int vocab,
                             int* slot_table, const int* state_slots, const int* seq_lens, int num_requests,
                             int num_slots, hipStream_t stream) {
  MI_REQUIRE(n >= 0 && num_requests >= 0 && vocab >= 1, "begin_step: bad sizes n=%d requests=%d vocab=%d", n,
             num_requests, vocab);
  MI_REQUIRE(from_rows == nullptr || (source != nullptr && source_len >= 1 && ids != nullptr),
             "begin_step: tokens taken from the device need their source");
  MI_REQUIRE(slot_table == nullptr || (state_slots != nullptr && seq_lens != nullptr && num_slots >= 1),
             "begin_step: the slot table needs slot ids and lengths");
  const int work = max(from_rows ? n : 0, slot_table ? num_requests : 0);
  if (work == 0) return MI_OK;
  begin_step_kernel<<<ceil_div(work, 256), 256, 0, stream>>>(ids, from_rows, source, n, source_len, vocab,
                                                             slot_table, state_slots, seq_lens, num_requests,
                                                             num_slots);
  MI_CHECK_LAUNCH("begin_step");
  return MI_OK;
}

// ---------------------------------------------------------------------------
// residual add + RMSNorm
//   s = residual[r] + delta[r]           (float32; stored back unless `rows` is given)
//   out[b] = weight * s * rsqrt(mean(s^2) + eps)
// One block per output row; with `rows`, output row b reads input row rows[b].
// The delta may come in pieces: `partials` [num_partials][all rows][hidden] float32, the
// sums of a product over ranges of K (gemm_mid_bf16.hip); they are added in order and
// rounded to T, which gives the delta the product would have written itself.
// ---------------------------------------------------------------------------

// The norm of float32 elements (the 32-bit path) takes its statistics and scales in 64-bit and
// rounds each output once (in float32 throughout it measured 5.7e-8 from exact on average,
// against 2.5e-8 for the one rounding).  bfloat16 elements: float32, as said at the top.
template <typename T>
__device__ __forceinline__ float norm_scale(float weight, float value, float inv, double inv_wide) {
  if constexpr (sizeof(T) == 4) return (float)((double)weight * ((double)value * inv_wide));
  else return weight * (value * inv);
}

__device__ __forceinline__ double block_sum_wide(double v, double* scratch) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, MI_WAVE);
  const int wave = threadIdx.x / MI_WAVE, lane = threadIdx.x % MI_WAVE;
  const int n_waves = (blockDim.x + MI_WAVE - 1) / MI_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  double total = 0.0;
  for (int w = 0; w < n_waves; ++w) total += scratch[w];
  return total;
}

// rsqrt(sum / hidden + eps) from a thread's share of the sum of squares: both widths
template <typename T>
__device__ __forceinline__ void norm_factor(float squares, double squares_wide, int hidden, float eps,
                                            float* scratch, double* scratch_wide, float& inv, double& inv_wide) {
  if constexpr (sizeof(T) == 4) {
    inv_wide = 1.0 / sqrt(block_sum_wide(squares_wide, scratch_wide) / (double)hidden + (double)eps);
    inv = (float)inv_wide;
  } else {
    inv = rsqrtf(block_sum(squares, scratch) / (float)hidden + eps);
    inv_wide = 0.0;
  }
}

template <typename T, int VEC, bool PIECES>
__global__ __launch_bounds__(1024) void add_rmsnorm_kernel(
    const T* __restrict__ delta, float* __restrict__ residual, const T* __restrict__ weight,
    T* __restrict__ out, const int* __restrict__ rows, int hidden, float eps,
    const float* __restrict__ partials, int num_partials, int64_t partial_stride) {
  __shared__ float scratch[16];
  __shared__ double scratch_wide[16];
  constexpr bool WIDE = sizeof(T) == 4;
  const int b = blockIdx.x;
  const int64_t r = rows ? rows[b] : b;
  float* res = residual + r * hidden;
  const T* dl = delta ? delta + r * hidden : nullptr;
  const float* pt = PIECES ? partials + r * hidden : nullptr;
  T* o = out + (int64_t)b * hidden;
  const bool has_delta = PIECES || dl != nullptr;
  const bool store_sum = (rows == nullptr) && has_delta;
  // 4 consecutive values of the delta at i (VEC == 4 paths)
  auto delta4 = [&](int i, float* d) {
    if constexpr (PIECES) {
      float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
      for (int p = 0; p < num_partials; ++p) {  // the loads do not wait for one another
        float piece[4];
        load4(pt + (int64_t)p * partial_stride + i, piece);
#pragma unroll
        for (int k = 0; k < 4; ++k) sum[k] += piece[k];
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) d[k] = to_f32(from_f32<T>(sum[k]));
    } else {
      load4(dl + i, d);
    }
  };
  auto delta1 = [&](int i) -> float {
    if constexpr (PIECES) {
      float sum = 0.f;
#pragma unroll 8
      for (int p = 0; p < num_partials; ++p) sum += pt[(int64_t)p * partial_stride + i];
      return to_f32(from_f32<T>(sum));
    } else {
      return to_f32(dl[i]);
    }
  };

  if (VEC == 4 && hidden <= (int)blockDim.x * 4) {
    // the whole row is one vector per thread: it stays in registers between the two
    // passes (no second trip to memory), and the weight is requested before the
    // reduction instead of after it
    const int i = threadIdx.x * 4;
    const bool mine = i < hidden;
    float s[4] = {0.f, 0.f, 0.f, 0.f}, w[4] = {0.f, 0.f, 0.f, 0.f};
    if (mine) {
      load4(res + i, s);
      load4(weight + i, w);
      if (has_delta) {
        float d[4];
        delta4(i, d);
#pragma unroll
        for (int k = 0; k < 4; ++k) s[k] += d[k];
        if (store_sum) store4(res + i, s);
      }
    }
    float squares = 0.f;
    double squares_wide = 0.0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      if constexpr (WIDE) squares_wide += (double)s[k] * (double)s[k];
      else squares += s[k] * s[k];
    }
    float inv_one;
    double inv_one_wide;
    norm_factor<T>(squares, squares_wide, hidden, eps, scratch, scratch_wide, inv_one, inv_one_wide);
    if (mine) {
#pragma unroll
      for (int k = 0; k < 4; ++k) s[k] = norm_scale<T>(w[k], s[k], inv_one, inv_one_wide);
      store4(o + i, s);
    }
    return;
  }

  float sumsq = 0.f;
  double sumsq_wide = 0.0;
  if (VEC == 4) {
    for (int i = threadIdx.x * 4; i < hidden; i += blockDim.x * 4) {
      float s[4];
      load4(res + i, s);
      if (has_delta) {
        float d[4];
        delta4(i, d);
#pragma unroll
        for (int k = 0; k < 4; ++k) s[k] += d[k];
        if (store_sum) store4(res + i, s);
      }
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if constexpr (WIDE) sumsq_wide += (double)s[k] * (double)s[k];
        else sumsq += s[k] * s[k];
      }
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      float s = res[i];
      if (has_delta) {
        s += delta1(i);
        if (store_sum) res[i] = s;
      }
      if constexpr (WIDE) sumsq_wide += (double)s * (double)s;
      else sumsq += s * s;
    }
  }
  float inv;
  double inv_wide;
  norm_factor<T>(sumsq, sumsq_wide, hidden, eps, scratch, scratch_wide, inv, inv_wide);
  const bool re_add = has_delta && !store_sum;

  if (VEC == 4) {
    for (int i = threadIdx.x * 4; i < hidden; i += blockDim.x * 4) {
      float s[4], w[4];
      load4(res + i, s);
      if (re_add) {
        float d[4];
        delta4(i, d);
#pragma unroll
        for (int k = 0; k < 4; ++k) s[k] += d[k];
      }
      load4(weight + i, w);
#pragma unroll
      for (int k = 0; k < 4; ++k) s[k] = norm_scale<T>(w[k], s[k], inv, inv_wide);
      store4(o + i, s);
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      float s = res[i];
      if (re_add) s += delta1(i);
      o[i] = from_f32<T>(norm_scale<T>(to_f32(weight[i]), s, inv, inv_wide));
    }
  }
}

template <typename T>
static int add_rmsnorm_launch(const void* delta, float* residual, const void* weight, void* out,
                              const int* rows, int num_out_rows, int hidden, float eps,
                              const float* partials, int num_partials, int64_t partial_stride,
                              hipStream_t stream) {
  if (num_out_rows == 0) return MI_OK;
  if (hidden % 4 == 0) {
    // one vector of 4 per thread and pass where the row allows: fewer dependent steps
    const int threads = min(1024, max(256, ceil_div(hidden / 4, 64) * 64));
    if (partials)
      add_rmsnorm_kernel<T, 4, true><<<num_out_rows, threads, 0, stream>>>(
          (const T*)delta, residual, (const T*)weight, (T*)out, rows, hidden, eps, partials, num_partials,
          partial_stride);
    else
      add_rmsnorm_kernel<T, 4, false><<<num_out_rows, threads, 0, stream>>>(
          (const T*)delta, residual, (const T*)weight, (T*)out, rows, hidden, eps, nullptr, 0, 0);
  } else {
    if (partials)
      add_rmsnorm_kernel<T, 1, true><<<num_out_rows, 256, 0, stream>>>(
          (const T*)delta, residual, (const T*)weight, (T*)out, rows, hidden, eps, partials, num_partials,
          partial_stride);
    else
      add_rmsnorm_kernel<T, 1, false><<<num_out_rows, 256, 0, stream>>>(
          (const T*)delta, residual, (const T*)weight, (T*)out, rows, hidden, eps, nullptr, 0, 0);
  }
  MI_CHECK_LAUNCH("add_rmsnorm");
  return MI_OK;
}

// `delta` (element type) or `partials` (float32 [num_partials][all rows][hidden],
// `partial_stride` = all rows * hidden) or neither; never both.
extern "C" int mi_add_rmsnorm(int dtype, const void* delta, float* residual, const void* weight,
                              void* out, const int* rows, int num_out_rows, int hidden, float eps,
                              const float* partials, int num_partials, int64_t partial_stride,
                              hipStream_t stream) {
  MI_REQUIRE(num_out_rows >= 0 && hidden > 0, "add_rmsnorm: bad sizes rows=%d hidden=%d",
             num_out_rows, hidden);
  MI_REQUIRE(!(delta && partials), "add_rmsnorm: a delta or its partial sums, not both");
  MI_REQUIRE(!partials || (num_partials >= 1 && num_partials <= 16 && partial_stride >= hidden),
             "add_rmsnorm: bad partial sums count=%d stride=%lld", num_partials, (long long)partial_stride);
  MI_REQUIRE(eps > 0.f, "add_rmsnorm: eps must be positive, got %g", (double)eps);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "add_rmsnorm: unknown dtype %d", dtype);
  if (dtype == MI_F32)
    return add_rmsnorm_launch<float>(delta, residual, weight, out, rows, num_out_rows, hidden, eps, partials,
                                     num_partials, partial_stride, stream);
  return add_rmsnorm_launch<bf16_t>(delta, residual, weight, out, rows, num_out_rows, hidden, eps, partials,
                                    num_partials, partial_stride, stream);
}

// ---------------------------------------------------------------------------
// rotation tables: angle = float(position) * inv_freq[j]; cos and sin in float32
// ---------------------------------------------------------------------------

__global__ void rope_table_kernel(const int* __restrict__ positions,
                                  const float* __restrict__ inv_freq, float* __restrict__ cos_t,
                                  float* __restrict__ sin_t, int half) {
  const int t = blockIdx.x;
  const float pos = (float)positions[t];
  for (int j = threadIdx.x; j < half; j += blockDim.x) {
    const float angle = pos * inv_freq[j];
    float s, c;
    sincosf(angle, &s, &c);
    cos_t[(int64_t)t * half + j] = c;
    sin_t[(int64_t)t * half + j] = s;
  }
}

extern "C" int mi_rope_table(const int* positions, const float* inv_freq, float* cos_t,
                             float* sin_t, int num_tokens, int half, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && half > 0, "rope_table: bad sizes tokens=%d half=%d", num_tokens, half);
  if (num_tokens == 0) return MI_OK;
  rope_table_kernel<<<num_tokens, 64, 0, stream>>>(positions, inv_freq, cos_t, sin_t, half);
  MI_CHECK_LAUNCH("rope_table");
  return MI_OK;
}

// ---------------------------------------------------------------------------
// rotary encoding of q (in place) and k, and the write of k and v into pages.
//   row layout of qkv: [q heads | k heads | v heads], each head `head_dim` wide.
//   pairing: half rotation pairs dim j with j + rotary_dim/2; interleaved pairs
//   2j with 2j+1.  Dims at and beyond rotary_dim pass through.
//   pages: [num_pages, kv_heads, page_size, head_dim]; slot = page*page_size + offset;
//   a negative slot writes nothing.  With v_transposed, values are stored
//   [num_pages, kv_heads, head_dim, page_size] (what the matrix-core attention reads).
// ---------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_kernel(
    T* __restrict__ qkv, int64_t row_stride, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int* __restrict__ slot_mapping, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int q_heads, int kv_heads, int head_dim, int rotary_dim,
    int interleaved, int page_size, int v_transposed) {
  const int t = blockIdx.x;
  // the blocks along y share a token's work items
  const int first = blockIdx.y * blockDim.x + threadIdx.x;
  const int stride = blockDim.x * gridDim.y;
  const int half = rotary_dim / 2;
  T* row = qkv + (int64_t)t * row_stride;
  const float* c = cos_t + (int64_t)t * half;
  const float* s = sin_t + (int64_t)t * half;

  for (int e = first; e < q_heads * half; e += stride) {
    const int h = e / half, j = e % half;
    const int i0 = interleaved ? 2 * j : j;
    const int i1 = interleaved ? 2 * j + 1 : j + half;
    T* x = row + h * head_dim;
    const float x0 = to_f32(x[i0]), x1 = to_f32(x[i1]);
    x[i0] = from_f32<T>(x0 * c[j] - x1 * s[j]);
    x[i1] = from_f32<T>(x1 * c[j] + x0 * s[j]);
  }

  if (kv_heads == 0 || slot_mapping == nullptr) return;
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const int page = slot / page_size, off = slot % page_size;
  const T* k_row = row + (int64_t)q_heads * head_dim;
  const T* v_row = k_row + (int64_t)kv_heads * head_dim;

  for (int e = first; e < kv_heads * half; e += stride) {
    const int h = e / half, j = e % half;
    const int i0 = interleaved ? 2 * j : j;
    const int i1 = interleaved ? 2 * j + 1 : j + half;
    const T* x = k_row + h * head_dim;
    T* dst = k_pages + (((int64_t)page * kv_heads + h) * page_size + off) * head_dim;
    const float x0 = to_f32(x[i0]), x1 = to_f32(x[i1]);
    dst[i0] = from_f32<T>(x0 * c[j] - x1 * s[j]);
    dst[i1] = from_f32<T>(x1 * c[j] + x0 * s[j]);
  }
  const int pass = head_dim - rotary_dim;
  for (int e = first; e < kv_heads * pass; e += stride) {
    const int h = e / pass, d = rotary_dim + e % pass;
    k_pages[(((int64_t)page * kv_heads + h) * page_size + off) * head_dim + d] = k_row[h * head_dim + d];
  }
  for (int e = first; e < kv_heads * head_dim; e += stride) {
    const int h = e / head_dim, d = e % head_dim;
    const int64_t chunk = ((int64_t)page * kv_heads + h) * page_size * head_dim;
    const int64_t at = v_transposed ? chunk + (int64_t)d * page_size + off : chunk + (int64_t)off * head_dim + d;
    v_pages[at] = v_row[h * head_dim + d];
  }
}

// The same for the usual layout (halves paired, every size a multiple of 4), four
// elements per thread and step: 8- and 16-byte loads and stores instead of single
// elements.  Arithmetic and rounding are those of the kernel above.
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_vec;

template <typename T>
__global__ __launch_bounds__(256) void rope_kv_write_vec4_kernel(
    T* __restrict__ qkv, int64_t row_stride, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, const int* __restrict__ slot_mapping, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int q_heads, int kv_heads, int head_dim, int rotary_dim, int page_size,
    int v_transposed, int num_tokens, int blocks_y) {
  const int t = blockIdx.x;
  const int first = blockIdx.y * blockDim.x + threadIdx.x;
  const int stride = blockDim.x * blocks_y;
  const int half = rotary_dim / 2;
  const int half4 = half / 4;
  T* row = qkv + (int64_t)t * row_stride;
  const float* c = cos_t + (int64_t)t * half;
  const float* s = sin_t + (int64_t)t * half;

  auto rotate4 = [&](const T* x, int j, float lo[4], float hi[4]) {
    float x0[4], x1[4], cj[4], sj[4];
    load4(x + j, x0);
    load4(x + half + j, x1);
    load4(c + j, cj);
    load4(s + j, sj);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo[i] = x0[i] * cj[i] - x1[i] * sj[i];
      hi[i] = x1[i] * cj[i] + x0[i] * sj[i];
    }
  };

  for (int e = first; e < q_heads * half4; e += stride) {
    const int h = e / half4, j = (e % half4) * 4;
    T* x = row + h * head_dim;
    float lo[4], hi[4];
    rotate4(x, j, lo, hi);
    store4(x + j, lo);
    store4(x + half + j, hi);
  }

  if (kv_heads == 0 || slot_mapping == nullptr) return;
  const int slot = slot_mapping[t];
  if (slot < 0) return;
  const int page = slot / page_size, off = slot % page_size;
  const T* k_row = row + (int64_t)q_heads * head_dim;
  const T* v_row = k_row + (int64_t)kv_heads * head_dim;

  for (int e = first; e < kv_heads * half4; e += stride) {
    const int h = e / half4, j = (e % half4) * 4;
    T* dst = k_pages + (((int64_t)page * kv_heads + h) * page_size + off) * head_dim;
    float lo[4], hi[4];
    rotate4(k_row + h * head_dim, j, lo, hi);
    store4(dst + j, lo);
    store4(dst + half + j, hi);
  }
  const int pass4 = (head_dim - rotary_dim) / 4;
  for (int e = first; e < kv_heads * pass4; e += stride) {
    const int h = e / pass4, d = rotary_dim + (e % pass4) * 4;
    float x[4];
    load4(k_row + h * head_dim + d, x);
    store4(k_pages + (((int64_t)page * kv_heads + h) * page_size + off) * head_dim + d, x);
  }
  if (v_transposed && page_size % 8 == 0) {
    // Transposed value pages keep a dim's slots side by side: where this step's tokens fill a
    // whole page in order (a prompt's portion), a dim's row of the page is written at once
    // (page_size elements in a row instead of one at a time); the page's tokens share the
    // (head, dim) rows among them, each taking one page_size-th of them (all of them on the
    // page's first token measured 18.1 us for 2,048 tokens of 8 heads of 128, shared out 11 us).
    const int lead = t - off;
    bool whole_page = lead >= 0 && lead + page_size <= num_tokens;
    if (whole_page) {
      for (int i = 0; i < page_size; ++i) whole_page = whole_page && slot_mapping[lead + i] == page * page_size + i;
    }
    if (whole_page) {
      const int64_t v_off = (int64_t)(q_heads + kv_heads) * head_dim;
      const int rows_each = (kv_heads * head_dim + page_size - 1) / page_size;
      const int e_end = min((off + 1) * rows_each, kv_heads * head_dim);
      for (int e = off * rows_each + first; e < e_end; e += stride) {
        const int h = e / head_dim, d = e % head_dim;
        T* dst = v_pages + ((int64_t)page * kv_heads + h) * page_size * head_dim + (int64_t)d * page_size;
        const T* src = qkv + (int64_t)lead * row_stride + v_off + h * head_dim + d;
        for (int i0 = 0; i0 < page_size; i0 += 8) {
          if constexpr (sizeof(T) == 2) {
            bf16x8_vec x;
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = src[(int64_t)(i0 + i) * row_stride];
            *reinterpret_cast<bf16x8_vec*>(dst + i0) = x;
          } else {
#pragma unroll
            for (int i = 0; i < 8; ++i) dst[i0 + i] = src[(int64_t)(i0 + i) * row_stride];
          }
        }
      }
      return;
    }
  }
  const int dim4 = head_dim / 4;
  for (int e = first; e < kv_heads * dim4; e += stride) {
    const int h = e / dim4, d = (e % dim4) * 4;
    const int64_t chunk = ((int64_t)page * kv_heads + h) * page_size * head_dim;
    if (v_transposed) {
#pragma unroll
      for (int i = 0; i < 4; ++i) v_pages[chunk + (int64_t)(d + i) * page_size + off] = v_row[h * head_dim + d + i];
    } else {
      float x[4];
      load4(v_row + h * head_dim + d, x);
      store4(v_pages + chunk + (int64_t)off * head_dim + d, x);
    }
  }
}

extern "C" int mi_rope_kv_write(int dtype, void* qkv, int64_t row_stride, const float* cos_t,
                                const float* sin_t, const int* slot_mapping, void* k_pages,
                                void* v_pages, int num_tokens, int q_heads, int kv_heads,
                                int head_dim, int rotary_dim, int interleaved, int page_size,
                                int num_pages, int v_transposed, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && q_heads >= 0 && kv_heads >= 0 && head_dim > 0,
             "rope_kv_write: bad sizes tokens=%d q_heads=%d kv_heads=%d head_dim=%d", num_tokens,
             q_heads, kv_heads, head_dim);
  MI_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
             "rope_kv_write: rotary_dim=%d must be even and at most head_dim=%d", rotary_dim, head_dim);
  MI_REQUIRE(row_stride >= (int64_t)(q_heads + 2 * kv_heads) * head_dim,
             "rope_kv_write: row stride %lld is shorter than (q+2kv)*head_dim", (long long)row_stride);
  MI_REQUIRE(kv_heads == 0 || slot_mapping == nullptr || (page_size > 0 && num_pages > 0 && k_pages && v_pages),
             "rope_kv_write: pages are needed to write keys and values");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "rope_kv_write: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  // the usual layout, everything a multiple of 4 elements and 16-byte aligned: four elements a thread
  const size_t elem = dtype == MI_F32 ? 4 : 2;
  const bool aligned = ((uintptr_t)qkv | (uintptr_t)cos_t | (uintptr_t)sin_t | (uintptr_t)k_pages |
                        (uintptr_t)v_pages | (uintptr_t)(row_stride * elem)) % 16 == 0;
  if (!interleaved && aligned && head_dim % 4 == 0 && rotary_dim % 8 == 0) {
    const int items = max(q_heads * (rotary_dim / 8), kv_heads * (head_dim / 4));
    const int blocks_y = min((num_tokens >= 512) ? 2 : 16, max(1, ceil_div(items, 256)));
    dim3 grid(num_tokens, blocks_y);
    if (dtype == MI_F32) {
      rope_kv_write_vec4_kernel<float><<<grid, 256, 0, stream>>>(
          (float*)qkv, row_stride, cos_t, sin_t, slot_mapping, (float*)k_pages, (float*)v_pages,
          q_heads, kv_heads, head_dim, rotary_dim, page_size, v_transposed, num_tokens, blocks_y);
    } else {
      rope_kv_write_vec4_kernel<bf16_t><<<grid, 256, 0, stream>>>(
          (bf16_t*)qkv, row_stride, cos_t, sin_t, slot_mapping, (bf16_t*)k_pages, (bf16_t*)v_pages,
          q_heads, kv_heads, head_dim, rotary_dim, page_size, v_transposed, num_tokens, blocks_y);
    }
    MI_CHECK_LAUNCH("rope_kv_write");
    return MI_OK;
  }
  // few tokens (decode): spread each token's heads over several blocks
  const int items = max(q_heads * (rotary_dim / 2), kv_heads * head_dim);
  const int blocks_y = min((num_tokens >= 512) ? 4 : 16, max(1, ceil_div(items, 256)));
  dim3 grid(num_tokens, blocks_y);
  if (dtype == MI_F32) {
    rope_kv_write_kernel<float><<<grid, 256, 0, stream>>>(
        (float*)qkv, row_stride, cos_t, sin_t, slot_mapping, (float*)k_pages, (float*)v_pages,
        q_heads, kv_heads, head_dim, rotary_dim, interleaved, page_size, v_transposed);
  } else {
    rope_kv_write_kernel<bf16_t><<<grid, 256, 0, stream>>>(
        (bf16_t*)qkv, row_stride, cos_t, sin_t, slot_mapping, (bf16_t*)k_pages, (bf16_t*)v_pages,
        q_heads, kv_heads, head_dim, rotary_dim, interleaved, page_size, v_transposed);
  }
  MI_CHECK_LAUNCH("rope_kv_write");
  return MI_OK;
}

// ---------------------------------------------------------------------------
// out[t, i] = silu(gate_up[t, i]) * gate_up[t, I + i],  silu(g) = g / (1 + exp(-g))
// ---------------------------------------------------------------------------

// (float32 elements: evaluated in 64-bit and rounded once; the float32 exponential and two more
// roundings put the result 4.7e-8 away on average, twice what rounding alone costs)
template <typename T>
__device__ __forceinline__ float silu_times(float g, float u) {
  if constexpr (sizeof(T) == 4) return (float)((double)g / (1.0 + exp(-(double)g)) * (double)u);
  else return g / (1.f + expf(-g)) * u;
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void silu_mul_kernel(const T* __restrict__ gate_up,
                                                       T* __restrict__ out, int inter) {
  const int t = blockIdx.x;
  const T* g = gate_up + (int64_t)t * 2 * inter;
  const T* u = g + inter;
  T* o = out + (int64_t)t * inter;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * VEC;
  if (i >= inter) return;
  if (VEC == 4) {
    float gv[4], uv[4];
    load4(g + i, gv);
    load4(u + i, uv);
#pragma unroll
    for (int k = 0; k < 4; ++k) gv[k] = silu_times<T>(gv[k], uv[k]);
    store4(o + i, gv);
  } else {
    const float gv = to_f32(g[i]);
    o[i] = from_f32<T>(silu_times<T>(gv, to_f32(u[i])));
  }
}

extern "C" int mi_silu_mul(int dtype, const void* gate_up, void* out, int num_tokens, int inter,
                           hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && inter > 0, "silu_mul: bad sizes tokens=%d inter=%d", num_tokens, inter);
  MI_REQUIRE(ceil_div(inter, 256) <= 65535, "silu_mul: intermediate size %d is too large", inter);
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "silu_mul: unknown dtype %d", dtype);
  if (num_tokens == 0) return MI_OK;
  const int vec = (inter % 4 == 0) ? 4 : 1;
  dim3 grid(num_tokens, ceil_div(inter, 256 * vec));
  if (dtype == MI_F32) {
    if (vec == 4) silu_mul_kernel<float, 4><<<grid, 256, 0, stream>>>((const float*)gate_up, (float*)out, inter);
    else silu_mul_kernel<float, 1><<<grid, 256, 0, stream>>>((const float*)gate_up, (float*)out, inter);
  } else {
    if (vec == 4) silu_mul_kernel<bf16_t, 4><<<grid, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, inter);
    else silu_mul_kernel<bf16_t, 1><<<grid, 256, 0, stream>>>((const bf16_t*)gate_up, (bf16_t*)out, inter);
  }
  MI_CHECK_LAUNCH("silu_mul");
  return MI_OK;
}
