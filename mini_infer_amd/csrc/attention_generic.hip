// Paged causal attention, plain-FMA version: the float32 path of the engine and
// the fallback for sizes the matrix-core kernels refuse.  One 64-lane wave per
// (query token, key/value head, up to 4 query heads of its group, key split).
// Lanes own keys while scores are computed (one key row per lane, q broadcast
// from LDS) and own output dims while values are accumulated.  The softmax is an
// online one (running max).  For bfloat16 inputs the scores, the softmax's sum and the
// value sum are float32.  For float32 inputs (the engine's 32-bit path) they are kept in
// 64-bit: a float32 sum over thousands of keys is rounded at every key, which alone put
// the relative error of a 2,000-key row at 6e-7, twenty-five times what rounding the
// result once costs (and more than everything else in a layer together); in 64-bit the
// row is rounded once, when it is written.
//
// Head sizes: any even one up to 256.  Multiples of 16 read keys and values 16 bytes at a
// time; the others read them in pairs of elements (rows of an even head size are always
// aligned to that) and guard every access past the row's end.
//
// Semantics follow the reference's oracle (cache/packed_attention.py:296-338):
// query head h reads key/value head h / (Hq/Hkv); a query at absolute position p
// sees keys 0..p, or p-window+1..p with a window.  With `slopes` (one float per
// query head, may be null) the score of the key at position j gets
// slopes[h] * (j - p) added before the softmax: a bias linear in the distance.
//
// Layout: q rows [token][head][head_dim] with a row stride; pages
// [num_pages][kv_heads][page_size][head_dim]; block_table[request][i] is the page
// of that request's keys i*page_size .. (i+1)*page_size-1.
#include "common.h"
#include "entry_points.h"

#include <math.h>

#include <mutex>

#define GT 4  // query heads handled together by one wave

template <typename T, int N>
struct alignas(sizeof(T) * N) Pack {
  T v[N];
};

// what sums are kept in: see the note at the top
template <typename T>
struct SumType {
  using type = float;
};
template <>
struct SumType<float> {
  using type = double;
};

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, MI_WAVE);
  return v;
}

// VEC: head_dim is a multiple of 16 (16-byte loads, no guards inside a row)
template <typename T, int VPL, bool VEC>
__global__ __launch_bounds__(64) void attn_generic_kernel(
    const T* __restrict__ q, int64_t q_row_stride, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, const int* __restrict__ block_table, int max_blocks,
    const int* __restrict__ token_request, const int* __restrict__ positions, T* __restrict__ out,
    int64_t out_row_stride, float* __restrict__ part_acc, float* __restrict__ part_ml, int q_heads,
    int kv_heads, int head_dim, int page_size, float scale, int window, int num_splits,
    const float* __restrict__ slopes) {
  using S = typename SumType<T>::type;
  extern __shared__ __align__(8) unsigned char q_lds_bytes[];
  S* q_lds = reinterpret_cast<S*>(q_lds_bytes);  // [GT][head_dim], pre-multiplied by the scale
  constexpr int KV = VEC ? 16 / sizeof(T) : 4;  // elements per step along a key row

  const int t = blockIdx.x;
  const int group = q_heads / kv_heads;
  const int head_blocks = (group + GT - 1) / GT;
  const int kvh = blockIdx.y / head_blocks;
  const int g0 = (blockIdx.y % head_blocks) * GT;
  const int nh = min(GT, group - g0);
  const int head0 = kvh * group + g0;
  const int split = blockIdx.z;
  const int lane = threadIdx.x;

  const T* q_row = q + (int64_t)t * q_row_stride + (int64_t)head0 * head_dim;
  for (int i = lane; i < GT * head_dim; i += MI_WAVE)
    q_lds[i] = (i < nh * head_dim) ? (S)to_f32(q_row[i]) * (S)scale : (S)0;
  __syncthreads();

  const int pos = positions[t];
  const int req = token_request[t];
  const int lo = (window > 0) ? max(0, pos - window + 1) : 0;
  const int hi = pos + 1;
  int chunk = (hi - lo + num_splits - 1) / num_splits;
  chunk = (chunk + MI_WAVE - 1) / MI_WAVE * MI_WAVE;
  const int a = lo + split * chunk;
  const int b = min(a + chunk, hi);
  const int* bt = block_table + (int64_t)req * max_blocks;

  float m[GT];
  S l[GT], acc[GT][VPL];
#pragma unroll
  for (int g = 0; g < GT; ++g) {
    m[g] = -INFINITY;
    l[g] = 0;
#pragma unroll
    for (int v = 0; v < VPL; ++v) acc[g][v] = 0;
  }
  const bool owns_dims = lane * VPL < head_dim;
  float slope[GT];
#pragma unroll
  for (int g = 0; g < GT; ++g) slope[g] = (slopes != nullptr && g < nh) ? slopes[head0 + g] : 0.f;

  for (int base = a; base < b; base += MI_WAVE) {
    const int key = base + lane;
    const bool valid = key < b;
    int row_idx = 0;
    float s[GT];  // the score less nothing yet; below: less the running maximum
    S s_sum[GT];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      s[g] = -INFINITY;
      s_sum[g] = 0;
    }
    if (valid) {
      const int page = bt[key / page_size];
      row_idx = (page * kv_heads + kvh) * page_size + key % page_size;
      const T* k_row = k_pages + (int64_t)row_idx * head_dim;
      // four running sums per score (dims d, d+1, d+2, d+3 of every group of four), added
      // at the end: shorter chains of roundings than one sum over the whole head
      S s4[GT][4];
#pragma unroll
      for (int g = 0; g < GT; ++g)
#pragma unroll
        for (int e = 0; e < 4; ++e) s4[g][e] = 0;
      for (int d = 0; d < head_dim; d += KV) {
        float kf[KV];
        if constexpr (VEC) {
          const Pack<T, KV> kk = *reinterpret_cast<const Pack<T, KV>*>(k_row + d);
#pragma unroll
          for (int e = 0; e < KV; ++e) kf[e] = to_f32(kk.v[e]);
        } else {
          // pairs of elements; an even head size ends after the first or the second pair
          const Pack<T, 2> k0 = *reinterpret_cast<const Pack<T, 2>*>(k_row + d);
          kf[0] = to_f32(k0.v[0]);
          kf[1] = to_f32(k0.v[1]);
          kf[2] = kf[3] = 0.f;
          if (d + 2 < head_dim) {
            const Pack<T, 2> k1 = *reinterpret_cast<const Pack<T, 2>*>(k_row + d + 2);
            kf[2] = to_f32(k1.v[0]);
            kf[3] = to_f32(k1.v[1]);
          }
        }
#pragma unroll
        for (int e = 0; e < KV; ++e) {
          if (!VEC && d + e >= head_dim) break;
#pragma unroll
          for (int g = 0; g < GT; ++g) {
            const S qv = q_lds[g * head_dim + d + e];
            if constexpr (sizeof(S) == 8) s4[g][e % 4] = fma(qv, (S)kf[e], s4[g][e % 4]);
            else s4[g][e % 4] = fmaf(qv, kf[e], s4[g][e % 4]);
          }
        }
      }
      const S distance = (S)(key - pos);
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        s_sum[g] = (s4[g][0] + s4[g][1]) + (s4[g][2] + s4[g][3]);
        s_sum[g] += (S)slope[g] * distance;
        s[g] = (float)s_sum[g];
      }
    }
    float p[GT];
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      const float m_new = fmaxf(m[g], wave_max(s[g]));
      const float alpha = expf(m[g] - m_new);
      // (64-bit sums: the difference is taken and the exponential made before anything is
      // rounded to float32, so a key's weight is off by one rounding, not by the score's)
      if constexpr (sizeof(S) == 8) p[g] = valid ? (float)exp(s_sum[g] - (S)m_new) : 0.f;
      else p[g] = valid ? expf(s_sum[g] - m_new) : 0.f;
      l[g] = l[g] * (S)alpha + wave_sum((S)p[g]);
#pragma unroll
      for (int v = 0; v < VPL; ++v) acc[g][v] *= (S)alpha;
      m[g] = m_new;
    }
    const int n_valid = min(MI_WAVE, b - base);
    for (int j = 0; j < n_valid; ++j) {
      const int rj = __shfl(row_idx, j, MI_WAVE);
      float vv[VPL];
#pragma unroll
      for (int v = 0; v < VPL; ++v) vv[v] = 0.f;
      if (owns_dims) {
        const T* v_row = v_pages + (int64_t)rj * head_dim + lane * VPL;
        if constexpr (VEC || VPL <= 2) {  // (an even head size: a pair never straddles the row's end)
          const Pack<T, VPL> pk = *reinterpret_cast<const Pack<T, VPL>*>(v_row);
#pragma unroll
          for (int v = 0; v < VPL; ++v) vv[v] = to_f32(pk.v[v]);
        } else {
#pragma unroll
          for (int v = 0; v < VPL; v += 2) {
            if (lane * VPL + v < head_dim) {
              const Pack<T, 2> pk = *reinterpret_cast<const Pack<T, 2>*>(v_row + v);
              vv[v] = to_f32(pk.v[0]);
              vv[v + 1] = to_f32(pk.v[1]);
            }
          }
        }
      }
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        const float pj = __shfl(p[g], j, MI_WAVE);
#pragma unroll
        for (int v = 0; v < VPL; ++v) acc[g][v] += (S)pj * (S)vv[v];
      }
    }
  }

  if (num_splits == 1) {
    if (owns_dims) {
#pragma unroll
      for (int g = 0; g < GT; ++g) {
        if (g < nh) {
          T* o = out + (int64_t)t * out_row_stride + (int64_t)(head0 + g) * head_dim + lane * VPL;
          const S inv = (S)1 / l[g];
#pragma unroll
          for (int v = 0; v < VPL; ++v)
            if (VEC || lane * VPL + v < head_dim) o[v] = from_f32<T>((float)(acc[g][v] * inv));
        }
      }
    }
  } else {
#pragma unroll
    for (int g = 0; g < GT; ++g) {
      if (g < nh) {
        const int64_t slot = ((int64_t)t * q_heads + head0 + g) * num_splits + split;
        if (owns_dims) {
#pragma unroll
          for (int v = 0; v < VPL; ++v)
            if (VEC || lane * VPL + v < head_dim) part_acc[slot * head_dim + lane * VPL + v] = (float)acc[g][v];
        }
        if (lane == 0) {
          part_ml[slot * 2] = m[g];
          part_ml[slot * 2 + 1] = (float)l[g];
        }
      }
    }
  }
}

// Combine the splits of one (token, head): one wave; lanes first share the work of
// reading the splits' (max, sum) pairs, then own output dims.  The order of the sums
// is fixed, so the result does not depend on timing.
template <typename T>
__global__ __launch_bounds__(64) void attn_reduce_kernel(const float* __restrict__ part_acc,
                                                         const float* __restrict__ part_ml,
                                                         T* __restrict__ out, int64_t out_row_stride,
                                                         int q_heads, int head_dim, int num_splits) {
  using S = typename SumType<T>::type;
  const int t = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x;
  const int64_t base = ((int64_t)t * q_heads + h) * num_splits;
  constexpr int BATCH = 8;
  // Few splits of a head of at most 128 dims (the usual decode step): every partial value
  // this lane needs is requested up front, together with the (max, sum) pairs, so the
  // kernel waits for memory once.
  const bool small = num_splits <= BATCH && head_dim <= 2 * MI_WAVE;
  float early[2][BATCH];
  if (small) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int d = half * MI_WAVE + lane;
#pragma unroll
      for (int i = 0; i < BATCH; ++i) {
        const int sp = min(i, num_splits - 1);  // past the end: re-read the last split, weight 0 below
        early[half][i] = (d < head_dim) ? part_acc[(base + sp) * head_dim + d] : 0.f;
      }
    }
  }
  // num_splits <= 64: lane s holds split s
  const float m_s = (lane < num_splits) ? part_ml[(base + lane) * 2] : -INFINITY;
  const float l_s = (lane < num_splits) ? part_ml[(base + lane) * 2 + 1] : 0.f;
  const float m_all = wave_max(m_s);
  const float w_s = (lane < num_splits) ? expf(m_s - m_all) : 0.f;
  S l_all = 0;
  for (int s = 0; s < num_splits; ++s) l_all += (S)__shfl(l_s, s, MI_WAVE) * (S)__shfl(w_s, s, MI_WAVE);
  const S inv = (S)1 / l_all;
  // The partial accumulators are read in batches of independent loads (a load per split
  // issued one after the other's use would cost a memory latency per split) and added in
  // split order.
  if (small) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int d = half * MI_WAVE + lane;
      S o = 0;
#pragma unroll
      for (int i = 0; i < BATCH; ++i) {
        const float w = __shfl(w_s, i, MI_WAVE);
        if (i < num_splits) o += (S)early[half][i] * (S)w;
      }
      if (d < head_dim) out[(int64_t)t * out_row_stride + (int64_t)h * head_dim + d] = from_f32<T>((float)(o * inv));
    }
    return;
  }
  for (int d0 = 0; d0 < head_dim; d0 += MI_WAVE) {  // all lanes stay in the loop for the shuffles
    const int d = d0 + lane;
    const bool active = d < head_dim;
    const float* src = part_acc + base * head_dim + (active ? d : 0);
    S o = 0;
    for (int s0 = 0; s0 < num_splits; s0 += BATCH) {
      float v[BATCH];
#pragma unroll
      for (int i = 0; i < BATCH; ++i) {
        const int sp = min(s0 + i, num_splits - 1);  // past the end: re-read the last split, weight 0 below
        v[i] = src[(int64_t)sp * head_dim];
      }
#pragma unroll
      for (int i = 0; i < BATCH; ++i) {
        const float w = __shfl(w_s, min(s0 + i, MI_WAVE - 1), MI_WAVE);
        if (s0 + i < num_splits) o += (S)v[i] * (S)w;
      }
    }
    if (active) out[(int64_t)t * out_row_stride + (int64_t)h * head_dim + d] = from_f32<T>((float)(o * inv));
  }
}

template <typename T>
static int attn_generic_launch(const void* q, int64_t q_row_stride, const void* k_pages,
                               const void* v_pages, const int* block_table, int max_blocks,
                               const int* token_request, const int* positions, void* out,
                               int64_t out_row_stride, float* part_acc, float* part_ml,
                               int num_tokens, int q_heads, int kv_heads, int head_dim,
                               int page_size, float scale, int window, int num_splits,
                               const float* slopes, hipStream_t stream) {
  const int group = q_heads / kv_heads;
  dim3 grid(num_tokens, kv_heads * ceil_div(group, GT), num_splits);
  const size_t lds = sizeof(typename SumType<T>::type) * GT * head_dim;
  const bool vec = head_dim % 16 == 0;
#define MI_ATTN_LAUNCH(VPL, VEC)                                                                  \
  attn_generic_kernel<T, VPL, VEC><<<grid, MI_WAVE, lds, stream>>>(                               \
      (const T*)q, q_row_stride, (const T*)k_pages, (const T*)v_pages, block_table, max_blocks,   \
      token_request, positions, (T*)out, out_row_stride, part_acc, part_ml, q_heads, kv_heads,    \
      head_dim, page_size, scale, window, num_splits, slopes)
  if (head_dim <= 64) { if (vec) MI_ATTN_LAUNCH(1, true); else MI_ATTN_LAUNCH(1, false); }
  else if (head_dim <= 128) { if (vec) MI_ATTN_LAUNCH(2, true); else MI_ATTN_LAUNCH(2, false); }
  else { if (vec) MI_ATTN_LAUNCH(4, true); else MI_ATTN_LAUNCH(4, false); }
#undef MI_ATTN_LAUNCH
  MI_CHECK_LAUNCH("attn_generic");
  if (num_splits > 1) {
    dim3 rgrid(num_tokens, q_heads);
    attn_reduce_kernel<T><<<rgrid, MI_WAVE, 0, stream>>>(part_acc, part_ml, (T*)out, out_row_stride,
                                                         q_heads, head_dim, num_splits);
    MI_CHECK_LAUNCH("attn_reduce");
  }
  return MI_OK;
}

static int attn_generic_check(int dtype, int64_t q_row_stride, int max_blocks, int64_t out_row_stride,
                              int num_tokens, int q_heads, int kv_heads, int head_dim, int page_size,
                              int num_pages, int window, int num_splits) {
  MI_REQUIRE(num_tokens >= 0 && q_heads > 0 && kv_heads > 0, "attn_generic: bad sizes tokens=%d q_heads=%d kv_heads=%d",
             num_tokens, q_heads, kv_heads);
  MI_REQUIRE(q_heads % kv_heads == 0, "attn_generic: q_heads=%d is not a multiple of kv_heads=%d",
             q_heads, kv_heads);
  MI_REQUIRE(head_dim > 0 && head_dim % 2 == 0 && head_dim <= 256,
             "attn_generic: head_dim=%d must be even and at most 256", head_dim);
  MI_REQUIRE(page_size > 0 && num_pages > 0 && max_blocks > 0, "attn_generic: bad page sizes page_size=%d num_pages=%d max_blocks=%d",
             page_size, num_pages, max_blocks);
  MI_REQUIRE((int64_t)num_pages * kv_heads * page_size < (int64_t)1 << 31,
             "attn_generic: the cache has too many key rows for 32-bit row indices");
  MI_REQUIRE(window >= 0, "attn_generic: window=%d must be 0 (none) or positive", window);
  MI_REQUIRE(num_splits >= 1 && num_splits <= 64, "attn_generic: num_splits=%d must be 1..64", num_splits);
  MI_REQUIRE(q_row_stride >= (int64_t)q_heads * head_dim && out_row_stride >= (int64_t)q_heads * head_dim,
             "attn_generic: row strides shorter than q_heads*head_dim");
  MI_REQUIRE(kv_heads * ceil_div(q_heads / kv_heads, GT) <= 65535, "attn_generic: too many heads");
  MI_REQUIRE(dtype == MI_F32 || dtype == MI_BF16, "attn_generic: unknown dtype %d", dtype);
  return MI_OK;
}

// part_acc holds num_tokens*q_heads*num_splits*head_dim floats and part_ml
// num_tokens*q_heads*num_splits*2 floats; both may be null when num_splits == 1.
// `slopes` (q_heads floats) may be null.
extern "C" int mi_attn_generic(int dtype, const void* q, int64_t q_row_stride, const void* k_pages,
                               const void* v_pages, const int* block_table, int max_blocks,
                               const int* token_request, const int* positions, void* out,
                               int64_t out_row_stride, float* part_acc, float* part_ml,
                               int num_tokens, int q_heads, int kv_heads, int head_dim,
                               int page_size, int num_pages, float scale, int window,
                               int num_splits, const float* slopes, hipStream_t stream) {
  const int bad = attn_generic_check(dtype, q_row_stride, max_blocks, out_row_stride, num_tokens, q_heads,
                                     kv_heads, head_dim, page_size, num_pages, window, num_splits);
  if (bad != MI_OK) return bad;
  MI_REQUIRE(num_splits == 1 || (part_acc && part_ml), "attn_generic: split keys need partial buffers");
  if (num_tokens == 0) return MI_OK;
  if (dtype == MI_F32)
    return attn_generic_launch<float>(q, q_row_stride, k_pages, v_pages, block_table, max_blocks,
                                      token_request, positions, out, out_row_stride, part_acc, part_ml,
                                      num_tokens, q_heads, kv_heads, head_dim, page_size, scale, window,
                                      num_splits, slopes, stream);
  return attn_generic_launch<bf16_t>(q, q_row_stride, k_pages, v_pages, block_table, max_blocks,
                                     token_request, positions, out, out_row_stride, part_acc, part_ml,
                                     num_tokens, q_heads, kv_heads, head_dim, page_size, scale, window,
                                     num_splits, slopes, stream);
}

// The combining step alone, for partials written by the matrix-core kernel.
extern "C" int mi_attn_reduce_bf16(const float* part_acc, const float* part_ml, void* out,
                                   int64_t out_row_stride, int num_tokens, int q_heads,
                                   int head_dim, int num_splits, hipStream_t stream) {
  if (num_tokens == 0) return MI_OK;
  MI_REQUIRE(q_heads <= 65535, "attn_reduce: too many heads");
  dim3 rgrid(num_tokens, q_heads);
  attn_reduce_kernel<bf16_t><<<rgrid, MI_WAVE, 0, stream>>>(part_acc, part_ml, (bf16_t*)out,
                                                            out_row_stride, q_heads, head_dim,
                                                            num_splits);
  MI_CHECK_LAUNCH("attn_reduce");
  return MI_OK;
}

// ---------------------------------------------------------------------------------------
// The same attention for callers that cannot allocate: the partial results of the key
// ranges lie in an array of the library's own.
//
// `scratch` below is, in host code, only a stand-in for the device symbol: its device
// address differs per GPU and is asked for once per device with hipGetSymbolAddress;
// host code passes that address, never the array's name, to kernels.

#define MI_MAX_DEVICES 64

static __device__ __align__(256) unsigned char scratch[MI_ATTN_STATIC_SCRATCH_BYTES];

static std::mutex g_scratch_mutex;
static void* g_scratch_ptr[MI_MAX_DEVICES] = {};

// The address of this device's copy of `scratch` (asked for at the first call on the device).
static int scratch_of_current_device(float** ptr) {
  int device = -1;
  hipError_t err = hipGetDevice(&device);
  if (err != hipSuccess || device < 0 || device >= MI_MAX_DEVICES) {
    mi_set_error("attn_generic_static: cannot tell the current device (%s, device %d)",
                 hipGetErrorString(err), device);
    return MI_ERR_LAUNCH;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[device] == nullptr) {
    void* address = nullptr;
    err = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
    if (err != hipSuccess || address == nullptr) {
      mi_set_error("attn_generic_static: hipGetSymbolAddress failed on device %d: %s", device,
                   hipGetErrorString(err));
      return MI_ERR_LAUNCH;
    }
    g_scratch_ptr[device] = address;
  }
  *ptr = (float*)g_scratch_ptr[device];
  return MI_OK;
}

extern "C" int mi_attn_generic_static(int dtype, const void* q, int64_t q_row_stride, const void* k_pages,
                                      const void* v_pages, const int* block_table, int max_blocks,
                                      const int* token_request, const int* positions, void* out,
                                      int64_t out_row_stride, int num_tokens, int q_heads, int kv_heads,
                                      int head_dim, int page_size, int num_pages, float scale, int window,
                                      int num_splits, const float* slopes, hipStream_t stream) {
  const int bad = attn_generic_check(dtype, q_row_stride, max_blocks, out_row_stride, num_tokens, q_heads,
                                     kv_heads, head_dim, page_size, num_pages, window, num_splits);
  if (bad != MI_OK) return bad;
  if (num_tokens == 0) return MI_OK;
  const int64_t slots = (int64_t)num_tokens * q_heads * num_splits;
  const int64_t bytes = slots * (head_dim + 2) * (int64_t)sizeof(float);
  if (num_splits > 1 && bytes > (int64_t)MI_ATTN_STATIC_SCRATCH_BYTES) {
    mi_set_error("attn_generic_static: %d tokens x %d heads x %d key ranges x head_dim %d need %lld bytes "
                 "of partial results, the library's array holds %u",
                 num_tokens, q_heads, num_splits, head_dim, (long long)bytes, MI_ATTN_STATIC_SCRATCH_BYTES);
    return MI_ERR_LIMIT;
  }
  float* part_acc = nullptr;
  float* part_ml = nullptr;
  if (num_splits > 1) {
    float* base = nullptr;
    const int status = scratch_of_current_device(&base);
    if (status != MI_OK) return status;
    part_acc = base;                     // [slots][head_dim]
    part_ml = base + slots * head_dim;  // [slots][2]
  }
  if (dtype == MI_F32)
    return attn_generic_launch<float>(q, q_row_stride, k_pages, v_pages, block_table, max_blocks,
                                      token_request, positions, out, out_row_stride, part_acc, part_ml,
                                      num_tokens, q_heads, kv_heads, head_dim, page_size, scale, window,
                                      num_splits, slopes, stream);
  return attn_generic_launch<bf16_t>(q, q_row_stride, k_pages, v_pages, block_table, max_blocks,
                                     token_request, positions, out, out_row_stride, part_acc, part_ml,
                                     num_tokens, q_heads, kv_heads, head_dim, page_size, scale, window,
                                     num_splits, slopes, stream);
}
