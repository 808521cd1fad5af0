// Shared helpers of the HIP kernels: element types, wave reductions, error reporting.
// Everything here is written for gfx950 (CDNA4): 64-lane waves, 160 KB LDS per CU.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;

#define MI_WAVE 64

// Every entry point returns 0 on success.  On refusal it returns a negative code
// and leaves a message that mi_last_error() returns.
#define MI_OK 0
#define MI_ERR_SHAPE (-1)
#define MI_ERR_LAUNCH (-2)
#define MI_ERR_LIMIT (-3)

void mi_set_error(const char* fmt, ...);

#define MI_REQUIRE(cond, ...)        \
  do {                               \
    if (!(cond)) {                   \
      mi_set_error(__VA_ARGS__);     \
      return MI_ERR_SHAPE;           \
    }                                \
  } while (0)

#define MI_CHECK_LAUNCH(name)                                               \
  do {                                                                      \
    hipError_t mi_err_ = hipGetLastError();                                 \
    if (mi_err_ != hipSuccess) {                                            \
      mi_set_error("%s: launch failed: %s", name, hipGetErrorString(mi_err_)); \
      return MI_ERR_LAUNCH;                                                 \
    }                                                                       \
  } while (0)

// dtype codes shared with the Python side
#define MI_F32 0
#define MI_BF16 1

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return (float)v; }

template <typename T>
__device__ __forceinline__ T from_f32(float v);
template <>
__device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) { return (bf16_t)v; }

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef int int32x4_t __attribute__((ext_vector_type(4)));

// How a weight-streaming product reads its weights ("LINES" in the kernels).  The matrix-core
// operand wants, per k-step (32 elements), 16 bytes of each of 16 weight rows in every 16
// lanes: four lanes a row, 64 bytes, half a cache line; the other half is asked for by the
// next k-step's load.  Whole lines per load run faster, and non-temporal loads (the weights
// are read once) faster again, but only on whole lines.  Measured on MI355X, microseconds for
// 6144 x 4096 / 4096 x 14336 / 28672 x 4096 / 128256 x 4096 at 8 rows, weights not in any
// cache: half lines 13.5 / 30.1 / 46.3 / 192; non-temporal on half lines slower (28672 x
// 4096: 47.5-50.1 in a kernel that only reads); whole lines with every 16 lanes on 8 lines and
// an exchange inside the 16 lanes 14.8 / 27.7 / 42.3 / 168; whole lines with every 8 lanes
// on one line (this) 11.4 / 23.8 / 40.0 / 168.  A long plain read reaches 6.1-6.3 TB/s, a
// non-temporal one 7.0-7.1 TB/s.
// So a load takes 8 rows x 128 bytes (two k-steps): lane l reads 16-byte chunk l % 8 of the
// line of row l / 8 of the tile's lower or upper 8 rows.  Of a pair of such loads (lower rows,
// upper rows) the lanes with chunks 4-7 of the first and those with chunks 0-3 of the second
// change places (inside every 16 lanes: two DPP moves), which sorts the chunks by k-step; then
// every lane fetches its operand's 16 bytes from the lane that holds them (ds_bpermute, which
// moves data between lanes through the LDS crossbar without touching LDS memory).
// Needs: rows of the matrix on 128-byte boundaries, k-steps taken in even-aligned pairs.
__device__ __forceinline__ void lines_to_operands(bf16x8_t& lower_rows, bf16x8_t& upper_rows) {
  int32x4_t lo = __builtin_bit_cast(int32x4_t, lower_rows), hi = __builtin_bit_cast(int32x4_t, upper_rows);
  // operand lane (quad, col) wants row col, chunk quad of its k-step: after the exchange that
  // is lane 8 * (col % 8) + 4 * (col / 8) + quad
  const int lane = threadIdx.x % MI_WAVE, col = lane % 16, quad = lane / 16;
  const int from = 4 * (8 * (col % 8) + 4 * (col / 8) + quad);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int lo_was = lo[e];
    // row_shr:4 into lanes 4-7 and 12-15 of every 16: the upper rows' chunks 0-3 (first k-step)
    lo[e] = __builtin_amdgcn_update_dpp(lo[e], hi[e], 0x114, 0xF, 0xA, false);
    // row_shl:4 into lanes 0-3 and 8-11: the lower rows' chunks 4-7 (second k-step)
    hi[e] = __builtin_amdgcn_update_dpp(hi[e], lo_was, 0x104, 0xF, 0x5, false);
    lo[e] = __builtin_amdgcn_ds_bpermute(from, lo[e]);
    hi[e] = __builtin_amdgcn_ds_bpermute(from, hi[e]);
  }
  lower_rows = __builtin_bit_cast(bf16x8_t, lo);  // operand of the pair's first k-step
  upper_rows = __builtin_bit_cast(bf16x8_t, hi);  // operand of its second
}

// The row (0..7 of the lower or upper 8) whose line a lane reads, and its 16-byte chunk of
// that line as a byte offset.
__device__ __forceinline__ int line_row_of_lane(int lane) { return lane / 8; }
__device__ __forceinline__ uint32_t line_chunk_of_lane(int lane) { return (uint32_t)(lane % 8) * 16u; }

// The two loads of a pair of k-steps, non-temporal: base (uniform, kept in scalar registers) + the
// lane's offsets.
__device__ __forceinline__ void load_line_pair(const void* matrix, int64_t first_kstep, uint32_t lower_at,
                                               uint32_t upper_at, bf16x8_t& lower_rows, bf16x8_t& upper_rows) {
  using global_bytes = const __attribute__((address_space(1))) char;
  using global_chunk = const __attribute__((address_space(1))) bf16x8_t;
  uint64_t base_bits = reinterpret_cast<uint64_t>(matrix) + (uint64_t)first_kstep * 64u;
  asm("" : "+s"(base_bits));  // scalar: the lanes add their 32-bit offsets
  global_bytes* base = (global_bytes*)base_bits;
  // (opaque to the compiler, or it widens the offsets to 64 bits once and for all and adds
  // whole addresses in vector registers for every load)
  asm("" : "+v"(lower_at), "+v"(upper_at));
  lower_rows = __builtin_nontemporal_load((global_chunk*)(base + lower_at));
  upper_rows = __builtin_nontemporal_load((global_chunk*)(base + upper_at));
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, MI_WAVE));
  return v;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = MI_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, MI_WAVE);
  return v;
}

// Sum over a whole block in a fixed order: lanes by butterfly, waves one after another.
// `scratch` holds at least blockDim.x / 64 floats.  All threads get the result.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / MI_WAVE;
  const int lane = threadIdx.x % MI_WAVE;
  const int n_waves = (blockDim.x + MI_WAVE - 1) / MI_WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < n_waves; ++w) total += scratch[w];
  return total;
}

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
static inline int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }
