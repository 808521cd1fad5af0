// Weight-streaming matrix product for few rows (decode): C[M,N] = A[M,K] * W[N,K]^T,
// bfloat16 in and out, float32 accumulate on the matrix cores, M <= 16.
//
// At these sizes the product is bound by reading W once from HBM.  A block owns 8 to 64
// output features and all of K: its 8 waves each stream one eighth of every one of
// its weight rows (16 contiguous bytes per lane and k-step, MFMA 16x16x32 with
// the weights as the A operand and the activations, transposed, as the B operand),
// then add their partial tiles through LDS in a fixed order, so the result does not
// depend on timing.  Activations are small and come from the cache hierarchy.
// What comes before and after a product in a decoder layer is folded into it where that
// saves a launch: the RMS norm of the input (PRO_NORM), the SiLU-gated product
// (EPI_GATED), the add into the float32 residual with the next norm's statistics
// (EPI_RESIDUAL).
//
// This stands where the reference's engine calls the vendor BLAS
// (distributed/linear.py:167); that library's kernels reach about half of the HBM
// rate at these shapes.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;

#define SK_WAVES 8
#define SK_MAX_ROWS 16
#define SK_STAT_ROWS 16  // row slots per entry of a sum-of-squares table

// Where the activations come from.
//   PRO_PLAIN: a[m, k] in bfloat16.
//   PRO_NORM:  the RMS-normalized float32 residual rows x[m, k]:
//              a = bf16(norm_weight * (x * rsqrt(mean(x^2) + eps))), the formula of the
//              stand-alone norm kernel, made on the fly; mean(x^2) comes from a table of
//              partial sums of squares [slots][16 rows] that the producer of x wrote
//              (EPI_RESIDUAL below), added up in a fixed order.
enum { PRO_PLAIN = 0, PRO_NORM = 1 };
// What happens to the products.
//   EPI_STORE:    c[m, n] = bf16(product).
//   EPI_GATED:    W holds two stacked matrices [gate; up] of n rows each and
//                 c = silu(gate . a) * (up . a): a block computes both halves of its
//                 features, so the [m, 2n] intermediate is never written.  Both sums are
//                 rounded to bfloat16 before the activation, exactly as when the product
//                 and the activation run as two kernels.
//   EPI_RESIDUAL: residual[m, n] (float32) += bf16(product), and the block's share of every
//                 row's sum of squares of the NEW residual goes to stats_out[block][row]:
//                 the add of the next norm is done here, and its statistics are ready.
enum { EPI_STORE = 0, EPI_GATED = 1, EPI_RESIDUAL = 2 };

struct SkinnyArgs {
  const bf16_t* a;  // PRO_PLAIN
  const float* x;  // PRO_NORM
  int64_t ld_in;  // row stride of a or x, in elements
  const bf16_t* norm_weight;  // PRO_NORM: [k]
  const float* stats_in;  // PRO_NORM: [stats_slots][SK_STAT_ROWS]
  int stats_slots;
  float eps;
  const bf16_t* w;
  int64_t ldw;
  bf16_t* c;  // EPI_STORE, EPI_GATED
  float* residual;  // EPI_RESIDUAL
  int64_t ld_out;  // row stride of c or residual
  float* stats_out;  // EPI_RESIDUAL: [gridDim.x][SK_STAT_ROWS]
  int m, n, k, features_per_block;
};

// NT = 16-feature tiles of the OUTPUT per block (the activations a wave loads are used
// for every weight tile of the block), U = k-steps whose loads are issued together
// before their products run.  Register use is kept low on purpose: many resident waves,
// each with U*(tiles+1) loads in flight, hide the memory latency better than a deeper
// pipeline in fewer waves.
template <int NT, int U, int PRO, int EPI>
__global__ __launch_bounds__(64 * SK_WAVES) void gemm_skinny_bf16_kernel(const SkinnyArgs p) {
  constexpr int WT = (EPI == EPI_GATED) ? 2 * NT : NT;  // weight tiles per block
  __shared__ float red[SK_WAVES][WT][256];

  const int wave = threadIdx.x / MI_WAVE;
  const int lane = threadIdx.x % MI_WAVE;
  const int col = lane % 16;
  const int quad = lane / 16;
  const int m = p.m, n = p.n, k = p.k;
  // the block's features [n0, n_end): up to 16*NT, a multiple of 4 chosen by the host so
  // that the blocks spread evenly over the CUs (rows past n_end repeat the last one)
  const int n0 = blockIdx.x * p.features_per_block;
  const int n_end = min(n0 + p.features_per_block, n);

  const int ksteps = k / 32;
  const int per_wave = (ksteps + SK_WAVES - 1) / SK_WAVES;
  const int s_begin = min(wave * per_wave, ksteps);
  const int s_end = min(s_begin + per_wave, ksteps);

  // weights: lane reads feature n0 + 16*nt + col (and its twin n rows further down when
  // gated), 8 consecutive k
  const bf16_t* wp[WT];
#pragma unroll
  for (int t = 0; t < WT; ++t) {
    const int row = min(n0 + (t % NT) * 16 + col, n_end - 1) + (t / NT) * n;
    wp[t] = p.w + (int64_t)row * p.ldw + quad * 8;
  }
  // activations: lane reads token `col`; lanes past M re-read the last token (the same
  // cache lines as its own lane, so no extra traffic) and their columns are never stored
  const int a_row = min(col, m - 1);
  const bf16_t* ap = (PRO == PRO_PLAIN) ? p.a + (int64_t)a_row * p.ld_in + quad * 8 : nullptr;
  const float* xp = (PRO == PRO_NORM) ? p.x + (int64_t)a_row * p.ld_in + quad * 8 : nullptr;
  const bf16_t* gp = (PRO == PRO_NORM) ? p.norm_weight + quad * 8 : nullptr;

  float inv_rms = 0.f;
  if (PRO == PRO_NORM) {
    // every block adds up the table the same way: 32 strided partial sums per row, then those in order
    __shared__ float stat_part[32][SK_STAT_ROWS];
    __shared__ float stat_inv[SK_STAT_ROWS];
    {
      const int row = threadIdx.x % SK_STAT_ROWS, part = threadIdx.x / SK_STAT_ROWS;  // 512 threads: 32 parts
      float sum = 0.f;
      for (int slot = part; slot < p.stats_slots; slot += 32) sum += p.stats_in[slot * SK_STAT_ROWS + row];
      stat_part[part][row] = sum;
    }
    __syncthreads();
    if (threadIdx.x < SK_STAT_ROWS) {
      float total = 0.f;
#pragma unroll
      for (int part = 0; part < 32; ++part) total += stat_part[part][threadIdx.x];
      stat_inv[threadIdx.x] = rsqrtf(total / (float)k + p.eps);
    }
    __syncthreads();
    inv_rms = stat_inv[a_row];
  }

  // the activation operand of k-step s
  auto load_plain = [&](int s) -> bf16x8_t { return *reinterpret_cast<const bf16x8_t*>(ap + (int64_t)s * 32); };
  struct RawNorm {
    f32x4_t lo, hi;
    bf16x8_t g;
  };
  auto load_norm = [&](int s) -> RawNorm {
    RawNorm r;
    r.lo = *reinterpret_cast<const f32x4_t*>(xp + (int64_t)s * 32);
    r.hi = *reinterpret_cast<const f32x4_t*>(xp + (int64_t)s * 32 + 4);
    r.g = *reinterpret_cast<const bf16x8_t*>(gp + (int64_t)s * 32);
    return r;
  };
  auto finish_norm = [&](const RawNorm& r) -> bf16x8_t {
    bf16x8_t out;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[i] = (bf16_t)((float)r.g[i] * (r.lo[i] * inv_rms));
      out[4 + i] = (bf16_t)((float)r.g[4 + i] * (r.hi[i] * inv_rms));
    }
    return out;
  };

  f32x4_t acc[WT];
#pragma unroll
  for (int t = 0; t < WT; ++t) acc[t] = (f32x4_t){0.f, 0.f, 0.f, 0.f};

  int s = s_begin;
  for (; s + U <= s_end; s += U) {
    bf16x8_t w_reg[U][WT];
    bf16x8_t a_reg[U];
    RawNorm raw[PRO == PRO_NORM ? U : 1];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < WT; ++t)
        w_reg[u][t] = *reinterpret_cast<const bf16x8_t*>(wp[t] + (int64_t)(s + u) * 32);
      if (PRO == PRO_NORM) raw[u] = load_norm(s + u);
      else a_reg[u] = load_plain(s + u);
    }
    if (PRO == PRO_NORM) {
#pragma unroll
      for (int u = 0; u < U; ++u) a_reg[u] = finish_norm(raw[u]);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < WT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_reg[u][t], a_reg[u], acc[t], 0, 0, 0);
  }
  for (; s < s_end; ++s) {  // fewer than U k-steps left
    const bf16x8_t a_tail = (PRO == PRO_NORM) ? finish_norm(load_norm(s)) : load_plain(s);
#pragma unroll
    for (int t = 0; t < WT; ++t) {
      const bf16x8_t w_tail = *reinterpret_cast<const bf16x8_t*>(wp[t] + (int64_t)s * 32);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_tail, a_tail, acc[t], 0, 0, 0);
    }
  }

  // acc[t][r] = C^T[feature n0 + 16*(t % NT) + 4*quad + r][token col]; add the 8 waves in order
#pragma unroll
  for (int t = 0; t < WT; ++t) {
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][t][(quad * 4 + r) * 16 + col] = acc[t][r];
  }
  __syncthreads();
  // 256*NT outputs, each a sum of 8 (two such when gated): a thread takes 4 consecutive
  // features of one token (NT*64 <= 256 threads have work)
  static_assert(NT * 64 <= 64 * SK_WAVES, "one output item per thread at most");
  __shared__ float square_part[EPI == EPI_RESIDUAL ? NT * 4 : 1][SK_STAT_ROWS];
  const int item = threadIdx.x;
  const int nt = item / 64;
  const int token = (item % 64) % 16;
  const int fq = (item % 64) / 16;
  if (item < NT * 64 && token < m) {
    float sum[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int wv = 0; wv < SK_WAVES; ++wv)
#pragma unroll
      for (int r = 0; r < 4; ++r) sum[r] += red[wv][nt][(fq * 4 + r) * 16 + token];
    if (EPI == EPI_GATED) {
      float up[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int wv = 0; wv < SK_WAVES; ++wv)
#pragma unroll
        for (int r = 0; r < 4; ++r) up[r] += red[wv][NT + nt][(fq * 4 + r) * 16 + token];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float g = (float)(bf16_t)sum[r];
        sum[r] = g / (1.f + expf(-g)) * (float)(bf16_t)up[r];
      }
    }
    const int feature = n0 + nt * 16 + fq * 4;
    if (EPI == EPI_RESIDUAL) {
      float* dst = p.residual + (int64_t)token * p.ld_out + feature;
      float squares = 0.f;
      if (feature + 3 < n_end && (p.ld_out % 4 == 0)) {
        f32x4_t x = *reinterpret_cast<const f32x4_t*>(dst);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          x[r] += (float)(bf16_t)sum[r];
          squares += x[r] * x[r];
        }
        *reinterpret_cast<f32x4_t*>(dst) = x;
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          if (feature + r < n_end) {
            const float x = dst[r] + (float)(bf16_t)sum[r];
            dst[r] = x;
            squares += x * x;
          }
        }
      }
      square_part[nt * 4 + fq][token] = squares;
    } else {
      bf16_t* dst = p.c + (int64_t)token * p.ld_out + feature;
      if (feature + 3 < n_end && (p.ld_out % 4 == 0)) {
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
  }
  if (EPI == EPI_RESIDUAL) {
    __syncthreads();
    if (threadIdx.x < SK_STAT_ROWS) {
      float total = 0.f;
      if ((int)threadIdx.x < m) {
#pragma unroll
        for (int i = 0; i < NT * 4; ++i) total += square_part[i][threadIdx.x];
      }
      p.stats_out[(int64_t)blockIdx.x * SK_STAT_ROWS + threadIdx.x] = total;  // rows past m: 0
    }
  }
}

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

extern "C" int mi_gemm_skinny_bf16_supported(int m, int n, int k, int64_t lda, int64_t ldw) {
  return (m >= 1 && m <= SK_MAX_ROWS && n >= 1 && k >= 32 && k % 32 == 0 && lda % 8 == 0 && ldw % 8 == 0) ? 1 : 0;
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

static int max_tiles_for(int epilogue) { return epilogue == EPI_GATED ? 2 : 4; }  // gated: two weight tiles per output tile

// Blocks the product of n output features will run as = entries of the sum-of-squares
// table an EPI_RESIDUAL product writes.  0 if the device cannot be asked.
extern "C" int mi_gemm_skinny_blocks(int n, int epilogue) {
  const int cus = compute_units();
  if (cus <= 0 || n <= 0) return 0;
  return ceil_div(n, features_per_block_for(n, cus, max_tiles_for(epilogue)));
}

// The general entry point.  `in` is a[m, k] bfloat16 (prologue 0) or the float32 residual
// x[m, k] (prologue 1, with norm_weight[k], stats_in[stats_slots][16] and eps); `out` is
// c[m, n] bfloat16 (epilogue 0 and 1) or the float32 residual [m, n] to add into (epilogue
// 2, with stats_out[mi_gemm_skinny_blocks(n, 2)][16]).  w is [n, k], or [2n, k] when gated.
extern "C" int mi_gemm_skinny_fused_bf16(int prologue, int epilogue, const void* in, int64_t ld_in,
                                         const void* norm_weight, const float* stats_in, int stats_slots,
                                         float eps, const void* w, int64_t ldw, void* out, int64_t ld_out,
                                         float* stats_out, int m, int n, int k, hipStream_t stream) {
  MI_REQUIRE(prologue == PRO_PLAIN || prologue == PRO_NORM, "gemm_skinny: unknown prologue %d", prologue);
  MI_REQUIRE(epilogue >= EPI_STORE && epilogue <= EPI_RESIDUAL, "gemm_skinny: unknown epilogue %d", epilogue);
  MI_REQUIRE(!(prologue == PRO_NORM && epilogue == EPI_RESIDUAL), "gemm_skinny: norm prologue with residual epilogue is not built");
  MI_REQUIRE(m >= 1 && m <= SK_MAX_ROWS && n >= 1 && k >= 32 && k % 32 == 0,
             "gemm_skinny: takes 1 <= m <= 16 and k a multiple of 32; got m=%d n=%d k=%d", m, n, k);
  MI_REQUIRE(ldw % 8 == 0 && ldw >= k, "gemm_skinny: weight rows must be 16-byte aligned and hold k; ldw=%lld", (long long)ldw);
  MI_REQUIRE(ld_in >= k && ld_in % (prologue == PRO_NORM ? 4 : 8) == 0,
             "gemm_skinny: input rows must be 16-byte aligned and hold k; ld=%lld", (long long)ld_in);
  MI_REQUIRE(ld_out >= n, "gemm_skinny: output rows are shorter than n; ld=%lld", (long long)ld_out);
  MI_REQUIRE(in && w && out, "gemm_skinny: null operand");
  if (prologue == PRO_NORM) {
    MI_REQUIRE(norm_weight && stats_in && stats_slots >= 1, "gemm_skinny: the norm prologue needs its weight and the sums of squares");
  }
  if (epilogue == EPI_RESIDUAL) MI_REQUIRE(stats_out != nullptr, "gemm_skinny: the residual epilogue needs a table for the sums of squares");
  const int cus = compute_units();
  MI_REQUIRE(cus > 0, "gemm_skinny: cannot read the device's compute unit count");
  SkinnyArgs p;
  p.a = prologue == PRO_PLAIN ? (const bf16_t*)in : nullptr;
  p.x = prologue == PRO_NORM ? (const float*)in : nullptr;
  p.ld_in = ld_in;
  p.norm_weight = (const bf16_t*)norm_weight;
  p.stats_in = stats_in;
  p.stats_slots = stats_slots;
  p.eps = eps;
  p.w = (const bf16_t*)w;
  p.ldw = ldw;
  p.c = epilogue == EPI_RESIDUAL ? nullptr : (bf16_t*)out;
  p.residual = epilogue == EPI_RESIDUAL ? (float*)out : nullptr;
  p.ld_out = ld_out;
  p.stats_out = stats_out;
  p.m = m;
  p.n = n;
  p.k = k;
  p.features_per_block = features_per_block_for(n, cus, max_tiles_for(epilogue));
  const int blocks = ceil_div(n, p.features_per_block);
  const int threads = 64 * SK_WAVES;
  const int tiles = ceil_div(p.features_per_block, 16);
#define SK_LAUNCH(NT_, U_, PRO_, EPI_) gemm_skinny_bf16_kernel<NT_, U_, PRO_, EPI_><<<blocks, threads, 0, stream>>>(p)
  if (epilogue == EPI_GATED) {
    if (prologue == PRO_NORM) {
      if (tiles == 1) SK_LAUNCH(1, 4, PRO_NORM, EPI_GATED); else SK_LAUNCH(2, 2, PRO_NORM, EPI_GATED);
    } else {
      if (tiles == 1) SK_LAUNCH(1, 4, PRO_PLAIN, EPI_GATED); else SK_LAUNCH(2, 2, PRO_PLAIN, EPI_GATED);
    }
  } else if (epilogue == EPI_RESIDUAL) {
    switch (tiles) {
      case 1: SK_LAUNCH(1, 8, PRO_PLAIN, EPI_RESIDUAL); break;
      case 2: SK_LAUNCH(2, 8, PRO_PLAIN, EPI_RESIDUAL); break;
      case 3: SK_LAUNCH(3, 4, PRO_PLAIN, EPI_RESIDUAL); break;
      default: SK_LAUNCH(4, 2, PRO_PLAIN, EPI_RESIDUAL); break;
    }
  } else if (prologue == PRO_NORM) {
    switch (tiles) {  // fewer k-steps in flight: the float32 rows take three registers where bfloat16 takes one
      case 1: SK_LAUNCH(1, 4, PRO_NORM, EPI_STORE); break;
      case 2: SK_LAUNCH(2, 4, PRO_NORM, EPI_STORE); break;
      case 3: SK_LAUNCH(3, 2, PRO_NORM, EPI_STORE); break;
      default: SK_LAUNCH(4, 2, PRO_NORM, EPI_STORE); break;
    }
  } else {
    switch (tiles) {
      case 1: SK_LAUNCH(1, 8, PRO_PLAIN, EPI_STORE); break;
      case 2: SK_LAUNCH(2, 8, PRO_PLAIN, EPI_STORE); break;
      case 3: SK_LAUNCH(3, 4, PRO_PLAIN, EPI_STORE); break;
      default: SK_LAUNCH(4, 2, PRO_PLAIN, EPI_STORE); break;
    }
  }
#undef SK_LAUNCH
  MI_CHECK_LAUNCH("gemm_skinny");
  return MI_OK;
}

extern "C" int mi_gemm_skinny_bf16(const void* a, int64_t lda, const void* w, int64_t ldw, void* c,
                                   int64_t ldc, int m, int n, int k, hipStream_t stream) {
  return mi_gemm_skinny_fused_bf16(PRO_PLAIN, EPI_STORE, a, lda, nullptr, nullptr, 0, 0.f, w, ldw, c, ldc,
                                   nullptr, m, n, k, stream);
}

// out[m, n] = silu(a . gate^T) * (a . up^T) with w = [gate; up] stacked, [2n, k].
extern "C" int mi_gemm_skinny_swiglu_bf16(const void* a, int64_t lda, const void* w, int64_t ldw, void* out,
                                          int64_t ldo, int m, int n, int k, hipStream_t stream) {
  return mi_gemm_skinny_fused_bf16(PRO_PLAIN, EPI_GATED, a, lda, nullptr, nullptr, 0, 0.f, w, ldw, out, ldo,
                                   nullptr, m, n, k, stream);
}
