// Matrix products y = x * W^T (+ bias) for gfx950, W stored [N, K] row-major as checkpoints
// hold it.
//  * cw_gemm_f32: true float32 (VALU FMA, float32 operands and accumulation, no reduced-precision
//    matrix mode). The order in which the products of one output element are summed depends on N
//    and K alone, never on M, so a row's result does not depend on what else is in the batch.
#include "common.h"

#define GT_BM 64
#define GT_BN 64
#define GT_BK 16

// C[M, N] = A[M, K] * W[N, K]^T + bias[N]. 256 threads, each a 4x4 tile of a 64x64 block.
// K is summed in ``splits`` parts of k_per_split values (a multiple of 16), and the parts in their
// order: ((p_0 + p_1) + ...) + bias. gridDim.z == 1: a block does so by itself. gridDim.z ==
// splits: block z makes part z alone and writes it to C + z * part_stride (no bias), and
// gemm_f32_sum_kernel adds the parts up in the same order, so both ways give the same bits.
// ONE_PART: a block makes one part (gridDim.z == splits, or there is only one part).
template <bool ONE_PART>
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ A, int64_t lda,
                                                       const float* __restrict__ W,
                                                       const float* __restrict__ bias,
                                                       float* __restrict__ C, int64_t ldc, int M,
                                                       int N, int K, int splits, int k_per_split,
                                                       int64_t part_stride) {
  __shared__ float As[GT_BK][GT_BM + 4];
  __shared__ float Ws[GT_BK][GT_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * GT_BM, n0 = blockIdx.x * GT_BN;
  const bool parallel = gridDim.z > 1;  // part blockIdx.z of several
  const int z_first = ONE_PART ? blockIdx.z : 0, z_last = ONE_PART ? blockIdx.z : splits - 1;
  float total[4][4];
  // each thread loads 4 elements of A and 4 of W per K step: row = tid / 4, k = (tid % 4) * 4 .. +3
  const int lr = tid >> 2, lk = (tid & 3) * 4;
  const bool k_vec_ok = (K % 4 == 0) && (lda % 4 == 0);
  for (int z = z_first; z <= z_last; ++z) {
  const int k_begin = z * k_per_split;
  const int k_end = min(K, k_begin + k_per_split);
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
  for (int k0 = k_begin; k0 < k_end; k0 += GT_BK) {
    {
      const int m = m0 + lr, k = k0 + lk;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (m < M) {
        const float* p = A + (int64_t)m * lda + k;
        if (k_vec_ok && k + 3 < k_end) {
          const float4 q = *reinterpret_cast<const float4*>(p);
          v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) if (k + j < k_end) v[j] = p[j];
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) As[lk + j][lr] = v[j];
    }
    {
      const int n = n0 + lr, k = k0 + lk;
      float v[4] = {0.f, 0.f, 0.f, 0.f};
      if (n < N) {
        const float* p = W + (int64_t)n * K + k;
        if (K % 4 == 0 && k + 3 < k_end) {
          const float4 q = *reinterpret_cast<const float4*>(p);
          v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) if (k + j < k_end) v[j] = p[j];
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) Ws[lk + j][lr] = v[j];
    }
    __syncthreads();
    // the 16 products of a K step are summed on their own and then added to the total: a long K
    // (8960 in a feed-forward) then rounds about sqrt(16) + sqrt(K / 16) times instead of sqrt(K)
    float part[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) part[i][j] = 0.0f;
#pragma unroll
    for (int kk = 0; kk < GT_BK; ++kk) {
      const float4 a = *reinterpret_cast<const float4*>(&As[kk][ty * 4]);
      const float4 w = *reinterpret_cast<const float4*>(&Ws[kk][tx * 4]);
      const float av[4] = {a.x, a.y, a.z, a.w};
      const float wv[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(av[i], wv[j], part[i][j]);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] += part[i][j];
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) total[i][j] = (ONE_PART || z == z_first) ? acc[i][j] : total[i][j] + acc[i][j];
  }
  float* out = parallel ? C + (int64_t)blockIdx.z * part_stride : C;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) out[(int64_t)m * ldc + n] = total[i][j] + (bias && !parallel ? bias[n] : 0.0f);
    }
  }
}

// C[m, n] = ((p_0 + p_1) + ... + p_{splits-1}) + bias[n] over the partial sums p_z[m, n] (rows of N
// floats, part_stride floats between two splits): always in the order of the splits.
__global__ __launch_bounds__(256) void gemm_f32_sum_kernel(const float* __restrict__ parts, int splits,
                                                           int64_t part_stride, const float* __restrict__ bias,
                                                           float* __restrict__ C, int64_t ldc, int rows, int N) {
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)rows * N) return;
  const int m = (int)(idx / N), n = (int)(idx - (int64_t)m * N);
  float total = parts[idx];
  for (int z = 1; z < splits; ++z) total += parts[z * part_stride + idx];
  C[(int64_t)m * ldc + n] = total + (bias ? bias[n] : 0.0f);
}

// Up to this many rows of x the parts of K are made by blocks of their own (beyond, there are
// blocks enough without, and a block sums its parts itself).
#define GT_SPLIT_ROWS 256

// How the float32 product cuts K for an [N, K] weight matrix: a narrow output (24 blocks of 64
// columns for a width of 1536) with few rows of x would leave most compute units without work and
// stream the matrix through the few that have some, so K is cut until there are about 512 blocks
// per 64 rows, with at least 256 values of K each. A function of N and K alone: the order of the
// sums must not depend on how many rows the step has.
static void gemm_f32_plan(int N, int K, int* splits, int* k_per_split) {
  const int col_blocks = (N + GT_BN - 1) / GT_BN;
  int s = (512 + col_blocks / 2) / col_blocks;
  if (s > K / 256) s = K / 256;
  if (s < 1) s = 1;
  const int per = ((K + s - 1) / s + GT_BK - 1) / GT_BK * GT_BK;
  *k_per_split = per;
  *splits = (K + per - 1) / per;
}

// Floats of workspace cw_gemm_f32 needs for this product (0: none).
CW_EXPORT int64_t cw_gemm_f32_workspace_floats(int M, int N, int K) {
  int splits, per;
  if (M <= 0 || M > GT_SPLIT_ROWS || N <= 0 || K <= 0) return 0;
  gemm_f32_plan(N, K, &splits, &per);
  return splits <= 1 ? 0 : (int64_t)splits * M * N;
}

CW_EXPORT int cw_gemm_f32(const float* A, int64_t lda, const float* W, const float* bias, float* C,
                          int64_t ldc, int M, int N, int K, float* workspace, int64_t workspace_floats,
                          hipStream_t stream) {
  if (M < 0 || N <= 0 || K <= 0 || lda < K || ldc < N) return CW_ERR_ARG;
  if (M == 0) return CW_OK;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return CW_ERR_ARG;
  int splits, per;
  gemm_f32_plan(N, K, &splits, &per);
  const dim3 block(256);
  dim3 grid((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM);
  if (grid.y > 65535) return CW_ERR_SIZE;
  if (splits <= 1) {
    hipLaunchKernelGGL(gemm_f32_kernel<true>, grid, block, 0, stream, A, lda, W, bias, C, ldc, M, N, K, 1, per, (int64_t)0);
    return cw_launch_status();
  }
  if (M > GT_SPLIT_ROWS) {
    hipLaunchKernelGGL(gemm_f32_kernel<false>, grid, block, 0, stream, A, lda, W, bias, C, ldc, M, N, K, splits, per,
                       (int64_t)0);
    return cw_launch_status();
  }
  const int64_t part_stride = (int64_t)M * N;
  if (workspace == nullptr || workspace_floats < splits * part_stride) return CW_ERR_ARG;
  grid.z = splits;
  hipLaunchKernelGGL(gemm_f32_kernel<true>, grid, block, 0, stream, A, lda, W, nullptr, workspace, (int64_t)N, M, N, K,
                     splits, per, part_stride);
  hipLaunchKernelGGL(gemm_f32_sum_kernel, dim3((unsigned)((part_stride + 255) / 256)), block, 0, stream, workspace,
                     splits, part_stride, bias, C, ldc, M, N);
  return cw_launch_status();
}

// =====================================================================================
// bfloat16 products with few rows of x (decode: 1 to 64 tokens): the weight matrix is streamed
// once at memory speed. A workgroup of WAVES waves owns RT * 16 weight rows; its waves split the K
// loop and are summed through LDS at the end, in a fixed order (no atomics: the result does not
// depend on timing). Few weight rows (a narrow output) get more waves each, so that enough loads
// are in flight on every compute unit that has work.
// Each wave feeds 16 weight rows x 32 k-values to one MFMA (v_mfma_f32_16x16x32_bf16) as the A
// operand, loaded from global memory directly in operand layout (lane = row l%16, 8 consecutive
// k at slot l/16), and 16 tokens x the same k-values as the B operand.
//
// MODE 0: y bfloat16 [M, N]; MODE 1: y float32 [M, N] (logits); MODE 2: W is [2I, K] with gate
// rows first, y[m, i] = silu(gate_i) * up_i as bfloat16 [M, I]: a row tile holds 8 gate rows and
// the 8 up rows that belong to them. MODE 3: K is also split over gridDim.y workgroups, each
// writing its float32 partial product [split, M, N]; whoever reads y next sums the partials in
// order (the residual-add + norm kernel does): a narrow output with a long K (96 row tiles for
// 27 MB of weights) then streams on all compute units instead of 96.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// How these kernels load operands. An MFMA operand wants lane l to hold row l % 16 of a tile and
// the 8 k-values of slot l / 16: loaded that way every lane asks for 16 bytes of a row of its own,
// 64 requests an instruction to a compute unit's load path, which takes in about 30 GB/s of such.
// So a lane loads row l / 4, slot l % 4 instead (four neighbouring lanes cover 64 bytes of one row:
// 16 requests an instruction), and the lanes swap what they hold afterwards, lane (r, s) taking
// from lane 4 r + s (ds_bpermute: through the LDS unit's crossbar, no memory). Measured on the
// 1.5B shape's gate/up product: 12.8 -> 11.7 us with 8 rows of x, 19.8 -> 17.5 us with 64.
typedef __attribute__((ext_vector_type(4))) int cw_i32x4_t;
__device__ __forceinline__ bf16x8_t cw_to_operand_layout(const bf16x8_t& v, int lane) {
  const int r = lane & 15, s = lane >> 4;
  const int from = (r * 4 + s) * 4;  // byte address of the lane that loaded what lane (r, s) multiplies
  const cw_i32x4_t q = __builtin_bit_cast(cw_i32x4_t, v);
  cw_i32x4_t t;
#pragma unroll
  for (int d = 0; d < 4; ++d) t[d] = __builtin_amdgcn_ds_bpermute(from, q[d]);
  return __builtin_bit_cast(bf16x8_t, t);
}

// ROWS (16, 8 or 4) is the number of weight rows a tile really holds: a narrow output with a long K
// is cut into more, smaller tiles so that every compute unit streams a share of the matrix (the
// unused rows of the MFMA tile are zeros). MODE 2 needs ROWS == 16.
template <int MT, int RT, int MODE, int WAVES, int ROWS>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_bf16_kernel(const bf16_t* __restrict__ X, int64_t ldx,
                                                               const bf16_t* __restrict__ W,
                                                               void* __restrict__ C, int64_t ldc,
                                                               int M, int N, int K) {
  __shared__ float red[WAVES][RT * MT * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, s = lane >> 4;
  const int lr = lane >> 2, ls = lane & 3;  // the row of a tile and the slot of a k-step that this lane loads
  const int I = N / 2;  // MODE 2 only

  // weight rows that this lane loads, one per row tile
  const bf16_t* wrow[RT];
  bool wok[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    int64_t n;
    if (MODE == 2) {
      const int64_t i = ((int64_t)blockIdx.x * RT + rt) * 8 + (lr & 7);
      n = (lr < 8) ? i : I + i;
      wok[rt] = i < I;
    } else {
      n = ((int64_t)blockIdx.x * RT + rt) * ROWS + lr;
      wok[rt] = lr < ROWS && n < N;
    }
    wrow[rt] = W + (wok[rt] ? n : 0) * K;
  }
  // x: one tile of tokens is few bytes beside the weights and is loaded in operand layout as it is
  // (a swap would only add to the wait before the first product); several tiles are loaded like the weights
  constexpr bool X_SWAP = MT > 1;
  const int xr = X_SWAP ? lr : r, xs = X_SWAP ? ls : s;
  const bf16_t* xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + xr;
    xok[mt] = m < M;
    xrow[mt] = X + (int64_t)(xok[mt] ? m : 0) * ldx;
  }

  f32x4_t acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[rt][mt] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};

  bf16x8_t zero;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero[e] = (__bf16)0.0f;

  const int k_steps = (K + 31) / 32;
  constexpr int U = 4;  // k-steps in flight per wave
  const int n_ksplit = MODE == 3 ? gridDim.y : 1;
  for (int ks0 = ((MODE == 3 ? blockIdx.y : 0) * WAVES + wave) * U; ks0 < k_steps; ks0 += n_ksplit * WAVES * U) {
    bf16x8_t wf[U][RT], xf[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (ks0 + u) * 32 + ls * 8;
      const bool kok = (ks0 + u) < k_steps && k + 8 <= K;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
        wf[u][rt] = (kok && wok[rt]) ? *reinterpret_cast<const bf16x8_t*>(wrow[rt] + k) : zero;
      const int kx = (ks0 + u) * 32 + xs * 8;
      const bool kxok = (ks0 + u) < k_steps && kx + 8 <= K;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        xf[u][mt] = (kxok && xok[mt]) ? *reinterpret_cast<const bf16x8_t*>(xrow[mt] + kx) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      bf16x8_t xo[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) xo[mt] = X_SWAP ? cw_to_operand_layout(xf[u][mt], lane) : xf[u][mt];
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const bf16x8_t wo = cw_to_operand_layout(wf[u][rt], lane);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[rt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wo, xo[mt], acc[rt][mt], 0, 0, 0);
      }
    }
  }

  // D tile of (rt, mt): lane (r, s) holds weight rows 4s..4s+3 of token r -> red[wave][tile][row][token]
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][(rt * MT + mt) * 256 + (4 * s + i) * 16 + r] = acc[rt][mt][i];
  __syncthreads();
  for (int idx = threadIdx.x; idx < RT * MT * 256; idx += WAVES * 64) {
    float sum = red[0][idx];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) sum += red[w][idx];
    red[0][idx] = sum;
  }
  __syncthreads();

  if (MODE == 2) {
    // outputs: 8 per row tile and token; idx -> (token, rt, j) with j fastest
    for (int idx = threadIdx.x; idx < RT * MT * 128; idx += WAVES * 64) {
      const int j = idx & 7, rt = (idx >> 3) % RT, m = idx / (8 * RT);
      const int mt = m >> 4, tok = m & 15;
      const int64_t i = ((int64_t)blockIdx.x * RT + rt) * 8 + j;
      if (m >= M || i >= I) continue;
      const float g = red[0][(rt * MT + mt) * 256 + j * 16 + tok];
      const float u = red[0][(rt * MT + mt) * 256 + (j + 8) * 16 + tok];
      ((bf16_t*)C)[(int64_t)m * ldc + i] = __float2bfloat16(g / (1.0f + __expf(-g)) * u);
    }
  } else {
    for (int idx = threadIdx.x; idx < RT * MT * 256; idx += WAVES * 64) {
      const int j = idx & 15, rt = (idx >> 4) % RT, m = idx / (16 * RT);
      const int mt = m >> 4, tok = m & 15;
      const int64_t n = ((int64_t)blockIdx.x * RT + rt) * ROWS + j;
      if (m >= M || n >= N || j >= ROWS) continue;
      const float v = red[0][(rt * MT + mt) * 256 + j * 16 + tok];
      if (MODE == 3) ((float*)C)[((int64_t)blockIdx.y * M + m) * ldc + n] = v;
      else if (MODE == 1) ((float*)C)[(int64_t)m * ldc + n] = v;
      else ((bf16_t*)C)[(int64_t)m * ldc + n] = __float2bfloat16(v);
    }
  }
}

// The same product with the x fragments of a wave's whole share of the K loop (up to 24 steps of
// 32, as many as its registers hold beside MT tiles of 16 tokens) kept in registers for good, so
// that only weights move.
// A workgroup walks over row tiles blockIdx.x, blockIdx.x + gridDim.x, ...; the weights of its
// next tile are on their way while the current one is reduced through LDS (one barrier per tile
// while the reduction buffer can be doubled, two for MT = 4). Loads are never conditional: a row
// or k-step outside the matrix reads a valid address instead and meets zeros in x or is not
// stored, which lets the compiler wait for exactly the loads a product needs. Wave w of k-split
// blockIdx.y owns k-steps [(blockIdx.y * WAVES + w) * SPW, + SPW). Modes and layouts as in
// gemm_skinny_bf16_kernel.
// NORM (MT = 1, no k-split): x is not read but made here, x = rmsnorm(resid + delta) * weight over
// the K elements of a row, with the rounding steps of the stand-alone norm kernel; every
// workgroup does so for itself (the rows are few and come from L2), nothing is written back.
struct StreamNormIn {
  const float* resid;    // [M, K] float32
  const bf16_t* delta;   // [M, K] bfloat16
  const void* weight;    // [K] bfloat16 or float32
  int weight_f32;
  float eps;
};

// Weight fragments of a tile are fetched CH steps at a time (two sets in flight), while the x
// fragments of all SPW steps stay in registers: a long K costs registers for x only.
constexpr int cw_stream_chunk(int spw) { return spw <= 8 ? spw : (spw <= 12 ? spw / 2 : spw / 4); }

template <int MODE, int WAVES, int SPW, int MT, bool NORM = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_stream_bf16_kernel(const bf16_t* __restrict__ X, int64_t ldx,
                                                               const bf16_t* __restrict__ W,
                                                               void* __restrict__ C, int64_t ldc,
                                                               int M, int N, int K, int n_tiles, StreamNormIn nin) {
  constexpr int NBUF = MT <= 2 ? 2 : 1;
  constexpr int CH = cw_stream_chunk(SPW), NC = SPW / CH;
  static_assert(SPW % CH == 0, "the steps of a wave are whole chunks");
  __shared__ __align__(16) float red[NBUF][WAVES][MT * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, s = lane >> 4;
  const int I = N / 2;  // MODE 2 only

  // Loads as cw_to_operand_layout describes: this lane loads row lr of a tile, slot ls of a k-step.
  const int lr = lane >> 2, ls = lane & 3;
  auto to_operand = [&](const bf16x8_t& v) __attribute__((always_inline)) -> bf16x8_t {
    return cw_to_operand_layout(v, lane);
  };
  int koff[SPW];  // the loading lane's 8 k-values of each step; a step outside K reads k = 0 and meets zeros in x
#pragma unroll
  for (int u = 0; u < SPW; ++u) {
    const int k = ((blockIdx.y * WAVES + wave) * SPW + u) * 32 + ls * 8;
    koff[u] = k + 8 <= K ? k : 0;
  }
  auto wrow = [&](int tile) __attribute__((always_inline)) -> const bf16_t* {
    int64_t n;
    if (MODE == 2) {  // gate and up rows alternate, so that a pair lies side by side in the tile
      const int64_t i = min((int64_t)tile * 8 + (lr >> 1), (int64_t)I - 1);
      n = (lr & 1) ? I + i : i;
    } else {
      n = min((int64_t)tile * 16 + lr, (int64_t)N - 1);
    }
    return W + n * K;
  };
  // the first tile's weights are requested before anything else: x, and with NORM the norm's
  // statistics, are fetched in their shadow
  int tile = blockIdx.x;
  bf16x8_t cur[CH], nxt[CH];
  const bf16_t* w_tile = wrow(tile);
#pragma unroll
  for (int u = 0; u < CH; ++u) cur[u] = *reinterpret_cast<const bf16x8_t*>(w_tile + koff[u]);

  bf16x8_t xf[SPW][MT];
  if constexpr (NORM) {
    static_assert(MT == 1 && SPW <= 4, "the fused norm serves one tile of tokens and rows of up to 2048 elements");
    __shared__ float ssq[WAVES][16];
    float v[SPW][8], wv[SPW][8];  // resid + delta and the norm weight at the lane's elements
    float ss = 0.0f;
#pragma unroll
    for (int u = 0; u < SPW; ++u) {
      const int k = (wave * SPW + u) * 32 + s * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) v[u][e] = wv[u][e] = 0.0f;
      if (k + 8 <= K && r < M) {
        const float4 a = *reinterpret_cast<const float4*>(nin.resid + (int64_t)r * K + k);
        const float4 b = *reinterpret_cast<const float4*>(nin.resid + (int64_t)r * K + k + 4);
        const bf16x8_t d = *reinterpret_cast<const bf16x8_t*>(nin.delta + (int64_t)r * K + k);
        v[u][0] = a.x + (float)d[0]; v[u][1] = a.y + (float)d[1]; v[u][2] = a.z + (float)d[2]; v[u][3] = a.w + (float)d[3];
        v[u][4] = b.x + (float)d[4]; v[u][5] = b.y + (float)d[5]; v[u][6] = b.z + (float)d[6]; v[u][7] = b.w + (float)d[7];
        if (nin.weight_f32) {
          const float4 w0 = *reinterpret_cast<const float4*>((const float*)nin.weight + k);
          const float4 w1 = *reinterpret_cast<const float4*>((const float*)nin.weight + k + 4);
          wv[u][0] = w0.x; wv[u][1] = w0.y; wv[u][2] = w0.z; wv[u][3] = w0.w;
          wv[u][4] = w1.x; wv[u][5] = w1.y; wv[u][6] = w1.z; wv[u][7] = w1.w;
        } else {
          const bf16x8_t w8 = *reinterpret_cast<const bf16x8_t*>((const bf16_t*)nin.weight + k);
#pragma unroll
          for (int e = 0; e < 8; ++e) wv[u][e] = (float)w8[e];
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += v[u][e] * v[u][e];
      }
    }
    ss = cw_quad_sum(ss);
    if (s == 0) ssq[wave][r] = ss;
    __syncthreads();
    float total = 0.0f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) total += ssq[w][r];
    const float inv = 1.0f / sqrtf(total / (float)K + nin.eps);
#pragma unroll
    for (int u = 0; u < SPW; ++u)
#pragma unroll
      for (int e = 0; e < 8; ++e) xf[u][0][e] = (__bf16)(wv[u][e] * (float)(__bf16)(v[u][e] * inv));
  } else {
    // Every workgroup pulls all of x from L2 (with 64 rows that is as many bytes as its weights),
    // loaded like the weights, four lanes to a row's step, and swapped into operand layout. The
    // loads are unconditional, from clamped addresses; what lies past M or K is zeroed first.
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + lr;
      const bf16_t* xrow = X + (int64_t)min(m, M - 1) * ldx;
#pragma unroll
      for (int u = 0; u < SPW; ++u) {
        const bool ok = ((blockIdx.y * WAVES + wave) * SPW + u) * 32 + ls * 8 + 8 <= K && m < M;
        bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(xrow + koff[u]);
        if (!ok) {
#pragma unroll
          for (int e = 0; e < 8; ++e) v[e] = (__bf16)0.0f;
        }
        xf[u][mt] = to_operand(v);
      }
    }
  }
  // what the waves' partial tiles of ``tile`` (in red[buf]) become: summed over the waves, then
  // stored as the mode says. One barrier before; a second after, when the buffer is not doubled.
  auto finish_tile = [&](const f32x4_t (&acc)[MT], int tile, int buf) __attribute__((always_inline)) {
    // lane (r, s) holds weight rows 4s..4s+3 of token r of tile mt -> red[buf][wave][mt][token][row]:
    // one 16-byte store a lane, the lanes of a wave side by side (no bank is hit twice)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      *reinterpret_cast<f32x4_t*>(&red[buf][wave][mt * 256 + r * 16 + 4 * s]) = acc[mt];
    cw_lds_barrier();  // not __syncthreads(): the next tile's weights stay in flight across it
    if (MODE == 2) {
      if (threadIdx.x < MT * 128) {  // (token, j): the gate and the up value of output j are neighbours
        const int j = threadIdx.x & 7, m = threadIdx.x >> 3;
        float g = 0.0f, up = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
          const float2 gu = *reinterpret_cast<const float2*>(&red[buf][w][m * 16 + 2 * j]);
          g += gu.x;
          up += gu.y;
        }
        const int64_t i = (int64_t)tile * 8 + j;
        if (m < M && i < I) ((bf16_t*)C)[(int64_t)m * ldc + i] = __float2bfloat16(g / (1.0f + __expf(-g)) * up);
      }
    } else {
      for (int idx = threadIdx.x; idx < MT * 256; idx += WAVES * 64) {  // (token, j): 16 outputs side by side
        const int j = idx & 15, m = idx >> 4;
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) v += red[buf][w][idx];
        const int64_t n = (int64_t)tile * 16 + j;
        if (m < M && n < N) {
          if (MODE == 3) ((float*)C)[((int64_t)blockIdx.y * M + m) * ldc + n] = v;
          else if (MODE == 1) ((float*)C)[(int64_t)m * ldc + n] = v;
          else ((bf16_t*)C)[(int64_t)m * ldc + n] = __float2bfloat16(v);
        }
      }
    }
    if (NBUF == 1) cw_lds_barrier();
  };
  int buf = 0;
  if constexpr (NC == 1) {
    // A wave's whole share of a tile is one set of fragments. Two sets take turns, without a
    // copy between them (a copy has to wait for the loads it copies): the loads of the tile
    // after this one are issued before this tile's products and are waited for only when their
    // own products begin, so they are in flight during the whole of this tile's products,
    // reduction and stores. Past the last tile a valid address is read and dropped.
    auto load_set = [&](bf16x8_t (&dst)[CH], int t) __attribute__((always_inline)) {
      const bf16_t* w = wrow(min(t, n_tiles - 1));
#pragma unroll
      for (int u = 0; u < CH; ++u) dst[u] = *reinterpret_cast<const bf16x8_t*>(w + koff[u]);
    };
    auto products = [&](const bf16x8_t (&w)[CH], f32x4_t (&acc)[MT]) __attribute__((always_inline)) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int u = 0; u < CH; ++u) {
        const bf16x8_t wu = to_operand(w[u]);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wu, xf[u][mt], acc[mt], 0, 0, 0);
      }
    };
    const int stride = (int)gridDim.x;
    while (tile < n_tiles) {
      f32x4_t acc[MT];
      load_set(nxt, tile + stride);
      __builtin_amdgcn_sched_barrier(0);  // the loads stay in front of the products
      products(cur, acc);
      finish_tile(acc, tile, buf);
      buf = (buf + 1) % NBUF;
      tile += stride;
      if (tile >= n_tiles) break;
      load_set(cur, tile + stride);
      __builtin_amdgcn_sched_barrier(0);
      products(nxt, acc);
      finish_tile(acc, tile, buf);
      buf = (buf + 1) % NBUF;
      tile += stride;
    }
  } else {
    for (; tile < n_tiles; tile += gridDim.x) {
      const bf16_t* w_next = wrow(min(tile + (int)gridDim.x, n_tiles - 1));
      f32x4_t acc[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        // the chunk after this one: of this tile, or the first of the workgroup's next tile
#pragma unroll
        for (int u = 0; u < CH; ++u)
          nxt[u] = *reinterpret_cast<const bf16x8_t*>((c + 1 < NC ? w_tile + koff[(c + 1) * CH + u] : w_next + koff[u]));
#pragma unroll
        for (int u = 0; u < CH; ++u) {
          const bf16x8_t wu = to_operand(cur[u]);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wu, xf[c * CH + u][mt], acc[mt], 0, 0, 0);
        }
#pragma unroll
        for (int u = 0; u < CH; ++u) cur[u] = nxt[u];
      }
      w_tile = w_next;
      finish_tile(acc, tile, buf);
      buf = (buf + 1) % NBUF;
    }
  }
}

static int cw_num_compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) return 256;
    cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
  }
  return cus;
}

// Do a wave's x fragments, two sets of weight fragments and the accumulators fit its registers?
constexpr bool cw_stream_fits(int waves, int spw, int mt) {
  return spw * mt * 4 + cw_stream_chunk(spw) * 8 + mt * 4 <= (waves == 16 ? 100 : 220);
}

// Steps per wave the kernel is built for: every count up to 8, then even counts, then multiples of 4.
constexpr int cw_stream_round_spw(int spw) {
  return spw <= 8 ? spw : (spw <= 12 ? (spw + 1) / 2 * 2 : (spw + 3) / 4 * 4);
}

template <int MODE, int WAVES, int SPW, int MT>
static int launch_stream_one(dim3 grid, const bf16_t* X, int64_t ldx, const bf16_t* W, void* C, int64_t ldc,
                             int M, int N, int K, int n_tiles, hipStream_t stream) {
  if constexpr (cw_stream_fits(WAVES, SPW, MT)) {
    hipLaunchKernelGGL((gemm_stream_bf16_kernel<MODE, WAVES, SPW, MT>), grid, dim3(WAVES * 64), 0, stream, X, ldx,
                       W, C, ldc, M, N, K, n_tiles, StreamNormIn{});
    return cw_launch_status();
  } else {
    return CW_ERR_SIZE;
  }
}

template <int MODE, int WAVES, int MT>
static int launch_stream(int spw, dim3 grid, const bf16_t* X, int64_t ldx, const bf16_t* W, void* C, int64_t ldc,
                         int M, int N, int K, int n_tiles, hipStream_t stream) {
#define CW_STREAM(SPW_) \
  case SPW_: return launch_stream_one<MODE, WAVES, SPW_, MT>(grid, X, ldx, W, C, ldc, M, N, K, n_tiles, stream)
  switch (spw) {
    CW_STREAM(1); CW_STREAM(2); CW_STREAM(3); CW_STREAM(4); CW_STREAM(5); CW_STREAM(6); CW_STREAM(7); CW_STREAM(8);
    CW_STREAM(10); CW_STREAM(12); CW_STREAM(16); CW_STREAM(20); CW_STREAM(24);
    default: return CW_ERR_SIZE;
  }
#undef CW_STREAM
}

template <int MODE, int WAVES>
static int launch_stream_mt(int mt, int spw, dim3 grid, const bf16_t* X, int64_t ldx, const bf16_t* W, void* C,
                            int64_t ldc, int M, int N, int K, int n_tiles, hipStream_t stream) {
  if (mt == 1) return launch_stream<MODE, WAVES, 1>(spw, grid, X, ldx, W, C, ldc, M, N, K, n_tiles, stream);
  if (mt == 2) return launch_stream<MODE, WAVES, 2>(spw, grid, X, ldx, W, C, ldc, M, N, K, n_tiles, stream);
  return launch_stream<MODE, WAVES, 4>(spw, grid, X, ldx, W, C, ldc, M, N, K, n_tiles, stream);
}

// Shape of the streaming kernel's launch for this product, or false if it does not apply: a
// wave's share of K must be short enough for its registers and there must be enough row tiles.
static bool plan_stream(int mode, int M, int N, int K, int k_splits, int* mt, int* spw, dim3* grid, int* n_tiles) {
  const int k_steps = (K + 31) / 32;
  *n_tiles = mode == 2 ? (N / 2 + 7) / 8 : (N + 15) / 16;
  const int waves = mode == 3 ? 8 : 16;
  *mt = M <= 16 ? 1 : (M <= 32 ? 2 : 4);
  *spw = cw_stream_round_spw((k_steps + k_splits * waves - 1) / (k_splits * waves));
  if (M > 64 || *spw > 24 || !cw_stream_fits(waves, *spw, *mt) || (mode != 3 && k_steps < 2 * waves)) return false;
  // tiles per workgroup: one workgroup on every compute unit (a second round of these large
  // workgroups costs more than it brings), each with the same share
  // (up to 16 rows the one-tile kernels are as fast below two rounds; beyond, the alternative
  // is a library product that is slower as soon as every compute unit has a tile)
  const int slots = cw_num_compute_units();
  if ((int64_t)*n_tiles * k_splits < (M <= 16 ? 2 * slots : slots)) return false;
  const int per = (*n_tiles * k_splits + slots - 1) / slots;
  *grid = dim3((*n_tiles + per - 1) / per, k_splits);
  return true;
}

static int try_stream(int mode, const bf16_t* X, int64_t ldx, const bf16_t* W, void* C, int64_t ldc,
                      int M, int N, int K, int k_splits, hipStream_t stream) {
  int mt, spw, n_tiles;
  dim3 grid;
  if (!plan_stream(mode, M, N, K, k_splits, &mt, &spw, &grid, &n_tiles)) return CW_ERR_SIZE;
  switch (mode) {
    case 0: return launch_stream_mt<0, 16>(mt, spw, grid, X, ldx, W, C, ldc, M, N, K, n_tiles, stream);
    case 1: return launch_stream_mt<1, 16>(mt, spw, grid, X, ldx, W, C, ldc, M, N, K, n_tiles, stream);
    case 2: return launch_stream_mt<2, 16>(mt, spw, grid, X, ldx, W, C, ldc, M, N, K, n_tiles, stream);
    default: return launch_stream_mt<3, 8>(mt, spw, grid, X, ldx, W, C, ldc, M, N, K, n_tiles, stream);
  }
}

#define CW_SKINNY_MAX_M 64

template <int MT, int RT, int WAVES, int ROWS = 16>
static int launch_skinny(int mode, const bf16_t* X, int64_t ldx, const bf16_t* W, void* C, int64_t ldc,
                         int M, int N, int K, int k_splits, hipStream_t stream) {
  const int rows_per_group = (mode == 2 ? 8 : ROWS) * RT;
  const int rows = mode == 2 ? N / 2 : N;
  dim3 grid((rows + rows_per_group - 1) / rows_per_group, mode == 3 ? k_splits : 1), block(WAVES * 64);
  if (mode == 0) hipLaunchKernelGGL((gemm_skinny_bf16_kernel<MT, RT, 0, WAVES, ROWS>), grid, block, 0, stream, X, ldx, W, C, ldc, M, N, K);
  else if (mode == 1) hipLaunchKernelGGL((gemm_skinny_bf16_kernel<MT, RT, 1, WAVES, ROWS>), grid, block, 0, stream, X, ldx, W, C, ldc, M, N, K);
  else if (mode == 3) hipLaunchKernelGGL((gemm_skinny_bf16_kernel<MT, RT, 3, WAVES, ROWS>), grid, block, 0, stream, X, ldx, W, C, ldc, M, N, K);
  else if (ROWS == 16) hipLaunchKernelGGL((gemm_skinny_bf16_kernel<MT, RT, 2, WAVES, 16>), grid, block, 0, stream, X, ldx, W, C, ldc, M, N, K);
  else return CW_ERR_ARG;
  return cw_launch_status();
}

// How many ways cw_gemm_bf16_skinny would split K for a partial-sum product of this shape
// (1: not worth it). The caller allocates [splits, M, N] float32 and passes mode 3.
CW_EXPORT int cw_gemm_bf16_skinny_ksplits(int M, int N, int K) {
  const int tiles = (N + 15) / 16;
  const int k_steps = (K + 31) / 32;
  if (M > 64 || tiles > 512) return 1;
  if (M > 16) {
    // Only the streaming kernel takes partial sums of more than 16 rows, and the alternative is a
    // library product that leaves most compute units idle on so narrow an output. Split K far
    // enough that every compute unit gets a tile (two for a long K) and that a wave's share of x
    // fits its registers, down to 8 steps of 32 per split.
    // (an output wide enough for half the compute units is split only if K is much longer still)
    if (tiles > 128 && K < 2 * N) return 1;
    const int mt = M <= 32 ? 2 : 4;
    int s = (cw_num_compute_units() + tiles - 1) / tiles;
    if (K >= 4096 && s < 512 / tiles) s = 512 / tiles;
    if (s > 8) s = 8;
    while (s < 16 && !cw_stream_fits(8, cw_stream_round_spw((k_steps + s * 8 - 1) / (s * 8)), mt)) ++s;
    while (s > 1 && K / s < 256) --s;
    int mt_, spw, n_tiles;
    dim3 grid;
    if (s <= 1 || !plan_stream(3, M, N, K, s, &mt_, &spw, &grid, &n_tiles)) return 1;
    return s;
  }
  if (K < 4096) return 1;
  int s = 512 / tiles;  // about two workgroups per compute unit,
  if (s > 8) s = 8;
  const int for_registers = (k_steps + 8 * 16 - 1) / (8 * 16);  // and at most 16 steps for each of 8 waves
  if (s < for_registers) s = for_registers;
  if (s > 16) s = 16;
  while (s > 1 && K / s < 1024) --s;
  if (s < 1) s = 1;
  // One split more if that is what brings the streaming kernel in (two tiles for every compute unit):
  // it keeps x in registers and its next tile's weights in flight, which the one-tile kernel does not
  // (the 1.5B shape's down product with the norm behind it: 13.2 us with 5 splits, 11.3 with 6).
  int mt, spw, n_tiles;
  dim3 grid;
  if (s < 16 && K / (s + 1) >= 1024 && !plan_stream(3, M, N, K, s, &mt, &spw, &grid, &n_tiles) &&
      plan_stream(3, M, N, K, s + 1, &mt, &spw, &grid, &n_tiles))
    ++s;
  return s;
}

// 1 if cw_gemm_bf16_skinny streams the weights once for this shape at full speed: every shape
// with M <= 16, and the shapes with 16 < M <= 64 that the streaming kernel takes (other shapes of
// that range run, but a library product is faster). mode 3 is answered by ..._ksplits() > 1.
CW_EXPORT int cw_gemm_bf16_skinny_fast(int mode, int M, int N, int K) {
  if (M <= 16) return 1;
  if (mode < 0 || mode > 2) return 0;
  int mt, spw, n_tiles;
  dim3 grid;
  return plan_stream(mode, M, N, K, 1, &mt, &spw, &grid, &n_tiles) ? 1 : 0;
}

// 1 if cw_gemm_bf16_swiglu_normed takes this shape (the streaming kernel with one tile of tokens).
CW_EXPORT int cw_gemm_bf16_swiglu_normed_ok(int M, int N, int K) {
  int mt, spw, n_tiles;
  dim3 grid;
  // rows of up to 2048 elements: a lane holds its share of a row in registers over the statistics
  return M >= 1 && M <= 16 && !(N & 1) && !(K & 7) && plan_stream(2, M, N, K, 1, &mt, &spw, &grid, &n_tiles) &&
                 spw <= 4
             ? 1
             : 0;
}

// y[m, i] = silu(gate_i . x_m) * (up_i . x_m) with x = rmsnorm(resid + delta) * norm_weight made
// inside the product kernel: resid float32 [M, K], delta bfloat16 [M, K], norm_weight [K]
// bfloat16 (norm_weight_f32 = 0) or float32, W [N = 2 I, K] with the gate rows first, y bfloat16
// [M, I] with row stride ldc. resid is not changed: whoever adds delta to it must still do so.
CW_EXPORT int cw_gemm_bf16_swiglu_normed(const float* resid, const void* delta, const void* norm_weight,
                                         int norm_weight_f32, float eps, const void* W, void* C, int64_t ldc,
                                         int M, int N, int K, hipStream_t stream) {
  if (!cw_gemm_bf16_swiglu_normed_ok(M, N, K)) return CW_ERR_SIZE;
  if (!resid || !delta || !norm_weight || !W || !C || ldc < N / 2) return CW_ERR_ARG;
  if (((uintptr_t)resid & 15) || ((uintptr_t)delta & 15) || ((uintptr_t)norm_weight & 15) || ((uintptr_t)W & 15))
    return CW_ERR_ARG;
  int mt, spw, n_tiles;
  dim3 grid;
  plan_stream(2, M, N, K, 1, &mt, &spw, &grid, &n_tiles);
  const StreamNormIn nin{resid, (const bf16_t*)delta, norm_weight, norm_weight_f32, eps};
#define CW_NORMED(SPW_)                                                                                        \
  case SPW_:                                                                                                   \
    if constexpr (cw_stream_fits(16, SPW_, 1))                                                                 \
      hipLaunchKernelGGL((gemm_stream_bf16_kernel<2, 16, SPW_, 1, true>), grid, dim3(16 * 64), 0, stream,      \
                         (const bf16_t*)nullptr, (int64_t)K, (const bf16_t*)W, C, ldc, M, N, K, n_tiles, nin); \
    break
  switch (spw) {
    CW_NORMED(1); CW_NORMED(2); CW_NORMED(3); CW_NORMED(4);
    default: return CW_ERR_SIZE;
  }
#undef CW_NORMED
  return cw_launch_status();
}

// y = x W^T for M <= 64 rows of bfloat16 x [M, K] (row stride ldx) and bfloat16 W [N, K].
// mode 0: y bfloat16 [M, N]; 1: y float32 [M, N]; 2: y = silu(gate) * up, bfloat16 [M, N / 2];
// 3: float32 partial products [splits, M, N], splits = ``k_splits`` if that is positive (up to 16
// rows of x; what a caller has measured to be the best for the shape), else
// cw_gemm_bf16_skinny_ksplits(M, N, K). K must be a multiple of 8 (16-byte rows).
CW_EXPORT int cw_gemm_bf16_skinny(int mode, const void* X, int64_t ldx, const void* W, void* C,
                                  int64_t ldc, int M, int N, int K, int k_splits, hipStream_t stream) {
  if (M < 0 || N <= 0 || K <= 0 || mode < 0 || mode > 3) return CW_ERR_ARG;
  if (M > CW_SKINNY_MAX_M) return CW_ERR_SIZE;
  if ((K & 7) || (ldx & 7) || ((uintptr_t)X & 15) || ((uintptr_t)W & 15)) return CW_ERR_ARG;
  if (mode == 2 && (N & 1)) return CW_ERR_ARG;
  if (ldx < K || ldc < (mode == 2 ? N / 2 : N)) return CW_ERR_ARG;
  if (M == 0) return CW_OK;
  const bf16_t* x = (const bf16_t*)X;
  const bf16_t* w = (const bf16_t*)W;
  const int rows = mode == 2 ? N / 2 : N;
  const int tiles = (rows + (mode == 2 ? 7 : 15)) / (mode == 2 ? 8 : 16);
  if (mode == 3) {
    const int ks = k_splits > 0 ? k_splits : cw_gemm_bf16_skinny_ksplits(M, N, K);
    if (ks > 16 || K / ks < 32) return CW_ERR_ARG;
    const int rc = try_stream(3, x, ldx, w, C, ldc, M, N, K, ks, stream);
    if (rc != CW_ERR_SIZE) return rc;
    if (M > 16) return CW_ERR_SIZE;
    return launch_skinny<1, 1, 8>(3, x, ldx, w, C, ldc, M, N, K, ks, stream);
  }
  {
    const int rc = try_stream(mode, x, ldx, w, C, ldc, M, N, K, 1, stream);
    if (rc != CW_ERR_SIZE) return rc;
  }
  if (M <= 16) {
    // few tiles: many waves on each tile keep enough loads in flight
    if (tiles <= 256 && K >= 1024) return launch_skinny<1, 1, 16>(mode, x, ldx, w, C, ldc, M, N, K, 1, stream);
    // very many tiles: several per workgroup, so that x is fetched from L2 less often
    if (tiles >= 4096) return launch_skinny<1, 4, 4>(mode, x, ldx, w, C, ldc, M, N, K, 1, stream);
    if (tiles <= 1024 && K >= 512) return launch_skinny<1, 1, 8>(mode, x, ldx, w, C, ldc, M, N, K, 1, stream);
    return launch_skinny<1, 1, 4>(mode, x, ldx, w, C, ldc, M, N, K, 1, stream);
  }
  if (M <= 32) {
    if (tiles <= 256 && K >= 1024) return launch_skinny<2, 1, 16>(mode, x, ldx, w, C, ldc, M, N, K, 1, stream);
    return rows >= 4096 ? launch_skinny<2, 2, 4>(mode, x, ldx, w, C, ldc, M, N, K, 1, stream)
                        : launch_skinny<2, 1, 4>(mode, x, ldx, w, C, ldc, M, N, K, 1, stream);
  }
  if (tiles <= 256 && K >= 1024) return launch_skinny<4, 1, 8>(mode, x, ldx, w, C, ldc, M, N, K, 1, stream);
  return rows >= 4096 ? launch_skinny<4, 2, 4>(mode, x, ldx, w, C, ldc, M, N, K, 1, stream)
                      : launch_skinny<4, 1, 4>(mode, x, ldx, w, C, ldc, M, N, K, 1, stream);
}

// =====================================================================================
// Fused q/k/v product + bias + rotary encoding + cache write for few rows of x (decode).
// The weight-streaming product above with another row order and epilogue: a tile of a q or k
// head holds rows (i .. i+7) and (i + hd/2 .. i + hd/2 + 7) of that head, so both elements of
// every rotary pair (half-split pairing, full rotary dimension) end up in one workgroup. The
// epilogue adds the bias, rotates by float32(pos) * inv_freq[i] and writes q to ``q_out``
// [M, nh * hd], rotated k and plain v to their cache rows ``slots[m]`` ([rows, nkv, hd]).
template <int WAVES, int MT>
__global__ __launch_bounds__(WAVES * 64) void gemm_qkv_rope_bf16_kernel(
    const bf16_t* __restrict__ X, int64_t ldx, const bf16_t* __restrict__ W, const void* __restrict__ bias,
    int bias_f32, const int* __restrict__ positions, const int* __restrict__ slots,
    const float* __restrict__ inv_freq, bf16_t* __restrict__ q_out, bf16_t* __restrict__ k_cache,
    bf16_t* __restrict__ v_cache, int64_t cache_rows, int M, int K, int nh, int nkv, int hd) {
  __shared__ __align__(16) float red[WAVES][MT * 256];  // [wave][token tile][token][tile row]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, s = lane >> 4;
  const int half = hd / 2;
  const int tiles_per_head = hd / 16;
  const int head = blockIdx.x / tiles_per_head;   // 0 .. nh + 2 nkv - 1
  const int tile = blockIdx.x % tiles_per_head;
  const bool is_v = head >= nh + nkv;
  // the weight row inside the head that this lane loads: row lr of the tile (see cw_to_operand_layout)
  const int lr = lane >> 2, ls = lane & 3;
  const int row_in_head = is_v ? tile * 16 + lr : (lr < 8 ? tile * 8 + lr : half + tile * 8 + (lr - 8));
  const bf16_t* wrow = W + ((int64_t)head * hd + row_in_head) * K;
  constexpr bool X_SWAP = MT > 1;  // one tile of tokens is loaded in operand layout as it is (see gemm_skinny_bf16_kernel)
  const int xr = X_SWAP ? lr : r, xs = X_SWAP ? ls : s;
  bool xok[MT];
  const bf16_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    xok[mt] = mt * 16 + xr < M;
    xrow[mt] = X + (int64_t)(xok[mt] ? mt * 16 + xr : 0) * ldx;
  }

  auto bias_at = [&](int col) -> float {
    if (bias == nullptr) return 0.0f;
    return bias_f32 ? ((const float*)bias)[col] : __bfloat162float(((const bf16_t*)bias)[col]);
  };
  // MT == 1: what this thread's part of the epilogue needs (position, slot, frequency, bias) is
  // requested here, beside the weights, and not after the product, where it would be one more
  // trip to memory with nothing else to do meanwhile
  int e_pos = 0;
  int64_t e_slot = -1;
  float e_inv = 0.0f, e_ba = 0.0f, e_bb = 0.0f;
  if constexpr (MT == 1) {
    if (is_v) {
      const int j = threadIdx.x & 15, m = threadIdx.x >> 4;
      if (m < 16 && m < M) {
        e_slot = slots[m];
        e_ba = bias_at(head * hd + tile * 16 + j);
      }
    } else {
      const int p = threadIdx.x & 7, m = threadIdx.x >> 3;
      if (m < 16 && m < M) {
        const int i = tile * 8 + p;
        e_pos = positions[m];
        e_slot = slots[m];
        e_inv = inv_freq[i];
        e_ba = bias_at(head * hd + i);
        e_bb = bias_at(head * hd + half + i);
      }
    }
  }

  f32x4_t acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};
  bf16x8_t zero;
#pragma unroll
  for (int e = 0; e < 8; ++e) zero[e] = (__bf16)0.0f;
  const int k_steps = (K + 31) / 32;
  constexpr int U = MT == 1 ? 4 : 2;
  for (int ks0 = wave * U; ks0 < k_steps; ks0 += WAVES * U) {
    bf16x8_t wf[U], xf[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (ks0 + u) * 32 + ls * 8;
      const bool kok = (ks0 + u) < k_steps && k + 8 <= K;
      wf[u] = kok ? *reinterpret_cast<const bf16x8_t*>(wrow + k) : zero;
      const int kx = (ks0 + u) * 32 + xs * 8;
      const bool kxok = (ks0 + u) < k_steps && kx + 8 <= K;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        xf[u][mt] = (kxok && xok[mt]) ? *reinterpret_cast<const bf16x8_t*>(xrow[mt] + kx) : zero;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const bf16x8_t wo = cw_to_operand_layout(wf[u], lane);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wo, X_SWAP ? cw_to_operand_layout(xf[u][mt], lane) : xf[u][mt],
                                                          acc[mt], 0, 0, 0);
    }
  }
  // lane (r, s) holds tile rows 4s..4s+3 of token r: one 16-byte store, no bank hit twice
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) *reinterpret_cast<f32x4_t*>(&red[wave][mt * 256 + r * 16 + 4 * s]) = acc[mt];
  __syncthreads();
  // MT * 256 values [token tile][token][tile row]; each is summed over the waves by one thread
  for (int idx = threadIdx.x; idx < MT * 256; idx += WAVES * 64) {
    float sum = red[0][idx];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) sum += red[w][idx];
    red[0][idx] = sum;
  }
  __syncthreads();
  auto summed = [&](int row, int m) -> float { return red[0][m * 16 + row]; };
  if constexpr (MT == 1) {
    // every thread has at most one output (v: 256 of them, q and k: 128 pairs)
    if (is_v) {
      const int j = threadIdx.x & 15, m = threadIdx.x >> 4;
      if (m < 16 && m < M && e_slot >= 0 && e_slot < cache_rows) {
        const int d = tile * 16 + j;
        v_cache[(e_slot * nkv + (head - nh - nkv)) * hd + d] = __float2bfloat16(summed(j, m) + e_ba);
      }
    } else {
      const int p = threadIdx.x & 7, m = threadIdx.x >> 3;
      if (m < 16 && m < M) {
        const int i = tile * 8 + p;
        const float a = summed(p, m) + e_ba;
        const float b = summed(p + 8, m) + e_bb;
        float sn, cs;
        sincosf((float)e_pos * e_inv, &sn, &cs);
        const bf16_t oa = __float2bfloat16(a * cs - b * sn), ob = __float2bfloat16(b * cs + a * sn);
        if (head < nh) {
          bf16_t* q = q_out + (int64_t)m * nh * hd + head * hd;
          q[i] = oa;
          q[i + half] = ob;
        } else if (e_slot >= 0 && e_slot < cache_rows) {
          bf16_t* kd = k_cache + (e_slot * nkv + (head - nh)) * hd;
          kd[i] = oa;
          kd[i + half] = ob;
        }
      }
    }
    return;
  }
  if (is_v) {
    // idx -> (token m, row j), j fastest: 16 consecutive elements of a cache row
    for (int idx = threadIdx.x; idx < MT * 256; idx += WAVES * 64) {
      const int j = idx & 15, m = idx >> 4;
      if (m >= M) continue;
      const int64_t slot = slots[m];
      if (slot < 0 || slot >= cache_rows) continue;
      const int d = tile * 16 + j;
      const float v = summed(j, m) + bias_at(head * hd + d);
      v_cache[(slot * nkv + (head - nh - nkv)) * hd + d] = __float2bfloat16(v);
    }
  } else {
    // idx -> (token m, pair p): elements i = tile * 8 + p and i + half
    for (int idx = threadIdx.x; idx < MT * 128; idx += WAVES * 64) {
      const int p = idx & 7, m = idx >> 3;
      if (m >= M) continue;
      const int i = tile * 8 + p;
      const float a = summed(p, m) + bias_at(head * hd + i);
      const float b = summed(p + 8, m) + bias_at(head * hd + half + i);
      float sn, cs;
      sincosf((float)positions[m] * inv_freq[i], &sn, &cs);
      const bf16_t oa = __float2bfloat16(a * cs - b * sn), ob = __float2bfloat16(b * cs + a * sn);
      if (head < nh) {
        bf16_t* q = q_out + (int64_t)m * nh * hd + head * hd;
        q[i] = oa;
        q[i + half] = ob;
      } else {
        const int64_t slot = slots[m];
        if (slot < 0 || slot >= cache_rows) continue;
        bf16_t* kd = k_cache + (slot * nkv + (head - nh)) * hd;
        kd[i] = oa;
        kd[i + half] = ob;
      }
    }
  }
}

// x [M <= 64, K] bfloat16, W [(nh + 2 nkv) * hd, K] bfloat16 (q heads, k heads, v heads), hd a
// multiple of 16, rotary dimension == hd. bias: nullptr, bfloat16 or float32 [(nh + 2 nkv) * hd].
CW_EXPORT int cw_gemm_qkv_rope_bf16(const void* X, int64_t ldx, const void* W, const void* bias,
                                    int bias_f32, const int* positions, const int* slots,
                                    const float* inv_freq, void* q_out, void* k_cache, void* v_cache,
                                    int64_t cache_rows, int M, int K, int nh, int nkv, int hd,
                                    hipStream_t stream) {
  if (M < 0 || M > 64 || K <= 0 || nh <= 0 || nkv <= 0 || hd <= 0 || (hd & 15)) return CW_ERR_ARG;
  if ((K & 7) || (ldx & 7) || ldx < K || ((uintptr_t)X & 15) || ((uintptr_t)W & 15)) return CW_ERR_ARG;
  if (!positions || !slots || !inv_freq || !q_out || !k_cache || !v_cache) return CW_ERR_ARG;
  if (M == 0) return CW_OK;
  const int tiles = (nh + 2 * nkv) * (hd / 16);
  dim3 grid(tiles);
  const bf16_t* x = (const bf16_t*)X;
  const bf16_t* w = (const bf16_t*)W;
#define CW_QKV(WAVES_, MT_)                                                                              \
  hipLaunchKernelGGL((gemm_qkv_rope_bf16_kernel<WAVES_, MT_>), grid, dim3(WAVES_ * 64), 0, stream, x, ldx, \
                     w, bias, bias_f32, positions, slots, inv_freq, (bf16_t*)q_out, (bf16_t*)k_cache,    \
                     (bf16_t*)v_cache, cache_rows, M, K, nh, nkv, hd)
  if (M > 32) {  // the reduction buffer is WAVES * MT KB
    if (K >= 512) CW_QKV(8, 4);
    else CW_QKV(4, 4);
  } else if (M > 16) {
    if (tiles <= 256 && K >= 1024) CW_QKV(16, 2);
    else if (K >= 512) CW_QKV(8, 2);
    else CW_QKV(4, 2);
  } else {
    if (tiles <= 256 && K >= 1024) CW_QKV(16, 1);
    else if (K >= 512) CW_QKV(8, 1);
    else CW_QKV(4, 1);
  }
#undef CW_QKV
  return cw_launch_status();
}
