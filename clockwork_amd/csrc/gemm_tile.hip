// bfloat16 matrix product y = x * W^T for many rows of x (portions of prompts) on the gfx950
// matrix cores, LDS tiled: x [M, K] row-major, W [N, K] row-major as checkpoints hold it.
//
// A workgroup of 4 waves owns a 128 x 128 tile of y and walks K in steps of 64. The x and W tiles
// of a step (128 rows x 64 elements each) go from global memory through registers into LDS, double
// buffered: the loads of step t + 1 are in flight while step t is multiplied, and one barrier per
// step separates writing a buffer from reading it. A wave owns a 64 x 64 quarter: per 32 elements
// of K it reads 4 + 4 fragments of 16 rows from LDS (16-byte reads; rows are padded by 16 bytes so
// that 16 lanes reading 16 different rows hit different banks) and issues 16
// v_mfma_f32_16x16x32_bf16. W is the first operand, so a lane ends up with 4 consecutive columns
// of one row of y, which it stores as 8 bytes. With quarters of this size the LDS reads (1 KB per
// 4 matrix instructions) hold the matrix cores to about a fifth of their peak: half of what the
// library's 256 x 256 tiles reach on the same shapes, so the engine takes this kernel only when it
// is asked to (``hip_products``) and the library product otherwise.
//
// What is fused in is chosen by MODE:
//   0  y bfloat16 [M, N], + bias [N] (bfloat16 or float32) when given;
//   2  W = [gate; up] stacked ([2 I, K]), y[m, i] = silu(gate_i . x_m) * (up_i . x_m), bfloat16
//      [M, I]: the tile holds 64 gate rows and the 64 up rows that belong to them, arranged so
//      that a lane holds both values of an output;
// Accumulation is float32; the K loop of an output runs in the same order whatever else is in
// the batch.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

#define GT_BM 128
#define GT_BN 128
#define GT_BK 64
#define GT_ROW (GT_BK + 8)  // LDS row in elements

struct TileArgs {
  const bf16_t* X;
  int64_t ldx;
  const bf16_t* W;
  const void* bias;   // nullptr, or [N]
  int bias_f32;
  void* C;
  int64_t ldc;
  int M, N, K;
};

// Row of W that row ``rb`` (0..127) of the workgroup's W tile ``tn`` is. MODE 2: a wave's 64 tile
// rows are 32 gate rows followed by the 32 up rows with the same indices.
template <int MODE>
__device__ __forceinline__ int64_t gt_w_row(int tn, int rb, int N, bool* ok) {
  if (MODE == 2) {
    const int I = N / 2;
    const int wn = rb >> 6, q = rb & 63;
    const int64_t i = (int64_t)tn * 64 + wn * 32 + (q & 31);
    *ok = i < I;
    return (q < 32 ? i : I + i);
  }
  const int64_t n = (int64_t)tn * GT_BN + rb;
  *ok = n < N;
  return n;
}

template <int MODE>
__global__ __launch_bounds__(256, 2) void gemm_tile_bf16_kernel(TileArgs a) {
  extern __shared__ __align__(16) unsigned char gt_smem[];
  bf16_t* As = reinterpret_cast<bf16_t*>(gt_smem);        // [2][128][GT_ROW]
  bf16_t* Bs = As + 2 * GT_BM * GT_ROW;                    // [2][128][GT_ROW]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int c = lane & 15, s = lane >> 4;
  const int tn = blockIdx.x, tm = blockIdx.y;
  const int M = a.M, N = a.N, K = a.K;

  // ---- global -> registers -> LDS: thread -> 16-byte chunk (tid & 7) of rows (tid >> 3) + 32 i
  const int chunk = tid & 7, row0 = tid >> 3;
  const bf16_t* xp[4];
  const bf16_t* wp[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = min((int64_t)tm * GT_BM + row0 + 32 * i, (int64_t)M - 1);  // a row past the end repeats the last one
    xp[i] = a.X + m * a.ldx + chunk * 8;
    bool ok;
    int64_t n = gt_w_row<MODE>(tn, row0 + 32 * i, N, &ok);
    if (!ok) n = 0;  // never stored
    wp[i] = a.W + n * K + chunk * 8;
  }
  u32x4_t gx[4], gw[4];
  const int k_tiles = (K + GT_BK - 1) / GT_BK;
  auto fetch = [&](int kt) __attribute__((always_inline)) {
    const int k = kt * GT_BK + chunk * 8;
    const bool ok = k + 8 <= K;        // K is a multiple of 8: a chunk is inside or outside
    const int at = ok ? kt * GT_BK : 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      gx[i] = *reinterpret_cast<const u32x4_t*>(xp[i] + at);
      gw[i] = *reinterpret_cast<const u32x4_t*>(wp[i] + at);
      if (!ok) {
        gx[i] = (u32x4_t){0u, 0u, 0u, 0u};
        gw[i] = (u32x4_t){0u, 0u, 0u, 0u};
      }
    }
  };
  auto stash = [&](int stage) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<u32x4_t*>(As + (stage * GT_BM + row0 + 32 * i) * GT_ROW + chunk * 8) = gx[i];
      *reinterpret_cast<u32x4_t*>(Bs + (stage * GT_BN + row0 + 32 * i) * GT_ROW + chunk * 8) = gw[i];
    }
  };

  f32x4_t acc[4][4];  // [block of 16 rows of x][block of 16 rows of W]
#pragma unroll
  for (int mi = 0; mi < 4; ++mi)
#pragma unroll
    for (int ni = 0; ni < 4; ++ni) acc[mi][ni] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};

  auto multiply = [&](int stage) __attribute__((always_inline)) {
    const bf16_t* as = As + (stage * GT_BM + wm * 64 + c) * GT_ROW + s * 8;
    const bf16_t* bs = Bs + (stage * GT_BN + wn * 64 + c) * GT_ROW + s * 8;
#pragma unroll
    for (int kk = 0; kk < GT_BK / 32; ++kk) {
      bf16x8_t xf[4], wf[4];
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) xf[mi] = *reinterpret_cast<const bf16x8_t*>(as + mi * 16 * GT_ROW + kk * 32);
#pragma unroll
      for (int ni = 0; ni < 4; ++ni) wf[ni] = *reinterpret_cast<const bf16x8_t*>(bs + ni * 16 * GT_ROW + kk * 32);
#pragma unroll
      for (int mi = 0; mi < 4; ++mi)
#pragma unroll
        for (int ni = 0; ni < 4; ++ni)
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[ni], xf[mi], acc[mi][ni], 0, 0, 0);
    }
  };
  fetch(0);
  stash(0);
  __syncthreads();
  for (int kt = 0; kt < k_tiles; ++kt) {
    if (kt + 1 < k_tiles) fetch(kt + 1);  // in flight while this step is multiplied
    multiply(kt & 1);
    if (kt + 1 < k_tiles) stash((kt + 1) & 1);
    __syncthreads();
  }

  // ---- lane (c, s) holds y[m = .. + mi * 16 + c][4 s + e of W block ni], e = 0..3
#pragma unroll
  for (int mi = 0; mi < 4; ++mi) {
    const int64_t m = (int64_t)tm * GT_BM + wm * 64 + mi * 16 + c;
    if (m >= M) continue;
    if (MODE == 2) {
      const int I = N / 2;
#pragma unroll
      for (int ni = 0; ni < 2; ++ni) {
        const int64_t i0 = (int64_t)tn * 64 + wn * 32 + ni * 16 + 4 * s;
        if (i0 >= I) continue;
        uint16_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float g = acc[mi][ni][e], up = acc[mi][ni + 2][e];
          o[e] = cw_float_to_bf16_bits(g / (1.0f + __expf(-g)) * up);
        }
        bf16_t* dst = (bf16_t*)a.C + m * a.ldc + i0;
        if (i0 + 4 <= I && !(a.ldc & 3)) {
          uint2 pk;
          pk.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
          pk.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
          *reinterpret_cast<uint2*>(dst) = pk;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (i0 + e < I) reinterpret_cast<uint16_t*>(dst)[e] = o[e];
        }
      }
    } else {
#pragma unroll
      for (int ni = 0; ni < 4; ++ni) {
        const int64_t n0 = (int64_t)tn * GT_BN + wn * 64 + ni * 16 + 4 * s;
        if (n0 >= N) continue;
        uint16_t o[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          float v = acc[mi][ni][e];
          if (a.bias != nullptr && n0 + e < N)
            v += a.bias_f32 ? ((const float*)a.bias)[n0 + e] : __bfloat162float(((const bf16_t*)a.bias)[n0 + e]);
          o[e] = cw_float_to_bf16_bits(v);
        }
        bf16_t* dst = (bf16_t*)a.C + m * a.ldc + n0;
        if (n0 + 4 <= N && !(a.ldc & 3)) {
          uint2 pk;
          pk.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
          pk.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
          *reinterpret_cast<uint2*>(dst) = pk;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n0 + e < N) reinterpret_cast<uint16_t*>(dst)[e] = o[e];
        }
      }
    }
  }
}

static const size_t GT_SMEM = (size_t)2 * (GT_BM + GT_BN) * GT_ROW * sizeof(bf16_t);

template <int MODE>
static int gt_launch(const TileArgs& a, hipStream_t stream) {
  static bool raised = false;
  if (!raised) {
    if (hipFuncSetAttribute((const void*)gemm_tile_bf16_kernel<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)GT_SMEM) != hipSuccess)
      return CW_ERR_LAUNCH;
    raised = true;
  }
  const int out_cols = MODE == 2 ? a.N / 2 : a.N;
  const int per_tile = MODE == 2 ? 64 : GT_BN;
  dim3 grid((out_cols + per_tile - 1) / per_tile, (a.M + GT_BM - 1) / GT_BM);
  if (grid.y > 65535) return CW_ERR_SIZE;
  hipLaunchKernelGGL((gemm_tile_bf16_kernel<MODE>), grid, dim3(256), GT_SMEM, stream, a);
  return cw_launch_status();
}

// y = x W^T (+ bias) for bfloat16 x [M, K] (row stride ldx) and W [N, K]; K a multiple of 8.
// mode 0: y bfloat16 [M, N] (row stride ldc), bias nullptr or [N] bfloat16 / float32 (bias_f32);
// mode 2: y = silu(gate) * up, bfloat16 [M, N / 2], W = [gate; up], no bias.
CW_EXPORT int cw_gemm_bf16_tiled(int mode, const void* X, int64_t ldx, const void* W, const void* bias,
                                 int bias_f32, void* C, int64_t ldc, int M, int N, int K, hipStream_t stream) {
  if (M < 0 || N <= 0 || K <= 0 || (mode != 0 && mode != 2)) return CW_ERR_ARG;
  if ((K & 7) || (ldx & 7) || ldx < K || ((uintptr_t)X & 15) || ((uintptr_t)W & 15) || ((uintptr_t)C & 7))
    return CW_ERR_ARG;
  if (mode == 2 && ((N & 1) || bias != nullptr)) return CW_ERR_ARG;
  if (ldc < (mode == 2 ? N / 2 : N)) return CW_ERR_ARG;
  if (M == 0) return CW_OK;
  TileArgs a{(const bf16_t*)X, ldx, (const bf16_t*)W, bias, bias_f32, C, ldc, M, N, K};
  return mode == 2 ? gt_launch<2>(a, stream) : gt_launch<0>(a, stream);
}
