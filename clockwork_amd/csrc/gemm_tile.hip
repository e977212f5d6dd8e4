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
//
// The second kernel of this file, gemm_wide_bf16_kernel, is the one the engine takes by itself
// for the gate/up product of long portions (it is as fast as the library's kernels there, and the
// gate costs no pass of its own): 256 x 192 tiles, K in stages of 32 that go from global memory
// straight into LDS (buffer loads with the LDS target, no registers between), a ring of five
// stages, and workgroups that stay and walk over their share of the tiles. It is described where
// it stands.
#include "common.h"
#include <type_traits>

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
    xp[i] = a.X + m * a.ldx;
    bool ok;
    int64_t n = gt_w_row<MODE>(tn, row0 + 32 * i, N, &ok);
    if (!ok) n = 0;  // never stored
    wp[i] = a.W + n * K;
  }
  u32x4_t gx[4], gw[4];
  const int k_tiles = (K + GT_BK - 1) / GT_BK;
  auto fetch = [&](int kt) __attribute__((always_inline)) {
    const int k = kt * GT_BK + chunk * 8;
    const bool ok = k + 8 <= K;        // K is a multiple of 8: a chunk is inside or outside
    const int at = ok ? k : 0;         // a chunk outside reads the row's first one (inside the tensor) and is zeroed
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


// ------------------------------------------------------------------------------------------------
// Wide tiles. One workgroup of 4 waves per compute unit owns 256 rows of x by 192 rows of W; a
// wave owns 128 x 96 of it in 8 x 6 accumulators of 16 x 16 (192 registers; with 512 registers a
// wave a SIMD holds this one wave, so everything that has a latency is overlapped by hand).
//
// K goes in stages of 32 elements: 16 KB of x and 12 KB of W, as 28 fragment blocks of 16 rows x
// 64 bytes. A block comes in by ONE buffer load with the LDS target (buffer_load_dwordx4 ... lds):
// lane l writes its 16 bytes at block + 16 l, no register and no LDS store instruction between.
// Four lanes next to each other take the 64 bytes of one row, so the cache sees one request for
// them (lanes that take 16 bytes of four different rows cost four; measured: 2.4 times the step
// time), and the four granules of row r change places by w_swizzle(r), so that the 16 lanes that
// later read one granule column of 16 rows with ds_read_b128 touch every bank once. The
// descriptors end with the matrices, so rows past the end read as zeros.
//
// Five stages are in LDS (140 KB). In iteration t a wave multiplies stage t from registers (48
// matrix instructions), reads the 14 fragments of stage t + 1 from LDS into the other register
// set, one read after every 3 matrix instructions, and takes part in bringing stages t + 4 and
// t + 5 in: two stages share their rows' 128-byte lines, so their loads are issued next to each
// other (six matrix instructions apart), spread over both iterations of the pair (the texture
// path takes a load every 16 cycles; eight of them in a row stall the wave). The loop is bound by
// these loads as much as by the matrix cores: without any matrix instruction or fragment read
// the kernel still takes 0.7 to 0.8 of its time, 50 to 78 GB/s into each compute unit. An even iteration ends when all loads but its own have
// landed (stages t + 2, t + 3), then a barrier; the waits and barriers are bare instructions,
// since a fence would wait for every load in flight. Measured on an MI355X: 0.52 us a stage
// against 0.45 us for the matrix instructions alone.
//
// The workgroups of a launch are dealt to the 8 XCDs in turn; each XCD takes a run of consecutive
// tiles (8 row tiles by 4 W tiles at a time: 176 KB a stage through one L2), each workgroup every
// 32nd tile of the run. Before a workgroup stores a tile it asks for the first four stages of its
// next one, which arrive while the results go out. A lane holds 4 columns of a row; two blocks
// change places between lane rows (v_permlane16_swap) so that it stores 16 bytes and four lanes
// 64 bytes of a row.
//
// MODE as above; K a multiple of 64, at least 256; both matrices below 4 GiB. MODE 3: the product
// of a narrow output with a long K (too few tiles to fill the card) summed in k_splits runs of K,
// each run of every tile a work item of its own; the items write float32 planes of partial sums
// [k_splits, M, N] that the next norm kernel adds up in their order.
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((address_space(3))) void lds_void_t;

#define W_NB 6                             // blocks of 16 W rows per wave
#define W_BM 256
#define W_BN (32 * W_NB)
#define W_BK 32
#define W_BLOCK 1024                       // bytes of a fragment block: 16 rows x 32 elements
#define W_XHALF (16 * W_BLOCK)             // x of a stage: 256 rows x 32 elements
#define W_WHALF (2 * W_NB * W_BLOCK)
#define W_STAGE (W_XHALF + W_WHALF)
#define W_SLOTS 5
#define W_LOADS (4 + W_NB / 2)             // loads of a wave per stage
#define W_GROUP_M 8                        // row tiles that run side by side

struct WideArgs {
  const bf16_t* X;
  int64_t ldx;
  const bf16_t* W;
  const void* bias;
  int bias_f32;
  void* C;
  int64_t ldc;
  int M, N, K;
  int tiles_m, tiles_n;
  int k_splits;  // MODE 3: K is cut into this many runs, each a tile of its own with a float32 plane of partial sums
};

// Row of W that row ``rb`` of W tile ``tn`` is. MODE 2: a wave's 96 rows are 48 gate rows followed
// by the up rows with the same indices.
template <int MODE>
__device__ __forceinline__ int64_t w_row_of(int tn, int rb, int N) {
  if (MODE == 2) {
    const int I = N / 2;
    const int wn = rb / (W_BN / 2), q = rb % (W_BN / 2);
    const int64_t i = (int64_t)tn * (W_BN / 2) + wn * (W_BN / 4) + (q % (W_BN / 4));
    return (q < W_BN / 4 ? i : I + i);
  }
  return (int64_t)tn * W_BN + rb;
}

// Which of a row's four 16-byte granules changes places with which in LDS: rows that lie 128 or 256
// bytes apart (r + 2, r + 4, ...) get different values, so that 8 or 16 lanes that read the same
// granule of neighbouring rows touch every bank once.
__device__ __forceinline__ int w_swizzle(int r) { return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1); }

__device__ __forceinline__ uint32_t w_pack_bf16(float lo, float hi) {
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));  // v_cvt_pk_bf16_f32
}

// s_waitcnt for "at most n vector-memory operations in flight" and nothing else
#define W_WAIT_LOADS(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))
// a barrier without a fence: what it orders is said at each use
#define W_BARRIER()                 \
  do {                              \
    asm volatile("" ::: "memory"); \
    __builtin_amdgcn_s_barrier();   \
    asm volatile("" ::: "memory"); \
  } while (0)

template <int MODE>
__global__ __launch_bounds__(256) void gemm_wide_bf16_kernel(WideArgs a) {
  extern __shared__ __align__(1024) unsigned char w_smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int c = lane & 15, s = lane >> 4;
  const int M = a.M, N = a.N, K = a.K;
  const int per_split = a.tiles_m * a.tiles_n;
  const int total = per_split * (MODE == 3 ? a.k_splits : 1);
  const int xcd = blockIdx.x & 7, local = blockIdx.x >> 3, per_xcd = gridDim.x >> 3;
  const int run = total >> 3, rest = total & 7;
  const int run_begin = xcd * run + min(xcd, rest), run_end = run_begin + run + (xcd < rest ? 1 : 0);
  // tile id -> (row tile, W tile): groups of W_GROUP_M row tiles, inside a group the row tiles
  // of one W tile next to each other
  auto tile_of = [&](int id, int* tm, int* tn) __attribute__((always_inline)) {
    if (MODE == 3) id %= per_split;  // the runs of K one after the other, each over all tiles
    const int per_group = W_GROUP_M * a.tiles_n;
    const int group = id / per_group, within = id - group * per_group;
    const int rows = min(W_GROUP_M, a.tiles_m - group * W_GROUP_M);
    *tn = within / rows;
    *tm = group * W_GROUP_M + (within - *tn * rows);
  };

  uint32_t xo[4], wo[W_NB / 2];
  const int lrow = lane >> 2, lsub = (lane & 3) ^ w_swizzle(lane >> 2);
#pragma unroll
  for (int j = 0; j < 4; ++j) xo[j] = (uint32_t)(((int64_t)(wave * 64 + j * 16 + lrow) * a.ldx + lsub * 8) * 2);
#pragma unroll
  for (int j = 0; j < W_NB / 2; ++j) {
    const int64_t n = w_row_of<MODE>(0, wave * (W_BN / 4) + j * 16 + lrow, N);  // the same in every tile
    wo[j] = (uint32_t)((n * K + lsub * 8) * 2);
  }
  const int k_run = MODE == 3 ? K / a.k_splits : K;  // elements of K that one work item sums
  const int k_tiles = k_run / W_BK;
  __amdgpu_buffer_rsrc_t xr, wr;
  auto aim = [&](int id) __attribute__((always_inline)) {
    int tm, tn;
    tile_of(id, &tm, &tn);
    const int64_t k0 = MODE == 3 ? (int64_t)(id / per_split) * k_run : 0;
    const int64_t x_row0 = (int64_t)tm * W_BM;
    const int64_t w_row0 = w_row_of<MODE>(tn, 0, N);
    // the descriptors begin at the run's first element of the tile's first row and end with the
    // run's last element of the matrix's last row: rows past the end read as zeros
    xr = __builtin_amdgcn_make_buffer_rsrc((void*)(a.X + x_row0 * a.ldx + k0), 0,
                                           (int)(uint32_t)(((M - x_row0 - 1) * a.ldx + k_run) * 2), 0x00020000);
    wr = __builtin_amdgcn_make_buffer_rsrc((void*)(a.W + w_row0 * K + k0), 0,
                                           (int)(uint32_t)(((N - w_row0 - 1) * (int64_t)K + k_run) * 2), 0x00020000);
  };
  // load i of a wave's W_LOADS for stage kt: its four x blocks, then its three W blocks
  auto fetch_one = [&](int kt, int i) __attribute__((always_inline)) {
    unsigned char* slot = w_smem + (kt % W_SLOTS) * W_STAGE;
    if (i < 4)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(xr, (lds_void_t*)(slot + (wave * 4 + i) * W_BLOCK), 16, xo[i], kt * (W_BK * 2), 0, 0);
    else
      __builtin_amdgcn_raw_ptr_buffer_load_lds(wr, (lds_void_t*)(slot + W_XHALF + (wave * (W_NB / 2) + i - 4) * W_BLOCK), 16,
                                               wo[i - 4], kt * (W_BK * 2), 0, 0);
  };
  auto fetch_first_stages = [&]() __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
      fetch_one(0, i);
      fetch_one(1, i);
    }
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
      fetch_one(2, i);
      fetch_one(3, i);
    }
  };

  f32x4_t acc[8][W_NB];
  bf16x8_t xf[2][8], wf[2][W_NB];
  // read i of the 8 + W_NB fragment reads of a stage: W first, in the order of their use
  auto read_one = [&](int kt, int set, int i) __attribute__((always_inline)) {
    const unsigned char* slot = w_smem + (kt % W_SLOTS) * W_STAGE + c * 64 + ((s ^ w_swizzle(c)) * 16);
    if (i < W_NB) wf[set][i] = *reinterpret_cast<const bf16x8_t*>(slot + W_XHALF + (wn * W_NB + i) * W_BLOCK);
    else xf[set][i - W_NB] = *reinterpret_cast<const bf16x8_t*>(slot + (wm * 8 + i - W_NB) * W_BLOCK);
  };
  // Iteration t, as described above. ``set`` is t % 2: the register set of stage t's fragments.
  auto iteration = [&](int t, auto set_c, auto fetch_c, auto read_c) __attribute__((always_inline)) {
    constexpr int set = decltype(set_c)::value;
    constexpr bool with_fetch = decltype(fetch_c)::value, with_read = decltype(read_c)::value;
#pragma unroll
    for (int g = 0; g < 16; ++g) {
      const int mi = g >> 1;
#pragma unroll
      for (int q = 0; q < W_NB / 2; ++q) {
        const int ni = (g & 1) * (W_NB / 2) + q;
        acc[mi][ni] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[set][ni], xf[set][mi], acc[mi][ni], 0, 0, 0);
      }
      // the order of issue is the order written here: the scheduler may move nothing across
      __builtin_amdgcn_sched_barrier(0);
      if (with_read && g < 8 + W_NB) read_one(t + 1, set ^ 1, g);
      if (with_fetch && (g & 1) == 0) {
        // a load after every second group: four pairs of loads in the even iteration, three in the
        // odd one, the two halves of a line six matrix instructions apart
        const int i = (g >> 2) + (set ? 4 : 0);
        if (i < W_LOADS) fetch_one(t + 4 - set + ((g >> 1) & 1), i);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (set == 0) {
      if (with_fetch) W_WAIT_LOADS(8);  // all but the 8 loads just issued: stages t + 2 and t + 3 are in
      else W_WAIT_LOADS(0);
    } else {
      // the next iteration asks for stage t + 6, which lands in the slot of stage t + 1: this wave's
      // fragment reads of that stage (issued above) have to be back before any wave may do so
      __builtin_amdgcn_s_waitcnt(0xC07F);
    }
    // every wave's loads of stage t + 2 are in LDS, and every wave has read stage t + 1
    W_BARRIER();
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using Yes = std::true_type;
  using No = std::false_type;

  int id = run_begin + local;
  if (id >= run_end) return;
  aim(id);
  fetch_first_stages();
  for (; id < run_end; id += per_xcd) {
    int tm, tn;
    tile_of(id, &tm, &tn);
#pragma unroll
    for (int mi = 0; mi < 8; ++mi)
#pragma unroll
      for (int ni = 0; ni < W_NB; ++ni) acc[mi][ni] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};
    W_WAIT_LOADS(0);
    W_BARRIER();  // the first four stages are in LDS
#pragma unroll
    for (int i = 0; i < 8 + W_NB; ++i) read_one(0, 0, i);
    // the first iteration's loads go into stage 0's slot: every wave has to have read it
    __builtin_amdgcn_s_waitcnt(0xC07F);
    W_BARRIER();
    int t = 0;
    for (; t + 4 < k_tiles; t += 2) {
      iteration(t, I0{}, Yes{}, Yes{});
      iteration(t + 1, I1{}, Yes{}, Yes{});
    }
    iteration(t, I0{}, No{}, Yes{});
    iteration(t + 1, I1{}, No{}, Yes{});
    iteration(t + 2, I0{}, No{}, Yes{});
    iteration(t + 3, I1{}, No{}, No{});
    // every slot is free: the first stages of the next tile come in while this one's results go out
    if (id + per_xcd < run_end) {
      aim(id + per_xcd);
      fetch_first_stages();
    }

    // ---- lane (c, s) holds y[m = .. + mi * 16 + c][4 s + e of W block ni], e = 0..3
    const int I = N / 2;
    const int out_cols = MODE == 2 ? I : N;
    constexpr int OUT_BLOCKS = MODE == 2 ? W_NB / 2 : W_NB;
    const int64_t col0 = MODE == 2 ? (int64_t)tn * (W_BN / 2) + wn * (W_BN / 4) : (int64_t)tn * W_BN + wn * (W_BN / 2);
    auto packed = [&](int mi, int ni, uint32_t* lo, uint32_t* hi) __attribute__((always_inline)) {
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (MODE == 2) {
          const float g = acc[mi][ni][e], up = acc[mi][ni + W_NB / 2][e];
          v[e] = g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)) * up;
        } else {
          v[e] = acc[mi][ni][e];
          const int64_t n = col0 + ni * 16 + 4 * s + e;
          if (a.bias != nullptr && n < N)
            v[e] += a.bias_f32 ? ((const float*)a.bias)[n] : __bfloat162float(((const bf16_t*)a.bias)[n]);
        }
      }
      *lo = w_pack_bf16(v[0], v[1]);
      *hi = w_pack_bf16(v[2], v[3]);
    };
    if constexpr (MODE == 3) {
      // the lane's four neighbouring columns of a row as they are: 16 bytes of the run's plane
      float* plane = (float*)a.C + (int64_t)(id / per_split) * M * a.ldc;
      const bool vec_ok = !(a.ldc & 3) && !((uintptr_t)a.C & 15);
#pragma unroll
      for (int mi = 0; mi < 8; ++mi) {
        const int64_t m = (int64_t)tm * W_BM + wm * 128 + mi * 16 + c;
        if (m >= M) continue;
#pragma unroll
        for (int ni = 0; ni < W_NB; ++ni) {
          const int64_t n0 = col0 + ni * 16 + 4 * s;
          if (n0 >= N) continue;
          float* dst = plane + m * a.ldc + n0;
          if (n0 + 4 <= N && vec_ok) {
            *reinterpret_cast<f32x4_t*>(dst) = acc[mi][ni];
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n0 + e < N) dst[e] = acc[mi][ni][e];
          }
        }
      }
      continue;
    }
    const bool wide_ok = !(a.ldc & 7) && !((uintptr_t)a.C & 15);
#pragma unroll
    for (int mi = 0; mi < 8; ++mi) {
      const int64_t m = (int64_t)tm * W_BM + wm * 128 + mi * 16 + c;
#pragma unroll
      for (int ni = 0; ni + 1 < OUT_BLOCKS; ni += 2) {
        uint32_t a_lo, a_hi, b_lo, b_hi;
        packed(mi, ni, &a_lo, &a_hi);
        packed(mi, ni + 1, &b_lo, &b_hi);
        // lane rows 1 and 3 of the first take lane rows 0 and 2 of the second: the lane then holds
        // columns 8 (s / 2) .. + 8 of block ni (s even) or of block ni + 1 (s odd)
        const cw_u32x2_t lo = __builtin_amdgcn_permlane16_swap(a_lo, b_lo, false, false);
        const cw_u32x2_t hi = __builtin_amdgcn_permlane16_swap(a_hi, b_hi, false, false);
        const int64_t n0 = col0 + (ni + (s & 1)) * 16 + 8 * (s >> 1);
        if (m >= M || n0 >= out_cols) continue;
        uint16_t* dst = (uint16_t*)a.C + m * a.ldc + n0;
        const uint32_t w4[4] = {lo[0], hi[0], lo[1], hi[1]};
        if (n0 + 8 <= out_cols && wide_ok) {
          *reinterpret_cast<uint4*>(dst) = make_uint4(w4[0], w4[1], w4[2], w4[3]);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n0 + e < out_cols) dst[e] = (uint16_t)(w4[e >> 1] >> ((e & 1) * 16));
        }
      }
      if (OUT_BLOCKS & 1) {
        constexpr int ni = OUT_BLOCKS - 1;
        uint32_t lo, hi;
        packed(mi, ni, &lo, &hi);
        const int64_t n0 = col0 + ni * 16 + 4 * s;
        if (m >= M || n0 >= out_cols) continue;
        uint16_t* dst = (uint16_t*)a.C + m * a.ldc + n0;
        if (n0 + 4 <= out_cols && !(a.ldc & 3)) {
          *reinterpret_cast<uint2*>(dst) = make_uint2(lo, hi);
        } else {
          const uint32_t w2[2] = {lo, hi};
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n0 + e < out_cols) dst[e] = (uint16_t)(w2[e >> 1] >> ((e & 1) * 16));
        }
      }
    }
  }
}

static const size_t W_SMEM = (size_t)W_SLOTS * W_STAGE;

static int w_tiles(int mode, int M, int N) {
  const int out_cols = mode == 2 ? N / 2 : N;
  const int per_tile = mode == 2 ? W_BN / 2 : W_BN;
  return ((M + W_BM - 1) / W_BM) * ((out_cols + per_tile - 1) / per_tile);
}

// Does the wide-tile kernel take this product? Returns its number of tiles, or 0.
CW_EXPORT int cw_gemm_bf16_wide_tiles(int mode, int M, int N, int K, int64_t ldx) {
  if (M <= 0 || N <= 0 || (mode != 0 && mode != 2) || (mode == 2 && (N & 1))) return 0;
  if ((K & 63) || K < 256 || (ldx & 7) || ldx < K) return 0;
  if ((int64_t)N * K * 2 >= (1ll << 32) || (int64_t)M * ldx * 2 >= (1ll << 32)) return 0;
  return w_tiles(mode, M, N);
}

// 1 if the wide-tile kernel sums this product in ``k_splits`` runs of K (cw_gemm_bf16_wide_partial).
CW_EXPORT int cw_gemm_bf16_wide_partial_ok(int M, int N, int K, int64_t ldx, int k_splits) {
  if (k_splits < 2 || k_splits > 16 || K % (64 * k_splits) || K / k_splits < 256) return 0;
  return cw_gemm_bf16_wide_tiles(0, M, N, K, ldx) > 0 ? 1 : 0;
}

template <int MODE>
static int w_launch(WideArgs a, int workgroups, hipStream_t stream) {
  static bool raised = false;
  if (!raised) {
    if (hipFuncSetAttribute((const void*)gemm_wide_bf16_kernel<MODE>, hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)W_SMEM) != hipSuccess)
      return CW_ERR_LAUNCH;
    raised = true;
  }
  const int out_cols = MODE == 2 ? a.N / 2 : a.N;
  const int per_tile = MODE == 2 ? W_BN / 2 : W_BN;
  a.tiles_n = (out_cols + per_tile - 1) / per_tile;
  a.tiles_m = (a.M + W_BM - 1) / W_BM;
  const int total = a.tiles_m * a.tiles_n * (MODE == 3 ? a.k_splits : 1);
  // a multiple of 8 workgroups, so that every XCD gets the same number of them
  int grid = total < workgroups ? total : workgroups;
  grid = (grid + 7) & ~7;
  hipLaunchKernelGGL((gemm_wide_bf16_kernel<MODE>), dim3(grid), dim3(256), W_SMEM, stream, a);
  return cw_launch_status();
}

// The same product as cw_gemm_bf16_tiled through the wide-tile kernel, for the shapes that
// cw_gemm_bf16_wide_tiles takes. ``workgroups``: how many to launch at most, the number of compute
// units of the GPU (one workgroup fills a unit).
CW_EXPORT int cw_gemm_bf16_wide(int mode, const void* X, int64_t ldx, const void* W, const void* bias, int bias_f32,
                                void* C, int64_t ldc, int M, int N, int K, int workgroups, hipStream_t stream) {
  if (M < 0 || N <= 0 || K <= 0 || (mode != 0 && mode != 2) || workgroups < 8) return CW_ERR_ARG;
  if (((uintptr_t)X & 15) || ((uintptr_t)W & 15) || ((uintptr_t)C & 7)) return CW_ERR_ARG;
  if (mode == 2 && ((N & 1) || bias != nullptr)) return CW_ERR_ARG;
  if (ldc < (mode == 2 ? N / 2 : N)) return CW_ERR_ARG;
  if (M == 0) return CW_OK;
  if (cw_gemm_bf16_wide_tiles(mode, M, N, K, ldx) == 0) return CW_ERR_SIZE;
  WideArgs a{(const bf16_t*)X, ldx, (const bf16_t*)W, bias, bias_f32, C, ldc, M, N, K, 0, 0, 1};
  return mode == 2 ? w_launch<2>(a, workgroups, stream) : w_launch<0>(a, workgroups, stream);
}

// parts[z] = x[:, run z of K] W[:, run z of K]^T for z < k_splits: float32 planes [k_splits, M, N]
// (rows ldc floats apart) whose sum, taken in the order of z, is the product. For the shapes that
// cw_gemm_bf16_wide_partial_ok takes.
CW_EXPORT int cw_gemm_bf16_wide_partial(const void* X, int64_t ldx, const void* W, float* parts, int64_t ldc, int M,
                                        int N, int K, int k_splits, int workgroups, hipStream_t stream) {
  if (M < 0 || N <= 0 || K <= 0 || workgroups < 8 || !parts || ldc < N) return CW_ERR_ARG;
  if (((uintptr_t)X & 15) || ((uintptr_t)W & 15) || ((uintptr_t)parts & 15)) return CW_ERR_ARG;
  if (M == 0) return CW_OK;
  if (!cw_gemm_bf16_wide_partial_ok(M, N, K, ldx, k_splits)) return CW_ERR_SIZE;
  WideArgs a{(const bf16_t*)X, ldx, (const bf16_t*)W, nullptr, 0, parts, ldc, M, N, K, 0, 0, k_splits};
  return w_launch<3>(a, workgroups, stream);
}
