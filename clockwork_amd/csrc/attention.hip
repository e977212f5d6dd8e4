// Causal attention over a paged key/value cache for gfx950, one head size per build
// (compile with -DCW_HD=<head_dim>, a multiple of 16 from 16 to 256).
//
// One kernel serves portions of prompts and single decoded tokens: a work item is a run of
// consecutive query tokens of one request; a workgroup takes one item, one key/value head and
// all (or a chunk of) the query heads of that head's group, so a key/value tile is fetched once
// for the whole group. The key range of an item can be cut into splits that run in parallel
// and are merged by a second kernel (decode with few requests and long contexts).
//
// Scores, softmax and the output accumulation are float32 whatever the cache type is.
// A token at position p reads keys j <= p, and j > p - window when a window is set. Pages are
// found through the request's block table; positions outside an item's key range are never
// dereferenced (their table entries may be stale or -1).
#include "common.h"

#ifndef CW_HD
#error "compile with -DCW_HD=<head_dim>"
#endif
static_assert(CW_HD % 16 == 0 && CW_HD >= 16 && CW_HD <= 256, "head_dim: multiples of 16 up to 256");

struct AttnParams {
  const void* q;          // [tokens, q_stride] query heads at column head * HD
  int64_t q_stride;
  void* out;              // [tokens, out_stride]
  int64_t out_stride;
  const void* k_cache;    // [slots, nkv, HD]
  const void* v_cache;
  const int* block_tables;  // [requests, table_stride]
  int table_stride;
  const int* ctx_lens;    // [requests] keys of the request after this step
  const int* cu_q;        // [requests + 1] offsets of each request's tokens in the batch
  const int* items;       // [n_items, 4]: request, first token (relative), tokens, part | parts << 8 (prefill kernel)
  int nh, nkv, block_size;
  int bs_shift;           // log2(block_size) when it is a power of two, else -1
  int gh;                 // query heads of a group handled by one workgroup
  int n_chunks;           // ceil(group / gh)
  int n_splits;
  int window;             // 0: none
  float scale;
  float* part_o;          // [n_items, nkv * n_chunks, n_splits, ROWS, HD] unnormalised outputs
  float* part_ml;         // [n_items, nkv * n_chunks, n_splits, ROWS, 2] running max, sum
  const void* zeros;      // at least HD zero elements: what a masked key or value row is loaded from
  // decode kernel only
  int identity;           // 1: item i is request i and its one token is row i of the batch (items, cu_q unread)
  int split_keys;         // > 0: split s takes keys [s * split_keys, (s + 1) * split_keys), a multiple of 32
};

// page of a position and the offset inside it; POW2: the page size is a power of two (shift given)
template <bool POW2> __device__ __forceinline__ int cw_page_index(int pos, int bs, int shift) {
  return POW2 ? pos >> shift : pos / bs;
}
template <bool POW2> __device__ __forceinline__ int cw_page_offset(int pos, int bs, int shift) {
  return POW2 ? pos & (bs - 1) : pos % bs;
}
static inline int cw_log2_or_minus1(int v) {
  for (int s = 0; s < 31; ++s) if ((1 << s) == v) return s;
  return -1;
}

template <typename T> struct Vec16;
template <> struct Vec16<float> {
  static constexpr int N = 4;
  __device__ static void load(const float* p, float* o) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
};
template <> struct Vec16<bf16_t> {
  static constexpr int N = 8;
  __device__ static void load(const bf16_t* p, float* o) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = __uint_as_float(w[i] << 16);
      o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
};

template <int HD, int ROWS, int BN> struct TileShape {
  static constexpr int QS = HD + 4;   // query row stride in floats (16-byte rows)
  static constexpr int KS = HD + 1;   // key row stride: odd, so a column read hits distinct banks
  static constexpr int VS = HD + 4;   // value row stride (16-byte rows); also the buffer's row size
  static constexpr int SS = BN + 1;
  static constexpr int FLOATS = ROWS * QS + BN * VS + ROWS * SS + 3 * ROWS;
};

template <typename T, int HD, int ROWS, int BN>
__global__ __launch_bounds__(256) void attn_tile_kernel(AttnParams p) {
  using S = TileShape<HD, ROWS, BN>;
  extern __shared__ __align__(16) float smem[];
  float* Qs = smem;
  float* KVs = Qs + ROWS * S::QS;
  float* Ss = KVs + BN * S::VS;
  float* m_s = Ss + ROWS * S::SS;
  float* l_s = m_s + ROWS;
  float* a_s = l_s + ROWS;

  const int tid = threadIdx.x;
  const int item = blockIdx.x;
  const int kvh = blockIdx.y / p.n_chunks;
  const int chunk = blockIdx.y % p.n_chunks;
  const int split = blockIdx.z;
  const int req = p.items[4 * item], tok0 = p.items[4 * item + 1];
  const int ctx = p.ctx_lens[req];
  const int q_begin = p.cu_q[req];
  const int qlen = p.cu_q[req + 1] - q_begin;
  // an item may reach past the request's tokens (work items laid out for a longer portion than
  // the step brings): what lies past them is not computed
  const int ntok = min(p.items[4 * item + 2], qlen - tok0);
  if (ntok <= 0) return;
  const int group = p.nh / p.nkv;
  const int gh = p.gh;
  const int pos0 = ctx - qlen + tok0;  // absolute position of the item's first token
  const int kv_end = pos0 + ntok;
  const int kv_lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
  const int tile0 = kv_lo / BN;
  const int n_tiles = (kv_end + BN - 1) / BN - tile0;
  const int tps = (n_tiles + p.n_splits - 1) / p.n_splits;
  const int t_begin = tile0 + split * tps;
  const int t_end = min(tile0 + n_tiles, t_begin + tps);
  const T* qp = (const T*)p.q;
  const T* kc = (const T*)p.k_cache;
  const T* vc = (const T*)p.v_cache;
  const int* table = p.block_tables + (int64_t)req * p.table_stride;

  // ---- query tile: row r = (token r / gh, head chunk * gh + r % gh); unused rows are zero
  for (int idx = tid; idx < ROWS * HD; idx += 256) {
    const int r = idx / HD, d = idx - r * HD;
    const int tok = r / gh, hig = chunk * gh + (r - tok * gh);
    float v = 0.0f;
    if (tok < ntok && hig < group)
      v = cw_to_float(qp[(int64_t)(q_begin + tok0 + tok) * p.q_stride + (kvh * group + hig) * HD + d]);
    Qs[r * S::QS + d] = v;
  }
  if (tid < ROWS) { m_s[tid] = -INFINITY; l_s[tid] = 0.0f; a_s[tid] = 1.0f; }

  // ---- output accumulators: thread = (dg: 4 consecutive columns, stripe: rows stripe + k * NSTRIPE)
  constexpr int NDG = HD / 4;
  constexpr int NSTRIPE = 256 / NDG;
  constexpr int RPT = (ROWS + NSTRIPE - 1) / NSTRIPE;
  const int dg = tid % NDG, stripe = tid / NDG;
  const bool pv_active = stripe < NSTRIPE;
  float acc[RPT][4];
#pragma unroll
  for (int k = 0; k < RPT; ++k) { acc[k][0] = acc[k][1] = acc[k][2] = acc[k][3] = 0.0f; }

  constexpr int VEC = Vec16<T>::N;
  constexpr int CPR = HD / VEC;  // 16-byte chunks per cache row
  constexpr int NRG = 256 / BN;  // row groups of the score phase
  constexpr int RPT_S = ROWS / NRG;
  constexpr int TPR = 256 / ROWS;  // threads per row of the softmax phase
  static_assert(ROWS % NRG == 0 && 256 % ROWS == 0 && TPR <= 64, "tile shape");

  __syncthreads();
  for (int t = t_begin; t < t_end; ++t) {
    const int kv0 = t * BN;
    // ---- keys of the tile -> LDS as float32
    for (int idx = tid; idx < BN * CPR; idx += 256) {
      const int j = idx / CPR, ch = idx - j * CPR;
      const int pos = kv0 + j;
      float v[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] = 0.0f;
      if (pos >= kv_lo && pos < kv_end) {
        const int page = table[pos / p.block_size];
        if (page >= 0) {
          const int64_t slot = (int64_t)page * p.block_size + pos % p.block_size;
          Vec16<T>::load(kc + (slot * p.nkv + kvh) * HD + ch * VEC, v);
        }
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) KVs[j * S::KS + ch * VEC + e] = v[e];
    }
    __syncthreads();
    // ---- scores: thread = (key c, row group rg), rows rg + k * NRG
    {
      const int c = tid % BN, rg = tid / BN;
      float s[RPT_S];
#pragma unroll
      for (int k = 0; k < RPT_S; ++k) s[k] = 0.0f;
      const float* kr = KVs + c * S::KS;
      for (int d0 = 0; d0 < HD; d0 += 4) {
        const float k0 = kr[d0], k1 = kr[d0 + 1], k2 = kr[d0 + 2], k3 = kr[d0 + 3];
#pragma unroll
        for (int k = 0; k < RPT_S; ++k) {
          const float4 qv = *reinterpret_cast<const float4*>(&Qs[(rg + k * NRG) * S::QS + d0]);
          s[k] = fmaf(qv.x, k0, s[k]);
          s[k] = fmaf(qv.y, k1, s[k]);
          s[k] = fmaf(qv.z, k2, s[k]);
          s[k] = fmaf(qv.w, k3, s[k]);
        }
      }
      const int pos_k = kv0 + c;
#pragma unroll
      for (int k = 0; k < RPT_S; ++k) {
        const int r = rg + k * NRG;
        const int tok = r / gh, hig = chunk * gh + (r - tok * gh);
        const int prow = pos0 + tok;
        const int lo = p.window > 0 ? prow - p.window + 1 : 0;
        const bool ok = tok < ntok && hig < group && pos_k <= prow && pos_k >= lo;
        Ss[r * S::SS + c] = ok ? s[k] * p.scale : -INFINITY;
      }
    }
    __syncthreads();
    // ---- values of the tile -> LDS (the key rows are no longer read)
    for (int idx = tid; idx < BN * CPR; idx += 256) {
      const int j = idx / CPR, ch = idx - j * CPR;
      const int pos = kv0 + j;
      float v[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] = 0.0f;
      if (pos >= kv_lo && pos < kv_end) {
        const int page = table[pos / p.block_size];
        if (page >= 0) {
          const int64_t slot = (int64_t)page * p.block_size + pos % p.block_size;
          Vec16<T>::load(vc + (slot * p.nkv + kvh) * HD + ch * VEC, v);
        }
      }
#pragma unroll
      for (int e = 0; e < VEC; ++e) KVs[j * S::VS + ch * VEC + e] = v[e];
    }
    // ---- online softmax: TPR consecutive lanes share a row
    {
      const int r = tid / TPR, sub = tid % TPR;
      float* srow = Ss + r * S::SS;
      float tmax = -INFINITY;
      for (int c = sub; c < BN; c += TPR) tmax = fmaxf(tmax, srow[c]);
#pragma unroll
      for (int off = TPR / 2; off > 0; off >>= 1) tmax = fmaxf(tmax, __shfl_xor(tmax, off, 64));
      const float m_old = m_s[r];
      const float m_new = fmaxf(m_old, tmax);
      float alpha = 1.0f, sum = 0.0f;
      if (m_new == -INFINITY) {
        for (int c = sub; c < BN; c += TPR) srow[c] = 0.0f;
      } else {
        alpha = expf(m_old - m_new);
        for (int c = sub; c < BN; c += TPR) {
          const float e = expf(srow[c] - m_new);
          srow[c] = e;
          sum += e;
        }
      }
#pragma unroll
      for (int off = TPR / 2; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
      if (sub == 0) {
        m_s[r] = m_new;
        l_s[r] = l_s[r] * alpha + sum;
        a_s[r] = alpha;
      }
    }
    __syncthreads();
    // ---- out += P * V
    if (pv_active) {
#pragma unroll
      for (int k = 0; k < RPT; ++k) {
        const int r = stripe + k * NSTRIPE;
        const float a = r < ROWS ? a_s[r] : 1.0f;
        acc[k][0] *= a; acc[k][1] *= a; acc[k][2] *= a; acc[k][3] *= a;
      }
      for (int c = 0; c < BN; ++c) {
        const float4 v = *reinterpret_cast<const float4*>(&KVs[c * S::VS + dg * 4]);
#pragma unroll
        for (int k = 0; k < RPT; ++k) {
          const int r = stripe + k * NSTRIPE;
          const float pr = r < ROWS ? Ss[r * S::SS + c] : 0.0f;
          acc[k][0] = fmaf(pr, v.x, acc[k][0]);
          acc[k][1] = fmaf(pr, v.y, acc[k][1]);
          acc[k][2] = fmaf(pr, v.z, acc[k][2]);
          acc[k][3] = fmaf(pr, v.w, acc[k][3]);
        }
      }
    }
    __syncthreads();
  }

  // ---- write: final rows when there is one split, partial sums otherwise
  if (!pv_active) return;
  if (p.n_splits == 1) {
    T* op = (T*)p.out;
#pragma unroll
    for (int k = 0; k < RPT; ++k) {
      const int r = stripe + k * NSTRIPE;
      if (r >= ROWS) continue;
      const int tok = r / gh, hig = chunk * gh + (r - tok * gh);
      if (tok >= ntok || hig >= group) continue;
      const float inv = 1.0f / l_s[r];
      T* o = op + (int64_t)(q_begin + tok0 + tok) * p.out_stride + (kvh * group + hig) * HD + dg * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = cw_from_float<T>(acc[k][e] * inv);
    }
  } else {
    const int64_t base = ((int64_t)item * gridDim.y + blockIdx.y) * p.n_splits + split;
#pragma unroll
    for (int k = 0; k < RPT; ++k) {
      const int r = stripe + k * NSTRIPE;
      if (r >= ROWS) continue;
      float* o = p.part_o + (base * ROWS + r) * HD + dg * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = acc[k][e];
      if (dg == 0) {
        p.part_ml[(base * ROWS + r) * 2] = m_s[r];
        p.part_ml[(base * ROWS + r) * 2 + 1] = l_s[r];
      }
    }
  }
}

// Merge the splits of every (item, head) row: out = sum_s e^(m_s - M) o_s / sum_s e^(m_s - M) l_s,
// splits taken in ascending order.
template <typename T, int HD, int ROWS>
__global__ __launch_bounds__(256) void attn_merge_kernel(AttnParams p) {
  const int item = blockIdx.x;
  const int kvh = blockIdx.y / p.n_chunks;
  const int chunk = blockIdx.y % p.n_chunks;
  const int req = p.items[4 * item], tok0 = p.items[4 * item + 1];
  const int q_begin = p.cu_q[req];
  // as in the kernel above: an item may reach past the request's tokens, and those rows are nobody's
  const int ntok = min(p.items[4 * item + 2], p.cu_q[req + 1] - q_begin - tok0);
  const int group = p.nh / p.nkv;
  const int gh = p.gh;
  const int64_t base = ((int64_t)item * gridDim.y + blockIdx.y) * p.n_splits;
  T* op = (T*)p.out;
  for (int idx = threadIdx.x; idx < ROWS * HD; idx += 256) {
    const int r = idx / HD, d = idx - r * HD;
    const int tok = r / gh, hig = chunk * gh + (r - tok * gh);
    if (tok >= ntok || hig >= group) continue;
    float M = -INFINITY;
    for (int s = 0; s < p.n_splits; ++s) M = fmaxf(M, p.part_ml[((base + s) * ROWS + r) * 2]);
    float L = 0.0f, O = 0.0f;
    for (int s = 0; s < p.n_splits; ++s) {
      const float m = p.part_ml[((base + s) * ROWS + r) * 2];
      if (m == -INFINITY) continue;
      const float w = expf(m - M);
      L = fmaf(p.part_ml[((base + s) * ROWS + r) * 2 + 1], w, L);
      O = fmaf(p.part_o[((base + s) * ROWS + r) * HD + d], w, O);
    }
    op[(int64_t)(q_begin + tok0 + tok) * p.out_stride + (kvh * group + hig) * HD + d] =
        cw_from_float<T>(O / L);
  }
}

template <typename T, int ROWS, int BN>
static int launch_attention(const AttnParams& p, int n_items, hipStream_t stream) {
  constexpr int HD = CW_HD;
  const size_t smem = sizeof(float) * TileShape<HD, ROWS, BN>::FLOATS;
  static int limit = -1;
  if (limit < 0) {
    int dev = 0, v = 0;
    if (hipGetDevice(&dev) != hipSuccess) return CW_ERR_LAUNCH;
    if (hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) != hipSuccess)
      return CW_ERR_LAUNCH;
    limit = v;
  }
  if ((size_t)limit < smem) return CW_ERR_SIZE;
  static bool raised = false;
  if (!raised) {
    if (hipFuncSetAttribute((const void*)attn_tile_kernel<T, HD, ROWS, BN>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
      return CW_ERR_LAUNCH;
    raised = true;
  }
  dim3 grid(n_items, p.nkv * p.n_chunks, p.n_splits), block(256);
  hipLaunchKernelGGL((attn_tile_kernel<T, HD, ROWS, BN>), grid, block, smem, stream, p);
  if (p.n_splits > 1) {
    dim3 mgrid(n_items, p.nkv * p.n_chunks);
    hipLaunchKernelGGL((attn_merge_kernel<T, HD, ROWS>), mgrid, block, 0, stream, p);
  }
  return cw_launch_status();
}

CW_EXPORT int cw_attention_head_dim() { return CW_HD; }

// Floats of workspace a launch with these sizes needs (0 when n_splits == 1).
CW_EXPORT int64_t cw_attention_workspace_floats(int rows, int n_items, int nkv, int n_chunks, int n_splits) {
  if (n_splits <= 1) return 0;
  return (int64_t)n_items * nkv * n_chunks * n_splits * rows * (CW_HD + 2);
}

// rows: 64 (portions of prompts) or 16 (single tokens, few tokens). gh * tokens-per-item <= rows.
CW_EXPORT int cw_attention(int rows, int dtype, const void* q, int64_t q_stride, void* out,
                           int64_t out_stride, const void* k_cache, const void* v_cache,
                           const int* block_tables, int table_stride, const int* ctx_lens,
                           const int* cu_q, const int* items, int n_items, int nh, int nkv,
                           int block_size, int gh, int n_splits, int window, float scale,
                           float* workspace, int64_t workspace_floats, hipStream_t stream) {
  if (n_items < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || block_size <= 0 || table_stride <= 0)
    return CW_ERR_ARG;
  if (rows != 64 && rows != 16) return CW_ERR_ARG;
  const int group = nh / nkv;
  if (gh < 1 || gh > group || gh > rows || n_splits < 1 || n_splits > 65535 || window < 0) return CW_ERR_ARG;
  if (n_items == 0) return CW_OK;
  AttnParams p{};
  p.q = q; p.q_stride = q_stride; p.out = out; p.out_stride = out_stride;
  p.k_cache = k_cache; p.v_cache = v_cache; p.block_tables = block_tables;
  p.table_stride = table_stride; p.ctx_lens = ctx_lens; p.cu_q = cu_q; p.items = items;
  p.nh = nh; p.nkv = nkv; p.block_size = block_size; p.bs_shift = cw_log2_or_minus1(block_size); p.gh = gh;
  p.n_chunks = (group + gh - 1) / gh; p.n_splits = n_splits; p.window = window; p.scale = scale;
  if ((int64_t)nkv * p.n_chunks > 65535) return CW_ERR_SIZE;
  const int64_t need = cw_attention_workspace_floats(rows, n_items, nkv, p.n_chunks, n_splits);
  if (need > 0 && (workspace == nullptr || workspace_floats < need)) return CW_ERR_ARG;
  const int64_t n_o = need / (CW_HD + 2) * CW_HD;
  p.part_o = workspace;
  p.part_ml = workspace ? workspace + n_o : nullptr;
  p.zeros = nullptr;
  constexpr int BN = CW_HD <= 128 ? 64 : 32;
  if (dtype == CW_F32) {
    return rows == 64 ? launch_attention<float, 64, BN>(p, n_items, stream)
                      : launch_attention<float, 16, BN>(p, n_items, stream);
  } else if (dtype == CW_BF16) {
    return rows == 64 ? launch_attention<bf16_t, 64, BN>(p, n_items, stream)
                      : launch_attention<bf16_t, 16, BN>(p, n_items, stream);
  }
  return CW_ERR_DTYPE;
}

// =====================================================================================
// bfloat16 decode attention: one query token per work item, keys and values streamed at memory
// speed, all products on the matrix cores.
//
// A workgroup (4 waves) takes one (request, key/value head, split of the key range); its waves
// take turns on tiles of 32 keys. Per tile:
//   S^T[key, head] = K * Q^T        v_mfma_f32_16x16x32_bf16; the up to 16 heads of the group are
//                                   the columns, so every key is fetched once for the whole group;
//   softmax per head in float32: a lane holds 8 keys of one head, two shuffles finish a head;
//   V^T from V: V times a 0/1 selector matrix comes back with keys in the lane's registers
//                                   (the layout the next product needs), values bit-exact;
//   O^T[d, head] += V^T * P^T       P^T is the softmax output as it lies in the registers.
// K and V fragments are loaded from the pages straight into operand layout with 16-byte loads;
// the next tile's loads are issued before the current tile is computed. Waves are merged through
// LDS at the end; splits are merged by a second, small kernel.
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define DEC_WAVES 4

template <int HD, bool POW2>
__global__ __launch_bounds__(256) void attn_decode_bf16_kernel(AttnParams p) {
  constexpr int NF = HD / 32;  // 32-element steps over the head dimension
  constexpr int ND = HD / 16;  // 16-wide blocks of the head dimension
  extern __shared__ __align__(16) float dyn_s[];  // [waves][16 heads][HD] outputs, then this split's pages
  float* o_s = dyn_s;
  int* tbl = reinterpret_cast<int*>(dyn_s + DEC_WAVES * 16 * HD);
  __shared__ float M_s[DEC_WAVES][16];
  __shared__ float L_s[DEC_WAVES][16];

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c = lane & 15, s = lane >> 4;
  const int item = blockIdx.x;
  const int kvh = blockIdx.y / p.n_chunks, chunk = blockIdx.y % p.n_chunks;
  const int split = blockIdx.z;
  // Every trip to memory that depends on an earlier one costs about a microsecond, which is what
  // a short context takes in all: with ``identity`` and fixed key ranges per split, the context
  // length, the table entries and the query are fetched side by side, then keys and values.
  const bool ident = p.identity != 0;
  const int req = ident ? item : p.items[4 * item];
  const int tok0 = ident ? 0 : p.items[4 * item + 1];
  const int ctx = p.ctx_lens[req];
  const int q_begin = ident ? item : p.cu_q[req];
  const int qlen = ident ? 1 : p.cu_q[req + 1] - q_begin;
  const int group = p.nh / p.nkv;
  const int gh = p.gh;
  const bf16_t* kc = (const bf16_t*)p.k_cache;
  const bf16_t* vc = (const bf16_t*)p.v_cache;
  const bf16_t* zrow = (const bf16_t*)p.zeros;
  const int bs = p.block_size, sh = p.bs_shift;
  const int* table = p.block_tables + (int64_t)req * p.table_stride;
  int page0 = 0;
  if (p.split_keys > 0) {
    // the pages of this split's key range -> LDS, whatever the context length turns out to be
    const int k_first = split * p.split_keys;
    const int k_last = min(k_first + p.split_keys, p.table_stride * bs) - 1;
    page0 = cw_page_index<POW2>(k_first, bs, sh);
    const int n_pages = k_last >= k_first ? cw_page_index<POW2>(k_last, bs, sh) - page0 + 1 : 0;
    for (int i = threadIdx.x; i < n_pages; i += 256) tbl[i] = table[page0 + i];
  }
  const int pos = ctx - qlen + tok0;
  const int lo = p.window > 0 ? max(0, pos - p.window + 1) : 0;
  const int tile0 = lo / 32;
  const int n_tiles = pos / 32 + 1 - tile0;
  int t_begin, t_end;
  if (p.split_keys > 0) {
    t_begin = max(tile0, split * (p.split_keys / 32));
    t_end = min(tile0 + n_tiles, (split + 1) * (p.split_keys / 32));
  } else {
    const int tps = (n_tiles + p.n_splits - 1) / p.n_splits;
    t_begin = tile0 + split * tps;
    t_end = min(tile0 + n_tiles, t_begin + tps);
    // the pages of this split's keys -> LDS, so that no tile waits for a table entry from memory
    page0 = cw_page_index<POW2>(t_begin * 32, bs, sh);
    const int last_key = min(pos, t_end * 32 - 1);
    const int n_pages = t_end > t_begin ? cw_page_index<POW2>(last_key, bs, sh) - page0 + 1 : 0;
    for (int i = threadIdx.x; i < n_pages; i += 256) tbl[i] = table[page0 + i];
  }
  __syncthreads();

  // query fragments (B operand): lane (c, s) holds head c, elements (j * 4 + s) * 8 .. + 7
  bf16x8_t qf[NF];
  const int hig = chunk * gh + c;
  const bool head_ok = c < gh && hig < group;
  {
    const bf16_t* qrow = head_ok ? (const bf16_t*)p.q + (int64_t)(q_begin + tok0) * p.q_stride + (kvh * group + hig) * HD : zrow;
#pragma unroll
    for (int j = 0; j < NF; ++j) qf[j] = *reinterpret_cast<const bf16x8_t*>(qrow + (j * 4 + s) * 8);
  }
  // selectors (B operand) that pick elements 0..15 / 16..31 of a 32-element step: (k = 8s + e, n = c)
  bf16x8_t sel_lo, sel_hi;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    sel_lo[e] = (8 * s + e == c) ? (__bf16)1.0f : (__bf16)0.0f;
    sel_hi[e] = (8 * s + e == 16 + c) ? (__bf16)1.0f : (__bf16)0.0f;
  }

  // loads of one 32-key tile, always issued: a masked key is read from a row of zeros
  auto load_tile = [&](int t, bf16x8_t (*kf)[NF], bf16x8_t (*vf)[NF]) {
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      const int kp = t * 32 + kb * 16 + c;
      const bool ok = t < t_end && kp >= lo && kp <= pos;
      const int page = tbl[ok ? cw_page_index<POW2>(kp, bs, sh) - page0 : 0];
      const bool have = ok && page >= 0;
      const int64_t off = (((int64_t)page * bs + cw_page_offset<POW2>(kp, bs, sh)) * p.nkv + kvh) * HD;
      const bf16_t* kr = have ? kc + off : zrow;
      const bf16_t* vr = have ? vc + off : zrow;
#pragma unroll
      for (int j = 0; j < NF; ++j) kf[kb][j] = *reinterpret_cast<const bf16x8_t*>(kr + (j * 4 + s) * 8);
#pragma unroll
      for (int j = 0; j < NF; ++j) vf[kb][j] = *reinterpret_cast<const bf16x8_t*>(vr + j * 32 + s * 8);
    }
  };

  f32x4_t o[ND];
#pragma unroll
  for (int db = 0; db < ND; ++db) o[db] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};
  float m_run = -INFINITY, l_run = 0.0f;  // of head c, the same in all four lane groups
  bf16x8_t kf[2][NF], vf[2][NF], kf_n[2][NF], vf_n[2][NF];
  load_tile(t_begin + wave, kf, vf);
  for (int t = t_begin + wave; t < t_end; t += DEC_WAVES) {
    const int kv0 = t * 32;
    load_tile(t + DEC_WAVES, kf_n, vf_n);  // the wave's next tile is on its way meanwhile
    // ---- S^T = K Q^T, keys 4s..4s+3 of each 16-key block for head c
    float sv[8];
    float tmax = -INFINITY;
#pragma unroll
    for (int kb = 0; kb < 2; ++kb) {
      f32x4_t sc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int j = 0; j < NF; ++j) sc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[kb][j], qf[j], sc, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int kp = kv0 + kb * 16 + 4 * s + i;
        const float v = (kp >= lo && kp <= pos) ? sc[i] * p.scale : -INFINITY;
        sv[kb * 4 + i] = v;
        tmax = fmaxf(tmax, v);
      }
    }
    tmax = cw_quad_max(tmax);
    const float m_new = fmaxf(m_run, tmax);
    float alpha = 1.0f, psum = 0.0f;
    bf16x8_t pf;
#pragma unroll
    for (int e = 0; e < 8; ++e) pf[e] = (__bf16)0.0f;
    if (m_new != -INFINITY) {
      alpha = __expf(m_run - m_new);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float pe = __expf(sv[e] - m_new);
        psum += pe;
        pf[e] = (__bf16)pe;
      }
    }
    psum = cw_quad_sum(psum);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int db = 0; db < ND; ++db) o[db] *= alpha;
    }
    // ---- O^T += V^T P^T
#pragma unroll
    for (int j = 0; j < NF; ++j) {
      bf16x8_t vt_lo, vt_hi;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        const f32x4_t zero = {0.0f, 0.0f, 0.0f, 0.0f};
        const f32x4_t tl = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[kb][j], sel_lo, zero, 0, 0, 0);
        const f32x4_t th = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf[kb][j], sel_hi, zero, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          vt_lo[kb * 4 + i] = (__bf16)tl[i];
          vt_hi[kb * 4 + i] = (__bf16)th[i];
        }
      }
      o[2 * j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt_lo, pf, o[2 * j], 0, 0, 0);
      o[2 * j + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt_hi, pf, o[2 * j + 1], 0, 0, 0);
    }
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int j = 0; j < NF; ++j) { kf[kb][j] = kf_n[kb][j]; vf[kb][j] = vf_n[kb][j]; }
  }

  // a context beyond the fixed key ranges (the caller promised there is none) must not pass for a result
  if (p.split_keys > 0 && pos >= p.n_splits * p.split_keys) l_run = NAN;
  // ---- merge the waves: o_s[wave][head c][d], lane (c, s) holds d = db * 16 + 4s .. + 3
  if (s == 0) { M_s[wave][c] = m_run; L_s[wave][c] = l_run; }
#pragma unroll
  for (int db = 0; db < ND; ++db)
    *reinterpret_cast<f32x4_t*>(&o_s[(wave * 16 + c) * HD + db * 16 + 4 * s]) = o[db];
  __syncthreads();
  const int64_t base = ((int64_t)item * gridDim.y + blockIdx.y) * p.n_splits + split;
  for (int idx = threadIdx.x; idx < gh * HD; idx += 256) {
    const int g = idx / HD, d = idx - g * HD;
    const int hg = chunk * gh + g;
    if (hg >= group) continue;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) M = fmaxf(M, M_s[w][g]);
    float L = 0.0f, O = 0.0f;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) {
      const float mw = M_s[w][g];
      const float wgt = mw == -INFINITY ? 0.0f : __expf(mw - M);
      L = fmaf(L_s[w][g], wgt, L);
      O = fmaf(o_s[(w * 16 + g) * HD + d], wgt, O);
    }
    if (p.n_splits == 1) {
      ((bf16_t*)p.out)[(int64_t)(q_begin + tok0) * p.out_stride + (kvh * group + hg) * HD + d] =
          __float2bfloat16(O / L);
    } else {
      p.part_o[(base * gh + g) * HD + d] = O;
      if (d == 0) {
        p.part_ml[(base * gh + g) * 2] = M;
        p.part_ml[(base * gh + g) * 2 + 1] = L;
      }
    }
  }
}

// Merge of the decode kernel's splits: one workgroup per (item, head) of blockDim.x = G * HD
// threads. Thread (g, d) sums element d over splits g, g + G, ...; the G sums meet in LDS. The
// statistics of all splits go through LDS first, and partial outputs are fetched eight at a
// time, so the kernel is a few memory round trips long whatever the number of splits.
#define DEC_MAX_SPLITS 256

template <int HD>
__global__ __launch_bounds__(1024) void attn_decode_merge_kernel(AttnParams p) {
  __shared__ float ms[DEC_MAX_SPLITS], ls[DEC_MAX_SPLITS];
  __shared__ float o_s[1024], l_s[1024 / HD];
  const int gh = p.gh;
  const int item = blockIdx.x;
  const int y = blockIdx.y / gh, g = blockIdx.y % gh;
  const int kvh = y / p.n_chunks, chunk = y % p.n_chunks;
  const int group = p.nh / p.nkv;
  const int hg = chunk * gh + g;
  if (hg >= group) return;
  const bool ident = p.identity != 0;
  const int tok0 = ident ? 0 : p.items[4 * item + 1];
  const int q_begin = ident ? item : p.cu_q[p.items[4 * item]];
  const int64_t base = ((int64_t)item * (p.nkv * p.n_chunks) + y) * p.n_splits;
  const int G = blockDim.x / HD;
  const int tg = threadIdx.x / HD, d = threadIdx.x - tg * HD;
  // the thread's first eight partial outputs are requested together with the statistics: they do
  // not depend on them, and a trip to memory that waits for another is most of this kernel's time
  float ov[8];
#pragma unroll
  for (int u = 0; u < 8; ++u) {
    const int sp = tg + u * G;
    ov[u] = sp < p.n_splits ? p.part_o[((base + sp) * gh + g) * HD + d] : 0.0f;
  }
  for (int sp = threadIdx.x; sp < p.n_splits; sp += blockDim.x) {
    const float2 ml = *reinterpret_cast<const float2*>(&p.part_ml[((base + sp) * gh + g) * 2]);
    ms[sp] = ml.x;
    ls[sp] = ml.y;
  }
  __syncthreads();
  float M = -INFINITY;
  for (int sp = 0; sp < p.n_splits; ++sp) M = fmaxf(M, ms[sp]);
  float L = 0.0f, O = 0.0f;
  for (int sp0 = tg; sp0 < p.n_splits; sp0 += 8 * G) {
    if (sp0 != tg) {
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int sp = sp0 + u * G;
        ov[u] = sp < p.n_splits ? p.part_o[((base + sp) * gh + g) * HD + d] : 0.0f;
      }
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int sp = sp0 + u * G;
      if (sp >= p.n_splits) continue;
      const float mv = ms[sp];
      const float wgt = mv == -INFINITY ? 0.0f : __expf(mv - M);
      L = fmaf(ls[sp], wgt, L);
      O = fmaf(ov[u], wgt, O);
    }
  }
  if (G > 1) {
    o_s[threadIdx.x] = O;
    if (d == 0) l_s[tg] = L;
    __syncthreads();
    if (tg > 0) return;
    for (int w = 1; w < G; ++w) {
      O += o_s[w * HD + d];
      L += l_s[w];
    }
  }
  ((bf16_t*)p.out)[(int64_t)(q_begin + tok0) * p.out_stride + (kvh * group + hg) * HD + d] = __float2bfloat16(O / L);
}

#if CW_HD % 32 == 0
#define CW_HAS_DECODE 1
#else
#define CW_HAS_DECODE 0
#endif

// 1 when this head size has the bfloat16 decode kernel (multiples of 32).
CW_EXPORT int cw_attention_decode_supported() { return CW_HAS_DECODE; }

// The most splits cw_attention_decode_bf16 takes.
CW_EXPORT int cw_attention_decode_max_splits() { return DEC_MAX_SPLITS; }

// Heads of a group one workgroup of the decode kernel takes, for a group of this size.
CW_EXPORT int cw_attention_decode_gh(int group) { return group < 16 ? group : 16; }

CW_EXPORT int64_t cw_attention_decode_workspace_floats(int n_items, int nh, int nkv, int n_splits) {
  if (n_splits <= 1) return 0;
  const int group = nh / nkv;
  const int gh = cw_attention_decode_gh(group);
  const int n_chunks = (group + gh - 1) / gh;
  return (int64_t)n_items * nkv * n_chunks * n_splits * gh * (CW_HD + 2);
}

#if CW_HAS_DECODE
template <bool POW2>
static int launch_decode(AttnParams& p, int n_items, hipStream_t stream) {
  constexpr int HD = CW_HD;
  // keys of a split: at most ceil(tiles / splits) tiles of 32; their pages go to LDS
  const int64_t max_tiles = ((int64_t)p.table_stride * p.block_size + 31) / 32;
  const int64_t tiles_per_split = p.split_keys > 0 ? p.split_keys / 32 : (max_tiles + p.n_splits - 1) / p.n_splits;
  const int64_t pages = (tiles_per_split * 32 + p.block_size - 1) / p.block_size + 2;
  const size_t smem = sizeof(float) * DEC_WAVES * 16 * HD + sizeof(int) * (size_t)pages;
  if (smem > 160 * 1024) return CW_ERR_SIZE;
  static size_t raised = 0;
  if (smem > raised) {
    if (hipFuncSetAttribute((const void*)attn_decode_bf16_kernel<HD, POW2>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
      return CW_ERR_LAUNCH;
    raised = smem;
  }
  dim3 grid(n_items, p.nkv * p.n_chunks, p.n_splits), block(256);
  hipLaunchKernelGGL((attn_decode_bf16_kernel<HD, POW2>), grid, block, smem, stream, p);
  if (p.n_splits > 1) {
    dim3 mgrid(n_items, p.nkv * p.n_chunks * p.gh);
    // thread groups that share the splits: about eight splits for each, as many as 1024 threads hold
    int groups = p.n_splits / 8;
    if (groups > 1024 / HD) groups = 1024 / HD;
    if (groups < 1) groups = 1;
    hipLaunchKernelGGL((attn_decode_merge_kernel<HD>), mgrid, dim3(groups * HD), 0, stream, p);
  }
  return cw_launch_status();
}
#endif

// Single-token items (every item: one token), bfloat16. Same arguments as cw_attention;
// ``zeros``: at least CW_HD zero elements (16-byte aligned) that masked rows are read from.
// ``identity``: item i is request i and its token is row i (a batch of single tokens only): items
// and cu_q are not read. ``split_keys`` > 0 (a multiple of 32): split s takes keys
// [s * split_keys, (s + 1) * split_keys) instead of a share of each request's own length, and
// ``max_ctx``, the longest context among the requests, must not exceed n_splits * split_keys.
CW_EXPORT int cw_attention_decode_bf16(const void* q, int64_t q_stride, void* out, int64_t out_stride,
                                       const void* k_cache, const void* v_cache, const int* block_tables,
                                       int table_stride, const int* ctx_lens, const int* cu_q,
                                       const int* items, int n_items, int nh, int nkv, int block_size,
                                       int n_splits, int window, float scale, float* workspace,
                                       int64_t workspace_floats, const void* zeros, int identity,
                                       int split_keys, int max_ctx, hipStream_t stream) {
#if CW_HAS_DECODE
  if (n_items < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || block_size <= 0 || table_stride <= 0)
    return CW_ERR_ARG;
  if (n_splits < 1 || n_splits > DEC_MAX_SPLITS || window < 0) return CW_ERR_ARG;
  if (((uintptr_t)q & 15) || ((uintptr_t)k_cache & 15) || ((uintptr_t)v_cache & 15) || (q_stride & 7))
    return CW_ERR_ARG;
  if (zeros == nullptr || ((uintptr_t)zeros & 15)) return CW_ERR_ARG;
  // fixed key ranges must cover the longest context the caller will run
  if (split_keys < 0 || (split_keys & 31) || max_ctx < 0) return CW_ERR_ARG;
  if (split_keys > 0 && (int64_t)split_keys * n_splits < max_ctx) return CW_ERR_ARG;
  if (n_items == 0) return CW_OK;
  const int group = nh / nkv;
  AttnParams p{};
  p.q = q; p.q_stride = q_stride; p.out = out; p.out_stride = out_stride;
  p.k_cache = k_cache; p.v_cache = v_cache; p.block_tables = block_tables;
  p.table_stride = table_stride; p.ctx_lens = ctx_lens; p.cu_q = cu_q; p.items = items;
  p.nh = nh; p.nkv = nkv; p.block_size = block_size; p.bs_shift = cw_log2_or_minus1(block_size);
  p.identity = identity ? 1 : 0; p.split_keys = split_keys;
  p.gh = cw_attention_decode_gh(group);
  p.n_chunks = (group + p.gh - 1) / p.gh; p.n_splits = n_splits; p.window = window; p.scale = scale;
  if ((int64_t)nkv * p.n_chunks * p.gh > 65535) return CW_ERR_SIZE;
  const int64_t need = cw_attention_decode_workspace_floats(n_items, nh, nkv, n_splits);
  if (need > 0 && (workspace == nullptr || workspace_floats < need)) return CW_ERR_ARG;
  if ((uintptr_t)workspace & 7) return CW_ERR_ARG;
  p.part_o = workspace;
  p.part_ml = workspace ? workspace + need / (CW_HD + 2) * CW_HD : nullptr;
  p.zeros = zeros;
  return p.bs_shift >= 0 ? launch_decode<true>(p, n_items, stream) : launch_decode<false>(p, n_items, stream);
#else
  return CW_ERR_ARG;
#endif
}

// =====================================================================================
// bfloat16 attention for portions of prompts on the matrix cores.
//
// A workgroup takes a run of query tokens of one request and one key/value head. Four waves own
// 32 query rows each (row = token * gh + head of the group, so the group shares every key and
// value); for head sizes up to 128 a second set of four waves owns the same rows and the two sets
// split every stage's keys, so each SIMD holds two waves that hide each other's waits, and the
// sets' running states are merged through LDS at the end. All waves walk the same stages of keys,
// which are fetched once per workgroup into LDS, double buffered: the loads of stage t + 1 are in
// flight while stage t is computed.
//   S^T[key, row] = K * Q^T     v_mfma_f32_16x16x32_bf16; K fragments come from LDS in operand
//                               layout (lane = key l%16, 8 consecutive head elements at slot l/16),
//                               Q fragments are loaded once from global memory the same way;
//   softmax per row in float32: a lane holds 8 keys of one row; the running maximum is shared by
//                               the row's 4 lanes every tile, the running sum only at the end;
//                               tiles that no row masks skip the position tests;
//   O^T[d, row] += V^T * P^T    P^T is already in operand layout (the lane's 8 keys of its row).
//                               V^T fragments come from the row-major V tile through the LDS
//                               transposing read (ds_read_b64_tr_b16): in a group of 16 lanes, lane
//                               i receives element i%4 of what lanes i/4, 4 + i/4, 8 + i/4 and
//                               12 + i/4 addressed, so four lanes that point at one key's 16 head
//                               elements hand every lane its column of 4 keys.
// The element order inside an MFMA's k dimension is free as long as both operands agree; that
// is what lets every fragment be filled by plain 8- and 16-byte reads.
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;
typedef __attribute__((address_space(3))) s16x4_t lds_s16x4_t;

typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;

// RB: row blocks (waves that own 32 query rows each) of a workgroup, 4 or 2. With 2 the same eight
// waves cut a stage's keys four ways instead of two: half the rows per workgroup and half the
// time per stage, for launches whose portions would otherwise leave compute units without work
// and wait for the workgroups with the longest key ranges.
template <int HD, int RB>
struct PrefillTile {
  static_assert(RB == 4 || (RB == 2 && HD <= 128), "two row blocks only with the eight-wave workgroup");
  // The K tile lies in LDS as HD / 32 blocks of [key][32 elements]: the 64 lanes of a fragment
  // read (16 keys x 4 slots of 8 elements) and of a stash store (16 keys x 4 chunks) then touch
  // 1 KB without a gap, so no bank is hit twice and the rows need no padding.
  static constexpr int VROW = HD + 16;  // V rows: 32 bytes of padding, for the 8-byte transposing reads
  static constexpr int NH = HD <= 128 ? 8 / RB : 1;  // waves that share a row block and split its keys
  static constexpr int KW = HD <= 128 ? 128 / NH : 32;  // keys a wave takes from a stage
  static constexpr int KT = KW * NH;            // keys of one stage
  static constexpr int NT = 64 * RB * NH;       // threads of a workgroup
  static constexpr int STAGE = KT * (HD + VROW);  // elements of one stage: a K tile, then a V tile
  static constexpr size_t BYTES = 2 * STAGE * sizeof(bf16_t);
  static constexpr int TABLE = 2048;  // block-table entries held in LDS at a time
  // what the sets of waves exchange at the end: accumulators, then maxima and sums
  static constexpr size_t XO_BYTES = (size_t)(NH - 1) * RB * 2 * (HD / 16) * 64 * 16;
  static constexpr size_t XCHG_BYTES = XO_BYTES + (size_t)(NH - 1) * RB * 2 * 2 * 64 * 4;
  static_assert(XCHG_BYTES <= BYTES, "the exchange reuses the tiles' memory");
};

template <int HD, bool POW2, int RB>
__global__ __launch_bounds__((PrefillTile<HD, RB>::NT), (HD <= 128 ? 2 : 1)) void attn_prefill_bf16_kernel(AttnParams p) {
  using Tile = PrefillTile<HD, RB>;
  constexpr int NF = HD / 32;     // k-steps of the score product
  constexpr int ND = HD / 16;     // 16-wide blocks of the head dimension
  constexpr int VROW = Tile::VROW;
  constexpr int CPR = HD / 8;     // 16-byte chunks of a row
  constexpr int NH = Tile::NH, KW = Tile::KW, KT = Tile::KT, NT = Tile::NT;
  constexpr int NKB = KW / 16;  // 16-key blocks of a wave's keys
  extern __shared__ __align__(16) unsigned char smem_raw[];
  bf16_t* tiles = reinterpret_cast<bf16_t*>(smem_raw);  // [stage 2][K tile, V tile]
  int* tbl = reinterpret_cast<int*>(smem_raw + Tile::BYTES);

  const int lane = threadIdx.x & 63;
  const int wave = (threadIdx.x >> 6) % RB;  // the wave's row block
  const int half = threadIdx.x / (64 * RB);  // its share of a stage's keys
  const int c = lane & 15, s = lane >> 4;
  const int item = blockIdx.x;
  const int kvh = blockIdx.y / p.n_chunks, chunk = blockIdx.y % p.n_chunks;
  const int req = p.items[4 * item], tok0 = p.items[4 * item + 1];
  const int gh = p.gh;
  const int tpw = 32 / gh;  // tokens of a wave
  const int ctx = p.ctx_lens[req];
  const int q_begin = p.cu_q[req];
  const int qlen = p.cu_q[req + 1] - q_begin;
  // an item may reach past the request's tokens (work items laid out for a longer portion than
  // the step brings): what lies past them is not computed
  const int ntok = min(p.items[4 * item + 2], qlen - tok0);
  if (ntok <= 0) return;
  const int group = p.nh / p.nkv;
  const int pos0 = ctx - qlen + tok0;
  const int wg_last = pos0 + ntok - 1;
  const int wg_lo = p.window > 0 ? max(0, pos0 - p.window + 1) : 0;
  const int bs = p.block_size, sh = p.bs_shift;
  // the stages of keys this workgroup walks: all that its rows see, or one of ``parts`` runs of
  // them when the item's key range is shared among workgroups (the merge kernel puts the parts'
  // results together); a part may be empty
  int t_first = wg_lo / KT, t_last = wg_last / KT;
  const int packed = p.items[4 * item + 3];
  const int parts = p.part_o != nullptr ? max(1, (packed >> 8) & 0xff) : 1;  // no workspace: every part is the whole
  const int part = packed & 0xff;
  if (parts > 1) {
    const int per = (t_last - t_first + parts) / parts;
    t_first += part * per;
    t_last = min(t_last, t_first + per - 1);
  }
  // the pages of the keys this workgroup reads -> LDS, a window of Tile::TABLE entries at a time
  // (32k keys with pages of 16): no tile waits for a table entry from memory
  const int* table = p.block_tables + (int64_t)req * p.table_stride;
  const int page_last = cw_page_index<POW2>(wg_last, bs, sh);
  int page0 = cw_page_index<POW2>(min(max(t_first * KT, wg_lo), wg_last), bs, sh);  // the page of tbl[0]
  auto load_table = [&]() __attribute__((always_inline)) {
    const int n_pages = min(page_last - page0 + 1, Tile::TABLE);
    for (int i = threadIdx.x; i < n_pages; i += NT) tbl[i] = table[page0 + i];
  };
  load_table();
  __syncthreads();
  const bf16_t* kc = (const bf16_t*)p.k_cache;
  const bf16_t* vc = (const bf16_t*)p.v_cache;
  const bf16_t* zrow = (const bf16_t*)p.zeros;

  // ---- the wave's rows: block b, column c -> row b * 16 + c
  const bool wave_on = wave * tpw < ntok;
  const int p_first = pos0 + wave * tpw;
  const int p_last = pos0 + min(ntok, (wave + 1) * tpw) - 1;
  const int lo = p.window > 0 ? max(0, p_first - p.window + 1) : 0;
  int row_pos[2];      // position of the row's token, -1 for an unused row
  int64_t row_off[2];  // offset of the row's head in q / out, in elements
  bf16x8_t qf[2][NF];
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int row = b * 16 + c;
    const int tl = row / gh, g = row - tl * gh;
    const int tokw = wave * tpw + tl;
    const int hig = chunk * gh + g;
    const bool ok = wave_on && tl < tpw && tokw < ntok && hig < group;
    row_pos[b] = ok ? pos0 + tokw : -1;
    row_off[b] = ok ? (int64_t)(kvh * group + hig) * HD : 0;
    const bf16_t* qrow = ok ? (const bf16_t*)p.q + (int64_t)(q_begin + tok0 + tokw) * p.q_stride + row_off[b] : zrow;
#pragma unroll
    for (int j = 0; j < NF; ++j) qf[b][j] = *reinterpret_cast<const bf16x8_t*>(qrow + (j * 4 + s) * 8);
  }

  f32x4_t o[2][ND];
#pragma unroll
  for (int b = 0; b < 2; ++b)
#pragma unroll
    for (int db = 0; db < ND; ++db) o[b][db] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};
  // running maximum in units of the raw score (the scale is positive) and the lane's share of the sum
  float m_run[2] = {-INFINITY, -INFINITY}, l_run[2] = {0.0f, 0.0f};
  const float sl2 = p.scale * 1.4426950408889634f;  // exp(x * scale) = exp2(x * sl2)
  const float rescale_step = 8.0f / sl2;            // 8 in the exponent, in units of the raw score

  // ---- tile traffic: TPK threads share a key of the stage; thread j of them takes the 16-byte
  // chunks j, j + TPK, ... of its K row and of its V row, so a thread looks up one page and
  // builds one address per stage, and neighbouring lanes read neighbouring chunks (lanes spread
  // over 16 different rows, which would suit the LDS banks better, cost more in memory coalescing
  // than they saved: measured)
  constexpr int TPK = NT / KT;                  // threads per key
  constexpr int NCK = (CPR + TPK - 1) / TPK;    // chunks per thread and matrix
  const int f_key = threadIdx.x / TPK, f_ch = threadIdx.x % TPK;
  const int64_t row_elems = (int64_t)p.nkv * HD;
  // Two row blocks: the workgroups are short of work per stage, so a stage's loads get two stages
  // to arrive (a second register set); with four row blocks the registers are full and one is enough
  constexpr bool DEEP = RB == 2;
  u32x4_t gk[NCK], gv[NCK], gk1[DEEP ? NCK : 1], gv1[DEEP ? NCK : 1];
  auto fetch = [&](int t, u32x4_t* gk, u32x4_t* gv) __attribute__((always_inline)) {  // global -> registers; a masked key reads a row of zeros
    const int kp = t * KT + f_key;
    bool ok = kp >= wg_lo && kp <= wg_last;
    const int page = tbl[ok ? cw_page_index<POW2>(kp, bs, sh) - page0 : 0];
    ok = ok && page >= 0;
    const int64_t off = ((int64_t)page * bs + cw_page_offset<POW2>(kp, bs, sh)) * row_elems + kvh * HD + f_ch * 8;
    const bf16_t* kr = ok ? kc + off : zrow;
    const bf16_t* vr = ok ? vc + off : zrow;
    const int step = ok ? TPK * 8 : 0;  // the row of zeros is short: every chunk reads its start
#pragma unroll
    for (int i = 0; i < NCK; ++i) {
      const bool in_row = CPR % TPK == 0 || f_ch + i * TPK < CPR;
      gk[i] = *reinterpret_cast<const u32x4_t*>(kr + (in_row ? i * step : 0));
      gv[i] = *reinterpret_cast<const u32x4_t*>(vr + (in_row ? i * step : 0));
    }
  };
  auto stash = [&](int stage, const u32x4_t* gk, const u32x4_t* gv) __attribute__((always_inline)) {  // registers -> LDS
    bf16_t* ks = tiles + stage * Tile::STAGE + f_key * 32;
    bf16_t* vs = tiles + stage * Tile::STAGE + KT * HD + f_key * VROW + f_ch * 8;
#pragma unroll
    for (int i = 0; i < NCK; ++i) {
      if (CPR % TPK == 0 || f_ch + i * TPK < CPR) {
        const int ch = f_ch + i * TPK;  // 16-byte chunk of the row: block ch / 4, place ch % 4
        *reinterpret_cast<u32x4_t*>(ks + (ch >> 2) * (KT * 32) + (ch & 3) * 8) = gk[i];
        *reinterpret_cast<u32x4_t*>(vs + i * TPK * 8) = gv[i];
      }
    }
  };
  // the pages of stage tn must lie in the table window before it is fetched; every wave comes
  // here between the same two barriers and nobody reads the window meanwhile
  auto window_for = [&](int tn) __attribute__((always_inline)) {
    const int need = cw_page_index<POW2>(min(tn * KT + KT - 1, wg_last), bs, sh);
    if (need >= page0 + Tile::TABLE) {
      page0 = cw_page_index<POW2>(max(tn * KT, wg_lo), bs, sh);
      load_table();
      __syncthreads();
    }
  };
  auto compute = [&](int t, int stage) __attribute__((always_inline)) {
    const int kv0 = t * KT + half * KW;  // the wave's keys of this stage
    const bool active = wave_on && kv0 <= p_last && kv0 + KW - 1 >= lo;
    if (active) {
      const bf16_t* ks = tiles + stage * Tile::STAGE + half * KW * 32;
      const bf16_t* vs = tiles + stage * Tile::STAGE + KT * HD + half * KW * VROW;
      // ---- S^T = K Q^T
      f32x4_t sc[NKB][2];
#pragma unroll
      for (int kb = 0; kb < NKB; ++kb) {
        bf16x8_t kf[NF];
#pragma unroll
        for (int j = 0; j < NF; ++j)
          kf[j] = *reinterpret_cast<const bf16x8_t*>(ks + j * (KT * 32) + (kb * 16 + c) * 32 + s * 8);
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          sc[kb][b] = (f32x4_t){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
          for (int j = 0; j < NF; ++j)
            sc[kb][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[j], qf[b][j], sc[kb][b], 0, 0, 0);
        }
      }
      // ---- softmax per row; P^T packed as the B operand of the output product.
      // A tile needs the position tests only if some row of the wave masks some key of it.
      const bool masked = kv0 + KW - 1 > p_first || kv0 < wg_lo || (p.window > 0 && kv0 < p_last - p.window + 1);
      if (masked) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const int rp = row_pos[b];
          const int rlo = p.window > 0 ? rp - p.window + 1 : 0;
#pragma unroll
          for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int kp = kv0 + kb * 16 + 4 * s + i;
              if (!(kp <= rp && kp >= rlo)) sc[kb][b][i] = -INFINITY;
            }
        }
      }
      float tmax[2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        tmax[b] = fmaxf(fmaxf(sc[0][b][0], sc[0][b][1]), fmaxf(sc[0][b][2], sc[0][b][3]));
#pragma unroll
        for (int kb = 1; kb < NKB; ++kb)
          tmax[b] = fmaxf(tmax[b], fmaxf(fmaxf(sc[kb][b][0], sc[kb][b][1]), fmaxf(sc[kb][b][2], sc[kb][b][3])));
      }
#pragma unroll
      for (int b = 0; b < 2; ++b) tmax[b] = cw_quad_max(tmax[b]);
      bf16x8_t pf[2][NKB / 2];
      float alpha[2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        // The reference point of the exponentials moves only when the maximum has grown by more
        // than 2^8 in the exponent (or is the row's first): probabilities then reach 256 at most,
        // which float32 sums and bfloat16 products take without loss, and the accumulators are
        // rescaled a few times per row instead of in most tiles. The result is the same quotient.
        const float m_new = tmax[b] > m_run[b] + rescale_step ? tmax[b] : m_run[b];
        // a row that has seen no key yet keeps m = -inf; its probabilities are zero
        const float msc = m_new == -INFINITY ? 0.0f : m_new * sl2;
        const float a = __builtin_amdgcn_exp2f(m_run[b] * sl2 - msc);
        float psum = 0.0f;
#pragma unroll
        for (int kb = 0; kb < NKB; ++kb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float pe = __builtin_amdgcn_exp2f(fmaf(sc[kb][b][i], sl2, -msc));
            psum += pe;
            pf[b][kb / 2][(kb & 1) * 4 + i] = (__bf16)pe;
          }
        l_run[b] = l_run[b] * a + psum;
        m_run[b] = m_new;
        alpha[b] = a;
      }
      if (__any(alpha[0] != 1.0f || alpha[1] != 1.0f)) {
#pragma unroll
        for (int b = 0; b < 2; ++b)
#pragma unroll
          for (int db = 0; db < ND; ++db) o[b][db] *= alpha[b];
      }
      // ---- O^T += V^T P^T, one 16-wide block of the head dimension at a time
      const bf16_t* vlane = vs + (4 * s + (c >> 2)) * VROW + 4 * (c & 3);
#pragma unroll
      for (int k2 = 0; k2 < NKB / 2; ++k2)
#pragma unroll
        for (int db = 0; db < ND; ++db) {
          const bf16_t* vp = vlane + k2 * 32 * VROW + db * 16;
          const s16x4_t v0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)vp);
          const s16x4_t v1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_t*)(vp + 16 * VROW));
          const bf16x8_t vt = __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
          for (int b = 0; b < 2; ++b) o[b][db] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vt, pf[b][k2], o[b][db], 0, 0, 0);
        }
    }
  };

  fetch(t_first, gk, gv);
  stash(0, gk, gv);
  // Every load so far (the query fragments among them) has to be home before the loop starts:
  // the loop's first use of a fragment would otherwise carry a wait for "all loads but the last
  // few", and in every later round that wait would sit on the stage just requested, in order.
  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0)
  if constexpr (DEEP) {
    // set 0 holds stage t + 1 while an even round computes stage t, set 1 stage t + 2; each set is
    // stashed at the end of the round before its stage is computed and filled again at once
    if (t_first + 1 <= t_last) fetch(t_first + 1, gk, gv);
    if (t_first + 2 <= t_last) fetch(t_first + 2, gk1, gv1);
    __syncthreads();
    // The two waves of a SIMD (sets h and h + NH / 2) would walk through a round in step, both in
    // the score product, then both in the softmax, each waiting for the unit the other holds. The
    // later sets move their tile traffic to the start of the round (the buffer it writes was last
    // read before the barrier), so their phases fall beside other ones of the earlier sets:
    // 2048 tokens of 12 heads on 2 key/value heads 44.5 -> 42.6 us.
    const bool late = half >= NH / 2;
    for (int t = t_first; t <= t_last; t += 2) {
      if (!late) compute(t, 0);
      if (t + 1 <= t_last) stash(1, gk, gv);
      if (t + 3 <= t_last) {
        window_for(t + 3);
        fetch(t + 3, gk, gv);
      }
      if (late) compute(t, 0);
      __syncthreads();
      if (t + 1 > t_last) break;
      if (!late) compute(t + 1, 1);
      if (t + 2 <= t_last) stash(0, gk1, gv1);
      if (t + 4 <= t_last) {
        window_for(t + 4);
        fetch(t + 4, gk1, gv1);
      }
      if (late) compute(t + 1, 1);
      __syncthreads();
    }
  } else {
    __syncthreads();
    for (int t = t_first; t <= t_last; ++t) {
      const int stage = (t - t_first) & 1;
      if (t < t_last) {
        window_for(t + 1);
        fetch(t + 1, gk, gv);  // in flight while this tile is computed
      }
      compute(t, stage);
      if (t < t_last) stash(stage ^ 1, gk, gv);  // tile t + 1, read in the next round; nobody reads that buffer now
      __syncthreads();
    }
  }

  // ---- the other sets of waves hand their rows' state to the first set through LDS (the tiles
  // are dead after the loop's last barrier): o, then m and l, lanes side by side; the first set
  // merges them in a fixed order
  if constexpr (NH > 1) {
    constexpr int SET = RB * 2 * ND * 64;  // accumulator vectors of one set
    f32x4_t* xo = reinterpret_cast<f32x4_t*>(smem_raw);
    float* xml = reinterpret_cast<float*>(smem_raw + Tile::XO_BYTES);
    if (half > 0) {
#pragma unroll
      for (int b = 0; b < 2; ++b) {
#pragma unroll
        for (int db = 0; db < ND; ++db) xo[(half - 1) * SET + ((wave * 2 + b) * ND + db) * 64 + lane] = o[b][db];
        xml[(((half - 1) * RB + wave) * 2 + b) * 128 + lane] = m_run[b];
        xml[(((half - 1) * RB + wave) * 2 + b) * 128 + 64 + lane] = l_run[b];
      }
    }
    __syncthreads();
    if (half > 0) return;
#pragma unroll 1
    for (int h = 0; h < NH - 1; ++h) {
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const float m1 = xml[((h * RB + wave) * 2 + b) * 128 + lane];
        const float l1 = xml[((h * RB + wave) * 2 + b) * 128 + 64 + lane];
        const float m = fmaxf(m_run[b], m1);
        const float msc = m == -INFINITY ? 0.0f : m * sl2;
        const float a0 = __builtin_amdgcn_exp2f(m_run[b] * sl2 - msc);
        const float a1 = __builtin_amdgcn_exp2f(m1 * sl2 - msc);
        l_run[b] = l_run[b] * a0 + l1 * a1;
        m_run[b] = m;
#pragma unroll
        for (int db = 0; db < ND; ++db) {
          const f32x4_t o1 = xo[h * SET + ((wave * 2 + b) * ND + db) * 64 + lane];
          o[b][db] = o[b][db] * a0 + o1 * a1;
        }
      }
    }
  }

  // ---- a part of the key range: unnormalised sums, maximum and sum of every row of the workgroup
  // (unused rows too: zeros) for the merge kernel
  if (parts > 1) {
    const int64_t slot = ((int64_t)item * gridDim.y + blockIdx.y) * (RB * 32);
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const float l = cw_quad_sum(l_run[b]);
      const int64_t row = slot + wave * 32 + b * 16 + c;
#pragma unroll
      for (int db = 0; db < ND; ++db) *reinterpret_cast<f32x4_t*>(p.part_o + row * HD + db * 16 + 4 * s) = o[b][db];
      if (s == 0) {
        p.part_ml[row * 2] = m_run[b];
        p.part_ml[row * 2 + 1] = l;
      }
    }
    return;
  }

  // ---- out[row][d]: lane (c, s) holds d = db * 16 + 4s .. + 3 of row (b, c)
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    float l = l_run[b];
    l = cw_quad_sum(l);
    if (row_pos[b] < 0) continue;
    const float inv = 1.0f / l;
    bf16_t* orow = (bf16_t*)p.out + (int64_t)(q_begin + (row_pos[b] - (ctx - qlen))) * p.out_stride + row_off[b];
#pragma unroll
    for (int db = 0; db < ND; ++db) {
      uint2 packed;
      packed.x = (uint32_t)cw_float_to_bf16_bits(o[b][db][0] * inv) | ((uint32_t)cw_float_to_bf16_bits(o[b][db][1] * inv) << 16);
      packed.y = (uint32_t)cw_float_to_bf16_bits(o[b][db][2] * inv) | ((uint32_t)cw_float_to_bf16_bits(o[b][db][3] * inv) << 16);
      *reinterpret_cast<uint2*>(orow + db * 16 + 4 * s) = packed;
    }
  }
}

// Puts together the parts of items whose key range was shared among workgroups. One workgroup per
// (item, key/value head) as in the kernel above; the workgroups of an item's parts share its rows
// (part z takes rows z * ceil(rows / parts) ...), each reading those rows of every part. With few
// rows a workgroup its threads also share the parts: thread (row, 4 elements, slice) sums the parts
// slice, slice + S, ..., and the slices meet in LDS in a fixed order.
#define PREFILL_MAX_PARTS 255

template <int HD, int RB>
__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(AttnParams p) {
  constexpr int ROWS = RB * 32;
  constexpr int VEC = HD / 4;  // 16-byte pieces of a row
  __shared__ float ms[ROWS + PREFILL_MAX_PARTS + 1], ls[ROWS + PREFILL_MAX_PARTS + 1];
  __shared__ __align__(16) float red[256 * 4];
  const int packed = p.items[4 * blockIdx.x + 3];
  const int parts = (packed >> 8) & 0xff, part = packed & 0xff;
  if (parts <= 1) return;
  const int item = blockIdx.x - part;  // the item's part 0
  const int kvh = blockIdx.y / p.n_chunks, chunk = blockIdx.y % p.n_chunks;
  const int req = p.items[4 * item], tok0 = p.items[4 * item + 1];
  const int gh = p.gh, tpw = 32 / gh, group = p.nh / p.nkv;
  const int q_begin = p.cu_q[req];
  const int ntok = min(p.items[4 * item + 2], p.cu_q[req + 1] - q_begin - tok0);
  const float sl2 = p.scale * 1.4426950408889634f;
  const int rpb = (ROWS + parts - 1) / parts;  // rows of this workgroup
  const int row0 = part * rpb;
  if (row0 >= ROWS) return;
  auto slot = [&](int z, int row) { return ((int64_t)(item + z) * gridDim.y + blockIdx.y) * ROWS + row; };
  for (int i = threadIdx.x; i < rpb * parts; i += 256) {
    const int r = i / parts, z = i - r * parts;
    const bool in = row0 + r < ROWS;
    ms[i] = in ? p.part_ml[slot(z, row0 + r) * 2] : -INFINITY;
    ls[i] = in ? p.part_ml[slot(z, row0 + r) * 2 + 1] : 0.0f;
  }
  __syncthreads();
  const int n_pairs = rpb * VEC;                      // (row, 4 elements) pairs of this workgroup
  const int slices = n_pairs >= 256 ? 1 : 256 / n_pairs;
  for (int u0 = 0; u0 < n_pairs * slices; u0 += 256) {  // one round when the parts are shared
    const int u = u0 + threadIdx.x;
    const bool has = u < n_pairs * slices;
    const int pair = has ? u % n_pairs : 0, slice = has ? u / n_pairs : 0;
    const int r = pair / VEC, d = (pair - r * VEC) * 4;
    const int row = row0 + r;
    const int wave = row >> 5, rr = row & 31;
    const int tl = rr / gh, g = rr - tl * gh;
    const int tokw = wave * tpw + tl, hig = chunk * gh + g;
    const bool valid = has && row < ROWS && tl < tpw && tokw < ntok && hig < group;
    float m = -INFINITY, l = 0.0f;
    f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
    if (valid) {
      for (int z = 0; z < parts; ++z) m = fmaxf(m, ms[r * parts + z]);
      for (int z = 0; z < parts; ++z) {
        const float mz = ms[r * parts + z];
        l = fmaf(ls[r * parts + z], mz == -INFINITY ? 0.0f : __builtin_amdgcn_exp2f((mz - m) * sl2), l);
      }
      for (int z = slice; z < parts; z += slices) {
        const float mz = ms[r * parts + z];
        if (mz == -INFINITY) continue;
        acc += *reinterpret_cast<const f32x4_t*>(p.part_o + slot(z, row) * HD + d) * __builtin_amdgcn_exp2f((mz - m) * sl2);
      }
    }
    if (slices > 1) {
      *reinterpret_cast<f32x4_t*>(&red[threadIdx.x * 4]) = acc;
      __syncthreads();
      if (slice == 0)
        for (int sl = 1; sl < slices; ++sl) acc += *reinterpret_cast<const f32x4_t*>(&red[(sl * n_pairs + pair) * 4]);
    }
    if (valid && slice == 0) {
      const float inv = 1.0f / l;
      bf16_t* orow = (bf16_t*)p.out + (int64_t)(q_begin + tok0 + tokw) * p.out_stride + (int64_t)(kvh * group + hig) * HD;
      uint2 two;
      two.x = (uint32_t)cw_float_to_bf16_bits(acc[0] * inv) | ((uint32_t)cw_float_to_bf16_bits(acc[1] * inv) << 16);
      two.y = (uint32_t)cw_float_to_bf16_bits(acc[2] * inv) | ((uint32_t)cw_float_to_bf16_bits(acc[3] * inv) << 16);
      *reinterpret_cast<uint2*>(orow + d) = two;
    }
  }
}

#if CW_HD % 32 == 0
#define CW_HAS_PREFILL 1
#else
#define CW_HAS_PREFILL 0
#endif

// 1 when this head size has the bfloat16 matrix-core kernel for portions (multiples of 32).
CW_EXPORT int cw_attention_prefill_supported() { return CW_HAS_PREFILL; }

#if CW_HAS_PREFILL
template <bool POW2, int RB>
static int launch_prefill(const AttnParams& p, int n_items, int table_stride, hipStream_t stream) {
  using Tile = PrefillTile<CW_HD, RB>;
  dim3 grid(n_items, p.nkv * p.n_chunks), block(Tile::NT);
  // two stages of K and V tiles, then the window of the block table
  const size_t entries = (size_t)table_stride < (size_t)Tile::TABLE ? table_stride : Tile::TABLE;
  if ((Tile::KT + p.block_size - 1) / p.block_size + 1 > Tile::TABLE) return CW_ERR_SIZE;
  const size_t smem = Tile::BYTES + sizeof(int) * entries;
  if (smem > 160 * 1024) return CW_ERR_SIZE;
  static size_t raised = 0;
  if (smem > raised && smem > 48 * 1024) {
    if (hipFuncSetAttribute((const void*)attn_prefill_bf16_kernel<CW_HD, POW2, RB>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem) != hipSuccess)
      return CW_ERR_LAUNCH;
    raised = smem;
  }
  hipLaunchKernelGGL((attn_prefill_bf16_kernel<CW_HD, POW2, RB>), grid, block, smem, stream, p);
  if (p.part_o != nullptr)
    hipLaunchKernelGGL((attn_prefill_merge_kernel<CW_HD, RB>), grid, dim3(256), 0, stream, p);
  return cw_launch_status();
}
#endif

// Floats of workspace cw_attention_prefill_bf16 needs when some items are parts of a key range.
CW_EXPORT int64_t cw_attention_prefill_workspace_floats(int n_items, int nh, int nkv, int row_blocks) {
  if (n_items <= 0 || nh <= 0 || nkv <= 0) return 0;
  const int group = nh / nkv;
  const int gh = group < 32 ? group : 32;
  const int n_chunks = (group + gh - 1) / gh;
  return (int64_t)n_items * nkv * n_chunks * row_blocks * 32 * (CW_HD + 2);
}

// 1 if the kernel for portions can run with this many row blocks a workgroup (4, and 2 for head
// sizes up to 128).
CW_EXPORT int cw_attention_prefill_row_blocks_ok(int row_blocks) {
  return CW_HAS_PREFILL && (row_blocks == 4 || (row_blocks == 2 && CW_HD <= 128)) ? 1 : 0;
}

// Portions of prompts, bfloat16. items: (request, first token, tokens, part | parts << 8) with
// tokens <= row_blocks * (32 / gh), gh = min(group, 32) heads of a group per workgroup; tokens of
// an item beyond that are not computed. row_blocks: 4, or 2 (see PrefillTile). An item with
// parts > 1 stands ``parts`` times in the list, one after the other, as part 0, 1, ...: each takes
// a share of the keys that its tokens see, and a second kernel puts the shares together. Any item
// of that kind (``with_parts``) needs a float32 workspace of
// cw_attention_prefill_workspace_floats(n_items, ...) elements; parts at most 255.
CW_EXPORT int cw_attention_prefill_bf16(const void* q, int64_t q_stride, void* out, int64_t out_stride,
                                        const void* k_cache, const void* v_cache, const int* block_tables,
                                        int table_stride, const int* ctx_lens, const int* cu_q,
                                        const int* items, int n_items, int nh, int nkv, int block_size,
                                        int window, float scale, const void* zeros, int row_blocks,
                                        int with_parts, float* workspace, int64_t workspace_floats,
                                        hipStream_t stream) {
#if CW_HAS_PREFILL
  if (zeros == nullptr || ((uintptr_t)zeros & 15)) return CW_ERR_ARG;
  if (n_items < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || block_size <= 0 || table_stride <= 0 || window < 0)
    return CW_ERR_ARG;
  if (!cw_attention_prefill_row_blocks_ok(row_blocks)) return CW_ERR_ARG;
  if (((uintptr_t)q & 15) || ((uintptr_t)k_cache & 15) || ((uintptr_t)v_cache & 15) || ((uintptr_t)out & 7) ||
      (q_stride & 7) || (out_stride & 3))
    return CW_ERR_ARG;
  if (n_items == 0) return CW_OK;
  const int group = nh / nkv;
  AttnParams p{};
  p.q = q; p.q_stride = q_stride; p.out = out; p.out_stride = out_stride;
  p.k_cache = k_cache; p.v_cache = v_cache; p.block_tables = block_tables;
  p.table_stride = table_stride; p.ctx_lens = ctx_lens; p.cu_q = cu_q; p.items = items;
  p.nh = nh; p.nkv = nkv; p.block_size = block_size; p.bs_shift = cw_log2_or_minus1(block_size); p.gh = group < 32 ? group : 32;
  p.n_chunks = (group + p.gh - 1) / p.gh; p.n_splits = 1; p.window = window; p.scale = scale;
  p.part_o = nullptr; p.part_ml = nullptr; p.zeros = zeros;
  if ((int64_t)nkv * p.n_chunks > 65535) return CW_ERR_SIZE;
  if (with_parts) {
    const int64_t need = cw_attention_prefill_workspace_floats(n_items, nh, nkv, row_blocks);
    if (workspace == nullptr || workspace_floats < need || ((uintptr_t)workspace & 15)) return CW_ERR_ARG;
    p.part_o = workspace;
    p.part_ml = workspace + need / (CW_HD + 2) * CW_HD;
  }
#if CW_HD <= 128
  if (row_blocks == 2)
    return p.bs_shift >= 0 ? launch_prefill<true, 2>(p, n_items, table_stride, stream)
                           : launch_prefill<false, 2>(p, n_items, table_stride, stream);
#endif
  return p.bs_shift >= 0 ? launch_prefill<true, 4>(p, n_items, table_stride, stream)
                         : launch_prefill<false, 4>(p, n_items, table_stride, stream);
#else
  return CW_ERR_ARG;
#endif
}
