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
  const int* items;       // [n_items, 4]: request, first token (relative), tokens, unused
  int nh, nkv, block_size;
  int gh;                 // query heads of a group handled by one workgroup
  int n_chunks;           // ceil(group / gh)
  int n_splits;
  int window;             // 0: none
  float scale;
  float* part_o;          // [n_items, nkv * n_chunks, n_splits, ROWS, HD] unnormalised outputs
  float* part_ml;         // [n_items, nkv * n_chunks, n_splits, ROWS, 2] running max, sum
};

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
  const int req = p.items[4 * item], tok0 = p.items[4 * item + 1], ntok = p.items[4 * item + 2];
  const int ctx = p.ctx_lens[req];
  const int q_begin = p.cu_q[req];
  const int qlen = p.cu_q[req + 1] - q_begin;
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
  const int req = p.items[4 * item], tok0 = p.items[4 * item + 1], ntok = p.items[4 * item + 2];
  const int q_begin = p.cu_q[req];
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
  AttnParams p;
  p.q = q; p.q_stride = q_stride; p.out = out; p.out_stride = out_stride;
  p.k_cache = k_cache; p.v_cache = v_cache; p.block_tables = block_tables;
  p.table_stride = table_stride; p.ctx_lens = ctx_lens; p.cu_q = cu_q; p.items = items;
  p.nh = nh; p.nkv = nkv; p.block_size = block_size; p.gh = gh;
  p.n_chunks = (group + gh - 1) / gh; p.n_splits = n_splits; p.window = window; p.scale = scale;
  if ((int64_t)nkv * p.n_chunks > 65535) return CW_ERR_SIZE;
  const int64_t need = cw_attention_workspace_floats(rows, n_items, nkv, p.n_chunks, n_splits);
  if (need > 0 && (workspace == nullptr || workspace_floats < need)) return CW_ERR_ARG;
  const int64_t n_o = need / (CW_HD + 2) * CW_HD;
  p.part_o = workspace;
  p.part_ml = workspace ? workspace + n_o : nullptr;
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
