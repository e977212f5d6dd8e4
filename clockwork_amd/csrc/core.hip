// Row-wise and element-wise kernels of the forward pass for gfx950:
// embedding gather, fused residual-add + RMSNorm, rotary encoding fused with the
// key/value cache write, SiLU-gate multiply, page copies.
// All statistics, angles and the residual stream are float32; T is the activation type.
#include "common.h"

// ---------------------------------------------------------------- embedding
// resid[t, :] = table[ids[t], :] as float32. An id outside [0, V) yields a zero row
// (the host validates ids; this only keeps the kernel inside the table).
template <typename T>
__global__ void embedding_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                 float* __restrict__ resid, int H, int V) {
  const int t = blockIdx.x;
  const int id = ids[t];
  const bool ok = id >= 0 && id < V;
  const T* row = table + (int64_t)(ok ? id : 0) * H;
  float* out = resid + (int64_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = ok ? cw_to_float(row[i]) : 0.0f;
}

CW_EXPORT int cw_embedding(const void* table, int dtype, const int* ids, float* resid, int T,
                           int H, int V, hipStream_t stream) {
  if (T < 0 || H <= 0 || V <= 0) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  dim3 grid(T), block(256);
  if (dtype == CW_F32)
    hipLaunchKernelGGL(embedding_kernel<float>, grid, block, 0, stream, (const float*)table, ids, resid, H, V);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(embedding_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)table, ids, resid, H, V);
  else
    return CW_ERR_DTYPE;
  return cw_launch_status();
}

// ---------------------------------------------------------------- residual add + RMSNorm
// rows == nullptr: for every t < n: resid[t] += delta[t] (if delta), out[t] = norm(resid[t]).
// rows != nullptr: for i < n: x = resid[rows[i]] + delta[rows[i]], out[i] = norm(x); resid untouched.
// norm(x) = weight * cast_T(x * 1/sqrt(mean(x^2) + eps)): the cast to T comes before the weight
// multiply. The sum of squares of a row is reduced in an order that depends on H alone.
template <typename T, typename WT>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const T* __restrict__ delta,
                                   const WT* __restrict__ weight, float eps, T* __restrict__ out,
                                   const int* __restrict__ rows, int H) {
  __shared__ float partial[4];
  const int i = blockIdx.x;
  const int t = rows ? rows[i] : i;
  float* x = resid + (int64_t)t * H;
  const T* dl = delta ? delta + (int64_t)t * H : nullptr;
  T* o = out + (int64_t)i * H;
  const bool write_back = rows == nullptr && dl != nullptr;

  float ss = 0.0f;
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = x[j];
    if (dl) v += cw_to_float(dl[j]);
    if (write_back) x[j] = v;
    ss += v * v;
  }
  ss = cw_wave_sum(ss);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) partial[wave] = ss;
  __syncthreads();
  const float total = (partial[0] + partial[1]) + (partial[2] + partial[3]);
  const float inv = 1.0f / sqrtf(total / (float)H + eps);
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = x[j];
    if (dl && !write_back) v += cw_to_float(dl[j]);
    const T n = cw_from_float<T>(v * inv);
    o[j] = cw_from_float<T>(cw_to_float(weight[j]) * cw_to_float(n));
  }
}

CW_EXPORT int cw_add_rmsnorm(float* resid, const void* delta, const void* weight, int w_dtype,
                             float eps, void* out, int dtype, const int* rows, int n, int H,
                             hipStream_t stream) {
  if (n < 0 || H <= 0) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  dim3 grid(n), block(256);
#define CW_LAUNCH(T, WT)                                                                         \
  hipLaunchKernelGGL((add_rmsnorm_kernel<T, WT>), grid, block, 0, stream, resid, (const T*)delta, \
                     (const WT*)weight, eps, (T*)out, rows, H)
  if (dtype == CW_F32 && w_dtype == CW_F32) CW_LAUNCH(float, float);
  else if (dtype == CW_BF16 && w_dtype == CW_BF16) CW_LAUNCH(bf16_t, bf16_t);
  else if (dtype == CW_BF16 && w_dtype == CW_F32) CW_LAUNCH(bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- rotary + cache write
// qkv: [T, (nh + 2*nkv) * hd], one row per token: q heads, then k heads, then v heads, with an
// optional bias [(nh + 2*nkv) * hd] added first. The first rotary_dim elements of every q and k
// head are rotated in pairs (i, i + rotary_dim/2) by angle pos * inv_freq[i], computed in float32.
// q is rewritten in place; rotated k and plain v go to the flat cache rows
// k_cache/v_cache[slot, nkv, hd]. A negative slot writes no cache row. inv_freq == nullptr: no rotation.
template <typename T, typename BT>
__global__ void rope_kv_write_kernel(T* __restrict__ qkv, const BT* __restrict__ bias,
                                     const int* __restrict__ positions,
                                     const int* __restrict__ slots, const float* __restrict__ inv_freq,
                                     int rotary_dim, int nh, int nkv, int hd, T* __restrict__ k_cache,
                                     T* __restrict__ v_cache, int64_t cache_rows) {
  const int t = blockIdx.x;
  const int width = (nh + 2 * nkv) * hd;
  T* row = qkv + (int64_t)t * width;
  const float pos = (float)positions[t];
  int64_t slot = slots ? (int64_t)slots[t] : -1;
  if (slot >= cache_rows) slot = -1;
  const int half = rotary_dim / 2;
  const int rest = hd - rotary_dim;
  const int per_head = half + rest;  // work items of a q or k head: pairs, then pass-through
  const int n_qk = (nh + nkv) * per_head;
  for (int w = threadIdx.x; w < n_qk; w += blockDim.x) {
    const int head = w / per_head;
    const int i = w % per_head;
    T* h = row + head * hd;
    const BT* hb = bias ? bias + head * hd : nullptr;
    T* kdst = (head >= nh && slot >= 0)
                  ? k_cache + (slot * nkv + (head - nh)) * (int64_t)hd
                  : nullptr;
    if (i < half) {
      float a = cw_to_float(h[i]);
      float b = cw_to_float(h[i + half]);
      if (hb) { a += cw_to_float(hb[i]); b += cw_to_float(hb[i + half]); }
      float ra = a, rb = b;
      if (inv_freq) {
        float s, c;
        sincosf(pos * inv_freq[i], &s, &c);
        ra = a * c - b * s;
        rb = b * c + a * s;
      }
      const T oa = cw_from_float<T>(ra), ob = cw_from_float<T>(rb);
      if (head < nh) { h[i] = oa; h[i + half] = ob; }
      else if (kdst) { kdst[i] = oa; kdst[i + half] = ob; }
    } else {
      const int j = rotary_dim + (i - half);
      float a = cw_to_float(h[j]);
      if (hb) a += cw_to_float(hb[j]);
      const T oa = cw_from_float<T>(a);
      if (head < nh) h[j] = oa;
      else if (kdst) kdst[j] = oa;
    }
  }
  if (slot >= 0) {
    const int n_v = nkv * hd;
    const T* v = row + (nh + nkv) * hd;
    const BT* vb = bias ? bias + (nh + nkv) * hd : nullptr;
    T* vdst = v_cache + slot * nkv * (int64_t)hd;
    for (int w = threadIdx.x; w < n_v; w += blockDim.x) {
      float a = cw_to_float(v[w]);
      if (vb) a += cw_to_float(vb[w]);
      vdst[w] = cw_from_float<T>(a);
    }
  }
}

CW_EXPORT int cw_rope_kv_write(void* qkv, int dtype, const void* bias, int bias_dtype,
                               const int* positions, const int* slots, const float* inv_freq,
                               int rotary_dim, int T, int nh, int nkv, int hd, void* k_cache,
                               void* v_cache, int64_t cache_rows, hipStream_t stream) {
  if (T < 0 || nh <= 0 || nkv < 0 || hd <= 0 || rotary_dim < 0 || rotary_dim > hd || (rotary_dim & 1))
    return CW_ERR_ARG;
  if (slots && (!k_cache || !v_cache) && nkv > 0) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  dim3 grid(T), block(256);
#define CW_LAUNCH(T_, BT_)                                                                       \
  hipLaunchKernelGGL((rope_kv_write_kernel<T_, BT_>), grid, block, 0, stream, (T_*)qkv,          \
                     (const BT_*)bias, positions, slots, inv_freq, rotary_dim, nh, nkv, hd,      \
                     (T_*)k_cache, (T_*)v_cache, cache_rows)
  if (dtype == CW_F32 && (bias == nullptr || bias_dtype == CW_F32)) CW_LAUNCH(float, float);
  else if (dtype == CW_BF16 && (bias == nullptr || bias_dtype == CW_BF16)) CW_LAUNCH(bf16_t, bf16_t);
  else if (dtype == CW_BF16 && bias_dtype == CW_F32) CW_LAUNCH(bf16_t, float);
  else return CW_ERR_DTYPE;
#undef CW_LAUNCH
  return cw_launch_status();
}

// ---------------------------------------------------------------- SiLU(gate) * up
// gate_up: [T, 2*I] (gate columns first), out: [T, I]; silu(z) = z / (1 + exp(-z)) in float32.
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int64_t n, int I) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = idx / I;
    const int i = (int)(idx - t * I);
    const float g = cw_to_float(gate_up[t * 2 * I + i]);
    const float u = cw_to_float(gate_up[t * 2 * I + I + i]);
    out[idx] = cw_from_float<T>(g / (1.0f + expf(-g)) * u);
  }
}

CW_EXPORT int cw_silu_mul(const void* gate_up, void* out, int dtype, int T, int I, hipStream_t stream) {
  if (T < 0 || I <= 0) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  const int64_t n = (int64_t)T * I;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == CW_F32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (const float*)gate_up, (float*)out, n, I);
  else if (dtype == CW_BF16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gate_up, (bf16_t*)out, n, I);
  else
    return CW_ERR_DTYPE;
  return cw_launch_status();
}

// ---------------------------------------------------------------- page copies
// The pool is [planes, num_blocks, block_bytes]; for each pair (src, dst) copy the page in
// every plane (a plane is the keys or the values of one cache entry). block_bytes % 16 == 0.
__global__ void copy_pages_kernel(uint4* __restrict__ pool, int64_t plane_vec, int64_t block_vec,
                                  const int* __restrict__ pairs) {
  const int pair = blockIdx.x;
  const int plane = blockIdx.y;
  const int64_t src = pairs[2 * pair], dst = pairs[2 * pair + 1];
  uint4* base = pool + plane * plane_vec;
  for (int64_t i = threadIdx.x; i < block_vec; i += blockDim.x)
    base[dst * block_vec + i] = base[src * block_vec + i];
}

CW_EXPORT int cw_copy_pages(void* pool, int planes, int64_t num_blocks, int64_t block_bytes,
                            const int* pairs, int n_pairs, hipStream_t stream) {
  if (planes <= 0 || num_blocks <= 0 || block_bytes <= 0 || (block_bytes & 15) || n_pairs < 0)
    return CW_ERR_ARG;
  if (n_pairs == 0) return CW_OK;
  dim3 grid(n_pairs, planes), block(256);
  hipLaunchKernelGGL(copy_pages_kernel, grid, block, 0, stream, (uint4*)pool,
                     num_blocks * (block_bytes / 16), block_bytes / 16, pairs);
  return cw_launch_status();
}

// ---------------------------------------------------------------- casts
// out[i] = float(in[i]) for bfloat16 input (logits of a bfloat16 product to float32).
__global__ void bf16_to_f32_kernel(const bf16_t* __restrict__ in, float* __restrict__ out, int64_t n) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x)
    out[i] = __bfloat162float(in[i]);
}

CW_EXPORT int cw_bf16_to_f32(const void* in, float* out, int64_t n, hipStream_t stream) {
  if (n < 0) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipLaunchKernelGGL(bf16_to_f32_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                     (const bf16_t*)in, out, n);
  return cw_launch_status();
}
