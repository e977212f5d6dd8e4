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
// DT is the type of delta: T, or float when delta is a stack of ``parts`` float32 partial sums
// [parts, n_rows_of_resid, H] (a product whose K loop was split over workgroups) that are added in order.
template <typename DT>
__device__ __forceinline__ float delta_at(const DT* dl, int64_t part_stride, int parts, int j) {
  float v = cw_to_float(dl[j]);
  for (int q = 1; q < parts; ++q) v += cw_to_float(dl[q * part_stride + j]);
  return v;
}

template <typename T, typename WT, typename DT>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const T* __restrict__ delta0,
                                   const DT* __restrict__ delta, int parts,
                                   int64_t part_stride, const WT* __restrict__ weight, float eps,
                                   T* __restrict__ out, const int* __restrict__ rows, int H) {
  __shared__ float partial[4];
  const int i = blockIdx.x;
  const int t = rows ? rows[i] : i;
  float* x = resid + (int64_t)t * H;
  const T* d0 = delta0 ? delta0 + (int64_t)t * H : nullptr;
  const DT* dl = delta ? delta + (int64_t)t * H : nullptr;
  T* o = out + (int64_t)i * H;
  const bool write_back = rows == nullptr && (dl != nullptr || d0 != nullptr);

  float ss = 0.0f;
  for (int j = threadIdx.x; j < H; j += 256) {
    float v = x[j];
    if (d0) v += cw_to_float(d0[j]);
    if (dl) v += delta_at(dl, part_stride, parts, j);
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
    if (d0 && !write_back) v += cw_to_float(d0[j]);
    if (dl && !write_back) v += delta_at(dl, part_stride, parts, j);
    const T n = cw_from_float<T>(v * inv);
    o[j] = cw_from_float<T>(cw_to_float(weight[j]) * cw_to_float(n));
  }
}

// The same for rows of up to 4096 elements with H % 4 == 0: every thread keeps its (at most four)
// 4-element chunks of the row in registers, so the row is read once, and all loads are in flight
// together. The order of the sum of squares depends on H alone here too.
template <typename T> struct Chunk4;
template <> struct Chunk4<float> {
  __device__ static void load(const float* p, float* o) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x; o[1] = v.y; o[2] = v.z; o[3] = v.w;
  }
  __device__ static void store(float* p, const float* v) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct Chunk4<bf16_t> {
  __device__ static void load(const bf16_t* p, float* o) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    o[0] = __uint_as_float(v.x << 16); o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16); o[3] = __uint_as_float(v.y & 0xffff0000u);
  }
  __device__ static void store(bf16_t* p, const float* v) {
    uint2 u;
    u.x = (uint32_t)cw_float_to_bf16_bits(v[0]) | ((uint32_t)cw_float_to_bf16_bits(v[1]) << 16);
    u.y = (uint32_t)cw_float_to_bf16_bits(v[2]) | ((uint32_t)cw_float_to_bf16_bits(v[3]) << 16);
    *reinterpret_cast<uint2*>(p) = u;
  }
};

// KC: chunks of 4 elements a thread holds (rows of up to 1024 * KC elements)
template <typename T, typename WT, typename DT, int KC>
__global__ __launch_bounds__(256) void add_rmsnorm_vec_kernel(float* __restrict__ resid, const T* __restrict__ delta0,
                                                              const DT* __restrict__ delta,
                                                              int parts, int64_t part_stride,
                                                              const WT* __restrict__ weight, float eps,
                                                              T* __restrict__ out, const int* __restrict__ rows, int H) {
  __shared__ float partial[4];
  const int i = blockIdx.x;
  const int t = rows ? rows[i] : i;
  float* x = resid + (int64_t)t * H;
  const T* d0 = delta0 ? delta0 + (int64_t)t * H : nullptr;
  const DT* dl = delta ? delta + (int64_t)t * H : nullptr;
  T* o = out + (int64_t)i * H;
  const bool write_back = rows == nullptr && (dl != nullptr || d0 != nullptr);
  const int n_chunks = H / 4;
  float v[KC][4], w[KC][4];
#pragma unroll
  for (int k = 0; k < KC; ++k) {
    const int ch = threadIdx.x + k * 256;
    if (ch < n_chunks) {
      Chunk4<float>::load(x + ch * 4, v[k]);
      Chunk4<WT>::load(weight + ch * 4, w[k]);
    } else {
      v[k][0] = v[k][1] = v[k][2] = v[k][3] = 0.0f;
    }
  }
  if (d0) {  // an earlier branch's output that was not added yet: it comes first, as it would have
#pragma unroll
    for (int k = 0; k < KC; ++k) {
      const int ch = threadIdx.x + k * 256;
      if (ch < n_chunks) {
        float d[4];
        Chunk4<T>::load(d0 + ch * 4, d);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[k][e] += d[e];
      }
    }
  }
  if (dl) {
    // the partial sums are added in order, but fetched PU at a time: every trip to memory that
    // waits for the one before costs about a microsecond, more than the rest of this kernel
    constexpr int PU = KC <= 4 ? 4 : 2;
    float acc[KC][4];
    for (int q0 = 0; q0 < parts; q0 += PU) {
      float d[PU][KC][4];
#pragma unroll
      for (int u = 0; u < PU; ++u)
#pragma unroll
        for (int k = 0; k < KC; ++k) {
          const int ch = threadIdx.x + k * 256;
          if (q0 + u < parts && ch < n_chunks) Chunk4<DT>::load(dl + (q0 + u) * part_stride + ch * 4, d[u][k]);
          else d[u][k][0] = d[u][k][1] = d[u][k][2] = d[u][k][3] = 0.0f;
        }
#pragma unroll
      for (int u = 0; u < PU; ++u) {
        if (q0 + u >= parts) break;
#pragma unroll
        for (int k = 0; k < KC; ++k)
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[k][e] = q0 + u == 0 ? d[u][k][e] : acc[k][e] + d[u][k][e];
      }
    }
#pragma unroll
    for (int k = 0; k < KC; ++k)
#pragma unroll
      for (int e = 0; e < 4; ++e) v[k][e] += acc[k][e];
  }
  float ss = 0.0f;
#pragma unroll
  for (int k = 0; k < KC; ++k) {
    const int ch = threadIdx.x + k * 256;
    if (ch < n_chunks) {
      if (write_back) Chunk4<float>::store(x + ch * 4, v[k]);
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += v[k][e] * v[k][e];
    }
  }
  ss = cw_wave_sum(ss);
  if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float total = (partial[0] + partial[1]) + (partial[2] + partial[3]);
  const float inv = 1.0f / sqrtf(total / (float)H + eps);
#pragma unroll
  for (int k = 0; k < KC; ++k) {
    const int ch = threadIdx.x + k * 256;
    if (ch < n_chunks) {
      float r[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) r[e] = w[k][e] * cw_to_float(cw_from_float<T>(v[k][e] * inv));
      Chunk4<T>::store(o + ch * 4, r);
    }
  }
}

// delta: nullptr, or [T, H] in the activation type (delta_parts == 0), or float32 [delta_parts, T, H].
// delta0: nullptr, or [T, H] in the activation type, added to the residual before delta.
CW_EXPORT int cw_add_rmsnorm(float* resid, const void* delta0, const void* delta, int delta_parts, int T_rows,
                             const void* weight, int w_dtype, float eps, void* out, int dtype,
                             const int* rows, int n, int H, hipStream_t stream) {
  if (n < 0 || H <= 0 || delta_parts < 0 || delta_parts > 64) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  dim3 grid(n), block(256);
  const bool vec = (H % 4 == 0) && H <= 8192 && !((uintptr_t)resid & 15) && !((uintptr_t)out & 15) &&
                   !((uintptr_t)weight & 15) && !((uintptr_t)delta & 15) && !((uintptr_t)delta0 & 15);
  const int parts = delta_parts > 0 ? delta_parts : 1;
  const int64_t part_stride = (int64_t)T_rows * H;
#define CW_LAUNCH(T, WT, DT)                                                                           \
  do {                                                                                                 \
    if (vec && H <= 4096)                                                                              \
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, WT, DT, 4>), grid, block, 0, stream, resid,        \
                         (const T*)delta0, (const DT*)delta, parts, part_stride, (const WT*)weight, eps, \
                         (T*)out, rows, H);                                                            \
    else if (vec)                                                                                      \
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, WT, DT, 8>), grid, block, 0, stream, resid,        \
                         (const T*)delta0, (const DT*)delta, parts, part_stride, (const WT*)weight, eps, \
                         (T*)out, rows, H);                                                            \
    else                                                                                               \
      hipLaunchKernelGGL((add_rmsnorm_kernel<T, WT, DT>), grid, block, 0, stream, resid,               \
                         (const T*)delta0, (const DT*)delta, parts, part_stride, (const WT*)weight, eps, \
                         (T*)out, rows, H);                                                            \
  } while (0)
  if (delta_parts > 0) {
    if (dtype == CW_F32 && w_dtype == CW_F32) CW_LAUNCH(float, float, float);
    else if (dtype == CW_BF16 && w_dtype == CW_BF16) CW_LAUNCH(bf16_t, bf16_t, float);
    else if (dtype == CW_BF16 && w_dtype == CW_F32) CW_LAUNCH(bf16_t, float, float);
    else return CW_ERR_DTYPE;
  } else {
    if (dtype == CW_F32 && w_dtype == CW_F32) CW_LAUNCH(float, float, float);
    else if (dtype == CW_BF16 && w_dtype == CW_BF16) CW_LAUNCH(bf16_t, bf16_t, bf16_t);
    else if (dtype == CW_BF16 && w_dtype == CW_F32) CW_LAUNCH(bf16_t, float, bf16_t);
    else return CW_ERR_DTYPE;
  }
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
  // rotated pairs: thread = (pair i, head stripe); the angle of pair i is computed once per thread
  if (half > 0) {
    const int i = threadIdx.x % half;
    const int stripe = threadIdx.x / half;
    const int n_stripes = blockDim.x / half;
    if (stripe < n_stripes) {
      float sn = 0.0f, cs = 1.0f;
      if (inv_freq) sincosf(pos * inv_freq[i], &sn, &cs);
      for (int head = stripe; head < nh + nkv; head += n_stripes) {
        T* h = row + head * hd;
        float a = cw_to_float(h[i]);
        float b = cw_to_float(h[i + half]);
        if (bias) { a += cw_to_float(bias[head * hd + i]); b += cw_to_float(bias[head * hd + i + half]); }
        const T oa = cw_from_float<T>(a * cs - b * sn), ob = cw_from_float<T>(b * cs + a * sn);
        if (head < nh) { h[i] = oa; h[i + half] = ob; }
        else if (slot >= 0) {
          T* kdst = k_cache + (slot * nkv + (head - nh)) * (int64_t)hd;
          kdst[i] = oa; kdst[i + half] = ob;
        }
      }
    }
  }
  // elements past the rotary dimension pass through (bias added)
  for (int w = threadIdx.x; w < (nh + nkv) * rest; w += blockDim.x) {
    const int head = w / rest, j = rotary_dim + w % rest;
    T* h = row + head * hd;
    float a = cw_to_float(h[j]);
    if (bias) a += cw_to_float(bias[head * hd + j]);
    const T oa = cw_from_float<T>(a);
    if (head < nh) h[j] = oa;
    else if (slot >= 0) k_cache[(slot * nkv + (head - nh)) * (int64_t)hd + j] = oa;
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

// The same for bfloat16 rows whose heads are rotated whole (rotary_dim == hd, hd a multiple of 16):
// the token's hd / 2 angles are computed once, into LDS, and every thread then moves 8 pairs at a
// time with 16-byte loads and stores (the kernel above moves one pair of 2-byte elements a time,
// which is what a 2048-token portion's 17 MB took 7.8 us for).
template <typename BT>
__global__ __launch_bounds__(256) void rope_kv_write_vec_kernel(bf16_t* __restrict__ qkv, const BT* __restrict__ bias,
                                                                const int* __restrict__ positions,
                                                                const int* __restrict__ slots,
                                                                const float* __restrict__ inv_freq, int nh, int nkv, int hd,
                                                                bf16_t* __restrict__ k_cache, bf16_t* __restrict__ v_cache,
                                                                int64_t cache_rows) {
  __shared__ float cs[128], sn[128];
  const int t = blockIdx.x;
  const int width = (nh + 2 * nkv) * hd;
  bf16_t* row = qkv + (int64_t)t * width;
  const float pos = (float)positions[t];
  int64_t slot = slots ? (int64_t)slots[t] : -1;
  if (slot >= cache_rows) slot = -1;
  const int half = hd / 2;
  if ((int)threadIdx.x < half) {
    float s_ = 0.0f, c_ = 1.0f;
    if (inv_freq) sincosf(pos * inv_freq[threadIdx.x], &s_, &c_);
    sn[threadIdx.x] = s_;
    cs[threadIdx.x] = c_;
  }
  __syncthreads();
  auto load8 = [](const bf16_t* p, float* out) __attribute__((always_inline)) {
    const uint4 raw = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      out[2 * e] = cw_bf16_bits_to_float((uint16_t)(w[e] & 0xffffu));
      out[2 * e + 1] = cw_bf16_bits_to_float((uint16_t)(w[e] >> 16));
    }
  };
  auto add_bias8 = [&](int at, float* v) __attribute__((always_inline)) {
    if (!bias) return;
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] += cw_to_float(bias[at + e]);
  };
  auto store8 = [](bf16_t* p, const float* v) __attribute__((always_inline)) {
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bf16_t lo = __float2bfloat16(v[2 * e]), hi = __float2bfloat16(v[2 * e + 1]);
      w[e] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
    }
    *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
  };
  const int chunks = half / 8;  // chunks of 8 pairs per head
  for (int w = threadIdx.x; w < (nh + nkv) * chunks; w += blockDim.x) {
    const int head = w / chunks, i8 = (w - head * chunks) * 8;
    bf16_t* h = row + head * hd;
    float a[8], b[8], oa[8], ob[8];
    load8(h + i8, a);
    load8(h + i8 + half, b);
    add_bias8(head * hd + i8, a);
    add_bias8(head * hd + i8 + half, b);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float c_ = cs[i8 + e], s_ = sn[i8 + e];
      oa[e] = a[e] * c_ - b[e] * s_;
      ob[e] = b[e] * c_ + a[e] * s_;
    }
    if (head < nh) {
      store8(h + i8, oa);
      store8(h + i8 + half, ob);
    } else if (slot >= 0) {
      bf16_t* kdst = k_cache + (slot * nkv + (head - nh)) * (int64_t)hd;
      store8(kdst + i8, oa);
      store8(kdst + i8 + half, ob);
    }
  }
  if (slot >= 0) {
    const bf16_t* v = row + (nh + nkv) * hd;
    bf16_t* vdst = v_cache + slot * nkv * (int64_t)hd;
    for (int w = threadIdx.x * 8; w < nkv * hd; w += blockDim.x * 8) {
      if (bias) {
        float x[8];
        load8(v + w, x);
        add_bias8((nh + nkv) * hd + w, x);
        store8(vdst + w, x);
      } else {
        *reinterpret_cast<uint4*>(vdst + w) = *reinterpret_cast<const uint4*>(v + w);
      }
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
  // whole heads of bfloat16, everything on 16-byte boundaries: 8 pairs a thread
  if (dtype == CW_BF16 && rotary_dim == hd && hd % 16 == 0 && hd <= 256 && !((uintptr_t)qkv & 15) &&
      !((uintptr_t)k_cache & 15) && !((uintptr_t)v_cache & 15)) {
    if (bias == nullptr || bias_dtype == CW_BF16)
      hipLaunchKernelGGL((rope_kv_write_vec_kernel<bf16_t>), grid, block, 0, stream, (bf16_t*)qkv, (const bf16_t*)bias,
                         positions, slots, inv_freq, nh, nkv, hd, (bf16_t*)k_cache, (bf16_t*)v_cache, cache_rows);
    else if (bias_dtype == CW_F32)
      hipLaunchKernelGGL((rope_kv_write_vec_kernel<float>), grid, block, 0, stream, (bf16_t*)qkv, (const float*)bias,
                         positions, slots, inv_freq, nh, nkv, hd, (bf16_t*)k_cache, (bf16_t*)v_cache, cache_rows);
    else
      return CW_ERR_DTYPE;
    return cw_launch_status();
  }
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

// 8 (bfloat16) or 4 (float32) consecutive elements per thread, 16-byte loads and stores.
template <typename T> struct Vec16B;
template <> struct Vec16B<float> {
  static constexpr int N = 4;
  __device__ static void load(const float* p, float* o) { Chunk4<float>::load(p, o); }
  __device__ static void store(float* p, const float* v) { Chunk4<float>::store(p, v); }
};
template <> struct Vec16B<bf16_t> {
  static constexpr int N = 8;
  __device__ static void load(const bf16_t* p, float* o) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) { o[2 * i] = __uint_as_float(w[i] << 16); o[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u); }
  }
  __device__ static void store(bf16_t* p, const float* v) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)cw_float_to_bf16_bits(v[2 * i]) | ((uint32_t)cw_float_to_bf16_bits(v[2 * i + 1]) << 16);
    *reinterpret_cast<uint4*>(p) = make_uint4(w[0], w[1], w[2], w[3]);
  }
};

template <typename T>
__global__ void silu_mul_vec_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int64_t n_vec, int I) {
  constexpr int N = Vec16B<T>::N;
  const int per_row = I / N;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n_vec;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = idx / per_row;
    const int i = (int)(idx - t * per_row) * N;
    float g[N], u[N], r[N];
    Vec16B<T>::load(gate_up + t * 2 * I + i, g);
    Vec16B<T>::load(gate_up + t * 2 * I + I + i, u);
#pragma unroll
    for (int e = 0; e < N; ++e) r[e] = g[e] / (1.0f + expf(-g[e])) * u[e];
    Vec16B<T>::store(out + t * I + i, r);
  }
}

CW_EXPORT int cw_silu_mul(const void* gate_up, void* out, int dtype, int T, int I, hipStream_t stream) {
  if (T < 0 || I <= 0) return CW_ERR_ARG;
  if (T == 0) return CW_OK;
  const int vec_n = dtype == CW_BF16 ? 8 : 4;
  const bool vec = (I % vec_n == 0) && !((uintptr_t)gate_up & 15) && !((uintptr_t)out & 15);
  const int64_t n = vec ? (int64_t)T * (I / vec_n) : (int64_t)T * I;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 262144) blocks = 262144;
  dim3 grid((unsigned)blocks), block(256);
  if (dtype == CW_F32) {
    if (vec) hipLaunchKernelGGL(silu_mul_vec_kernel<float>, grid, block, 0, stream, (const float*)gate_up, (float*)out, n, I);
    else hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (const float*)gate_up, (float*)out, n, I);
  } else if (dtype == CW_BF16) {
    if (vec) hipLaunchKernelGGL(silu_mul_vec_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gate_up, (bf16_t*)out, n, I);
    else hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gate_up, (bf16_t*)out, n, I);
  } else {
    return CW_ERR_DTYPE;
  }
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

// ---------------------------------------------------------------- fresh state slots
// The state pool of a group is [entries, slots, row_bytes]. A request whose first token runs in
// this step (starts[r] == 0) begins from the fresh state: its slot's row is set, in every entry, to
// the row of the pool's template slot, by a kernel (no memset or copy node: the launch is part of
// steps that are captured as graphs). slots[r] < 0 or >= num_slots: the row belongs to no request,
// nothing is written.
__global__ void fresh_state_rows_kernel(uint32_t* __restrict__ pool, int64_t entry_words, int64_t row_words,
                                        int num_slots, int fresh_slot, const int* __restrict__ slots,
                                        const int* __restrict__ starts) {
  const int r = blockIdx.x, entry = blockIdx.y;
  const int slot = slots[r];
  if (starts[r] != 0 || slot < 0 || slot >= num_slots) return;
  uint32_t* row = pool + entry * entry_words + (int64_t)slot * row_words;
  const uint32_t* fresh = pool + entry * entry_words + (int64_t)fresh_slot * row_words;
  for (int64_t i = threadIdx.x; i < row_words; i += blockDim.x) row[i] = fresh[i];
}

// pool [entries, pool_slots, row_bytes]: slots [0, num_slots) may be set, slot ``fresh_slot`` (one of
// the pool's, outside that range) holds what a fresh state is.
CW_EXPORT int cw_fresh_state_rows(void* pool, int entries, int pool_slots, int num_slots, int fresh_slot,
                                  int64_t row_bytes, const int* slots, const int* starts, int n, hipStream_t stream) {
  if (entries <= 0 || num_slots <= 0 || row_bytes <= 0 || (row_bytes & 3) || n < 0 || !pool || !slots || !starts)
    return CW_ERR_ARG;
  if (num_slots > pool_slots || fresh_slot < num_slots || fresh_slot >= pool_slots) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  if (entries > 65535) return CW_ERR_SIZE;
  hipLaunchKernelGGL(fresh_state_rows_kernel, dim3(n, entries), dim3(256), 0, stream, (uint32_t*)pool,
                     (int64_t)pool_slots * (row_bytes / 4), row_bytes / 4, num_slots, fresh_slot, slots, starts);
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
