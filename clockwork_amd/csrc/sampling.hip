// Token selection over float32 logits rows for gfx950: arg-max, and temperature / top-k / top-p
// sampling with a counter-based random stream.
//
// Sampling order follows the reference (clockwork/engine/model_runner.py:147-164):
// logits / temperature -> top-k (ties at the k-th value survive) -> top-p (a token stays while
// the probability mass of the tokens strictly more likely than it is <= top_p) -> softmax -> draw.
// The draw is ours: u = Philox4x32-10(key = seed, counter = draw index) mapped to [0, 1), then
// the first index whose running sum of weights, taken in index order, exceeds u * total. A row's
// result depends on that row, its seed and its draw index only.
#include "common.h"

#define SAMPLE_THREADS 1024
#define SAMPLE_WAVES (SAMPLE_THREADS / 64)

__device__ __forceinline__ uint32_t order_key(float x) {
  if (x != x) x = -INFINITY;
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ float block_sum(float v, float* red) {
  v = cw_wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int i = 0; i < SAMPLE_WAVES; ++i) t += red[i];
  return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
  v = cw_wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = -INFINITY;
#pragma unroll
  for (int i = 0; i < SAMPLE_WAVES; ++i) t = fmaxf(t, red[i]);
  return t;
}
__device__ __forceinline__ int block_sum_int(int v, int* red) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  int t = 0;
#pragma unroll
  for (int i = 0; i < SAMPLE_WAVES; ++i) t += red[i];
  return t;
}

// ---------------------------------------------------------------- arg-max, two stages
// The first index wins among equal maxima (torch.argmax semantics, model_runner.py:137).
__device__ __forceinline__ void argmax_merge(float& bv, int& bi, float v, int i) {
  if (v > bv || (v == bv && i < bi)) { bv = v; bi = i; }
}

__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ logits,
                                                             int64_t row_stride, int V, int chunks,
                                                             float* __restrict__ pv,
                                                             int* __restrict__ pi) {
  __shared__ float sv[4];
  __shared__ int si[4];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const int per = (V + chunks - 1) / chunks;
  const int lo = chunk * per, hi = min(V, lo + per);
  const float* x = logits + (int64_t)row * row_stride;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = lo + threadIdx.x; i < hi; i += 256) {
    float v = x[i];
    if (v != v) v = -INFINITY;
    argmax_merge(bv, bi, v, i);
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    argmax_merge(bv, bi, ov, oi);
  }
  if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = bv; si[threadIdx.x >> 6] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) argmax_merge(bv, bi, sv[w], si[w]);
    pv[row * chunks + chunk] = bv;
    pi[row * chunks + chunk] = bi;
  }
}

__global__ void argmax_final_kernel(const float* __restrict__ pv, const int* __restrict__ pi,
                                    int chunks, int V, int* __restrict__ out) {
  const int row = blockIdx.x;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += 64) argmax_merge(bv, bi, pv[row * chunks + c], pi[row * chunks + c]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(bv, off, 64);
    const int oi = __shfl_xor(bi, off, 64);
    argmax_merge(bv, bi, ov, oi);
  }
  if (threadIdx.x == 0) out[row] = bi < V ? bi : 0;
}

#define ARGMAX_MAX_CHUNKS 64

// workspace: n * chunks floats followed by n * chunks ints; chunks = cw_argmax_chunks(V).
CW_EXPORT int cw_argmax_chunks(int V) {
  int c = (V + 4095) / 4096;
  return c < 1 ? 1 : (c > ARGMAX_MAX_CHUNKS ? ARGMAX_MAX_CHUNKS : c);
}

CW_EXPORT int cw_argmax(const float* logits, int64_t row_stride, int n, int V, int* out,
                        void* workspace, int64_t workspace_bytes, hipStream_t stream) {
  if (n < 0 || V <= 0 || row_stride < V) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  if (n > 65535) return CW_ERR_SIZE;
  const int chunks = cw_argmax_chunks(V);
  if (workspace == nullptr || workspace_bytes < (int64_t)n * chunks * 8) return CW_ERR_ARG;
  float* pv = (float*)workspace;
  int* pi = (int*)(pv + (int64_t)n * chunks);
  hipLaunchKernelGGL(argmax_partial_kernel, dim3(chunks, n), dim3(256), 0, stream, logits, row_stride, V, chunks, pv, pi);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(n), dim3(64), 0, stream, pv, pi, chunks, V, out);
  return cw_launch_status();
}

// ---------------------------------------------------------------- Philox4x32-10
__device__ __forceinline__ uint32_t philox_first_word(uint64_t seed, uint64_t counter) {
  uint32_t c0 = (uint32_t)counter, c1 = (uint32_t)(counter >> 32), c2 = 0u, c3 = 0u;
  uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return c0;
}

// ---------------------------------------------------------------- sampling, one workgroup per row
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int64_t row_stride, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const int64_t* __restrict__ seeds,
    const int64_t* __restrict__ draws, int* __restrict__ out) {
  __shared__ float red[SAMPLE_WAVES];
  __shared__ int redi[SAMPLE_WAVES];
  __shared__ float sums[SAMPLE_THREADS];
  __shared__ int pick_thread;
  __shared__ float pick_base;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  const float* x = logits + (int64_t)row * row_stride;
  const float temp = temperature[row];

  if (!(temp > 0.0f)) {  // greedy row inside a sampled batch
    float bv = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = tid; i < V; i += SAMPLE_THREADS) {
      float v = x[i];
      if (v != v) v = -INFINITY;
      argmax_merge(bv, bi, v, i);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, 64);
      const int oi = __shfl_xor(bi, off, 64);
      argmax_merge(bv, bi, ov, oi);
    }
    if ((tid & 63) == 0) { red[tid >> 6] = bv; redi[tid >> 6] = bi; }
    __syncthreads();
    if (tid == 0) {
      for (int w = 1; w < SAMPLE_WAVES; ++w) argmax_merge(bv, bi, red[w], redi[w]);
      out[row] = bi < V ? bi : 0;
    }
    return;
  }

  // ---- top-k: the k-th largest scaled logit, by bisection on the order-preserving key
  uint32_t key_floor = 0u;  // tokens with key < key_floor are masked
  const int k = top_k[row];
  if (k > 0 && k < V) {
    uint32_t K = 0u;
    for (int b = 31; b >= 0; --b) {
      const uint32_t cand = K | (1u << b);
      int cnt = 0;
      for (int i = tid; i < V; i += SAMPLE_THREADS) cnt += order_key(x[i] / temp) >= cand;
      if (block_sum_int(cnt, redi) >= k) K = cand;
    }
    key_floor = K;  // largest key with at least k tokens at or above it: the k-th largest
  }

  // ---- maximum of what is left
  float mx = -INFINITY;
  for (int i = tid; i < V; i += SAMPLE_THREADS) {
    const float v = x[i] / temp;
    if (order_key(v) >= key_floor && v == v) mx = fmaxf(mx, v);
  }
  mx = block_max(mx, red);

  // ---- top-p
  const float p = top_p[row];
  if (p < 1.0f) {
    float z = 0.0f;
    for (int i = tid; i < V; i += SAMPLE_THREADS) {
      const float v = x[i] / temp;
      if (order_key(v) >= key_floor) z += expf(v - mx);
    }
    z = block_sum(z, red);
    const float limit = p * z;  // compare unnormalised masses with top_p * total
    // largest key K with mass(keys > K) > limit; everything above it stays
    uint32_t K = 0u;
    bool any = false;
    for (int b = 31; b >= 0; --b) {
      const uint32_t cand = K | (1u << b);
      float mass = 0.0f;
      for (int i = tid; i < V; i += SAMPLE_THREADS) {
        const float v = x[i] / temp;
        const uint32_t key = order_key(v);
        if (key > cand && key >= key_floor) mass += expf(v - mx);
      }
      if (block_sum(mass, red) > limit) { K = cand; any = true; }
    }
    if (!any) {
      // is mass(keys > 0) > limit at all? if not, nothing is cut
      float mass = 0.0f;
      for (int i = tid; i < V; i += SAMPLE_THREADS) {
        const float v = x[i] / temp;
        const uint32_t key = order_key(v);
        if (key > 0u && key >= key_floor) mass += expf(v - mx);
      }
      any = block_sum(mass, red) > limit;
    }
    if (any && K + 1u > key_floor) key_floor = K + 1u;
  }

  // ---- draw: weights in index order, thread t owns [t * per, (t + 1) * per)
  const int per = (V + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int lo = min(V, tid * per), hi = min(V, lo + per);
  float w = 0.0f;
  for (int i = lo; i < hi; ++i) {
    const float v = x[i] / temp;
    if (order_key(v) >= key_floor) w += expf(v - mx);
  }
  sums[tid] = w;
  __syncthreads();
  if (tid == 0) {
    float total = 0.0f;
    for (int t = 0; t < SAMPLE_THREADS; ++t) total += sums[t];
    const uint32_t r = philox_first_word((uint64_t)seeds[row], (uint64_t)draws[row]);
    const float u = (float)(r >> 8) * (1.0f / 16777216.0f);
    const float target = u * total;
    float run = 0.0f;
    int chosen = -1;
    float base = 0.0f;
    int last_nonzero = 0;
    for (int t = 0; t < SAMPLE_THREADS; ++t) {
      if (sums[t] > 0.0f) last_nonzero = t;
      if (chosen < 0 && run + sums[t] > target && sums[t] > 0.0f) { chosen = t; base = run; }
      run += sums[t];
    }
    if (chosen < 0) {  // target fell on the total through rounding: take the last weighted chunk
      chosen = last_nonzero;
      base = -INFINITY;
    }
    pick_thread = chosen;
    pick_base = base;
    sums[0] = target;
  }
  __syncthreads();
  if (tid == pick_thread) {
    const float target = sums[0];
    float run = pick_base == -INFINITY ? 0.0f : pick_base;
    int chosen = -1, last = lo;
    for (int i = lo; i < hi; ++i) {
      const float v = x[i] / temp;
      if (order_key(v) < key_floor) continue;
      const float e = expf(v - mx);
      if (e > 0.0f) last = i;
      run += e;
      if (pick_base != -INFINITY && run > target && e > 0.0f) { chosen = i; break; }
    }
    out[row] = chosen >= 0 ? chosen : last;
  }
}

CW_EXPORT int cw_sample(const float* logits, int64_t row_stride, int n, int V,
                        const float* temperature, const int* top_k, const float* top_p,
                        const int64_t* seeds, const int64_t* draws, int* out, hipStream_t stream) {
  if (n < 0 || V <= 0 || row_stride < V) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  hipLaunchKernelGGL(sample_kernel, dim3(n), dim3(SAMPLE_THREADS), 0, stream, logits, row_stride, V,
                     temperature, top_k, top_p, seeds, draws, out);
  return cw_launch_status();
}
