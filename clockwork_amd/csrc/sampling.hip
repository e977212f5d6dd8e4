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
#include "sampling.h"

#include <mutex>


__device__ __forceinline__ uint32_t order_key(float x) {
  if (x != x) x = -INFINITY;
  const uint32_t u = __float_as_uint(x);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
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

// ---------------------------------------------------------------- arg-max without a workspace
// For callers that cannot allocate (see sampling.h): the partial results live in this array, one
// copy on every GPU that loads the library. In host code its name is only a handle for
// hipGetSymbolAddress; the kernels get the address that call returned for the current GPU.
static __device__ __align__(256) unsigned char scratch[CW_ARGMAX_STATIC_BYTES];
static_assert(CW_ARGMAX_STATIC_BYTES == CW_ARGMAX_STATIC_MAX_ROWS * ARGMAX_MAX_CHUNKS * 8, "scratch holds a value and an index per row and chunk");

#define ARGMAX_STATIC_MAX_DEVICES 64
static void* scratch_of_device[ARGMAX_STATIC_MAX_DEVICES];
static std::mutex scratch_lock;

// The array's address on the current GPU, looked up at the first call on that GPU.
static int argmax_static_scratch(void** out) {
  int device = -1;
  if (hipGetDevice(&device) != hipSuccess) return CW_ERR_LAUNCH;
  if (device < 0 || device >= ARGMAX_STATIC_MAX_DEVICES) return CW_ERR_SIZE;
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (scratch_of_device[device] == nullptr) {
    void* ptr = nullptr;
    if (hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)) != hipSuccess || ptr == nullptr) {
      (void)hipGetLastError();
      return CW_ERR_LAUNCH;
    }
    scratch_of_device[device] = ptr;
  }
  *out = scratch_of_device[device];
  return CW_OK;
}

CW_EXPORT int cw_argmax_static_init(void) {
  void* ptr = nullptr;
  return argmax_static_scratch(&ptr);
}

CW_EXPORT int cw_argmax_static(const float* logits, int64_t row_stride, int n, int V, int* out,
                               hipStream_t stream) {
  if (n < 0 || V <= 0 || row_stride < V || logits == nullptr || out == nullptr) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  if (n > CW_ARGMAX_STATIC_MAX_ROWS) return CW_ERR_SIZE;
  void* ptr = nullptr;
  const int status = argmax_static_scratch(&ptr);
  if (status != CW_OK) return status;
  const int chunks = cw_argmax_chunks(V);
  // values in the first half of the array, indices in the second, wherever n and chunks end
  float* pv = (float*)ptr;
  int* pi = (int*)((unsigned char*)ptr + CW_ARGMAX_STATIC_BYTES / 2);
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

// ---------------------------------------------------------------- sampling
// A row is cut into chunks and every step of the selection is one small kernel over
// (chunk, row), so a row's work is spread over many compute units and a step costs little more
// than its launch; what a step needs of the step before it goes through the workspace: the
// chunks add their histograms into the row's with integer atomics (a sum that no order changes),
// and every workgroup of the next step reads that one histogram.
//
//   MAX      per chunk: the largest logit and its first index (greedy rows end here);
//   TOPK 0-3 the k-th largest logit by radix selection, 8 bits of the order-preserving key a
//            step: per chunk a histogram of the next byte among the keys that share the bytes
//            found so far. Dividing by the temperature keeps the order, so the selection runs on
//            the raw logits and the floor of what is kept is (k-th largest) / temperature:
//            ties at the k-th value survive, also ties that the division makes;
//   ZSUM     per chunk: the sum of the weights exp(logit / T - max) of what top-k left;
//   TOPP 0-3 the same radix selection with weights instead of counts: the largest key K with
//            weight(keys >= K) > top_p * total; everything from K up stays, i.e. a token stays
//            while the tokens strictly more likely than it weigh <= top_p * total;
//   SUMS     the chunk sums again with the final floor (rows with top-p only);
//   LOCATE   u * total falls into a chunk, and in it on the first index whose running sum
//            exceeds it.
// Weights are integers, exp(.) * 2^40 rounded down: their sums do not depend on the order of
// addition, so every comparison above gives the same answer however the row is cut and however
// the additions are scheduled (LDS atomics included), run after run.
#define SAMPLE_THREADS 256
#define SAMPLE_MAX_CHUNKS 64
#define SAMPLE_WEIGHT_SCALE 1099511627776.0f  // 2^40

typedef unsigned long long u64_t;

struct SampleArgs {
  const float* logits;
  int64_t row_stride;
  int n, V, chunks, per;
  const float* temperature;
  const int* top_k;
  const float* top_p;
  const int64_t* seeds;
  const int64_t* draws;
  int* out;
  // workspace
  float* pmax;       // [n][chunks]
  int* pmax_i;       // [n][chunks]
  uint32_t* hist_k;  // [4 steps][n][256], zeroed by the MAX step
  u64_t* hist_p;     // [4 steps][n][256], zeroed by the MAX step
  uint32_t* state_k; // [2][n][2]: key bits found so far, rank still to go
  u64_t* state_p;    // [2][n][2]: key bits found so far, weight above them
  uint32_t* floor_k; // [n] scaled-key floor after top-k
  u64_t* psum;       // [n][chunks] chunk sums of weights
};

CW_EXPORT int cw_sample_chunks(int V) {
  int c = (V + 2047) / 2048;
  return c < 1 ? 1 : (c > SAMPLE_MAX_CHUNKS ? SAMPLE_MAX_CHUNKS : c);
}

CW_EXPORT int64_t cw_sample_workspace_bytes(int n, int V) {
  const int64_t rc = (int64_t)n * cw_sample_chunks(V);
  // hist_p, state_p, psum, the second psum with a floor per row; hist_k, state_k, floor_k, pmax, pmax_i
  return 8 * (4 * (int64_t)n * 256 + 4 * (int64_t)n + rc + rc + n) + 4 * (4 * (int64_t)n * 256 + 4 * (int64_t)n + n + 2 * rc) + 64;
}

__device__ __forceinline__ float key_to_float(uint32_t k) {
  return __uint_as_float((k & 0x80000000u) ? (k & 0x7fffffffu) : ~k);
}
__device__ __forceinline__ bool row_has_top_k(const SampleArgs& a, int row) {
  const int k = a.top_k[row];
  return k > 0 && k < a.V;
}
__device__ __forceinline__ bool row_has_top_p(const SampleArgs& a, int row) { return a.top_p[row] < 1.0f; }
__device__ __forceinline__ u64_t weight_of(float v, float mx) {
  const float e = expf(v - mx);  // NaN for inf - inf: no weight
  return e == e ? (u64_t)(e * SAMPLE_WEIGHT_SCALE) : 0;
}

// The row's largest logit (NaN counts as -inf) and its first index, from the chunk maxima: the
// first wave takes a chunk a lane (there are at most 64), every thread gets the result.
__device__ __forceinline__ void row_max(const SampleArgs& a, int row, float& bv, int& bi) {
  __shared__ float best_v;
  __shared__ int best_i;
  if (threadIdx.x < 64) {
    float v = -INFINITY;
    int i = 0x7fffffff;
    if ((int)threadIdx.x < a.chunks) {
      v = a.pmax[row * a.chunks + threadIdx.x];
      i = a.pmax_i[row * a.chunks + threadIdx.x];
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      const float ov = __shfl_xor(v, off, 64);
      const int oi = __shfl_xor(i, off, 64);
      argmax_merge(v, i, ov, oi);
    }
    if (threadIdx.x == 0) { best_v = v; best_i = i; }
  }
  __syncthreads();
  bv = best_v;
  bi = best_i;
  __syncthreads();
}

// For every thread b < 256: suf = sum of the bins b..255 of a row's histogram (a scan through
// LDS) and next = the bins above b.
template <typename T>
__device__ __forceinline__ T suffix_of_bins(const T* hist_row, T* sh, T& next) {
  const int b = threadIdx.x;
  const T t = hist_row[b];
  __syncthreads();
  sh[b] = t;
  __syncthreads();
  for (int off = 1; off < 256; off <<= 1) {
    const T add = b + off < 256 ? sh[b + off] : (T)0;
    __syncthreads();
    sh[b] += add;
    __syncthreads();
  }
  const T suf = sh[b];
  next = suf - t;
  return suf;
}

// MAX
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_max_kernel(SampleArgs a) {
  __shared__ float sv[SAMPLE_THREADS / 64];
  __shared__ int si[SAMPLE_THREADS / 64];
  const int row = blockIdx.y, chunk = blockIdx.x;
  if (chunk == 0) {  // the row's histograms start at zero
#pragma unroll
    for (int step = 0; step < 4; ++step) {
      a.hist_k[((int64_t)step * a.n + row) * 256 + threadIdx.x] = 0u;
      a.hist_p[((int64_t)step * a.n + row) * 256 + threadIdx.x] = 0;
    }
  }
  const int lo = chunk * a.per, hi = min(a.V, lo + a.per);
  const float* x = a.logits + (int64_t)row * a.row_stride;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = lo + threadIdx.x; i < hi; i += SAMPLE_THREADS) {
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
    for (int w = 1; w < SAMPLE_THREADS / 64; ++w) argmax_merge(bv, bi, sv[w], si[w]);
    a.pmax[row * a.chunks + chunk] = bv;
    a.pmax_i[row * a.chunks + chunk] = bi;
  }
}

// State of the top-k descent after `done` steps, from the state after done - 1 steps (in the
// workspace, written by the step before) and that step's histograms: (key bits, rank to go).
__device__ __forceinline__ void topk_state(const SampleArgs& a, int row, int done, uint32_t* sh, uint32_t& prefix,
                                           uint32_t& rank) {
  __shared__ uint32_t picked[2];
  if (done == 0) {
    prefix = 0u;
    rank = (uint32_t)a.top_k[row];
    return;
  }
  uint32_t p0 = 0u, r0 = (uint32_t)a.top_k[row];
  if (done > 1) {
    const uint32_t* st = a.state_k + ((int64_t)((done - 2) & 1) * a.n + row) * 2;
    p0 = st[0];
    r0 = st[1];
  }
  const uint32_t* hist = a.hist_k + ((int64_t)(done - 1) * a.n + row) * 256;
  if (threadIdx.x == 0) {  // what stands if no bin qualifies (it always does for counts that add up)
    picked[0] = 0u;
    picked[1] = r0;
  }
  uint32_t above;
  const uint32_t suf = suffix_of_bins<uint32_t>(hist, sh, above);
  // the bin that holds the rank-th largest: at least `rank` keys from it up, fewer above it
  if (suf >= r0 && above < r0) {
    picked[0] = threadIdx.x;
    picked[1] = r0 - above;
  }
  __syncthreads();
  prefix = p0 | (picked[0] << (24 - 8 * (done - 1)));
  rank = picked[1];
  __syncthreads();
}

// TOPK step `step` (0..3): histogram of byte `step` of the raw keys that share the bytes found.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_topk_kernel(SampleArgs a, int step) {
  __shared__ uint32_t sh[256];
  __shared__ uint32_t bins[SAMPLE_THREADS / 64][256];
  const int row = blockIdx.y, chunk = blockIdx.x;
  if (!(a.temperature[row] > 0.0f) || !row_has_top_k(a, row)) return;
  uint32_t prefix, rank;
  topk_state(a, row, step, sh, prefix, rank);
  if (chunk == 0 && threadIdx.x == 0 && step > 0) {
    uint32_t* st = a.state_k + ((int64_t)((step - 1) & 1) * a.n + row) * 2;
    st[0] = prefix;
    st[1] = rank;
  }
  for (int i = threadIdx.x; i < (SAMPLE_THREADS / 64) * 256; i += SAMPLE_THREADS) (&bins[0][0])[i] = 0u;
  __syncthreads();
  const int lo = chunk * a.per, hi = min(a.V, lo + a.per);
  const float* x = a.logits + (int64_t)row * a.row_stride;
  const int shift = 24 - 8 * step;
  const uint32_t mask = step == 0 ? 0u : (0xffffffffu << (shift + 8));
  uint32_t* mine = bins[threadIdx.x >> 6];
  for (int i0 = lo + threadIdx.x; i0 < hi; i0 += 4 * SAMPLE_THREADS) {  // four loads in flight
    float raw[4];
    bool in[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      in[u] = i0 + u * SAMPLE_THREADS < hi;
      raw[u] = in[u] ? x[i0 + u * SAMPLE_THREADS] : 0.0f;
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const uint32_t key = order_key(raw[u]);
      if (in[u] && (key & mask) == prefix) atomicAdd(&mine[(key >> shift) & 255u], 1u);
    }
  }
  __syncthreads();
  uint32_t t = 0u;
#pragma unroll
  for (int w = 0; w < SAMPLE_THREADS / 64; ++w) t += bins[w][threadIdx.x];
  if (t) atomicAdd(&a.hist_k[((int64_t)step * a.n + row) * 256 + threadIdx.x], t);
}

// The floor top-k leaves, as a key of the scaled logits (0: nothing is cut). Every thread of the
// workgroup gets it; after ZSUM it is in the workspace.
__device__ __forceinline__ uint32_t topk_floor(const SampleArgs& a, int row, float temp, uint32_t* sh) {
  if (!row_has_top_k(a, row)) return 0u;
  uint32_t key, rank;
  topk_state(a, row, 4, sh, key, rank);
  return order_key(key_to_float(key) / temp);
}

// Sum of the weights of the chunk's kept tokens, every thread gets it.
__device__ __forceinline__ u64_t chunk_weight(const SampleArgs& a, int row, int chunk, float temp, float mx,
                                              uint32_t floor_key, u64_t* red) {
  const int lo = chunk * a.per, hi = min(a.V, lo + a.per);
  const float* x = a.logits + (int64_t)row * a.row_stride;
  u64_t w = 0;
  for (int i0 = lo + threadIdx.x; i0 < hi; i0 += 4 * SAMPLE_THREADS) {  // four loads in flight
    float raw[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) raw[u] = i0 + u * SAMPLE_THREADS < hi ? x[i0 + u * SAMPLE_THREADS] : NAN;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float v = raw[u] / temp;
      if (v == v && order_key(v) >= floor_key) w += weight_of(v, mx);
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) w += __shfl_xor(w, off, 64);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = w;
  __syncthreads();
  u64_t t = 0;
#pragma unroll
  for (int i = 0; i < SAMPLE_THREADS / 64; ++i) t += red[i];
  return t;
}

// ZSUM
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_zsum_kernel(SampleArgs a) {
  __shared__ uint32_t sh[256];
  __shared__ u64_t red[SAMPLE_THREADS / 64];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const float temp = a.temperature[row];
  if (!(temp > 0.0f)) return;
  const uint32_t floor_key = topk_floor(a, row, temp, sh);
  if (chunk == 0 && threadIdx.x == 0) a.floor_k[row] = floor_key;
  float mraw;
  int mi;
  row_max(a, row, mraw, mi);
  const u64_t w = chunk_weight(a, row, chunk, temp, mraw / temp, floor_key, red);
  if (threadIdx.x == 0) a.psum[row * a.chunks + chunk] = w;
}

// State of the top-p descent after `done` steps: (key bits, weight of the keys above them).
__device__ __forceinline__ void topp_state(const SampleArgs& a, int row, int done, u64_t limit, u64_t* sh,
                                           uint32_t& prefix, u64_t& above_all) {
  __shared__ u64_t picked[2];
  if (done == 0) {
    prefix = 0u;
    above_all = 0;
    return;
  }
  uint32_t p0 = 0u;
  u64_t a0 = 0;
  if (done > 1) {
    const u64_t* st = a.state_p + ((int64_t)((done - 2) & 1) * a.n + row) * 2;
    p0 = (uint32_t)st[0];
    a0 = st[1];
  }
  const u64_t* hist = a.hist_p + ((int64_t)(done - 1) * a.n + row) * 256;
  if (threadIdx.x == 0) {  // what stands if no bin qualifies (a row without any weight)
    picked[0] = 0;
    picked[1] = a0;
  }
  u64_t above;
  const u64_t suf = suffix_of_bins<u64_t>(hist, sh, above);
  // the largest byte b with weight(keys >= (bytes so far, b, 0...)) > limit
  if (a0 + suf > limit && !(a0 + above > limit)) {
    picked[0] = threadIdx.x;
    picked[1] = a0 + above;
  }
  __syncthreads();
  prefix = p0 | ((uint32_t)picked[0] << (24 - 8 * (done - 1)));
  above_all = picked[1];
  __syncthreads();
}

// Sum of a row's chunk sums (order does not matter: integers); every thread gets it.
__device__ __forceinline__ u64_t row_total(const u64_t* sums, int chunks) {
  __shared__ u64_t total;
  if (threadIdx.x < 64) {
    u64_t t = (int)threadIdx.x < chunks ? sums[threadIdx.x] : 0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) t += __shfl_xor(t, off, 64);
    if (threadIdx.x == 0) total = t;
  }
  __syncthreads();
  const u64_t t = total;
  __syncthreads();
  return t;
}
__device__ __forceinline__ u64_t topp_limit(float p, u64_t total) { return (u64_t)((double)p * (double)total); }

// TOPP step `step` (0..3): weight per value of byte `step` among the kept raw keys that share
// the bytes found so far.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_topp_kernel(SampleArgs a, int step) {
  __shared__ u64_t sh[256];
  __shared__ u64_t bins[SAMPLE_THREADS / 64][256];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const float temp = a.temperature[row];
  if (!(temp > 0.0f) || !row_has_top_p(a, row)) return;
  const u64_t limit = topp_limit(a.top_p[row], row_total(a.psum + row * a.chunks, a.chunks));
  uint32_t prefix;
  u64_t above;
  topp_state(a, row, step, limit, sh, prefix, above);
  if (chunk == 0 && threadIdx.x == 0 && step > 0) {
    u64_t* st = a.state_p + ((int64_t)((step - 1) & 1) * a.n + row) * 2;
    st[0] = prefix;
    st[1] = above;
  }
  for (int i = threadIdx.x; i < (SAMPLE_THREADS / 64) * 256; i += SAMPLE_THREADS) (&bins[0][0])[i] = 0;
  __syncthreads();
  float mraw;
  int mi;
  row_max(a, row, mraw, mi);
  const float mx = mraw / temp;
  const uint32_t floor_key = a.floor_k[row];
  const int lo = chunk * a.per, hi = min(a.V, lo + a.per);
  const float* x = a.logits + (int64_t)row * a.row_stride;
  const int shift = 24 - 8 * step;
  const uint32_t mask = step == 0 ? 0u : (0xffffffffu << (shift + 8));
  u64_t* mine = bins[threadIdx.x >> 6];
  for (int i0 = lo + threadIdx.x; i0 < hi; i0 += 4 * SAMPLE_THREADS) {  // four loads in flight
    float raws[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) raws[u] = i0 + u * SAMPLE_THREADS < hi ? x[i0 + u * SAMPLE_THREADS] : NAN;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float raw = raws[u];
      const uint32_t key = order_key(raw);
      if (raw != raw || (key & mask) != prefix) continue;
      const float v = raw / temp;
      if (v == v && order_key(v) >= floor_key) atomicAdd(&mine[(key >> shift) & 255u], weight_of(v, mx));
    }
  }
  __syncthreads();
  u64_t t = 0;
#pragma unroll
  for (int w = 0; w < SAMPLE_THREADS / 64; ++w) t += bins[w][threadIdx.x];
  if (t) atomicAdd(&a.hist_p[((int64_t)step * a.n + row) * 256 + threadIdx.x], t);
}

// SUMS: the chunk sums with the floor that top-p adds (rows with top-p).
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_sums_kernel(SampleArgs a, u64_t* psum_out) {
  __shared__ u64_t sh[256];
  __shared__ u64_t red[SAMPLE_THREADS / 64];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const float temp = a.temperature[row];
  if (!(temp > 0.0f) || !row_has_top_p(a, row)) return;
  const u64_t limit = topp_limit(a.top_p[row], row_total(a.psum + row * a.chunks, a.chunks));
  uint32_t key;
  u64_t above;
  topp_state(a, row, 4, limit, sh, key, above);
  uint32_t floor_key = order_key(key_to_float(key) / temp);
  if (floor_key < a.floor_k[row]) floor_key = a.floor_k[row];
  float mraw;
  int mi;
  row_max(a, row, mraw, mi);
  const u64_t w = chunk_weight(a, row, chunk, temp, mraw / temp, floor_key, red);
  if (threadIdx.x == 0) {
    psum_out[row * a.chunks + chunk] = w;
    if (chunk == 0) psum_out[(int64_t)a.n * a.chunks + row] = floor_key;  // for LOCATE
  }
}

// LOCATE: one workgroup per row.
__global__ __launch_bounds__(SAMPLE_THREADS) void sample_locate_kernel(SampleArgs a, const u64_t* psum2) {
  __shared__ u64_t scan[SAMPLE_THREADS];
  __shared__ int found;
  const int row = blockIdx.x;
  const float temp = a.temperature[row];
  float mraw;
  int mi;
  row_max(a, row, mraw, mi);
  if (!(temp > 0.0f)) {  // greedy row inside a sampled batch
    if (threadIdx.x == 0) a.out[row] = mi < a.V ? mi : 0;
    return;
  }
  const bool with_p = row_has_top_p(a, row);
  const u64_t* sums = (with_p ? psum2 : a.psum) + row * a.chunks;
  const uint32_t floor_key = with_p ? (uint32_t)psum2[(int64_t)a.n * a.chunks + row] : a.floor_k[row];
  const u64_t total = row_total(sums, a.chunks);
  if (total == 0) {  // no token has any weight (every logit -inf or NaN): the first maximum, as greedy
    if (threadIdx.x == 0) a.out[row] = mi < a.V ? mi : 0;
    return;
  }
  const uint32_t r = philox_first_word((uint64_t)a.seeds[row], (uint64_t)a.draws[row]);
  // u = (r >> 8) / 2^24; the drawn token is the first whose running weight exceeds u * total
  u64_t target = (u64_t)((double)(r >> 8) * (1.0 / 16777216.0) * (double)total);
  if (target >= total) target = total - 1;  // (total >= 2^40: the largest logit weighs that much)
  // the chunk the target falls into: a running sum over the chunks in the first wave
  __shared__ int sel_chunk;
  __shared__ u64_t sel_base;
  if (threadIdx.x == 0) {
    sel_chunk = 0;
    sel_base = 0;
  }
  __syncthreads();
  if (threadIdx.x < 64) {
    const u64_t v = (int)threadIdx.x < a.chunks ? sums[threadIdx.x] : 0;
    u64_t incl = v;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const u64_t up = __shfl_up(incl, off, 64);
      if ((int)threadIdx.x >= off) incl += up;
    }
    if (v > 0 && incl - v <= target && target < incl) {
      sel_chunk = threadIdx.x;
      sel_base = incl - v;
    }
  }
  __syncthreads();
  const int chunk = sel_chunk;
  const u64_t base = sel_base;
  // in the chunk: thread t owns a run of consecutive tokens
  const float mx = mraw / temp;
  const int lo = chunk * a.per, hi = min(a.V, lo + a.per);
  const int run = (hi - lo + SAMPLE_THREADS - 1) / SAMPLE_THREADS;
  const int my_lo = min(hi, lo + (int)threadIdx.x * run), my_hi = min(hi, my_lo + run);
  const float* x = a.logits + (int64_t)row * a.row_stride;
  u64_t w = 0;
  for (int i = my_lo; i < my_hi; ++i) {
    const float v = x[i] / temp;
    if (v == v && order_key(v) >= floor_key) w += weight_of(v, mx);
  }
  scan[threadIdx.x] = w;
  if (threadIdx.x == 0) found = -1;
  __syncthreads();
  for (int off = 1; off < SAMPLE_THREADS; off <<= 1) {  // inclusive scan
    const u64_t add = threadIdx.x >= off ? scan[threadIdx.x - off] : 0;
    __syncthreads();
    scan[threadIdx.x] += add;
    __syncthreads();
  }
  const u64_t incl = base + scan[threadIdx.x], excl = incl - w;
  if (w > 0 && excl <= target && target < incl) {
    u64_t at = excl;
    int chosen = my_lo;
    for (int i = my_lo; i < my_hi; ++i) {
      const float v = x[i] / temp;
      if (!(v == v && order_key(v) >= floor_key)) continue;
      const u64_t q = weight_of(v, mx);
      if (q == 0) continue;
      chosen = i;
      at += q;
      if (at > target) break;
    }
    found = chosen;
  }
  __syncthreads();
  if (threadIdx.x == 0) a.out[row] = found >= 0 ? found : (mi < a.V ? mi : 0);
}

// flags: bit 0 some row may have top-k, bit 1 some row may have top-p (3 when unknown): the
// steps no row needs are not launched. workspace: cw_sample_workspace_bytes(n, V) bytes, 16-byte
// aligned.
CW_EXPORT int cw_sample(const float* logits, int64_t row_stride, int n, int V,
                        const float* temperature, const int* top_k, const float* top_p,
                        const int64_t* seeds, const int64_t* draws, int* out, void* workspace,
                        int64_t workspace_bytes, int flags, hipStream_t stream) {
  if (n < 0 || V <= 0 || row_stride < V) return CW_ERR_ARG;
  if (n == 0) return CW_OK;
  if (n > 65535) return CW_ERR_SIZE;
  if (workspace == nullptr || ((uintptr_t)workspace & 15) || workspace_bytes < cw_sample_workspace_bytes(n, V))
    return CW_ERR_ARG;
  SampleArgs a;
  a.logits = logits; a.row_stride = row_stride; a.n = n; a.V = V;
  a.chunks = cw_sample_chunks(V);
  a.per = (V + a.chunks - 1) / a.chunks;
  a.temperature = temperature; a.top_k = top_k; a.top_p = top_p; a.seeds = seeds; a.draws = draws; a.out = out;
  const int64_t rc = (int64_t)n * a.chunks;
  // 8-byte items first
  u64_t* p8 = (u64_t*)workspace;
  a.hist_p = p8; p8 += 4 * (int64_t)n * 256;
  a.state_p = p8; p8 += (int64_t)n * 4;
  a.psum = p8; p8 += rc;
  u64_t* psum2 = p8; p8 += rc + n;
  uint32_t* p4 = (uint32_t*)p8;
  a.hist_k = p4; p4 += 4 * (int64_t)n * 256;
  a.state_k = p4; p4 += (int64_t)n * 4;
  a.floor_k = p4; p4 += n;
  a.pmax = (float*)p4; p4 += rc;
  a.pmax_i = (int*)p4; p4 += rc;
  if ((char*)p4 > (char*)workspace + workspace_bytes) return CW_ERR_ARG;
  const dim3 grid(a.chunks, n), block(SAMPLE_THREADS);
  hipLaunchKernelGGL(sample_max_kernel, grid, block, 0, stream, a);
  if (flags & 1)
    for (int step = 0; step < 4; ++step) hipLaunchKernelGGL(sample_topk_kernel, grid, block, 0, stream, a, step);
  hipLaunchKernelGGL(sample_zsum_kernel, grid, block, 0, stream, a);
  if (flags & 2) {
    for (int step = 0; step < 4; ++step) hipLaunchKernelGGL(sample_topp_kernel, grid, block, 0, stream, a, step);
    hipLaunchKernelGGL(sample_sums_kernel, grid, block, 0, stream, a, psum2);
  }
  hipLaunchKernelGGL(sample_locate_kernel, dim3(n), block, 0, stream, a, psum2);
  return cw_launch_status();
}
