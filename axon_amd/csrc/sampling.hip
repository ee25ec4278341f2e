// Picking on the device: greedy argmax and the candidates of a sampled row.
//
// Both order logits by one 64-bit key, (order key of the logit) << 32 | id, as the
// reference's sampler does (src/sample.rs:280-305; src/cuda/sample.cu:124-220): a larger
// logit has a larger key, -0.0 ties +0.0, NaN is below everything, and of equal logits the
// larger id wins.  The largest key is the greedy pick: of equal maxima the last index, NaN
// never, all NaN gives n - 1 (src/generate.rs:222-264).  Keys are distinct, so selection is
// exact and has no order-dependent step: integer histograms only.
#include <mutex>

#include "api.h"
#include "common.h"

#define PICK_THREADS 1024

__device__ inline uint32_t order_key(float v) {
  if (v != v) return 0u;
  uint32_t b = v == 0.0f ? 0u : __float_as_uint(v);
  return (b >> 31) ? ~b : (b | 0x80000000u);
}

__device__ inline uint64_t key64(float v, int id) { return ((uint64_t)order_key(v) << 32) | (uint32_t)id; }

__device__ inline uint64_t wave_max_u64(uint64_t v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const uint32_t lo = __shfl_xor((uint32_t)v, off, AXON_WAVE);
    const uint32_t hi = __shfl_xor((uint32_t)(v >> 32), off, AXON_WAVE);
    const uint64_t o = ((uint64_t)hi << 32) | lo;
    v = o > v ? o : v;
  }
  return v;
}

// Two launches: blocks of 256 threads each take ARGMAX_CHUNK logits of one row and leave the
// largest key of their chunk; then one wave per row takes the largest of those.  The largest
// of 64-bit keys does not depend on the order in which they are compared.
#define ARGMAX_CHUNK 4096
#define ARGMAX_THREADS 256

__global__ void __launch_bounds__(ARGMAX_THREADS)
argmax_chunk_kernel(const float* __restrict__ logits, int stride, uint64_t* __restrict__ chunk_best, int n, int vec) {
  __shared__ uint64_t partial[ARGMAX_THREADS / AXON_WAVE];
  const float* row = logits + (size_t)blockIdx.y * stride;
  const int lo = blockIdx.x * ARGMAX_CHUNK, hi = min(n, lo + ARGMAX_CHUNK);
  uint64_t best = 0;
  if (vec && hi == lo + ARGMAX_CHUNK) {
#pragma unroll
    for (int j = 0; j < ARGMAX_CHUNK / (4 * ARGMAX_THREADS); ++j) {
      const int i = lo + (j * ARGMAX_THREADS + threadIdx.x) * 4;
      const float4 v = *reinterpret_cast<const float4*>(row + i);
      uint64_t k = key64(v.x, i);
      best = k > best ? k : best;
      k = key64(v.y, i + 1);
      best = k > best ? k : best;
      k = key64(v.z, i + 2);
      best = k > best ? k : best;
      k = key64(v.w, i + 3);
      best = k > best ? k : best;
    }
  } else {
    for (int i = lo + threadIdx.x; i < hi; i += ARGMAX_THREADS) {
      const uint64_t k = key64(row[i], i);
      best = k > best ? k : best;
    }
  }
  best = wave_max_u64(best);
  if ((threadIdx.x & (AXON_WAVE - 1)) == 0) partial[threadIdx.x / AXON_WAVE] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint64_t b = partial[0];
    for (int w = 1; w < ARGMAX_THREADS / AXON_WAVE; ++w) b = partial[w] > b ? partial[w] : b;
    chunk_best[(size_t)blockIdx.y * gridDim.x + blockIdx.x] = b;
  }
}

__global__ void __launch_bounds__(AXON_WAVE)
argmax_rows_kernel(const uint64_t* __restrict__ chunk_best, int n_chunks, int32_t* __restrict__ picks) {
  const uint64_t* mine = chunk_best + (size_t)blockIdx.x * n_chunks;
  uint64_t best = 0;
  for (int c = threadIdx.x; c < n_chunks; c += AXON_WAVE) best = mine[c] > best ? mine[c] : best;
  best = wave_max_u64(best);
  // every key of an all-NaN row is (0 << 32 | id): the largest id, n - 1, wins
  if (threadIdx.x == 0) picks[blockIdx.x] = (int32_t)(uint32_t)best;
}

extern "C" long axk_argmax_workspace(int n_rows, int n) {
  return (long)sizeof(uint64_t) * (long)(n_rows > 0 ? n_rows : 0) * ceil_div(n > 0 ? n : 1, ARGMAX_CHUNK);
}

extern "C" int axk_argmax(const float* logits, int logits_stride, int32_t* picks, int n_rows, int n, void* workspace,
                          void* stream) {
  AXK_REQUIRE(n_rows >= 0 && n > 0 && logits_stride >= n, "argmax: bad sizes rows=%d n=%d stride=%d", n_rows, n,
              logits_stride);
  AXK_REQUIRE(n_rows <= 65535, "argmax: %d rows are more than one launch takes", n_rows);
  AXK_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 7) == 0, "argmax: needs its workspace, 8-byte aligned");
  if (n_rows == 0) return 0;
  const int n_chunks = ceil_div(n, ARGMAX_CHUNK);
  const int vec = logits_stride % 4 == 0 && ((uintptr_t)logits & 15) == 0;
  argmax_chunk_kernel<<<dim3(n_chunks, n_rows), ARGMAX_THREADS, 0, (hipStream_t)stream>>>(
      logits, logits_stride, (uint64_t*)workspace, n, vec);
  AXK_LAUNCH_CHECK("argmax_chunk");
  argmax_rows_kernel<<<n_rows, AXON_WAVE, 0, (hipStream_t)stream>>>((const uint64_t*)workspace, n_chunks, picks);
  AXK_LAUNCH_CHECK("argmax_rows");
  return 0;
}

// ---------------------------------------------------------------------------- candidates
// (1) llama.cpp's repeat penalty on the distinct ids of the row's recent window, in place: a
// positive logit is divided by p, any other multiplied (src/sample.rs:307-326).  (2) The k
// largest of the row's 64-bit keys, exactly, in no particular order (the host sorts k pairs).
// Two launches: blocks of 256 threads each take a slice of TOPK_SLICE logits of one row into LDS,
// apply the penalty to the ids that lie in it and leave the slice's own k largest keys (the k
// largest of the row are among them); then one block per row takes the k largest of those.  A
// selection is an 8-pass radix select on the keys: integer histograms only, no step that depends
// on an order.
#define TOPK_SLICE 4096
#define TOPK_THREADS 256
#define TOPK_MERGE_THREADS 1024

// The k-th largest (k >= 1) of the distinct keys key_at(i), i < count, of which at least k are
// valid (key_at returns false for a place without a key).  Every thread of the block calls it
// and gets the same value.  hist: 256 ints of LDS, vars: 2 ints of LDS; blocks of at least 256 threads.
template <class KeyAt>
__device__ inline uint64_t kth_largest_key(KeyAt key_at, int count, int k, int* hist, int* vars) {
  __shared__ int wave_total[256 / AXON_WAVE];
  uint64_t prefix = 0, mask = 0;
  if (threadIdx.x == 0) vars[0] = k;                   // keys still wanted among those that match the prefix
  for (int pass = 7; pass >= 0; --pass) {
    const int shift = pass * 8;
    for (int b = threadIdx.x; b < 256; b += blockDim.x) hist[b] = 0;
    __syncthreads();
    for (int i = threadIdx.x; i < count; i += blockDim.x) {
      uint64_t key;
      if (key_at(i, key) && (key & mask) == prefix) atomicAdd(&hist[(int)((key >> shift) & 255u)], 1);
    }
    __syncthreads();
    // the digit whose bin holds the k-th largest: thread t owns bin 255 - t, counts the keys in the
    // bins above its own (a scan over the threads: within each wave, then the waves before it) and
    // the one thread whose bin the count crosses in says so
    const int remaining = vars[0];
    int mine = 0, upto = 0;
    if (threadIdx.x < 256) {
      mine = hist[255 - threadIdx.x];
      upto = mine;
      const int lane = threadIdx.x & (AXON_WAVE - 1);
#pragma unroll
      for (int off = 1; off < AXON_WAVE; off <<= 1) {
        const int other = __shfl_up(upto, off, AXON_WAVE);
        if (lane >= off) upto += other;
      }
      if (lane == AXON_WAVE - 1) wave_total[threadIdx.x / AXON_WAVE] = upto;
    }
    __syncthreads();
    if (threadIdx.x < 256) {
      for (int w = 0; w < (int)threadIdx.x / AXON_WAVE; ++w) upto += wave_total[w];
      const int above = upto - mine;
      if (above < remaining && upto >= remaining) {
        vars[1] = 255 - threadIdx.x;
        vars[0] = remaining - above;
      }
    }
    __syncthreads();
    prefix |= (uint64_t)vars[1] << shift;
    mask |= (uint64_t)255u << shift;
  }
  __syncthreads();
  return prefix;
}

// grid (slices, rows).  slice_keys [rows][slices][k_stride], slice_count [rows][slices].
__global__ void __launch_bounds__(TOPK_THREADS)
topk_slice_kernel(float* __restrict__ logits, int stride, const int32_t* __restrict__ recent, int recent_stride,
                  const int32_t* __restrict__ n_recent, const float* __restrict__ penalty,
                  const int32_t* __restrict__ k_of_row, uint64_t* __restrict__ slice_keys,
                  int32_t* __restrict__ slice_count, int k_stride, int n) {
  __shared__ float vals[TOPK_SLICE];
  __shared__ int hist[256];
  __shared__ int vars[2], s_count;
  const int r = blockIdx.y, s = blockIdx.x, slices = gridDim.x;
  const int lo = s * TOPK_SLICE, count = min(n - lo, TOPK_SLICE);
  float* row = logits + (size_t)r * stride;
  int k = min(min(k_of_row[r], n), k_stride);        // never past the places of a slice, whatever the caller asks
  if (k <= 0) return;
  for (int i = threadIdx.x; i < count; i += TOPK_THREADS) vals[i] = row[lo + i];
  __syncthreads();
  const float p = penalty[r];
  const int nr = n_recent[r];
  if (p != 1.0f && nr > 0) {
    const int32_t* rec = recent + (size_t)r * recent_stride;
    for (int j = threadIdx.x; j < nr; j += TOPK_THREADS) {
      const int id = rec[j];
      bool first = id >= lo && id < lo + count;         // the ids of this slice, each once
      for (int e = 0; e < j && first; ++e) first = rec[e] != id;
      if (first) {
        const float v = vals[id - lo];
        const float w = v > 0.0f ? v / p : v * p;
        vals[id - lo] = w;
        row[id] = w;
      }
    }
    __syncthreads();
  }
  k = min(k, count);
  auto key_at = [&](int i, uint64_t& key) {
    key = key64(vals[i], lo + i);
    return true;
  };
  const uint64_t least = k == count ? 0 : kth_largest_key(key_at, count, k, hist, vars);
  if (threadIdx.x == 0) s_count = 0;
  __syncthreads();
  uint64_t* dst = slice_keys + ((size_t)r * slices + s) * k_stride;
  for (int i = threadIdx.x; i < count; i += TOPK_THREADS) {
    const uint64_t key = key64(vals[i], lo + i);
    if (key >= least) {
      const int at = atomicAdd(&s_count, 1);
      if (at < k) dst[at] = key;
    }
  }
  if (threadIdx.x == 0) slice_count[r * slices + s] = k;
}

// One block per row: the k largest of the slices' keys.
__global__ void __launch_bounds__(TOPK_MERGE_THREADS)
topk_merge_kernel(const uint64_t* __restrict__ slice_keys, const int32_t* __restrict__ slice_count, int slices, int k_stride,
                  const int32_t* __restrict__ k_of_row, uint64_t* __restrict__ cands, int cands_stride, int n) {
  __shared__ int hist[256];
  __shared__ int vars[2], s_count;
  const int r = blockIdx.x;
  const int k = min(min(k_of_row[r], n), min(k_stride, cands_stride));   // never past the row of candidates
  if (k <= 0) return;
  const uint64_t* keys = slice_keys + (size_t)r * slices * k_stride;
  const int32_t* counts = slice_count + r * slices;
  const int places = slices * k_stride;
  auto key_at = [&](int i, uint64_t& key) {
    if (i % k_stride >= counts[i / k_stride]) return false;
    key = keys[i];
    return true;
  };
  const uint64_t least = kth_largest_key(key_at, places, k, hist, vars);
  if (threadIdx.x == 0) s_count = 0;
  __syncthreads();
  uint64_t* dst = cands + (size_t)r * cands_stride;
  for (int i = threadIdx.x; i < places; i += TOPK_MERGE_THREADS) {
    uint64_t key;
    if (key_at(i, key) && key >= least) {
      const int at = atomicAdd(&s_count, 1);
      if (at < k) dst[at] = key;
    }
  }
}

extern "C" long axk_topk_workspace(int n_rows, int n, int k_stride) {
  if (n_rows <= 0 || n <= 0 || k_stride <= 0) return 0;
  const long slices = ceil_div(n, TOPK_SLICE);
  return (long)n_rows * slices * ((long)k_stride * 8 + 8);       // the slices' keys, then their counts (8-byte places)
}

extern "C" int axk_topk(float* logits, int logits_stride, const int32_t* recent, int recent_stride,
                        const int32_t* n_recent, const float* penalty, const int32_t* k_of_row, uint64_t* cands,
                        int cands_stride, int n_rows, int n, void* workspace, void* stream) {
  AXK_REQUIRE(n_rows >= 0 && n > 0 && logits_stride >= n, "topk: bad sizes rows=%d n=%d stride=%d", n_rows, n,
              logits_stride);
  AXK_REQUIRE(cands_stride >= 1, "topk: candidate stride %d", cands_stride);
  AXK_REQUIRE(n_rows <= 65535, "topk: %d rows are more than one launch takes", n_rows);
  AXK_REQUIRE(workspace != nullptr && ((uintptr_t)workspace & 7) == 0, "topk: needs its workspace, 8-byte aligned");
  if (n_rows == 0) return 0;
  const int slices = ceil_div(n, TOPK_SLICE);
  uint64_t* slice_keys = (uint64_t*)workspace;
  int32_t* slice_count = (int32_t*)(slice_keys + (size_t)n_rows * slices * cands_stride);
  topk_slice_kernel<<<dim3(slices, n_rows), TOPK_THREADS, 0, (hipStream_t)stream>>>(
      logits, logits_stride, recent, recent_stride, n_recent, penalty, k_of_row, slice_keys, slice_count, cands_stride, n);
  AXK_LAUNCH_CHECK("topk_slice");
  topk_merge_kernel<<<n_rows, TOPK_MERGE_THREADS, 0, (hipStream_t)stream>>>(slice_keys, slice_count, slices, cands_stride,
                                                                           k_of_row, cands, cands_stride, n);
  AXK_LAUNCH_CHECK("topk_merge");
  return 0;
}

// ---------------------------------------------------------------------------- argmax without a workspace
// axk_argmax_static: axk_argmax for callers that cannot allocate or bring device memory beyond
// their inputs and outputs.  The chunks' best keys (what axk_argmax keeps in the caller's
// workspace) live in an array of the library's own, ARGMAX_STATIC_ROWS x ARGMAX_STATIC_CHUNKS
// keys = 128 KB that every GPU the library runs on holds until the process ends.  In host code
// the array's name is only a stand-in: the address on the current GPU comes from
// hipGetSymbolAddress, asked once per device, and that pointer is what the kernels are given.
// Nothing has to start at zero: the first launch writes every key the second reads.  All calls
// on one GPU share the array, so calls that overlap there (two streams, two threads) race.
#define ARGMAX_STATIC_ROWS 256
#define ARGMAX_STATIC_CHUNKS 64
#define ARGMAX_STATIC_DEVICES 64

static __device__ __align__(256) uint64_t argmax_scratch[ARGMAX_STATIC_ROWS * ARGMAX_STATIC_CHUNKS];
static uint64_t* argmax_scratch_at[ARGMAX_STATIC_DEVICES];     // per device; written once, under the lock
static std::mutex argmax_scratch_lock;

static int argmax_scratch_of_device(uint64_t** at) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess || device < 0 || device >= ARGMAX_STATIC_DEVICES) {
    axk_set_error("argmax_static: no current device (%s, device %d)", hipGetErrorString(e), device);
    return -2;
  }
  std::lock_guard<std::mutex> hold(argmax_scratch_lock);
  if (argmax_scratch_at[device] == nullptr) {
    uint64_t* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(argmax_scratch));
    if (e != hipSuccess || p == nullptr) {
      axk_set_error("argmax_static: the address of the scratch array on device %d: %s", device, hipGetErrorString(e));
      return -2;
    }
    argmax_scratch_at[device] = p;
  }
  *at = argmax_scratch_at[device];
  return 0;
}

extern "C" int axk_argmax_static_max_rows(void) { return ARGMAX_STATIC_ROWS; }
extern "C" int axk_argmax_static_max_n(void) { return ARGMAX_STATIC_CHUNKS * ARGMAX_CHUNK; }

extern "C" int axk_argmax_static(const float* logits, int logits_stride, int32_t* picks, int n_rows, int n,
                                 void* stream) {
  AXK_REQUIRE(n_rows >= 0 && n > 0 && logits_stride >= n, "argmax_static: bad sizes rows=%d n=%d stride=%d", n_rows, n,
              logits_stride);
  AXK_REQUIRE(n_rows <= ARGMAX_STATIC_ROWS && n <= ARGMAX_STATIC_CHUNKS * ARGMAX_CHUNK,
              "argmax_static: %d rows of %d logits; the library's own scratch takes up to %d rows of %d", n_rows, n,
              ARGMAX_STATIC_ROWS, ARGMAX_STATIC_CHUNKS * ARGMAX_CHUNK);
  AXK_REQUIRE(logits != nullptr && picks != nullptr, "argmax_static: logits or picks missing");
  if (n_rows == 0) return 0;
  uint64_t* scratch = nullptr;
  const int rc = argmax_scratch_of_device(&scratch);
  if (rc != 0) return rc;
  const int n_chunks = ceil_div(n, ARGMAX_CHUNK);
  const int vec = logits_stride % 4 == 0 && ((uintptr_t)logits & 15) == 0;
  argmax_chunk_kernel<<<dim3(n_chunks, n_rows), ARGMAX_THREADS, 0, (hipStream_t)stream>>>(logits, logits_stride,
                                                                                         scratch, n, vec);
  AXK_LAUNCH_CHECK("argmax_chunk");
  argmax_rows_kernel<<<n_rows, AXON_WAVE, 0, (hipStream_t)stream>>>(scratch, n_chunks, picks);
  AXK_LAUNCH_CHECK("argmax_rows");
  return 0;
}
