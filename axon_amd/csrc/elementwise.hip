// Row-wise kernels: embedding gather, RMSNorm, rotary tables, rotary + paged cache store,
// SwiGLU, fills.  Each computes a row the same way whatever other rows share the launch.
#include "api.h"
#include "common.h"
#include "instances.h"

// ---------------------------------------------------------------------------- embedding
// One block per token; the row is widened exactly (bf16 -> f32) or copied.
// Reference twin: embed_b (src/cuda/prefill.cu:52-56); no scaling for this architecture
// (src/model.rs:2657-2675).
// A tied head's matrix is kept packed for the products (see axk_pack_matrix): element (row, i) is
// then at ((row / 16 * dim / 32 + i / 32) * 64 + row % 16 + 16 (i % 32 / 8)) * 8 + i % 8.
__global__ void embed_kernel(const int32_t* __restrict__ tokens, const elem_t* __restrict__ table, int packed,
                             float* __restrict__ x, int dim) {
  const int t = blockIdx.x;
  const int token = tokens[t];
  float* dst = x + (size_t)t * dim;
  if (packed) {
    const elem_t* tile = table + (size_t)(token / 16) * (dim / 32) * 512 + (token % 16) * 8;
    for (int i = threadIdx.x; i < dim; i += blockDim.x)
      dst[i] = to_float(tile[(size_t)(i / 32) * 512 + ((i % 32) / 8) * 128 + i % 8]);
    return;
  }
  const elem_t* row = table + (size_t)token * dim;
  for (int i = threadIdx.x; i < dim; i += blockDim.x) dst[i] = to_float(row[i]);
}

extern "C" int axk_embed(const int32_t* tokens, const void* table, int packed, float* x, int n_tokens, int dim,
                         int vocab, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && dim > 0 && vocab > 0, "embed: bad sizes T=%d dim=%d vocab=%d", n_tokens, dim, vocab);
  AXK_REQUIRE(!packed || dim % 32 == 0, "embed: a packed table has rows of whole blocks of 32, not %d", dim);
  if (n_tokens == 0) return 0;
  embed_kernel<<<n_tokens, 256, 0, (hipStream_t)stream>>>(tokens, (const elem_t*)table, packed, x, dim);
  AXK_LAUNCH_CHECK("embed");
  return 0;
}

// ---------------------------------------------------------------------------- RMSNorm
// ss = sum x^2 (32-bit), ms = ss / n, inv = 1 / sqrt(ms + eps), out = (x * inv) * g: x times
// inv first, then the gain (src/model.rs:3888-3898).  The sum is a strided chain per thread,
// a butterfly per wave and the four waves in order: fixed by `dim` alone
// (the reference's GPU twin does the same: src/cuda/decode.cu:212-249).
#define NORM_THREADS 256
#define NORM_CACHED 4  // float4 a thread keeps in registers: rows up to 4096 wide are read once

__device__ inline void store4(elem_t* dst, float a, float b, float c, float d) {
#if AXON_BF16
  uint2 pk;
  pk.x = (uint32_t)float_to_bf16(a).bits | ((uint32_t)float_to_bf16(b).bits << 16);
  pk.y = (uint32_t)float_to_bf16(c).bits | ((uint32_t)float_to_bf16(d).bits << 16);
  *reinterpret_cast<uint2*>(dst) = pk;
#else
  *reinterpret_cast<float4*>(dst) = make_float4(a, b, c, d);
#endif
}

// Rows whose width is a multiple of 4: thread t takes the float4 t, t + 256, ...; the first
// NORM_CACHED of them stay in registers between the sum and the scaling.  The order of the
// sum depends on the width alone.
__global__ void __launch_bounds__(NORM_THREADS)
rmsnorm_vec_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows, const void* __restrict__ gain,
                   int gain_is_f32, elem_t* __restrict__ out, int dim, float eps) {
  __shared__ float partial[NORM_THREADS / AXON_WAVE];
  const int r = blockIdx.x, n4 = dim >> 2;
  const float4* src = reinterpret_cast<const float4*>(x + (size_t)(rows ? rows[r] : r) * dim);
  float4 kept[NORM_CACHED];
  float ss = 0.0f;
#pragma unroll
  for (int c = 0; c < NORM_CACHED; ++c) {
    const int i = threadIdx.x + c * NORM_THREADS;
    kept[c] = i < n4 ? src[i] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    ss = fmaf(kept[c].x, kept[c].x, ss);
    ss = fmaf(kept[c].y, kept[c].y, ss);
    ss = fmaf(kept[c].z, kept[c].z, ss);
    ss = fmaf(kept[c].w, kept[c].w, ss);
  }
  for (int i = threadIdx.x + NORM_CACHED * NORM_THREADS; i < n4; i += NORM_THREADS) {
    const float4 v = src[i];
    ss = fmaf(v.x, v.x, ss);
    ss = fmaf(v.y, v.y, ss);
    ss = fmaf(v.z, v.z, ss);
    ss = fmaf(v.w, v.w, ss);
  }
  const float total = block_sum_256(ss, partial);
  const float inv = 1.0f / sqrtf(total / (float)dim + eps);
  elem_t* dst = out + (size_t)r * dim;
#pragma unroll
  for (int c = 0; c < NORM_CACHED; ++c) {
    const int i = threadIdx.x + c * NORM_THREADS;
    if (i < n4) {
      const int e = i * 4;
      store4(dst + e, (kept[c].x * inv) * load_vec(gain, gain_is_f32, e), (kept[c].y * inv) * load_vec(gain, gain_is_f32, e + 1),
             (kept[c].z * inv) * load_vec(gain, gain_is_f32, e + 2), (kept[c].w * inv) * load_vec(gain, gain_is_f32, e + 3));
    }
  }
  for (int i = threadIdx.x + NORM_CACHED * NORM_THREADS; i < n4; i += NORM_THREADS) {
    const float4 v = src[i];
    const int e = i * 4;
    store4(dst + e, (v.x * inv) * load_vec(gain, gain_is_f32, e), (v.y * inv) * load_vec(gain, gain_is_f32, e + 1),
           (v.z * inv) * load_vec(gain, gain_is_f32, e + 2), (v.w * inv) * load_vec(gain, gain_is_f32, e + 3));
  }
}

// Any width.
__global__ void __launch_bounds__(NORM_THREADS)
rmsnorm_kernel(const float* __restrict__ x, const int32_t* __restrict__ rows, const void* __restrict__ gain,
               int gain_is_f32, elem_t* __restrict__ out, int dim, float eps) {
  __shared__ float partial[NORM_THREADS / AXON_WAVE];
  const int r = blockIdx.x;
  const float* src = x + (size_t)(rows ? rows[r] : r) * dim;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < dim; i += NORM_THREADS) {
    float v = src[i];
    ss = fmaf(v, v, ss);
  }
  const float total = block_sum_256(ss, partial);
  const float ms = total / (float)dim;
  const float inv = 1.0f / sqrtf(ms + eps);
  elem_t* dst = out + (size_t)r * dim;
  for (int i = threadIdx.x; i < dim; i += NORM_THREADS) {
    float g = load_vec(gain, gain_is_f32, i);
    dst[i] = from_float((src[i] * inv) * g);
  }
}

extern "C" int axk_rmsnorm(const float* x, const int32_t* rows, const void* gain, int gain_is_f32, void* out,
                           int n_rows, int dim, float eps, void* stream) {
  AXK_REQUIRE(n_rows >= 0 && dim > 0, "rmsnorm: bad sizes rows=%d dim=%d", n_rows, dim);
  if (n_rows == 0) return 0;
  const bool vec = dim % 4 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0;
  if (vec) {
    AXK_INSTANCE(INST_RMSNORM, 1);
    rmsnorm_vec_kernel<<<n_rows, NORM_THREADS, 0, (hipStream_t)stream>>>(x, rows, gain, gain_is_f32, (elem_t*)out, dim,
                                                                        eps);
  } else {
    AXK_INSTANCE(INST_RMSNORM, 0);
    rmsnorm_kernel<<<n_rows, NORM_THREADS, 0, (hipStream_t)stream>>>(x, rows, gain, gain_is_f32, (elem_t*)out, dim, eps);
  }
  AXK_LAUNCH_CHECK("rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------- rotary tables
// angle = pos * freq_i in float64, (sin, cos) in float64, rounded to float32 once
// (src/model.rs:2612-2621; GPU twin rope_table_b, src/cuda/prefill.cu:60-69).
__global__ void rope_table_kernel(const int32_t* __restrict__ positions, const double* __restrict__ freqs,
                                  float* __restrict__ table, int n_pairs) {
  const int t = blockIdx.x;
  const double pos = (double)positions[t];
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    double s, c;
    sincos(pos * freqs[i], &s, &c);
    table[((size_t)t * n_pairs + i) * 2 + 0] = (float)s;
    table[((size_t)t * n_pairs + i) * 2 + 1] = (float)c;
  }
}

extern "C" int axk_rope_table(const int32_t* positions, const double* freqs, float* table, int n_tokens,
                              int n_pairs, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_pairs > 0, "rope_table: bad sizes T=%d pairs=%d", n_tokens, n_pairs);
  if (n_tokens == 0) return 0;
  rope_table_kernel<<<n_tokens, 64, 0, (hipStream_t)stream>>>(positions, freqs, table, n_pairs);
  AXK_LAUNCH_CHECK("rope_table");
  return 0;
}

// ---------------------------------------------------------------------------- rotary + cache store
// One wave per (token, head slot), four waves a block: q heads are rotated in place, k heads rotated and stored
// in the request's page for that position, v heads stored as they are (transposed: a page of
// values is [dim][slot], so that the positions of one dim are contiguous).  Pair i of a head
// is (i, i + rotary_dim / 2): out_i = a cos - b sin, out_{i+half} = a sin + b cos, each
// product and sum rounded on its own (src/model.rs:3922-3929; src/cuda/prefill.cu:129-160).
__global__ void rope_kv_write_kernel(elem_t* __restrict__ qkv, const float* __restrict__ table,
                                     const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                                     const int32_t* __restrict__ block_table, int table_stride,
                                     elem_t* __restrict__ k_cache, elem_t* __restrict__ v_cache, int n_heads,
                                     int n_kv_heads, int head_dim, int rotary_dim, int page_size, int write_kv) {
  const int t = blockIdx.x;
  const int slot = blockIdx.y * 4 + threadIdx.x / AXON_WAVE;  // 0..nh: q heads; then k heads; then v heads
  const int lane = threadIdx.x % AXON_WAVE;
  if (slot >= n_heads + (write_kv ? 2 * n_kv_heads : 0)) return;
  const int half = rotary_dim / 2;
  const int row_elems = (n_heads + 2 * n_kv_heads) * head_dim;
  elem_t* src = qkv + (size_t)t * row_elems + (size_t)slot * head_dim;
  const float* tab = table + (size_t)t * half * 2;

  elem_t* dst = src;
  if (slot >= n_heads) {
    if (!write_kv) return;
    const int pos = positions[t];
    const int page = block_table[(size_t)seq_rows[t] * table_stride + pos / page_size];
    const int in_page = pos % page_size;
    const bool is_v = slot >= n_heads + n_kv_heads;
    const int kvh = slot - n_heads - (is_v ? n_kv_heads : 0);
    if (is_v) {
      // values are kept position-contiguous: [page][kv head][dim][slot in page]
      elem_t* vdst = v_cache + ((size_t)page * n_kv_heads + kvh) * head_dim * page_size + in_page;
      for (int i = lane; i < head_dim; i += AXON_WAVE) vdst[(size_t)i * page_size] = src[i];
      return;
    }
    dst = k_cache + (((size_t)page * n_kv_heads + kvh) * page_size + in_page) * head_dim;
  }
  for (int i = lane; i < half; i += AXON_WAVE) {
    const float s = tab[2 * i], c = tab[2 * i + 1];
    const float a = to_float(src[i]), b = to_float(src[i + half]);
    const float lo = __fsub_rn(__fmul_rn(a, c), __fmul_rn(b, s));
    const float hi = __fadd_rn(__fmul_rn(a, s), __fmul_rn(b, c));
    dst[i] = from_float(lo);
    dst[i + half] = from_float(hi);
  }
  if (dst != src)
    for (int i = rotary_dim + lane; i < head_dim; i += AXON_WAVE) dst[i] = src[i];
}

extern "C" int axk_rope_kv_write(void* qkv, const float* table, const int32_t* positions, const int32_t* seq_rows,
                                 const int32_t* block_table, int table_stride, void* k_cache, void* v_cache,
                                 int n_tokens, int n_heads, int n_kv_heads, int head_dim, int rotary_dim,
                                 int page_size, int write_kv, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && head_dim > 0 && page_size > 0,
              "rope_kv_write: bad sizes T=%d nh=%d nkv=%d hd=%d page=%d", n_tokens, n_heads, n_kv_heads, head_dim,
              page_size);
  AXK_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0,
              "rope_kv_write: rotary_dim %d must be even and at most head_dim %d", rotary_dim, head_dim);
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, ceil_div(n_heads + (write_kv ? 2 * n_kv_heads : 0), 4));
  rope_kv_write_kernel<<<grid, 4 * AXON_WAVE, 0, (hipStream_t)stream>>>((elem_t*)qkv, table, positions, seq_rows, block_table,
                                                            table_stride, (elem_t*)k_cache, (elem_t*)v_cache,
                                                            n_heads, n_kv_heads, head_dim, rotary_dim, page_size,
                                                            write_kv);
  AXK_LAUNCH_CHECK("rope_kv_write");
  return 0;
}

// ---------------------------------------------------------------------------- SwiGLU
__global__ void swiglu_kernel(const elem_t* __restrict__ gate_up, elem_t* __restrict__ out, int n_ffn) {
  const int t = blockIdx.y;
  const int f = blockIdx.x * blockDim.x + threadIdx.x;
  if (f >= n_ffn) return;
  const elem_t* row = gate_up + (size_t)t * 2 * n_ffn;
  out[(size_t)t * n_ffn + f] = from_float(swiglu1(to_float(row[f]), to_float(row[n_ffn + f])));
}

extern "C" int axk_swiglu(const void* gate_up, void* out, int n_tokens, int n_ffn, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_ffn > 0, "swiglu: bad sizes T=%d ffn=%d", n_tokens, n_ffn);
  AXK_REQUIRE(n_tokens <= 65535, "swiglu: %d tokens in one step (at most 65535)", n_tokens);
  if (n_tokens == 0) return 0;
  dim3 grid(ceil_div(n_ffn, 256), n_tokens);
  swiglu_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const elem_t*)gate_up, (elem_t*)out, n_ffn);
  AXK_LAUNCH_CHECK("swiglu");
  return 0;
}

// ---------------------------------------------------------------------------- fills
template <typename V>
__global__ void fill_kernel(V* dst, V value, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = value;
}

extern "C" int axk_fill_i32(int32_t* dst, int32_t value, int n, void* stream) {
  if (n <= 0) return 0;
  fill_kernel<int32_t><<<ceil_div(n, 256), 256, 0, (hipStream_t)stream>>>(dst, value, n);
  AXK_LAUNCH_CHECK("fill_i32");
  return 0;
}

extern "C" int axk_fill_f32(float* dst, float value, int n, void* stream) {
  if (n <= 0) return 0;
  fill_kernel<float><<<ceil_div(n, 256), 256, 0, (hipStream_t)stream>>>(dst, value, n);
  AXK_LAUNCH_CHECK("fill_f32");
  return 0;
}
