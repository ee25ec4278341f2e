// Paged causal attention over the cache.
//
// The order every variant keeps (the reference's rule for its attention kernels,
// src/cuda/decode.cu:1371-1400, 1650-1670): a token's positions are taken in blocks of 64
// aligned to absolute position (block b = positions 64b .. 64b+63), each block gives
// (m_b, l_b, o_b) = (max score, sum of exp(s - m_b), sum of exp(s - m_b) v), and blocks are
// folded in ascending order into running (M, L, O):
//     mn = max(M, m_b); alpha = exp(M - mn); w = exp(m_b - mn);
//     L = l_b w + L alpha;  O = o_b w + O alpha;  out = O / L.
// The block size does not depend on the page size, the batch or the context length, so a
// token's result is the same however the step was cut.
//
// attention_rows: one wave (or eight, see below) per (token, query head), any head_dim that is a
// multiple of 16 up to 256, any page size, any window.  Prefill portions and decode tokens alike.
#include <math.h>

#include "api.h"
#include "common.h"
#include "instances.h"

#define ATT_BLOCK 64
#define ATT_MAX_HD 256
// What a wave brings through LDS at a time (`staged`): 32 dims of its block's 64 keys, then all
// dims of 8 positions of values: loads in which neighbouring lanes read neighbouring bytes, where a
// lane walking its own key row (and a row of V^T a lane) asks for 64 cache lines an instruction.
#define ATT_KC 32
#define ATT_VP 8
#define ATT_STAGE (ATT_BLOCK * (ATT_KC + 4))   // floats a wave; also ATT_MAX_HD x (ATT_VP + 1)

__device__ inline const elem_t* cache_row(const elem_t* base, const int32_t* table_row, int pos, int page_size,
                                          int n_kv_heads, int kvh, int head_dim) {
  const int page = table_row[pos / page_size];
  return base + (((size_t)page * n_kv_heads + kvh) * page_size + (pos % page_size)) * head_dim;
}

// WAVES waves a block take WAVES neighbouring blocks of 64 positions at a time, each wave its own,
// and every wave then folds them in ascending order (all waves hold the same running values):
// the arithmetic of a wave alone, spread over more of the chip when tokens x heads are few.
template <int WAVES>
__global__ void __launch_bounds__(AXON_WAVE * WAVES)
attention_rows_kernel(const elem_t* __restrict__ q, int q_stride, const elem_t* __restrict__ k_cache,
                      const elem_t* __restrict__ v_cache, const int32_t* __restrict__ block_table, int table_stride,
                      const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                      elem_t* __restrict__ out, int n_heads, int n_kv_heads, int head_dim, int page_size, int window,
                      float scale, bool vec_k, bool staged) {
  static_assert(ATT_STAGE >= ATT_MAX_HD * (ATT_VP + 1), "the stage holds a step of either kind");
  __shared__ float qs[ATT_MAX_HD];
  __shared__ float es[WAVES][ATT_BLOCK];
  __shared__ const elem_t* vrow[WAVES][ATT_BLOCK];
  __shared__ float part[WAVES][WAVES > 1 ? ATT_MAX_HD + 2 : 1];   // a wave's block: o_b, then m_b and l_b
  extern __shared__ __align__(16) float stages[];                 // [WAVES][ATT_STAGE] if `staged`
  const int t = blockIdx.x, qh = blockIdx.y, lane = threadIdx.x % AXON_WAVE, wave = threadIdx.x / AXON_WAVE;
  float* stage = stages + wave * ATT_STAGE;
  const int kvh = qh / (n_heads / n_kv_heads);
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
  const int32_t* table_row = block_table + (size_t)seq_rows[t] * table_stride;

  const elem_t* qrow = q + (size_t)t * q_stride + (size_t)qh * head_dim;
  for (int d = threadIdx.x; d < head_dim; d += AXON_WAVE * WAVES) qs[d] = to_float(qrow[d]);
  __syncthreads();

  constexpr int DPL = ATT_MAX_HD / AXON_WAVE;  // output dims per lane at most
  float M = -INFINITY, L = 0.0f, O[DPL];
#pragma unroll
  for (int i = 0; i < DPL; ++i) O[i] = 0.0f;

  for (int g0 = (lo / ATT_BLOCK) * ATT_BLOCK; g0 <= pos; g0 += ATT_BLOCK * WAVES) {
    const int b0 = g0 + ATT_BLOCK * wave;   // this wave's block; beyond pos it only keeps the barriers' count
    const int p = b0 + lane;
    const bool live = p >= lo && p <= pos;
    float s = -INFINITY;
    if (staged) {
      // lane l fetches 16 bytes l % 8 of the chunk of rows l / 8 + 8 i; every wave of the block
      // passes the same barriers whether its block exists or not
      const int sub = (lane % 8) * 4;
      const elem_t* krow[ATT_BLOCK / 8];
#pragma unroll
      for (int i = 0; i < ATT_BLOCK / 8; ++i) {
        const int pr = b0 + lane / 8 + 8 * i;
        krow[i] = pr >= lo && pr <= pos ? cache_row(k_cache, table_row, pr, page_size, n_kv_heads, kvh, head_dim) + sub
                                        : nullptr;
      }
      float dot = 0.0f;
      for (int c0 = 0; c0 < head_dim; c0 += ATT_KC) {
        const int dims = min(ATT_KC, head_dim - c0);   // head_dim is a multiple of 16
#pragma unroll
        for (int i = 0; i < ATT_BLOCK / 8; ++i) {
          if (krow[i] == nullptr || sub >= dims) continue;
          float k4[4];
          load4_guarded(krow[i] + c0, 4, true, k4);
          *reinterpret_cast<float4*>(&stage[(lane / 8 + 8 * i) * (ATT_KC + 4) + sub]) = make_float4(k4[0], k4[1], k4[2], k4[3]);
        }
        __syncthreads();
        if (live) {
          for (int d = 0; d < dims; d += 4) {
            const float4 k4 = *reinterpret_cast<const float4*>(&stage[lane * (ATT_KC + 4) + d]);
            dot = fmaf(qs[c0 + d], k4.x, dot);
            dot = fmaf(qs[c0 + d + 1], k4.y, dot);
            dot = fmaf(qs[c0 + d + 2], k4.z, dot);
            dot = fmaf(qs[c0 + d + 3], k4.w, dot);
          }
        }
        __syncthreads();
      }
      if (live) s = dot * scale;
    } else if (live) {
      const elem_t* kr = cache_row(k_cache, table_row, p, page_size, n_kv_heads, kvh, head_dim);
      float dot = 0.0f;
      for (int d = 0; d < head_dim; d += 4) {   // head_dim is a multiple of 16
        float k4[4];
        load4_guarded(kr + d, 4, vec_k, k4);
#pragma unroll
        for (int i = 0; i < 4; ++i) dot = fmaf(qs[d + i], k4[i], dot);
      }
      s = dot * scale;
      vrow[wave][lane] =
          v_cache + ((size_t)table_row[p / page_size] * n_kv_heads + kvh) * head_dim * page_size + (p % page_size);
    }
    const float mb = wave_max(s);
    const float e = live ? expf(s - mb) : 0.0f;
    const float lb = wave_sum(e);
    es[wave][lane] = e;
    __syncthreads();
    float ob[DPL];
#pragma unroll
    for (int i = 0; i < DPL; ++i) ob[i] = 0.0f;
    const int first = max(lo - b0, 0), last = min(pos - b0, ATT_BLOCK - 1);
    if (staged) {
      // 8 positions at a time: lane l fetches four positions (the page size is a multiple of 4, so
      // they lie in one page) of dim (l + 64 i) / 2; a page that holds a live position is there whole
      for (int j0 = 0; j0 < ATT_BLOCK; j0 += ATT_VP) {
#pragma unroll
        for (int i = 0; i < ATT_MAX_HD * 2 / AXON_WAVE; ++i) {
          const int g = lane + AXON_WAVE * i, d = g >> 1, p4 = b0 + j0 + 4 * (g & 1);
          if (d >= head_dim || p4 > pos || p4 + 3 < lo) continue;
          const elem_t* src = v_cache + ((size_t)table_row[p4 / page_size] * n_kv_heads + kvh) * head_dim * page_size +
                              (size_t)d * page_size + (p4 % page_size);
          float v4[4];
          load4_guarded(src, 4, true, v4);
#pragma unroll
          for (int e = 0; e < 4; ++e) stage[d * (ATT_VP + 1) + 4 * (g & 1) + e] = v4[e];
        }
        __syncthreads();
        for (int j = max(first, j0); j <= min(last, j0 + ATT_VP - 1); ++j) {
          const float ej = es[wave][j];
#pragma unroll
          for (int i = 0; i < DPL; ++i) {
            const int d = lane + i * AXON_WAVE;
            if (d < head_dim) ob[i] = fmaf(ej, stage[d * (ATT_VP + 1) + j - j0], ob[i]);
          }
        }
        __syncthreads();
      }
    } else {
      for (int j = first; j <= last; ++j) {
        const float ej = es[wave][j];
        const elem_t* vr = vrow[wave][j];
#pragma unroll
        for (int i = 0; i < DPL; ++i) {
          const int d = lane + i * AXON_WAVE;
          if (d < head_dim) ob[i] = fmaf(ej, to_float(vr[(size_t)d * page_size]), ob[i]);
        }
      }
    }
    if (WAVES > 1) {
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        const int d = lane + i * AXON_WAVE;
        if (d < head_dim) part[wave][d] = ob[i];
      }
      if (lane == 0) {
        part[wave][ATT_MAX_HD] = mb;
        part[wave][ATT_MAX_HD + 1] = lb;
      }
    }
    __syncthreads();
    for (int w = 0; w < WAVES && g0 + ATT_BLOCK * w <= pos; ++w) {
      const float m_w = WAVES > 1 ? part[w][ATT_MAX_HD] : mb, l_w = WAVES > 1 ? part[w][ATT_MAX_HD + 1] : lb;
      const float mn = fmaxf(M, m_w);
      const float alpha = expf(M - mn);
      const float wgt = expf(m_w - mn);
      L = fmaf(l_w, wgt, L * alpha);
#pragma unroll
      for (int i = 0; i < DPL; ++i) {
        const int d = lane + i * AXON_WAVE;
        const float o_w = WAVES > 1 ? (d < head_dim ? part[w][d] : 0.0f) : ob[i];
        O[i] = fmaf(o_w, wgt, O[i] * alpha);
      }
      M = mn;
    }
    if (WAVES > 1) __syncthreads();   // the loop's next turn writes `part` again
  }

  if (wave != 0) return;
  elem_t* orow = out + ((size_t)t * n_heads + qh) * head_dim;
#pragma unroll
  for (int i = 0; i < DPL; ++i) {
    const int d = lane + i * AXON_WAVE;
    if (d < head_dim) orow[d] = from_float(O[i] / L);
  }
}

extern "C" int axk_attention(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                             const int32_t* block_table, int table_stride, const int32_t* positions,
                             const int32_t* seq_rows, void* out, int n_tokens, int n_heads, int n_kv_heads,
                             int head_dim, int page_size, int window, float scale, void* stream) {
  AXK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv_heads > 0 && page_size > 0,
              "attention: bad sizes T=%d nh=%d nkv=%d page=%d", n_tokens, n_heads, n_kv_heads, page_size);
  AXK_REQUIRE(n_heads % n_kv_heads == 0, "attention: %d query heads are not a multiple of %d kv heads", n_heads,
              n_kv_heads);
  AXK_REQUIRE(head_dim > 0 && head_dim % 16 == 0 && head_dim <= ATT_MAX_HD,
              "attention: head_dim %d is not a multiple of 16 up to %d", head_dim, ATT_MAX_HD);
  AXK_REQUIRE(n_heads <= 65535, "attention: %d heads (at most 65535)", n_heads);
  AXK_REQUIRE(window >= 0, "attention: window %d is negative", window);
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, n_heads);
  const bool vec_k = (uintptr_t)k_cache % (4 * sizeof(elem_t)) == 0;
  // keys and values through LDS in whole 16-byte (bfloat16: 8-byte) loads where the layout allows
  const bool staged = vec_k && page_size % 4 == 0 && (uintptr_t)v_cache % (4 * sizeof(elem_t)) == 0;
#define ROWS_LAUNCH(WAVES)                                                                                         \
  {                                                                                                                \
    constexpr int lds_bytes = WAVES * ATT_STAGE * (int)sizeof(float);                                              \
    auto kernel = &attention_rows_kernel<WAVES>;                                                                   \
    static bool configured = lds_bytes <= 48 * 1024;                                                               \
    if (!configured) {                                                                                             \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),                                    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);                   \
      if (e != hipSuccess) {                                                                                       \
        axk_set_error("attention_rows: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));      \
        return -2;                                                                                                 \
      }                                                                                                            \
      configured = true;                                                                                           \
    }                                                                                                              \
    AXK_INSTANCE(INST_ATTENTION_ROWS, AXON_BF16, WAVES);                                                           \
    kernel<<<grid, AXON_WAVE * WAVES, staged ? lds_bytes : 0, (hipStream_t)stream>>>(                              \
        (const elem_t*)q, q_stride, (const elem_t*)k_cache, (const elem_t*)v_cache, block_table, table_stride,    \
        positions, seq_rows, (elem_t*)out, n_heads, n_kv_heads, head_dim, page_size, window, scale, vec_k, staged); \
  }
  // few tokens x heads (a decoding step): eight waves each, so that the chip has waves to run
  if ((long)n_tokens * n_heads < 1024) ROWS_LAUNCH(8) else ROWS_LAUNCH(1)
#undef ROWS_LAUNCH
  AXK_LAUNCH_CHECK("attention_rows");
  return 0;
}
