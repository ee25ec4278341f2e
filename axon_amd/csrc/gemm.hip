// Matrix products out = X [M, K] . W [N, K]^T with a bias / residual epilogue.
//
// The rule every variant keeps: the K-reduction of one output element is one chain in
// ascending k that does not depend on M, on the tile shape or on what else is in the batch
// (the reference states the rule for its own kernels: src/cuda/decode.cu:352-369,
// src/cuda/prefill.cu:6-16).  Rows only ride along.
//
// gemm_fma: any M, N, K and strides, 32-bit FMA, one chain per output: the float32 build's
// product (true 32-bit), and the bfloat16 build's fallback for shapes the MFMA kernels refuse.
#include "api.h"
#include "common.h"
#include "instances.h"

#define FMA_BN 64
#define FMA_BK 16
#define FMA_THREADS 256

// BM rows x 64 columns per block of 256 threads; thread (ty, tx) owns RM = BM / 16 rows and
// 4 columns.  K is walked in steps of 16 through LDS; inside a step k ascends.
template <int BM, bool GLU>
__global__ void __launch_bounds__(FMA_THREADS)
gemm_fma_kernel(const elem_t* __restrict__ x, int x_stride, const elem_t* __restrict__ w, const void* __restrict__ bias,
                int bias_is_f32, void* __restrict__ out, int out_stride, int M, int N, int K, int mode, bool vec_x,
                bool vec_w) {
  constexpr int RM = BM / 16;
  __shared__ float xs[FMA_BK][BM + 4];
  __shared__ float ws[FMA_BK][FMA_BN + 4];
  __shared__ float us[GLU ? FMA_BK : 1][FMA_BN + 4];  // the up rows of the same columns (GLU: W holds 2 N rows)
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * FMA_BN;

  float acc[RM][4], acc_up[GLU ? RM : 1][4];
#pragma unroll
  for (int i = 0; i < RM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      acc[i][j] = 0.0f;
      if (GLU) acc_up[i][j] = 0.0f;
    }

  // loader: each thread brings 4 consecutive k of one row, a step ahead of the products
  const int lrow = tid >> 2, lk = (tid & 3) * 4;
  float pw[4], pu[4], px[4];
  auto fetch = [&](int k0) {
    const int n = n0 + lrow, m = m0 + lrow;
    const int left = max(0, min(4, K - (k0 + lk)));
    load4_guarded(w + (size_t)n * K + k0 + lk, n < N ? left : 0, vec_w, pw);
    if (GLU) load4_guarded(w + (size_t)(N + n) * K + k0 + lk, n < N ? left : 0, vec_w, pu);
    if (lrow < BM) load4_guarded(x + (size_t)m * x_stride + k0 + lk, m < M ? left : 0, vec_x, px);
  };
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += FMA_BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ws[lk + i][lrow] = pw[i];
      if (GLU) us[lk + i][lrow] = pu[i];
      if (lrow < BM) xs[lk + i][lrow] = px[i];
    }
    __syncthreads();
    if (k0 + FMA_BK < K) fetch(k0 + FMA_BK);
#pragma unroll
    for (int kk = 0; kk < FMA_BK; ++kk) {
      float a[RM], b[4];
#pragma unroll
      for (int i = 0; i < RM; ++i) a[i] = xs[kk][ty * RM + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < RM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
      if (GLU) {
#pragma unroll
        for (int j = 0; j < 4; ++j) b[j] = us[kk][tx * 4 + j];
#pragma unroll
        for (int i = 0; i < RM; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j) acc_up[i][j] = fmaf(a[i], b[j], acc_up[i][j]);
      }
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < RM; ++i) {
    const int m = m0 + ty * RM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += load_vec(bias, bias_is_f32, n);
      const size_t at = (size_t)m * out_stride + n;
      if (GLU) ((elem_t*)out)[at] = from_float(swiglu1(v, acc_up[i][j]));
      else if (mode == MODE_STORE) ((elem_t*)out)[at] = from_float(v);
      else if (mode == MODE_ADD_F32) ((float*)out)[at] += v;
      else ((float*)out)[at] = v;
    }
  }
}

// Up to 16 rows (a decoding step): 16 rows x 16 columns a block, one output a thread, K in steps
// of 256 through LDS, the next step's loads in flight while this one is multiplied.  Such a
// product only waits for W, so it wants many blocks with much in flight each (the tile above
// gives N / 64 blocks with 4 KB each).  The chain of an output is the same: fmaf in ascending k.
#define FEW_BK 256
#define FEW_LD (FEW_BK + 4)   // rows 4 banks apart: the 16 rows a wave reads fall into all 64 banks
template <bool GLU>
__global__ void __launch_bounds__(FMA_THREADS)
gemm_fma_few_rows_kernel(const elem_t* __restrict__ x, int x_stride, const elem_t* __restrict__ w,
                         const void* __restrict__ bias, int bias_is_f32, void* __restrict__ out, int out_stride, int M,
                         int N, int K, int mode, bool vec_x, bool vec_w) {
  __shared__ __align__(16) float xs[16][FEW_LD];
  __shared__ __align__(16) float ws[16][FEW_LD];
  __shared__ __align__(16) float us[GLU ? 16 : 1][GLU ? FEW_LD : 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int n0 = blockIdx.x * 16;

  // loader: a tile is 16 rows of 64 groups of four k; a thread brings groups tid + 256 j
  float px[4][4], pw[4][4], pu[GLU ? 4 : 1][4];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int g = tid + FMA_THREADS * j, row = g >> 6, k = k0 + 4 * (g & 63);
      const int left = max(0, min(4, K - k)), n = n0 + row;
      load4_guarded(x + (size_t)row * x_stride + k, row < M ? left : 0, vec_x, px[j]);
      load4_guarded(w + (size_t)n * K + k, n < N ? left : 0, vec_w, pw[j]);
      if (GLU) load4_guarded(w + (size_t)(N + n) * K + k, n < N ? left : 0, vec_w, pu[j]);
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int g = tid + FMA_THREADS * j, row = g >> 6, kk = 4 * (g & 63);
      *reinterpret_cast<float4*>(&xs[row][kk]) = make_float4(px[j][0], px[j][1], px[j][2], px[j][3]);
      *reinterpret_cast<float4*>(&ws[row][kk]) = make_float4(pw[j][0], pw[j][1], pw[j][2], pw[j][3]);
      if (GLU) *reinterpret_cast<float4*>(&us[row][kk]) = make_float4(pu[j][0], pu[j][1], pu[j][2], pu[j][3]);
    }
  };

  float acc = 0.0f, acc_up = 0.0f;
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += FEW_BK) {
    stage();
    __syncthreads();
    if (k0 + FEW_BK < K) fetch(k0 + FEW_BK);
    const int k_end = min(FEW_BK, K - k0);   // beyond K the last group of four holds zeros
#pragma unroll 4
    for (int kk = 0; kk < k_end; kk += 4) {
      const float4 a = *reinterpret_cast<const float4*>(&xs[ty][kk]);
      const float4 b = *reinterpret_cast<const float4*>(&ws[tx][kk]);
      acc = fmaf(a.x, b.x, acc);
      acc = fmaf(a.y, b.y, acc);
      acc = fmaf(a.z, b.z, acc);
      acc = fmaf(a.w, b.w, acc);
      if (GLU) {
        const float4 u = *reinterpret_cast<const float4*>(&us[tx][kk]);
        acc_up = fmaf(a.x, u.x, acc_up);
        acc_up = fmaf(a.y, u.y, acc_up);
        acc_up = fmaf(a.z, u.z, acc_up);
        acc_up = fmaf(a.w, u.w, acc_up);
      }
    }
    __syncthreads();
  }

  const int m = ty, n = n0 + tx;
  if (m >= M || n >= N) return;
  float v = acc;
  if (bias) v += load_vec(bias, bias_is_f32, n);
  const size_t at = (size_t)m * out_stride + n;
  if (GLU) ((elem_t*)out)[at] = from_float(swiglu1(v, acc_up));
  else if (mode == MODE_STORE) ((elem_t*)out)[at] = from_float(v);
  else if (mode == MODE_ADD_F32) ((float*)out)[at] += v;
  else ((float*)out)[at] = v;
}

static int launch_fma(const elem_t* x, int x_stride, const elem_t* w, const void* bias, int bias_is_f32, void* out,
                      int out_stride, int m, int n, int k, int mode, hipStream_t stream) {
  const size_t vbytes = 4 * sizeof(elem_t);
  const bool vec_w = (k % 4 == 0) && ((uintptr_t)w % vbytes == 0);
  const bool vec_x = (k % 4 == 0) && (x_stride % 4 == 0) && ((uintptr_t)x % vbytes == 0);
#define FMA_LAUNCH(BM, GLU)                                                                                      \
  AXK_INSTANCE(INST_GEMM_FMA, BM, GLU);                                                                          \
  if (BM == 16)                                                                                                  \
    gemm_fma_few_rows_kernel<GLU><<<dim3(ceil_div(n, 16)), FMA_THREADS, 0, stream>>>(                            \
        x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, vec_x, vec_w);                        \
  else                                                                                                           \
    gemm_fma_kernel<64, GLU><<<dim3(ceil_div(n, FMA_BN), ceil_div(m, 64)), FMA_THREADS, 0, stream>>>(            \
        x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, vec_x, vec_w)
  if (mode == MODE_SWIGLU) {
    if (m <= 16) { FMA_LAUNCH(16, true); } else { FMA_LAUNCH(64, true); }
  } else {
    if (m <= 16) { FMA_LAUNCH(16, false); } else { FMA_LAUNCH(64, false); }
  }
#undef FMA_LAUNCH
  AXK_LAUNCH_CHECK("gemm_fma");
  return 0;
}

#if AXON_BF16
int launch_gemm_mfma(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                     int out_stride, int m, int n, int k, int mode, hipStream_t stream, const GemmNormFold* then_norm,
                     void* workspace, size_t workspace_bytes);
int gemm_pack_ok(int rows, int k, int gated);
int launch_pack_matrix(const bf16_t* src, bf16_t* dst, int rows, int k, hipStream_t stream);
size_t gemm_workspace_bytes(int m, int n, int k, int mode);
int gemm_segments(int tiles32, int k);
int gemm_then_norm_ok(int m, int n, int k);
int gemm_qkv_rope_ok(int m, int n, int k, int head_dim, int rotary_dim);
int launch_gemm_qkv_rope(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, bf16_t* out,
                         int out_stride, int m, int n, int k, const float* table, const int32_t* positions,
                         const int32_t* seq_rows, const int32_t* block_table, int table_stride, bf16_t* k_cache,
                         bf16_t* v_cache, int n_heads, int n_kv_heads, int head_dim, int page_size, void* workspace,
                         size_t workspace_bytes, hipStream_t stream);
int gemm_normed_ok(int m, int k);
int launch_gemm_normed_glu(const float* rows, int rows_stride, const bf16_t* gain, float eps, const bf16_t* w, bf16_t* out,
                           int out_stride, int m, int n, int k, hipStream_t stream);
int launch_gemm_normed_qkv_rope(const float* rows, int rows_stride, const bf16_t* gain, float eps,
                                const bf16_t* w, const void* bias, int bias_is_f32, bf16_t* out, int out_stride, int m, int n,
                                int k, const float* table, const int32_t* positions, const int32_t* seq_rows,
                                const int32_t* block_table, int table_stride, bf16_t* k_cache, bf16_t* v_cache, int n_heads,
                                int n_kv_heads, int head_dim, int page_size, hipStream_t stream);
#endif

static int gemm_checked(const void* x, int x_stride, const void* w, int w_packed, const void* bias, int bias_is_f32,
                        void* out, int out_stride, int m, int n, int k, int mode, const GemmNormFold* fold,
                        void* workspace, long workspace_bytes, void* stream) {
  AXK_REQUIRE(m >= 0 && n > 0 && k > 0, "gemm: bad sizes M=%d N=%d K=%d", m, n, k);
  AXK_REQUIRE(x_stride >= k && out_stride >= n, "gemm: strides x=%d (K=%d) out=%d (N=%d) too small", x_stride, k,
              out_stride, n);
  AXK_REQUIRE(mode >= 0 && mode <= 3, "gemm: unknown mode %d", mode);
  AXK_REQUIRE(mode != MODE_SWIGLU || bias == nullptr, "gemm: the gated epilogue takes no bias");
  AXK_REQUIRE(ceil_div(m, 16) <= 65535, "gemm: M=%d is more rows than one launch takes", m);
  if (m == 0) return 0;
  if (w_packed) {
#if AXON_BF16
    return launch_gemm_mfma((const bf16_t*)x, x_stride, (const bf16_t*)w, bias, bias_is_f32, out, out_stride, m, n, k, mode,
                            (hipStream_t)stream, fold, workspace, workspace_bytes > 0 ? (size_t)workspace_bytes : 0);
#else
    axk_set_error("gemm: packed matrices exist only in the bfloat16 build");
    return -1;
#endif
  }
  AXK_REQUIRE(fold == nullptr, "gemm: a norm follows only products with a packed matrix");
  return launch_fma((const elem_t*)x, x_stride, (const elem_t*)w, bias, bias_is_f32, out, out_stride, m, n, k, mode,
                    (hipStream_t)stream);
}

extern "C" long axk_gemm_workspace(int m, int n, int k, int mode) {
#if AXON_BF16
  return m > 0 && n > 0 && k > 0 ? (long)gemm_workspace_bytes(m, n, k, mode) : 0;
#else
  return 0;
#endif
}

extern "C" int axk_gemm(const void* x, int x_stride, const void* w, int w_packed, const void* bias, int bias_is_f32,
                        void* out, int out_stride, int m, int n, int k, int mode, void* workspace, long workspace_bytes,
                        void* stream) {
  return gemm_checked(x, x_stride, w, w_packed, bias, bias_is_f32, out, out_stride, m, n, k, mode, nullptr, workspace,
                      workspace_bytes, stream);
}

extern "C" int axk_pack_ok(int rows, int k, int gated) {
#if AXON_BF16
  return gemm_pack_ok(rows, k, gated);
#else
  return 0;   // the 32-bit build multiplies row-major matrices
#endif
}

extern "C" long axk_packed_elems(int rows, int k) { return (long)((rows + 15) / 16 * 16) * k; }

extern "C" int axk_pack_matrix(const void* src, void* dst, int rows, int k, void* stream) {
#if AXON_BF16
  AXK_REQUIRE(gemm_pack_ok(rows, k, 0), "pack_matrix: [%d, %d] cannot be packed", rows, k);
  AXK_REQUIRE(((uintptr_t)src & 15) == 0 && ((uintptr_t)dst & 15) == 0, "pack_matrix: operands must be 16-byte aligned");
  return launch_pack_matrix((const bf16_t*)src, (bf16_t*)dst, rows, k, (hipStream_t)stream);
#else
  axk_set_error("pack_matrix: only in the bfloat16 build");
  return -1;
#endif
}

// Segments K is cut into for a packed [n, k] matrix (gated: n is the width of the output, the
// matrix holds 2 n rows): the order of addition of every product with it.  1 where nothing is packed.
extern "C" int axk_gemm_segments(int n, int k, int gated) {
#if AXON_BF16
  if (n <= 0 || k <= 0 || !gemm_pack_ok(gated ? 2 * n : n, k, gated)) return 1;
  return gemm_segments(gated ? n / 16 : (n + 31) / 32, k);
#else
  return 1;
#endif
}

extern "C" int axk_gemm_then_norm_ok(int m, int n, int k) {
#if AXON_BF16
  return m > 0 && n > 0 && k > 0 && gemm_then_norm_ok(m, n, k);
#else
  return 0;   // the 32-bit build keeps the norm a pass of its own
#endif
}

extern "C" int axk_gemm_then_norm(const void* x, int x_stride, const void* w, const void* bias, int bias_is_f32,
                                  float* out, int out_stride, int m, int n, int k, const void* norm_gain,
                                  int norm_gain_is_f32, float norm_eps, void* norm_values, void* workspace,
                                  long workspace_bytes, void* stream) {
  AXK_REQUIRE(axk_gemm_then_norm_ok(m, n, k), "gemm: M=%d N=%d K=%d does not run with K split: the norm stays apart", m,
              n, k);
  AXK_REQUIRE(norm_gain && norm_values, "gemm: the norm behind the product needs its gain and its output");
  AXK_REQUIRE(out_stride % 4 == 0 && ((uintptr_t)out & 15) == 0 && ((uintptr_t)norm_values & 7) == 0,
              "gemm: the rows to add into must be 16-byte aligned (stride %d) and the norm's output 8-byte aligned",
              out_stride);
  const GemmNormFold fold = {norm_gain, norm_gain_is_f32, norm_values, norm_eps};
  return gemm_checked(x, x_stride, w, 1, bias, bias_is_f32, out, out_stride, m, n, k, MODE_ADD_F32, &fold, workspace,
                      workspace_bytes, stream);
}

extern "C" int axk_gemm_qkv_rope_ok(int m, int n, int k, int head_dim, int rotary_dim) {
#if AXON_BF16
  return n > 0 && k > 0 && head_dim > 0 && gemm_qkv_rope_ok(m, n, k, head_dim, rotary_dim);
#else
  return 0;   // the 32-bit build keeps the product, the rotation and the store apart
#endif
}

extern "C" int axk_gemm_qkv_rope(const void* x, int x_stride, const void* w, const void* bias, int bias_is_f32,
                                 void* qkv, int qkv_stride, int m, int k, const float* table, const int32_t* positions, const int32_t* seq_rows,
                                 const int32_t* block_table, int table_stride, void* k_cache, void* v_cache,
                                 int n_heads, int n_kv_heads, int head_dim, int page_size, int write_kv, void* workspace,
                                 long workspace_bytes, void* stream) {
#if AXON_BF16
  AXK_REQUIRE(n_heads > 0 && n_kv_heads > 0 && page_size > 0 && head_dim > 0, "gemm_qkv_rope: heads %d/%d of %d, page %d",
              n_heads, n_kv_heads, head_dim, page_size);
  const int n = (n_heads + (write_kv ? 2 * n_kv_heads : 0)) * head_dim;
  AXK_REQUIRE(axk_gemm_qkv_rope_ok(m, n, k, head_dim, head_dim), "gemm_qkv_rope: M=%d N=%d K=%d head_dim=%d are not taken",
              m, n, k, head_dim);
  AXK_REQUIRE(x_stride >= k && x_stride % 8 == 0 && qkv_stride >= n_heads * head_dim && qkv_stride % 4 == 0 &&
                  ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0 && ((uintptr_t)qkv & 7) == 0 &&
                  ((uintptr_t)table & 15) == 0,
              "gemm_qkv_rope: strides x=%d qkv=%d or the alignment of an operand are not taken", x_stride, qkv_stride);
  AXK_REQUIRE(table && positions && (!write_kv || (seq_rows && block_table && k_cache && v_cache)),
              "gemm_qkv_rope: a table, the positions or the cache is missing");
  return launch_gemm_qkv_rope((const bf16_t*)x, x_stride, (const bf16_t*)w, bias, bias_is_f32, (bf16_t*)qkv, qkv_stride,
                              m, n, k, table, positions, seq_rows, block_table, table_stride,
                              (bf16_t*)k_cache, (bf16_t*)v_cache, n_heads, n_kv_heads, head_dim, page_size, workspace,
                              workspace_bytes > 0 ? (size_t)workspace_bytes : 0, (hipStream_t)stream);
#else
  axk_set_error("gemm_qkv_rope: only in the bfloat16 build");
  return -1;
#endif
}

// ---------------------------------------------------------------------------- the norm inside the product
// Few rows (a decoding step): the gated product and the [q; k; v] product read the float32 rows
// themselves and apply the RMS norm on the way (the norm kernel's arithmetic, the same bits), so
// the norm is no launch of its own.  `ok` depends on the sizes alone.
extern "C" int axk_gemm_normed_ok(int m, int n, int k, int gated) {
#if AXON_BF16
  if (m <= 0 || n <= 0 || k <= 0 || !gemm_pack_ok(gated ? 2 * n : n, k, gated)) return 0;
  return gemm_normed_ok(m, k);
#else
  return 0;   // the 32-bit build keeps the norm a pass of its own
#endif
}

extern "C" int axk_gemm_normed_glu(const float* rows, int rows_stride, const void* gain, int gain_is_f32, float eps,
                                   const void* w, void* out, int out_stride, int m, int n, int k, void* stream) {
#if AXON_BF16
  AXK_REQUIRE(axk_gemm_normed_ok(m, n, k, 1), "gemm_normed_glu: M=%d N=%d K=%d are not taken", m, n, k);
  AXK_REQUIRE(!gain_is_f32, "gemm_normed_glu: the gain must be bfloat16");
  AXK_REQUIRE(rows && gain && w && out, "gemm_normed_glu: an operand is missing");
  AXK_REQUIRE(rows_stride >= k && rows_stride % 4 == 0 && out_stride >= n && ((uintptr_t)rows & 15) == 0 &&
                  ((uintptr_t)gain & 15) == 0 && ((uintptr_t)w & 15) == 0,
              "gemm_normed_glu: strides rows=%d out=%d or the alignment of an operand are not taken", rows_stride, out_stride);
  return launch_gemm_normed_glu(rows, rows_stride, (const bf16_t*)gain, eps, (const bf16_t*)w, (bf16_t*)out, out_stride, m, n,
                                k, (hipStream_t)stream);
#else
  axk_set_error("gemm_normed_glu: only in the bfloat16 build");
  return -1;
#endif
}

extern "C" int axk_gemm_normed_qkv_rope(const float* rows, int rows_stride, const void* gain, int gain_is_f32, float eps,
                                        const void* w, const void* bias, int bias_is_f32, void* qkv, int qkv_stride, int m,
                                        int k, const float* table, const int32_t* positions, const int32_t* seq_rows,
                                        const int32_t* block_table, int table_stride, void* k_cache, void* v_cache,
                                        int n_heads, int n_kv_heads, int head_dim, int page_size, int write_kv, void* stream) {
#if AXON_BF16
  AXK_REQUIRE(n_heads > 0 && n_kv_heads > 0 && page_size > 0 && head_dim > 0,
              "gemm_normed_qkv_rope: heads %d/%d of %d, page %d", n_heads, n_kv_heads, head_dim, page_size);
  const int n = (n_heads + (write_kv ? 2 * n_kv_heads : 0)) * head_dim;
  AXK_REQUIRE(axk_gemm_normed_ok(m, n, k, 0) && axk_gemm_qkv_rope_ok(m, n, k, head_dim, head_dim),
              "gemm_normed_qkv_rope: M=%d N=%d K=%d head_dim=%d are not taken", m, n, k, head_dim);
  AXK_REQUIRE(rows && gain && w && qkv, "gemm_normed_qkv_rope: an operand is missing");
  AXK_REQUIRE(!gain_is_f32, "gemm_normed_qkv_rope: the gain must be bfloat16");
  AXK_REQUIRE(rows_stride >= k && rows_stride % 4 == 0 && qkv_stride >= n_heads * head_dim && qkv_stride % 4 == 0 &&
                  ((uintptr_t)rows & 15) == 0 && ((uintptr_t)gain & 15) == 0 && ((uintptr_t)w & 15) == 0 &&
                  ((uintptr_t)qkv & 7) == 0 && ((uintptr_t)table & 15) == 0,
              "gemm_normed_qkv_rope: strides rows=%d qkv=%d or the alignment of an operand are not taken", rows_stride,
              qkv_stride);
  AXK_REQUIRE(table && positions && (!write_kv || (seq_rows && block_table && k_cache && v_cache)),
              "gemm_normed_qkv_rope: a table, the positions or the cache is missing");
  return launch_gemm_normed_qkv_rope(rows, rows_stride, (const bf16_t*)gain, eps, (const bf16_t*)w, bias, bias_is_f32,
                                     (bf16_t*)qkv, qkv_stride, m, n, k, table, positions, seq_rows, block_table, table_stride,
                                     (bf16_t*)k_cache, (bf16_t*)v_cache, n_heads, n_kv_heads, head_dim, page_size,
                                     (hipStream_t)stream);
#else
  axk_set_error("gemm_normed_qkv_rope: only in the bfloat16 build");
  return -1;
#endif
}
