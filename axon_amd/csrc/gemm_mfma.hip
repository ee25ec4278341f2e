// bfloat16 matrix products on the matrix cores: out = X [M, K] . W [N, K]^T, 32-bit accumulation.
// Only in the bfloat16 build.
//
// W is PACKED (axk_pack_matrix, once, when the weights are loaded): blocks of 16 rows x 32 k, each
// 1 KB in the order in which a wave holds them as an MFMA operand (lane l: row l % 16, the 8
// consecutive k from 8 (l / 16)); blocks ordered [row tile][k block]; rows padded to a multiple
// of 16 with zeros.  A wave instruction then reads 1 KB of consecutive memory (measured: 10 to 35 %
// more bandwidth than 16 rows x 64 bytes of a row-major matrix), lands in LDS without a
// permutation, and the same bytes serve the 16x16x32 and the 32x32x16 MFMA.
//
// Two kernels, chosen by the number of rows M alone, so that a given (N, K) always meets the same
// kernel and the same grouping of k for a given class of M:
//
// * gemm_skinny (M <= 16, decoding): bound by reading W once.  A block owns one or two row tiles
//   of W; its four waves split K between them and stream their share from memory straight into
//   MFMA operands (16x16x32), keeping a ring of steps in flight so that the memory pipe never
//   drains; each multiplies with up to 16 rows of X, and the waves' sums are added in wave
//   order through LDS.  No atomics, so the result does not depend on timing.  Epilogues: bias /
//   residual add / SwiGLU, an RMS norm folded in on either side, and the attention's qkv product
//   with the rotary encoding and the store into the paged cache.
//
// * gemm_tile (M > 16): a block of 4 or 8 waves owns a BM x BN tile of the output, walks K in
//   steps of 64 through LDS stages filled by direct global -> LDS loads (the next step's loads
//   in flight while this one multiplies), and each wave keeps a tile of 32x32x16 MFMA
//   accumulators.  X rows land in LDS with their 16-byte slots permuted so that fragment reads
//   of neighbouring rows fall into different banks; W blocks land as they are.  Blocks are
//   numbered so that the blocks of one XCD (every eighth block) share weight tiles in that
//   XCD's L2.  Tiles: 64 x 128 / 64 x 256 for 17 to 64 rows, 128 x 128 for 65 to 256, and 256 x 256
//   or 128 x 128 beyond, by how they fill the chip.  Where the output gives too few tiles for
//   256 CUs, K is split between blocks (by (N, K) alone within a class of M), the blocks' sums go
//   through a workspace and gemm_split_reduce adds them in block order and applies the epilogue.
//
// Classes of M: <= 16, 17..64, 65..256, 257..2048, > 2048.  Within a class a row's bits do not
// depend on the other rows of the batch; between classes they differ by the rounding of 32-bit
// sums (and only by that).
#include "api.h"
#include "common.h"

#if AXON_BF16

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ inline bf16x8 as_frag(uint4 v) {
  union { uint4 u; bf16x8 f; } c;
  c.u = v;
  return c.f;
}

typedef const __attribute__((address_space(1))) void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

__device__ inline bf16x8 as_frag(u32x4 v) { return __builtin_bit_cast(bf16x8, v); }

// ---------------------------------------------------------------------------- gemm_tile
// LDS holds STAGES stages; a stage is BM rows of X and the BN / 16 x BK / 32 packed blocks of W,
// written by direct global -> LDS loads of 16 bytes per lane (a wave instruction fills 1024
// bytes: 8 rows of X, or one block of W).  Every stage is filled before the loop, and the loads
// of step kt + STAGES go out as soon as step kt's stage is free, so the latency of L2 and of
// the path into LDS is covered by STAGES - 1 steps of MFMAs.
//
// A row of X in a stage is BK / 8 slots of 16 bytes, permuted so that fragment reads of
// neighbouring rows at one k chunk fall into different banks without padding (which direct
// loads could not skip).  LDS serves 256 bytes a cycle (64 banks): a 16-byte read of 16 consecutive lanes
// (16 consecutive rows, the same k chunk) is conflict-free when the rows' 16-byte positions
// modulo 256 differ.  With 128-byte rows (BK 64) that is slot = chunk ^ ((row >> 1) & 7); with
// 64-byte rows (BK 32) slot = chunk ^ ((row >> 2) & 3).
//
// GLU: W holds 2 N rows (gate rows, then up rows) and the output is silu(gate) * up, N wide.
// A block then owns BN / 2 output columns; each wave's share of the LDS tile holds the gate
// rows of its columns and, after them, the up rows of the same columns, so that a lane ends
// with both values of an output element.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool GLU, int BK, int STAGES>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_tile_kernel(const bf16_t* __restrict__ x, int x_stride, const bf16_t* __restrict__ w, const void* __restrict__ bias,
                 int bias_is_f32, void* __restrict__ out, int out_stride, int M, int N, int K, int mode, int m_blocks,
                 int n_blocks, float* __restrict__ partial) {
  extern __shared__ __align__(16) unsigned char smem[];
  static_assert(BK == 32 || BK == 64, "K steps of 32 or 64");
  constexpr int NW = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;  // a wave's tile
  constexpr int TM = WM / 32, TN = WN / 32;            // in 32 x 32 MFMA tiles
  constexpr int ROW = BK * 2;                          // bytes of a row
  constexpr int SLOTS = BK / 8;                        // 16-byte slots of a row
  constexpr int RPI = 1024 / ROW;                      // rows one wave instruction fills
  constexpr int KBT = BK / 32;                         // packed k blocks of a K tile
  constexpr int XQ = BM / RPI / NW, WQ = BN / 16 * KBT / NW;  // load instructions per wave and stage
  constexpr int STAGE = (BM + BN) * ROW;               // bytes per stage
  static_assert(XQ >= 1 && WQ >= 1 && (STAGES - 2) * (XQ + WQ) < 64, "tile too small or too many loads in flight");
  static_assert(BN / 16 * KBT % NW == 0 && WN % 32 == 0, "the 1 KB chunks of W are shared out evenly");
  static_assert(!GLU || TN % 2 == 0, "a wave's gate columns and up columns are whole MFMA tiles");
#define SWZ(row) (BK == 64 ? (((row) >> 1) & 7) : (((row) >> 2) & 3))

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;

  // Block numbering: every eighth block runs on the same XCD; give one XCD consecutive m
  // blocks of the same n block, so a weight tile is fetched into one L2 and reused there.
  const int bid = blockIdx.x;
  int mb, nb;
  if (bid < (n_blocks / 8) * 8 * m_blocks) {
    const int xcd = bid & 7, j = bid >> 3;
    nb = (j / m_blocks) * 8 + xcd;
    mb = j % m_blocks;
  } else {  // the last, incomplete group of n blocks: plain order
    const int r = bid - (n_blocks / 8) * 8 * m_blocks;
    nb = (n_blocks / 8) * 8 + r / m_blocks;
    mb = r % m_blocks;
  }
  const int m0 = mb * BM, n0 = nb * (GLU ? BN / 2 : BN);

  // what this lane fetches: row r = (q * NW + wave) * RPI + lane / SLOTS of a tile; it fills slot
  // lane % SLOTS of that row, which holds k chunk (lane % SLOTS) ^ SWZ(r)
  const int lrow = lane / SLOTS, lslot = lane % SLOTS;
  unsigned xoff[XQ], woff[WQ];
#pragma unroll
  for (int q = 0; q < XQ; ++q) {
    const int r = (q * NW + wave) * RPI + lrow;
    xoff[q] = (unsigned)min(m0 + r, M - 1) * (unsigned)x_stride + (lslot ^ SWZ(r)) * 8;
  }
  // W: chunk c = q * NW + wave of a stage is the packed block (row tile c / KBT, k block c % KBT)
  // of the tile, 1 KB as it lies in memory.  Row tiles past the matrix: its last one (the
  // epilogue drops those columns).
  const int KB = K / 32;
  const int row_tiles = GLU ? N / 16 : (N + 15) / 16;          // GLU: per half, N a multiple of 16
#pragma unroll
  for (int q = 0; q < WQ; ++q) {
    const int c = q * NW + wave;
    const int r = (c / KBT) * 16;                               // first row of the chunk in the LDS tile
    int tile;
    if (GLU) {
      const int owner = r / WN, within = r % WN;                // the wave whose columns these are
      const int col = n0 + owner * (WN / 2) + within % (WN / 2);
      tile = (within >= WN / 2 ? row_tiles : 0) + min(col / 16, row_tiles - 1);   // up rows follow the N gate rows
    } else {
      tile = min((n0 + r) / 16, row_tiles - 1);
    }
    woff[q] = ((unsigned)tile * (unsigned)KB + (c % KBT)) * 512 + lane * 8;
  }

  // Split K (gridDim.y > 1): this block multiplies the K tiles kt_begin .. kt_begin + nk - 1 and
  // leaves its sums in `partial`; gemm_split_reduce_kernel adds the blocks' sums in block order.
  const int kt_begin = (int)((long)blockIdx.y * (K / BK) / gridDim.y);
  const int nk = (int)((long)(blockIdx.y + 1) * (K / BK) / gridDim.y) - kt_begin;
  auto issue = [&](int kt) {     // kt counts from kt_begin
    unsigned char* stage = smem + (kt % STAGES) * STAGE;
    const int koff = (kt_begin + kt) * BK;
#pragma unroll
    for (int q = 0; q < XQ; ++q)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(x + xoff[q] + koff), (lds_ptr_t)(stage + (q * NW + wave) * 1024), 16,
                                       0, 0);
#pragma unroll
    for (int q = 0; q < WQ; ++q)
      __builtin_amdgcn_global_load_lds((global_ptr_t)(w + woff[q] + (kt_begin + kt) * (KBT * 512)),
                                       (lds_ptr_t)(stage + BM * ROW + (q * NW + wave) * 1024), 16, 0, 0);
  };

  f32x16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.0f;

  // fragment addresses: row = tile row + lane % 32, k chunk = 2 ks + lane / 32, slot = chunk ^ SWZ(row)
  const int frow = lane & 31, fhalf = lane >> 5, fsw = SWZ(frow);
  const unsigned lds0 = (unsigned)(size_t)(lds_ptr_t)smem;
  const unsigned xbase = lds0 + (wm * WM + frow) * ROW;
  // W fragment of k step ks: block (row tile of the lane's row, k block ks / 2), lane slot
  // 16 (2 (ks % 2) + lane / 32) + row % 16 of it: no permutation, 16 lanes read 256 consecutive bytes
  const unsigned wbase = lds0 + BM * ROW + ((wn * WN + frow) / 16) * KBT * 1024 + (fhalf * 16 + (frow & 15)) * 16;
  // The fragments of k step ks of a stage into one of two register sets.  The reads are written
  // as instructions: the compiler, which cannot tell the stage being read from the stage a
  // direct load is filling, would wait for every load in flight before each of its own reads,
  // and the loads of the next tile would never overlap the products of this one.
  u32x4 a[2][TM], b[2][TN];
  auto read_step = [&](int set, int stage_index, int ks) {
    read_frags<TM, 32 * ROW>(a[set], xbase + stage_index * STAGE + ((((ks * 2 + fhalf) ^ fsw)) << 4));
    read_frags<TN, 2 * KBT * 1024>(b[set], wbase + stage_index * STAGE + (ks / 2) * 1024 + (ks % 2) * 512);
  };
  auto multiply = [&](int set, int j_from, int j_to) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = j_from; j < j_to; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(a[set][i]), as_frag(b[set][j]), acc[i][j], 0, 0, 0);
  };

  // Every stage is filled before the loop; tile kt + STAGES is fetched into tile kt's stage as
  // soon as every wave has read that tile's last fragments, which is during its last k step:
  // the wait for the next tile, the barrier and the first reads of the next tile are hidden
  // behind that step's products (half of them before the barrier, half after the reads).
  constexpr int KS = BK / 16;
  static_assert(KS % 2 == 0, "the register sets alternate and start a tile at set 0");
#pragma unroll
  for (int d = 0; d < STAGES; ++d)
    if (d < nk) issue(d);
  if (nk >= STAGES) wait_vmcnt<(STAGES - 1) * (XQ + WQ)>();
  else wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();   // tile 0 is in LDS for every wave
  read_step(0, 0, 0);
  for (int kt = 0; kt < nk; ++kt) {
    const int stage_index = kt % STAGES;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < KS) {
        read_step(nxt, stage_index, ks + 1);
        wait_lgkmcnt<TM + TN>();          // this step's fragments (reads return in order)
        use_frags<TM>(a[cur]);
        use_frags<TN>(b[cur]);
        multiply(cur, 0, TN);
      } else {
        wait_lgkmcnt<0>();                // the last fragments of this tile: its stage is free
        use_frags<TM>(a[cur]);
        use_frags<TN>(b[cur]);
        multiply(cur, 0, TN / 2);
        if (kt + 1 < nk) {
          // this wave's part of tile kt + 1 has landed when only younger tiles are outstanding
          if (kt + STAGES < nk) wait_vmcnt<(STAGES - 2) * (XQ + WQ)>();
          else wait_vmcnt<0>();
          __builtin_amdgcn_s_barrier();   // tile kt + 1 is in LDS for every wave; nobody reads tile kt any more
          if (kt + STAGES < nk) issue(kt + STAGES);
          read_step(nxt, (kt + 1) % STAGES, 0);
        }
        multiply(cur, TN / 2, TN);
      }
    }
  }
#undef SWZ

  // epilogue: lane holds column n = lane % 32 of each tile and rows (e/4)*8 + (lane/32)*4 + e%4
  if (partial) {
    // [split][gate | up][M][N] (one part without GLU), 32-bit sums as they are
    constexpr int PARTS = GLU ? 2 : 1;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int part = GLU ? j / (TN / 2) : 0;
      const int n = GLU ? n0 + wn * (WN / 2) + (j % (TN / 2)) * 32 + (lane & 31) : n0 + wn * WN + j * 32 + (lane & 31);
      if (n >= N) continue;
      float* dst = partial + ((size_t)blockIdx.y * PARTS + part) * M * N + n;
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = m0 + wm * WM + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
          if (m < M) dst[(size_t)m * N] = acc[i][j][e];
        }
    }
    return;
  }
  if (GLU) {
#pragma unroll
    for (int j = 0; j < TN / 2; ++j) {
      const int n = n0 + wn * (WN / 2) + j * 32 + (lane & 31);
      if (n >= N) continue;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int m = m0 + wm * WM + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
          if (m >= M) continue;
          reinterpret_cast<bf16_t*>(out)[(size_t)m * out_stride + n] =
              float_to_bf16(swiglu1(acc[i][j][e], acc[i][j + TN / 2][e]));
        }
      }
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int n = n0 + wn * WN + j * 32 + (lane & 31);
    if (n >= N) continue;
    const float bv = bias ? load_vec(bias, bias_is_f32, n) : 0.0f;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int m = m0 + wm * WM + i * 32 + (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3);
        if (m >= M) continue;
        const float v = acc[i][j][e] + bv;
        const size_t at = (size_t)m * out_stride + n;
        if (mode == MODE_STORE) reinterpret_cast<bf16_t*>(out)[at] = float_to_bf16(v);
        else if (mode == MODE_ADD_F32) reinterpret_cast<float*>(out)[at] += v;
        else reinterpret_cast<float*>(out)[at] = v;
      }
    }
  }
}

// The sums of the split-K blocks, added in block order, then the epilogue of the product.
// One thread per 4 consecutive columns of a row (N is a multiple of 4 on this path).
__global__ void __launch_bounds__(256)
gemm_split_reduce_kernel(const float* __restrict__ partial, int splits, int M, int N, const void* __restrict__ bias,
                         int bias_is_f32, void* __restrict__ out, int out_stride, int mode) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  const int n4 = N / 4;
  if (idx >= M * n4) return;
  const int m = idx / n4, n = (idx % n4) * 4;
  const size_t plane = (size_t)M * N, at_in = (size_t)m * N + n;
  const int parts = mode == MODE_SWIGLU ? 2 : 1;
  // the blocks' sums in block order; four loads under way at a time
  auto summed = [&](const float* src, size_t step) {
    float4 g = *reinterpret_cast<const float4*>(src);
    int z = 1;
    for (; z + 3 < splits; z += 4) {
      const float4 a0 = *reinterpret_cast<const float4*>(src + (size_t)z * step);
      const float4 a1 = *reinterpret_cast<const float4*>(src + (size_t)(z + 1) * step);
      const float4 a2 = *reinterpret_cast<const float4*>(src + (size_t)(z + 2) * step);
      const float4 a3 = *reinterpret_cast<const float4*>(src + (size_t)(z + 3) * step);
      g.x += a0.x; g.y += a0.y; g.z += a0.z; g.w += a0.w;
      g.x += a1.x; g.y += a1.y; g.z += a1.z; g.w += a1.w;
      g.x += a2.x; g.y += a2.y; g.z += a2.z; g.w += a2.w;
      g.x += a3.x; g.y += a3.y; g.z += a3.z; g.w += a3.w;
    }
    for (; z < splits; ++z) {
      const float4 a = *reinterpret_cast<const float4*>(src + (size_t)z * step);
      g.x += a.x; g.y += a.y; g.z += a.z; g.w += a.w;
    }
    return g;
  };
  const float4 g = summed(partial + at_in, (size_t)parts * plane);
  const float4 u = parts == 2 ? summed(partial + plane + at_in, (size_t)parts * plane) : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
  float v[4] = {g.x, g.y, g.z, g.w};
  const size_t at = (size_t)m * out_stride + n;
  if (mode == MODE_SWIGLU) {
    const float uu[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) reinterpret_cast<bf16_t*>(out)[at + e] = float_to_bf16(swiglu1(v[e], uu[e]));
    return;
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (bias) v[e] += load_vec(bias, bias_is_f32, n + e);
    if (mode == MODE_STORE) reinterpret_cast<bf16_t*>(out)[at + e] = float_to_bf16(v[e]);
    else if (mode == MODE_ADD_F32) reinterpret_cast<float*>(out)[at + e] += v[e];
    else reinterpret_cast<float*>(out)[at + e] = v[e];
  }
}

// An RMS norm of the rows right after a split product that adds into them (the residual
// stream): the split-K sums, the bias and the addition as in gemm_split_reduce_kernel, then the
// norm of the new row, values = out * (1 / sqrt(mean(out^2) + eps)) * gain, in the same launch.
// A block of 1024 threads per row, a thread per 4 columns (and 4 more in a row wider than 4096):
// every load of the sums is independent of the others.  The new row goes through LDS to the
// first 256 threads, which add up its squares in the order of the norm's own kernel (thread t:
// the float4 t, t + 256, ...; then the lanes of a wave; then the four waves), so both ways give
// the same bits.
struct SplitNorm {
  const void* gain;
  int gain_is_f32;
  float eps;
  bf16_t* values;      // [M, N]
};

#define SRN_THREADS 1024
#define SRN_MAX_N 8192

__global__ void __launch_bounds__(SRN_THREADS)
gemm_split_reduce_norm_kernel(const float* __restrict__ partial, int splits, int M, int N, const void* __restrict__ bias,
                              int bias_is_f32, float* __restrict__ out, int out_stride, SplitNorm norm) {
  __shared__ float4 row[SRN_MAX_N / 4];
  __shared__ float sums[4];
  const int m = blockIdx.x, n4 = N / 4, tid = threadIdx.x;
  const size_t plane = (size_t)M * N;
  auto added = [&](int i) {
    const int n = i * 4;
    const float* src = partial + (size_t)m * N + n;
    float4 g = *reinterpret_cast<const float4*>(src);
    int z = 1;
    for (; z + 3 < splits; z += 4) {           // four loads under way at a time; added in block order
      const float4 a0 = *reinterpret_cast<const float4*>(src + (size_t)z * plane);
      const float4 a1 = *reinterpret_cast<const float4*>(src + (size_t)(z + 1) * plane);
      const float4 a2 = *reinterpret_cast<const float4*>(src + (size_t)(z + 2) * plane);
      const float4 a3 = *reinterpret_cast<const float4*>(src + (size_t)(z + 3) * plane);
      g.x += a0.x; g.y += a0.y; g.z += a0.z; g.w += a0.w;
      g.x += a1.x; g.y += a1.y; g.z += a1.z; g.w += a1.w;
      g.x += a2.x; g.y += a2.y; g.z += a2.z; g.w += a2.w;
      g.x += a3.x; g.y += a3.y; g.z += a3.z; g.w += a3.w;
    }
    for (; z < splits; ++z) {
      const float4 a = *reinterpret_cast<const float4*>(src + (size_t)z * plane);
      g.x += a.x; g.y += a.y; g.z += a.z; g.w += a.w;
    }
    if (bias) {
      g.x += load_vec(bias, bias_is_f32, n);
      g.y += load_vec(bias, bias_is_f32, n + 1);
      g.z += load_vec(bias, bias_is_f32, n + 2);
      g.w += load_vec(bias, bias_is_f32, n + 3);
    }
    float4* dst = reinterpret_cast<float4*>(out + (size_t)m * out_stride + n);
    float4 r = *dst;
    r.x += g.x; r.y += g.y; r.z += g.z; r.w += g.w;
    *dst = r;
    return r;
  };
  constexpr int MINE = SRN_MAX_N / 4 / SRN_THREADS;
  float4 mine[MINE];
#pragma unroll
  for (int c = 0; c < MINE; ++c) {
    const int i = tid + c * SRN_THREADS;
    if (i < n4) {
      mine[c] = added(i);
      row[i] = mine[c];
    }
  }
  __syncthreads();
  if (tid < 256) {
    float ss = 0.0f;
    for (int i = tid; i < n4; i += 256) {
      const float4 v = row[i];
      ss = fmaf(v.x, v.x, ss);
      ss = fmaf(v.y, v.y, ss);
      ss = fmaf(v.z, v.z, ss);
      ss = fmaf(v.w, v.w, ss);
    }
    ss = wave_sum(ss);
    if ((tid & (AXON_WAVE - 1)) == 0) sums[tid / AXON_WAVE] = ss;
  }
  __syncthreads();
  const float total = ((sums[0] + sums[1]) + sums[2]) + sums[3];
  const float inv = 1.0f / sqrtf(total / (float)N + norm.eps);
  bf16_t* dst = norm.values + (size_t)m * N;
#pragma unroll
  for (int c = 0; c < MINE; ++c) {
    const int i = tid + c * SRN_THREADS;
    if (i < n4) {
      const int e = i * 4;
      const float4 v = mine[c];
      uint2 pk;
      pk.x = pack2_bf16((v.x * inv) * load_vec(norm.gain, norm.gain_is_f32, e),
                        (v.y * inv) * load_vec(norm.gain, norm.gain_is_f32, e + 1));
      pk.y = pack2_bf16((v.z * inv) * load_vec(norm.gain, norm.gain_is_f32, e + 2),
                        (v.w * inv) * load_vec(norm.gain, norm.gain_is_f32, e + 3));
      *reinterpret_cast<uint2*>(dst + e) = pk;
    }
  }
}

struct RopeStore;
static int launch_split_reduce_rope(const float* partial, int splits, int m, int n, const void* bias, int bias_is_f32,
                                    void* out, int out_stride, const RopeStore& rope, hipStream_t stream);

template <int BM, int BN, int WAVES_M, int WAVES_N, bool GLU, int BK = 64, int STAGES = 2>
static int launch_tile(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                       int out_stride, int m, int n, int k, int mode, hipStream_t stream, int splits = 1,
                       float* partial = nullptr, const SplitNorm* norm = nullptr, const RopeStore* rope = nullptr) {
  static bool configured = false;
  constexpr int lds_bytes = STAGES * (BM + BN) * BK * 2;
  static_assert(lds_bytes <= 160 * 1024, "the stages do not fit the LDS of a CU");
  auto kernel = &gemm_tile_kernel<BM, BN, WAVES_M, WAVES_N, GLU, BK, STAGES>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       lds_bytes);
    if (e != hipSuccess) {
      axk_set_error("gemm_tile: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
      return -2;
    }
    configured = true;
  }
  const int m_blocks = ceil_div(m, BM), n_blocks = ceil_div(n, GLU ? BN / 2 : BN);
  kernel<<<dim3(m_blocks * n_blocks, splits), WAVES_M * WAVES_N * 64, lds_bytes, stream>>>(
      x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, m_blocks, n_blocks, splits > 1 ? partial : nullptr);
  AXK_LAUNCH_CHECK("gemm_tile");
  if (splits > 1 && rope != nullptr) return launch_split_reduce_rope(partial, splits, m, n, bias, bias_is_f32, out, out_stride, *rope, stream);
  if (splits > 1 && norm != nullptr) {
    gemm_split_reduce_norm_kernel<<<m, SRN_THREADS, 0, stream>>>(partial, splits, m, n, bias, bias_is_f32, (float*)out, out_stride,
                                                         *norm);
    AXK_LAUNCH_CHECK("gemm_split_reduce_norm");
  } else if (splits > 1) {
    gemm_split_reduce_kernel<<<ceil_div(m * (n / 4), 256), 256, 0, stream>>>(partial, splits, m, n, bias, bias_is_f32, out,
                                                                            out_stride, mode);
    AXK_LAUNCH_CHECK("gemm_split_reduce");
  }
  return 0;
}

// ---------------------------------------------------------------------------- gemm_skinny
// A block of WAVES waves owns NT16 row tiles (of 16) of W; wave v takes the k steps (of 64) v,
// v + WAVES, ...  C[n][m] tiles of 16 x 16: the MFMA's A operand is W (a packed block as it lies
// in memory), its B operand X (lane: row m = lane % 16, 8 consecutive k from (lane / 16) * 8).
// A lane ends with 4 consecutive n of one m: one vector store.
// GLU (NT16 = 2): the block's two tiles are the gate rows n0 .. n0 + 15 and the up rows of the
// same columns (W holds 2 N rows), and the output is silu(gate) * up.
//
// An RMS norm can be folded into the product on either side, which saves the norm's own pass
// over the rows (a launch each, between products that take microseconds):
// * in_squares: X holds x * gain, not yet scaled by its row's 1/rms, and in_squares [M, K / 16]
//   the sums of x^2 over the 16-column parts of each row.  Every block adds a row's parts (in
//   the same order, so all blocks agree) and multiplies the finished sums of products by
//   1/sqrt(sum / K + eps): the scale is common to the row, so it commutes with the product.
// * norm_gain (with the add-into-residual epilogue): beside out += result the block writes what
//   the next product's in_squares side takes: norm_values = out * norm_gain in bfloat16 and
//   norm_squares [M, ceil(N / 16)], the sums of out^2 over each tile's 16 columns.
struct NormFold {
  const float* in_squares;
  float in_eps;
  const void* norm_gain;
  int norm_gain_is_f32;
  bf16_t* norm_values;
  float* norm_squares;
};

// The product of the attention's fused [q; k; v] matrix with the rotary position encoding and the
// store into the paged cache as its epilogue (EPI_ROPE, NT16 = 2): W's rows are heads of
// head_dim; a block owns dims d0 .. d0 + 15 of one head and their rotation partners d0 + half ..,
// so that a lane ends with both values of a pair.  q heads go rotated to `out`, k heads rotated
// into the request's page of keys, v heads as they are into its page of values (kept
// position-contiguous, [dim][slot]).  The arithmetic is that of the rotary kernel after a
// plain product: the sums are rounded to bfloat16 first, and each product and sum of the
// rotation is rounded on its own.
struct RopeStore {
  const float* table;            // [M, half, 2]: sin, cos of each token's angles
  const int32_t* positions;      // [M]
  const int32_t* seq_rows;       // [M]: the row of the block table
  const int32_t* block_table;
  int table_stride;
  bf16_t* k_cache;
  bf16_t* v_cache;
  int n_heads, n_kv_heads, head_dim, page_size;
};

enum { EPI_PLAIN = 0, EPI_GLU = 1, EPI_ROPE = 2 };

// The sums of a split [q; k; v] product with the bias, the rotary encoding and the store into the
// pages: what gemm_split_reduce_kernel (storing bfloat16) and the rotary kernel do one after the
// other, bit for bit.  One wave per (token, head slot), four waves a block; q heads go rotated to
// `out`, k heads rotated into the request's page of keys, v heads as they are into its page of
// values.  Every head is rotated over its whole width.
__global__ void __launch_bounds__(256)
gemm_split_reduce_rope_kernel(const float* __restrict__ partial, int splits, int M, int N, const void* __restrict__ bias,
                              int bias_is_f32, bf16_t* __restrict__ out, int out_stride, RopeStore rope) {
  const int m = blockIdx.x, slot = blockIdx.y * 4 + threadIdx.x / AXON_WAVE, lane = threadIdx.x % AXON_WAVE;
  const int hd = rope.head_dim, half = hd / 2;
  if (slot * hd >= N) return;
  const size_t plane = (size_t)M * N;
  // a column's sum, rounded as the product's own store rounds it
  auto value = [&](int col) {
    const float* src = partial + (size_t)m * N + col;
    float g = src[0];
    for (int z = 1; z < splits; ++z) g += src[(size_t)z * plane];
    if (bias) g += load_vec(bias, bias_is_f32, col);
    return bf16_to_float(float_to_bf16(g));
  };
  bf16_t* dst;
  if (slot < rope.n_heads) {
    dst = out + (size_t)m * out_stride + (size_t)slot * hd;
  } else {
    const int pos = rope.positions[m];
    const int page = rope.block_table[(size_t)rope.seq_rows[m] * rope.table_stride + pos / rope.page_size];
    const int in_page = pos % rope.page_size;
    if (slot >= rope.n_heads + rope.n_kv_heads) {
      const int kvh = slot - rope.n_heads - rope.n_kv_heads;
      bf16_t* vdst = rope.v_cache + ((size_t)page * rope.n_kv_heads + kvh) * hd * rope.page_size + in_page;
      for (int i = lane; i < hd; i += AXON_WAVE) vdst[(size_t)i * rope.page_size] = float_to_bf16(value(slot * hd + i));
      return;
    }
    dst = rope.k_cache + (((size_t)page * rope.n_kv_heads + (slot - rope.n_heads)) * rope.page_size + in_page) * hd;
  }
  const float* tab = rope.table + (size_t)m * half * 2;
  for (int i = lane; i < half; i += AXON_WAVE) {
    const float sn = tab[2 * i], cs = tab[2 * i + 1];
    const float a = value(slot * hd + i), b = value(slot * hd + i + half);
    dst[i] = float_to_bf16(__fsub_rn(__fmul_rn(a, cs), __fmul_rn(b, sn)));
    dst[i + half] = float_to_bf16(__fadd_rn(__fmul_rn(a, sn), __fmul_rn(b, cs)));
  }
}

static int launch_split_reduce_rope(const float* partial, int splits, int m, int n, const void* bias, int bias_is_f32,
                                    void* out, int out_stride, const RopeStore& rope, hipStream_t stream) {
  const dim3 grid(m, ceil_div(n / rope.head_dim, 4));
  gemm_split_reduce_rope_kernel<<<grid, 256, 0, stream>>>(partial, splits, m, n, bias, bias_is_f32, (bf16_t*)out, out_stride,
                                                          rope);
  AXK_LAUNCH_CHECK("gemm_split_reduce_rope");
  return 0;
}

template <int NT16, int MT16, int WAVES, int DEPTH, int EPI>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_kernel(const bf16_t* __restrict__ x, int x_stride, const bf16_t* __restrict__ w,
                   const void* __restrict__ bias, int bias_is_f32, void* __restrict__ out, int out_stride, int M, int N,
                   int K, int mode, NormFold fold, RopeStore rope) {
  constexpr bool GLU = EPI == EPI_GLU, ROPE = EPI == EPI_ROPE;
  static_assert(EPI == EPI_PLAIN || NT16 == 2, "the paired epilogues own two tiles of W rows");
  __shared__ float partial[WAVES][NT16 * MT16][64][4];
  __shared__ float row_scale[MT16 * 16];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * (GLU ? 16 : NT16 * 16);
  const int r16 = lane & 15, kq = (lane >> 4) * 8;

  // the packed blocks of this block's row tiles: [row tile][k block of 32][lane][8]
  const int KB = K / 32;
  const bf16_t* wtile[NT16];
#pragma unroll
  for (int i = 0; i < NT16; ++i) {
    int tile;
    if (GLU) tile = i * (N / 16) + blockIdx.x;                 // gate rows, then the up rows of the same columns
    else if (ROPE) {
      const int half = rope.head_dim / 2, per_head = half / 16;
      tile = ((blockIdx.x / per_head) * rope.head_dim + i * half) / 16 + blockIdx.x % per_head;
    } else tile = min(n0 / 16 + i, (N + 15) / 16 - 1);         // past the matrix: its last tile (columns dropped below)
    wtile[i] = w + (size_t)tile * KB * 512 + lane * 8;
  }
  const bf16_t* xrow[MT16];
#pragma unroll
  for (int j = 0; j < MT16; ++j) xrow[j] = x + (size_t)min(j * 16 + r16, M - 1) * x_stride + kq;

  f32x4 acc[NT16][MT16];
#pragma unroll
  for (int i = 0; i < NT16; ++i)
#pragma unroll
    for (int j = 0; j < MT16; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  // This wave's steps (64 k each): wave, wave + WAVES, ...  A ring of DEPTH steps is kept in
  // flight: a step is multiplied as soon as ITS loads have landed (loads return in order), and
  // its place in the ring is refilled at once, so the memory pipe never drains.
  const int steps = K / 64;
  const int mine = steps > wave ? (steps - wave + WAVES - 1) / WAVES : 0;
  uint4 wf[DEPTH][NT16][2], xf[DEPTH][MT16][2];
  auto load = [&](int slot, int local) {
    const int k0 = (wave + local * WAVES) * 64;
#pragma unroll
    for (int i = 0; i < NT16; ++i) {
      wf[slot][i][0] = *reinterpret_cast<const uint4*>(wtile[i] + k0 * 16);          // k block k0 / 32: 512 elements each
      wf[slot][i][1] = *reinterpret_cast<const uint4*>(wtile[i] + k0 * 16 + 512);
    }
#pragma unroll
    for (int j = 0; j < MT16; ++j) {
      xf[slot][j][0] = *reinterpret_cast<const uint4*>(xrow[j] + k0);
      xf[slot][j][1] = *reinterpret_cast<const uint4*>(xrow[j] + k0 + 32);
    }
  };
  auto multiply = [&](int slot) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int i = 0; i < NT16; ++i)
#pragma unroll
        for (int j = 0; j < MT16; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(wf[slot][i][h]), as_frag(xf[slot][j][h]), acc[i][j],
                                                              0, 0, 0);
  };

  // The rows' scales.  Wave v takes rows v, v + WAVES, ...; a lane adds every 64th part, then the
  // lanes' sums are added.  Up to 256 parts (K <= 4096): one 16-byte load a lane and row, issued before the ring's,
  // so they return first (loads return in order) and are added up while the ring's first loads
  // are under way, and nothing between here and the main loop waits for the ring.  A wider K
  // is added up in a loop, before the ring starts.
  constexpr bool FOLDS = MT16 == 1;     // steps of up to 16 rows (see gemm_norm_fold_ok)
  constexpr int RW = FOLDS ? 16 / WAVES : 1;
  float4 sq[RW];
  const int parts = K / 16;             // a multiple of 4, as K is one of 64
  const bool fold_in = FOLDS && fold.in_squares != nullptr;
  const bool few_parts = parts <= 256;
  if (fold_in) {
    if (few_parts) {
#pragma unroll
      for (int i = 0; i < RW; ++i) {
        const int m = wave + i * WAVES;
        sq[i] = m < M && lane * 4 < parts ? *reinterpret_cast<const float4*>(fold.in_squares + (size_t)m * parts + lane * 4)
                                          : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
      }
    } else {
      for (int m = wave; m < M; m += WAVES) {
        float sum = 0.0f;
        for (int part = lane; part < parts; part += 64) sum += fold.in_squares[(size_t)m * parts + part];
        const float total = wave_sum_to_last(sum);
        if (lane == 63) row_scale[m] = 1.0f / sqrtf(total / (float)K + fold.in_eps);
      }
    }
  }
  if (mine > 0) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) load(d, min(d, mine - 1));   // beyond this wave's steps: a valid step again
  }
  if (fold_in && few_parts) {
#pragma unroll
    for (int i = 0; i < RW; ++i) {
      const float total = wave_sum_to_last((sq[i].x + sq[i].y) + (sq[i].z + sq[i].w));
      if (lane == 63) row_scale[wave + i * WAVES] = 1.0f / sqrtf(total / (float)K + fold.in_eps);
    }
  }
  if (mine > 0) {
    int base = 0;  // the ring holds local steps base .. base + DEPTH - 1
    for (; base + 2 * DEPTH <= mine; base += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        multiply(d);
        load(d, base + DEPTH + d);
      }
    }
    // the tail: what the ring holds, refilled only where a step is left, then those
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (base + d < mine) multiply(d);
      if (base + DEPTH + d < mine) load(d, base + DEPTH + d);
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (base + DEPTH + d < mine) multiply(d);
  }

#pragma unroll
  for (int i = 0; i < NT16; ++i)
#pragma unroll
    for (int j = 0; j < MT16; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) partial[wave][i * MT16 + j][lane][e] = acc[i][j][e];
  __syncthreads();

  if (ROPE) {
    const int hd = rope.head_dim, half = hd / 2, per_head = half / 16;
    const int slot = blockIdx.x / per_head;                  // q heads, then k heads, then v heads
    const int d = (blockIdx.x % per_head) * 16 + (lane >> 4) * 4;
    for (int j = wave; j < MT16; j += WAVES) {
      const int m = j * 16 + r16;
      if (m >= M) continue;
      const float scale = fold.in_squares ? row_scale[m] : 1.0f;
      float a[4], b[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float lo = partial[0][j][lane][e], hi = partial[0][MT16 + j][lane][e];
#pragma unroll
        for (int q = 1; q < WAVES; ++q) {
          lo += partial[q][j][lane][e];
          hi += partial[q][MT16 + j][lane][e];
        }
        if (fold.in_squares) {
          lo *= scale;
          hi *= scale;
        }
        if (bias) {
          lo += load_vec(bias, bias_is_f32, slot * hd + d + e);
          hi += load_vec(bias, bias_is_f32, slot * hd + half + d + e);
        }
        a[e] = bf16_to_float(float_to_bf16(lo));
        b[e] = bf16_to_float(float_to_bf16(hi));
      }
      bf16_t* dst;
      if (slot < rope.n_heads) {
        dst = reinterpret_cast<bf16_t*>(out) + (size_t)m * out_stride + (size_t)slot * hd;
      } else {
        const int pos = rope.positions[m];
        const int page = rope.block_table[(size_t)rope.seq_rows[m] * rope.table_stride + pos / rope.page_size];
        const int in_page = pos % rope.page_size;
        if (slot >= rope.n_heads + rope.n_kv_heads) {
          const int kvh = slot - rope.n_heads - rope.n_kv_heads;
          bf16_t* vdst = rope.v_cache + ((size_t)page * rope.n_kv_heads + kvh) * hd * rope.page_size + in_page;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            vdst[(size_t)(d + e) * rope.page_size] = float_to_bf16(a[e]);
            vdst[(size_t)(half + d + e) * rope.page_size] = float_to_bf16(b[e]);
          }
          continue;
        }
        const int kvh = slot - rope.n_heads;
        dst = rope.k_cache + (((size_t)page * rope.n_kv_heads + kvh) * rope.page_size + in_page) * hd;
      }
      const float4* tab = reinterpret_cast<const float4*>(rope.table + ((size_t)m * half + d) * 2);
      const float4 t0 = tab[0], t1 = tab[1];
      const float sn[4] = {t0.x, t0.z, t1.x, t1.z}, cs[4] = {t0.y, t0.w, t1.y, t1.w};
      float lo[4], hi[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo[e] = __fsub_rn(__fmul_rn(a[e], cs[e]), __fmul_rn(b[e], sn[e]));
        hi[e] = __fadd_rn(__fmul_rn(a[e], sn[e]), __fmul_rn(b[e], cs[e]));
      }
      uint2 pk;
      pk.x = pack2_bf16(lo[0], lo[1]);
      pk.y = pack2_bf16(lo[2], lo[3]);
      *reinterpret_cast<uint2*>(dst + d) = pk;
      pk.x = pack2_bf16(hi[0], hi[1]);
      pk.y = pack2_bf16(hi[2], hi[3]);
      *reinterpret_cast<uint2*>(dst + half + d) = pk;
    }
    return;
  }
  if (GLU) {
    // a wave takes both tiles of a column block: gate (tile j) and up (tile MT16 + j)
    for (int j = wave; j < MT16; j += WAVES) {
      const int m = j * 16 + r16;
      const int n = n0 + (lane >> 4) * 4;
      if (m >= M) continue;
      const float scale = fold.in_squares ? row_scale[m] : 1.0f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (n + e >= N) continue;
        float g = partial[0][j][lane][e], u = partial[0][MT16 + j][lane][e];
#pragma unroll
        for (int q = 1; q < WAVES; ++q) {
          g += partial[q][j][lane][e];
          u += partial[q][MT16 + j][lane][e];
        }
        if (fold.in_squares) {
          g *= scale;
          u *= scale;
        }
        reinterpret_cast<bf16_t*>(out)[(size_t)m * out_stride + n + e] = float_to_bf16(swiglu1(g, u));
      }
    }
    return;
  }
  // tiles are shared out between the waves; each sums the partials in wave order
  for (int t = wave; t < NT16 * MT16; t += WAVES) {
    const int i = t / MT16, j = t % MT16;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float sum = partial[0][t][lane][e];
#pragma unroll
      for (int q = 1; q < WAVES; ++q) sum += partial[q][t][lane][e];
      v[e] = sum;
    }
    const int m = j * 16 + r16;
    const int n = n0 + i * 16 + (lane >> 4) * 4;
    const bool row_ok = m < M;
    const float scale = fold.in_squares && row_ok ? row_scale[m] : 1.0f;
    float squares = 0.0f;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (!row_ok || n + e >= N) continue;
      float r = v[e];
      if (fold.in_squares) r *= scale;
      if (bias) r += load_vec(bias, bias_is_f32, n + e);
      const size_t at = (size_t)m * out_stride + n + e;
      if (mode == MODE_STORE) reinterpret_cast<bf16_t*>(out)[at] = float_to_bf16(r);
      else if (mode == MODE_ADD_F32) {
        const float sum = reinterpret_cast<float*>(out)[at] + r;
        reinterpret_cast<float*>(out)[at] = sum;
        if (fold.norm_gain) {
          fold.norm_values[(size_t)m * N + n + e] = float_to_bf16(sum * load_vec(fold.norm_gain, fold.norm_gain_is_f32, n + e));
          squares = fmaf(sum, sum, squares);
        }
      } else reinterpret_cast<float*>(out)[at] = r;
    }
    if (fold.norm_gain) {
      // the four lanes that hold a row's 16 columns of this tile: lane, lane ^ 16, lane ^ 32, lane ^ 48
      squares += __shfl_xor(squares, 16, AXON_WAVE);
      squares += __shfl_xor(squares, 32, AXON_WAVE);
      if (row_ok && lane < 16 && n0 + i * 16 < N) fold.norm_squares[(size_t)m * ((N + 15) >> 4) + (n0 >> 4) + i] = squares;
    }
  }
}

template <int NT16, int MT16, int WAVES, int DEPTH, int EPI = EPI_PLAIN>
static int launch_skinny(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                         int out_stride, int m, int n, int k, int mode, hipStream_t stream, const NormFold& fold,
                         const RopeStore& rope = RopeStore()) {
  gemm_skinny_kernel<NT16, MT16, WAVES, DEPTH, EPI><<<ceil_div(n, EPI == EPI_GLU ? 16 : NT16 * 16), WAVES * 64, 0, stream>>>(
      x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, fold, rope);
  AXK_LAUNCH_CHECK("gemm_skinny");
  return 0;
}

// Shapes the MFMA kernels take: K a multiple of 64 and 16-byte aligned rows.  Decided by (N, K)
// and the pointers' alignment, never by M, so a weight matrix always meets the same kernels.
// What can be packed: K in whole steps of 64, offsets inside the kernels in 32 bits, and for a
// [gate; up] matrix halves that are whole row tiles.
int gemm_pack_ok(int rows, int k, int gated) {
  if (rows <= 0 || k <= 0 || k % 64 != 0) return 0;
  if ((size_t)((rows + 15) / 16 * 16) * k >= (1ull << 32)) return 0;
  return !gated || (rows % 32 == 0);
}

// One thread per 16 bytes of the packed matrix: lane slot (row % 16) + 16 ((k % 32) / 8) of block
// (row / 16, k / 32).  Rows past the matrix are zeros.
__global__ void __launch_bounds__(256)
pack_matrix_kernel(const bf16_t* __restrict__ src, bf16_t* __restrict__ dst, int rows, int K) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;     // 16-byte slot of the packed matrix
  const int KB = K / 32;
  const size_t block = idx / 64;
  const int lane = (int)(idx % 64);
  const int tile = (int)(block / KB), kb = (int)(block % KB);
  if (tile >= (rows + 15) / 16) return;
  const int row = tile * 16 + (lane & 15), k = kb * 32 + (lane >> 4) * 8;
  uint4 v = uint4{0, 0, 0, 0};
  if (row < rows) v = *reinterpret_cast<const uint4*>(src + (size_t)row * K + k);
  *reinterpret_cast<uint4*>(dst + idx * 8) = v;
}

int launch_pack_matrix(const bf16_t* src, bf16_t* dst, int rows, int k, hipStream_t stream) {
  const size_t slots = (size_t)((rows + 15) / 16) * (k / 32) * 64;
  pack_matrix_kernel<<<(unsigned)((slots + 255) / 256), 256, 0, stream>>>(src, dst, rows, k);
  AXK_LAUNCH_CHECK("pack_matrix");
  return 0;
}

static bool skinny_takes(int m, int n, int k, int mode) { return m <= 16; }

// 17 to 64 rows: one tile of rows (gemm_tile with a 64-row block), K split between blocks so
// that the chip is full although the output is small; the blocks' sums go through a workspace
// and are added in block order.  The number of splits depends on (N, K) alone: a row's bits do
// not depend on how many rows ride along.
static int mid_splits(int n, int k, int mode) {
  if (n % 4 != 0) return 1;
  const int per_block = mode == MODE_SWIGLU ? 128 : (n >= 8192 ? 256 : 128);
  const int n_blocks = ceil_div(n, per_block), nk = k / 64;
  // a block a CU for the narrow tile, two for the wide one (measured); at least four K tiles a block
  int s = (per_block == 128 && mode != MODE_SWIGLU ? 256 : 512) / n_blocks;
  if (s > nk / 4) s = nk / 4;
  if (s > 32) s = 32;
  return s < 1 ? 1 : s;
}

// 65 to 256 rows: one or two rows of 128 x 128 tiles, which leave most CUs idle when N is small;
// K is split so that about a block a CU runs.  Again by (N, K) alone.
static int small_splits(int n, int k, int mode) {
  if (n % 4 != 0) return 1;
  const int n_blocks = ceil_div(n, mode == MODE_SWIGLU ? 64 : 128), nk = k / 64;
  int s = 256 / (2 * n_blocks);
  if (s > nk / 4) s = nk / 4;
  if (s > 16) s = 16;
  return s < 1 ? 1 : s;
}

// 257 to 2048 rows: a narrow output gives too few 256 x 256 tiles for 256 CUs, or a number of
// them that leaves the last round mostly idle; K is then cut into 2 to 4 parts.  By (N, K)
// alone (the tiles are counted for 2,048 rows).  The time of the product is the rounds of blocks
// over the parts; adding the parts' sums costs about 500 / K of the product's ideal time a
// part (twice that for [gate; up]).  A cut has to win 8 % and leave 24 K tiles a part.
static int long_k_splits(int n, int k, int mode) {
  if (n % 4 != 0) return 1;
  const bool glu = mode == MODE_SWIGLU;
  const int tiles = 8 * ceil_div(n, glu ? 128 : 256), nk = k / 64;
  int best = 1;
  double best_cost = (double)ceil_div(tiles, 256);
  for (int s = 2; s <= 4; ++s) {
    if (nk / s < 24) break;
    const double cost = (double)ceil_div(tiles * s, 256) / s + 500.0 * s / k * (tiles / 256.0) * (glu ? 2 : 1);
    if (cost < 0.92 * best_cost) {
      best = s;
      best_cost = cost;
    }
  }
  return best;
}

static int splits_of(int m, int n, int k, int mode) {
  if (m <= 16 || m > 2048) return 1;
  return m <= 64 ? mid_splits(n, k, mode) : m <= 256 ? small_splits(n, k, mode) : long_k_splits(n, k, mode);
}

size_t gemm_workspace_bytes(int m, int n, int k, int mode) {
  if (k % 64 != 0) return 0;
  const int s = splits_of(m, n, k, mode);
  return s > 1 ? (size_t)s * (mode == MODE_SWIGLU ? 2 : 1) * m * n * sizeof(float) : 0;
}

int gemm_norm_fold_ok(int m, int n, int k, int mode) {
  return gemm_pack_ok(mode == MODE_SWIGLU ? 2 * n : n, k, mode == MODE_SWIGLU) && skinny_takes(m, n, k, mode);
}

// Whether the product that adds into the rows runs with K split between blocks, so that the
// kernel that adds the blocks' sums can also norm the finished rows (gemm_split_reduce_norm_kernel:
// rows of up to SRN_MAX_N columns).
int gemm_then_norm_ok(int m, int n, int k) {
  return gemm_pack_ok(n, k, 0) && !skinny_takes(m, n, k, MODE_ADD_F32) && splits_of(m, n, k, MODE_ADD_F32) > 1 &&
         n <= SRN_MAX_N;
}

static int gemm_mfma_dispatch(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                              int out_stride, int m, int n, int k, int mode, hipStream_t stream,
                              const GemmNormFold* fold_in, void* workspace, size_t workspace_bytes,
                              const RopeStore* rope_after) {
  if (!gemm_pack_ok(mode == MODE_SWIGLU ? 2 * n : n, k, mode == MODE_SWIGLU)) {
    axk_set_error("gemm: N=%d K=%d is no shape of a packed matrix", n, k);
    return -1;
  }
  if (x_stride % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)w & 15) || (size_t)m * x_stride >= (1ull << 32)) {
    axk_set_error("gemm: with a packed matrix the rows of X must be 16-byte aligned and X below 2^32 elements "
                  "(stride %d, M=%d)", x_stride, m);
    return -1;
  }
  NormFold fold = {nullptr, 0.0f, nullptr, 0, nullptr, nullptr};
  if (fold_in) {
    fold.in_squares = fold_in->in_squares;
    fold.in_eps = fold_in->in_eps;
    fold.norm_gain = fold_in->norm_gain;
    fold.norm_gain_is_f32 = fold_in->norm_gain_is_f32;
    fold.norm_values = (bf16_t*)fold_in->norm_values;
    fold.norm_squares = fold_in->norm_squares;
  }
#define ARGS x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream
  if (skinny_takes(m, n, k, mode)) {
    if (mode == MODE_SWIGLU) return launch_skinny<2, 1, 4, 8, EPI_GLU>(ARGS, fold);
    // 32 rows of W per block where that still leaves 128 blocks or more, else 16; four waves
    // split K; the ring is as deep as the registers allow
    return n >= 32 * 128 ? launch_skinny<2, 1, 4, 8>(ARGS, fold) : launch_skinny<1, 1, 4, 8>(ARGS, fold);
  }
  // the tiled kernels: no norm on the way in; on the way out only a whole norm behind split sums
  SplitNorm after = {nullptr, 0, 0.0f, nullptr};
  const SplitNorm* norm = nullptr;
  if (fold_in) {
    const bool whole = fold_in->in_squares == nullptr && fold_in->norm_gain && fold_in->norm_values && !fold_in->norm_squares;
    if (!whole || mode != MODE_ADD_F32 || !gemm_then_norm_ok(m, n, k)) {
      axk_set_error("gemm: M=%d N=%d K=%d mode %d goes to the tiled kernel, which folds no such norm", m, n, k, mode);
      return -1;
    }
    after = SplitNorm{fold_in->norm_gain, fold_in->norm_gain_is_f32, fold_in->norm_eps, (bf16_t*)fold_in->norm_values};
    norm = &after;
  }
  const int splits = splits_of(m, n, k, mode);
  if (rope_after && (splits < 2 || mode != MODE_STORE)) {
    axk_set_error("gemm: M=%d N=%d K=%d does not run with K split: the rotary kernel stays apart", m, n, k);
    return -1;
  }
  const size_t need = gemm_workspace_bytes(m, n, k, mode);
  if (need > workspace_bytes || (need > 0 && (workspace == nullptr || ((uintptr_t)workspace & 15)))) {
    axk_set_error("gemm: M=%d N=%d K=%d needs a workspace of %zu bytes, 16-byte aligned (got %zu)", m, n, k, need,
                  workspace_bytes);
    return -1;
  }
  float* ws = (float*)workspace;
  if (m <= 256) {
    if (m > 64) {
      if (mode == MODE_SWIGLU) return launch_tile<128, 128, 2, 2, true>(ARGS, splits, ws);
      return launch_tile<128, 128, 2, 2, false>(ARGS, splits, ws, norm, rope_after);
    }
    if (mode == MODE_SWIGLU) return launch_tile<64, 256, 1, 4, true, 64, 2>(ARGS, splits, ws);
    if (n >= 8192) return launch_tile<64, 256, 1, 4, false, 64, 2>(ARGS, splits, ws, norm, rope_after);
    return launch_tile<64, 128, 1, 4, false, 64, 3>(ARGS, splits, ws, norm, rope_after);
  }
  // 256 x 256 tiles (8 waves) where they fill the chip: one round of at least 140 blocks (on 256
  // CUs), or several rounds of which the last is not mostly idle; else 128 x 128 tiles, four times
  // as many blocks at twice the traffic from L2 per product.  Thresholds are measured ones.
  const int n_per_block = mode == MODE_SWIGLU ? 128 : 256;
  const long big = (long)ceil_div(m, 256) * ceil_div(n, n_per_block) * splits;
  const long rounds = (big + 255) / 256;
  const bool use_big = big <= 256 ? big >= 140 : big * 10 >= rounds * 256 * 7;
  if (mode == MODE_SWIGLU) {
    if (use_big) return launch_tile<256, 256, 4, 2, true>(ARGS, splits, ws);
    return launch_tile<128, 128, 2, 2, true>(ARGS, splits, ws);
  }
  // one round of 256 x 256 tiles that leaves a quarter of the CUs idle, and N in whole tiles of
  // 192 columns that still fit one round: the narrower tile (measured 1.1 times the cost per
  // product, three quarters of the products per block).  The k order of a sum is the same.
  if (use_big && splits == 1 && big <= 192 && n % 192 == 0 && (long)ceil_div(m, 256) * (n / 192) <= 256)
    return launch_tile<256, 192, 4, 2, false>(ARGS, splits, ws, norm);
  if (use_big) return launch_tile<256, 256, 4, 2, false>(ARGS, splits, ws, norm, rope_after);
  return launch_tile<128, 128, 2, 2, false>(ARGS, splits, ws, norm, rope_after);
#undef ARGS
}

int launch_gemm_mfma(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                     int out_stride, int m, int n, int k, int mode, hipStream_t stream, const GemmNormFold* fold_in,
                     void* workspace, size_t workspace_bytes) {
  return gemm_mfma_dispatch(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream, fold_in, workspace,
                            workspace_bytes, nullptr);
}

// The [q; k; v] product with rotary encoding and cache store (see RopeStore): up to 16 rows in
// the epilogue of gemm_skinny, more rows where the product splits K (then the kernel that adds
// the parts' sums rotates and stores); every head rotated over its whole width, halves of a head
// a multiple of 16 wide.
int gemm_qkv_rope_ok(int m, int n, int k, int head_dim, int rotary_dim) {
  if (m < 1 || k % 64 != 0 || rotary_dim != head_dim || head_dim % 32 != 0 || n % head_dim != 0) return 0;
  if (m <= 16) return 1;
  return gemm_pack_ok(n, k, 0) && n % 4 == 0 && splits_of(m, n, k, MODE_STORE) > 1;
}

int launch_gemm_qkv_rope(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, bf16_t* out,
                         int out_stride, int m, int n, int k, const float* in_squares, float in_eps,
                         const float* table, const int32_t* positions, const int32_t* seq_rows,
                         const int32_t* block_table, int table_stride, bf16_t* k_cache, bf16_t* v_cache, int n_heads,
                         int n_kv_heads, int head_dim, int page_size, void* workspace, size_t workspace_bytes,
                         hipStream_t stream) {
  const NormFold fold = {in_squares, in_eps, nullptr, 0, nullptr, nullptr};
  const RopeStore rope = {table, positions, seq_rows, block_table, table_stride, k_cache, v_cache,
                          n_heads, n_kv_heads, head_dim, page_size};
  if (m > 16)
    return gemm_mfma_dispatch(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, MODE_STORE, stream, nullptr,
                              workspace, workspace_bytes, &rope);
#define ARGS x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, MODE_STORE, stream, fold, rope
  return launch_skinny<2, 1, 4, 8, EPI_ROPE>(ARGS);
#undef ARGS
}

#endif  // AXON_BF16
