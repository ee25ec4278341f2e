// bfloat16 matrix products on the matrix cores: out = X [M, K] . W [N, K]^T, 32-bit accumulation.
// Only in the bfloat16 build.
//
// W is PACKED (axk_pack_matrix, once, when the weights are loaded): blocks of 16 rows x 32 k, each
// 1 KB in the order in which a wave holds them as an MFMA operand (lane l: row l % 16, the 8
// consecutive k from 8 (l / 16)); blocks ordered [row tile][k block]; rows padded to a multiple
// of 16 with zeros.  A wave instruction then reads whole kilobytes of consecutive memory, the
// blocks land in LDS without a permutation, and the same bytes serve every kernel here.
//
// ONE ORDER OF ADDITION PER MATRIX.  Every output element of a product with a given W is
//     ((c_0 + c_1) + c_2) + ... + c_(S-1),   then the bias and the epilogue,
// where K is cut into S = gemm_segments(W's row tiles, K) contiguous segments (by the matrix
// alone, never by the number of rows M of X), and c_s is one chain of 32x32x16 MFMAs over
// the segment's k in ascending steps of 16, starting from zero.  Every kernel below computes
// exactly this, whatever its tiles, its number of waves or the way it spreads the segments over
// waves, blocks or registers: a row of X gives the same bits whether it comes alone, among 16
// rows or among 4,096 (src/lm.rs:272-278 asks this of a step; the reference's integer products
// get it from exact block sums, src/cuda/decode.cu:352-369).  The kernels are chosen by M, for
// speed alone:
//
// * gemm_stream (M <= 64): bound by reading W once.  A wave owns 32 rows of W and one segment of
//   K and streams its share from memory straight into MFMA operands, keeping a ring of steps
//   in flight; W is the A operand, up to 64 rows of X the B operand.  The waves of a block are
//   the segments of one tile of rows (or several tiles where S is small); their sums are added
//   in segment order through LDS.  Epilogues: bias / residual add / SwiGLU, and the attention's
//   qkv product with the rotary encoding and the store into the paged cache.
//
// * gemm_tile (M > 64): a block of 4 or 8 waves owns a BM x BN tile of the output, walks K in
//   steps of 64 through LDS stages filled by direct global -> LDS loads (the next step's loads
//   in flight while this one multiplies), and each wave keeps a tile of 32x32x16 MFMA
//   accumulators.  The segments are either kept apart in registers (a second set of
//   accumulators takes each finished segment's sums; SEG) or, where the output gives too few
//   tiles for 256 CUs, given to blocks of their own (gridDim.y = S), whose sums go through a
//   workspace and are added in segment order by gemm_split_reduce, which also applies the
//   epilogue.  X rows land in LDS with their 16-byte slots permuted so that fragment reads of
//   neighbouring rows fall into different banks; W blocks land as they are.  Blocks are numbered
//   so that the blocks of one XCD (every eighth block) share weight tiles in that XCD's L2.
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
//
// SEG: the block walks all of K and keeps the `segs` segments apart: at the end of a segment its
// sums are added to a second set of accumulators and the first starts from zero again.
template <int BM, int BN, int WAVES_M, int WAVES_N, bool GLU, int BK, int STAGES, bool SEG>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_tile_kernel(const bf16_t* __restrict__ x, int x_stride, const bf16_t* __restrict__ w, const void* __restrict__ bias,
                 int bias_is_f32, void* __restrict__ out, int out_stride, int M, int N, int K, int mode, int m_blocks,
                 int n_blocks, float* __restrict__ partial, int segs) {
  extern __shared__ __align__(16) unsigned char smem[];
  static_assert(BK == 64, "segments of K are counted in steps of 64");
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
  f32x16 total[SEG ? TM : 1][SEG ? TN : 1];     // SEG: the sums of the segments that are finished
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        acc[i][j][e] = 0.0f;
        if (SEG) total[i][j][e] = 0.0f;
      }
  int seg_at = 0, seg_end = SEG ? (int)((long)nk / segs) : 0;   // SEG: the segment under way ends before K tile seg_end

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
    if (SEG && kt + 1 == seg_end) {
      // a segment's chain is complete: its sums join the finished ones, in segment order
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            total[i][j][e] += acc[i][j][e];
            acc[i][j][e] = 0.0f;
          }
      ++seg_at;
      seg_end = (int)((long)(seg_at + 1) * nk / segs);
    }
  }
#undef SWZ
  if (SEG) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[i][j] = total[i][j];
  }

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

template <int BM, int BN, int WAVES_M, int WAVES_N, bool GLU, bool SEG = false, int BK = 64, int STAGES = 2>
static int launch_tile(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                       int out_stride, int m, int n, int k, int mode, hipStream_t stream, int segs = 1,
                       float* partial = nullptr, const SplitNorm* norm = nullptr, const RopeStore* rope = nullptr) {
  static bool configured = false;
  constexpr int lds_bytes = STAGES * (BM + BN) * BK * 2;
  static_assert(lds_bytes <= 160 * 1024, "the stages do not fit the LDS of a CU");
  auto kernel = &gemm_tile_kernel<BM, BN, WAVES_M, WAVES_N, GLU, BK, STAGES, SEG>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       lds_bytes);
    if (e != hipSuccess) {
      axk_set_error("gemm_tile: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
      return -2;
    }
    configured = true;
  }
  // SEG: every block walks all segments; else a block a segment (gridDim.y) and the sums through `partial`
  const int splits = SEG ? 1 : segs;
  const int m_blocks = ceil_div(m, BM), n_blocks = ceil_div(n, GLU ? BN / 2 : BN);
  kernel<<<dim3(m_blocks * n_blocks, splits), WAVES_M * WAVES_N * 64, lds_bytes, stream>>>(
      x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, m_blocks, n_blocks, splits > 1 ? partial : nullptr,
      segs);
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

// ---------------------------------------------------------------------------- gemm_stream
// Up to 64 rows of X: the product is bound by reading W once.  A wave owns one tile of 32 rows
// of W (two packed row tiles, A0 and A1) and one of the S segments of K.  Per step of 16 k it
// loads 1 KB of W (the A operand of a 32x32x16 MFMA: lane l holds row l % 32, the 8 consecutive
// k from 8 (l / 32); two pieces of 512 consecutive bytes, one in each packed tile) and, per 32
// rows of X, 1 KB of X (the B operand: lane l holds row l % 32 of X, the same 8 k), and
// multiplies; a ring of DEPTH steps is in flight, refilled as soon as a step is multiplied, so
// the memory pipe never drains.  The waves of a block are TILES tiles x SEGS segments; the
// segments' sums meet in LDS and are added in segment order, the 16 registers of a lane shared
// out between the tile's waves in units of 4 consecutive output columns.
//
// The accumulator of a 32 x 32 tile: lane l, register e holds W row 8 (e / 4) + 4 (l / 32) + e % 4
// and X row l % 32.  Rows 0..15 come from packed tile A0, rows 16..31 from A1, so register e + 8
// is the same row of A1 as register e of A0: the paired epilogues put partners there.
// * plain: A0, A1 = tiles 2t, 2t + 1: 32 consecutive columns of the output.
// * GLU: A0 = gate rows 16t .., A1 = the up rows of the same columns (W holds 2 N rows); the
//   output is silu(gate) * up.
// * ROPE (the attention's fused [q; k; v] matrix; W's rows are heads of head_dim): A0 = dims
//   16j .. of a head, A1 = their rotation partners 16j + half ..; q heads go rotated to `out`,
//   k heads rotated into the request's page of keys, v heads as they are into its page of
//   values (kept position-contiguous, [dim][slot]).  The arithmetic is that of the rotary kernel
//   after a plain product: the sums are rounded to bfloat16 first, and each product and sum of
//   the rotation is rounded on its own.
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

template <int MT32, int SEGS, int TILES, int DEPTH, int EPI>
__global__ void __launch_bounds__(SEGS * TILES * 64)
gemm_stream_kernel(const bf16_t* __restrict__ x, int x_stride, const bf16_t* __restrict__ w,
                   const void* __restrict__ bias, int bias_is_f32, void* __restrict__ out, int out_stride, int M, int N,
                   int K, int mode, int n_tiles, RopeStore rope) {
  constexpr bool GLU = EPI == EPI_GLU, ROPE = EPI == EPI_ROPE;
  constexpr int WAVES = SEGS * TILES;
  // [wave][32 rows of X][4 groups of 4 registers][lane]: a lane's 4 consecutive registers are one 16-byte slot
  __shared__ float4 sums[SEGS > 1 ? WAVES * MT32 * 4 * 64 : 1];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int tile = blockIdx.x * TILES + wave / SEGS, seg = wave % SEGS;
  const bool live = tile < n_tiles;                  // the last block may have tiles to spare
  const int t = live ? tile : n_tiles - 1;
  const int l32 = lane & 31, half = lane >> 5;

  // the two packed row tiles of this tile of 32 rows
  const int KB = K / 32;
  int a0, a1;
  if (GLU) {
    a0 = t;
    a1 = N / 16 + t;
  } else if (ROPE) {
    const int per_head = rope.head_dim / 32;
    a0 = (t / per_head) * (rope.head_dim / 16) + t % per_head;
    a1 = a0 + rope.head_dim / 32;
  } else {
    const int last = (N + 15) / 16 - 1;              // past the matrix: its last tile (columns dropped below)
    a0 = min(2 * t, last);
    a1 = min(2 * t + 1, last);
  }
  // step q (16 k from 16 q) of a packed row tile: the 512 bytes from 512 q; this lane's 16 of them
  const bf16_t* wp = w + (size_t)((lane & 16) ? a1 : a0) * KB * 512 + (half * 16 + (lane & 15)) * 8;
  const bf16_t* xp[MT32];
#pragma unroll
  for (int j = 0; j < MT32; ++j) xp[j] = x + (size_t)min(j * 32 + l32, M - 1) * x_stride + half * 8;

  // this wave's segment: the K tiles (of 64) nk seg / SEGS .. nk (seg + 1) / SEGS - 1, in steps of 16
  const int nk = K / 64;
  const int q0 = (int)((long)seg * nk / SEGS) * 4;
  const int steps = live ? (int)((long)(seg + 1) * nk / SEGS) * 4 - q0 : 0;

  f32x16 acc[MT32];
#pragma unroll
  for (int j = 0; j < MT32; ++j)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[j][e] = 0.0f;

  uint4 wf[DEPTH], xf[DEPTH][MT32];
  auto load = [&](int slot, int local) {
    const int q = q0 + local;
    wf[slot] = *reinterpret_cast<const uint4*>(wp + (size_t)q * 256);
#pragma unroll
    for (int j = 0; j < MT32; ++j) xf[slot][j] = *reinterpret_cast<const uint4*>(xp[j] + q * 16);
  };
  auto multiply = [&](int slot) {
#pragma unroll
    for (int j = 0; j < MT32; ++j)
      acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_frag(wf[slot]), as_frag(xf[slot][j]), acc[j], 0, 0, 0);
  };
  if (steps > 0) {
    // The ring holds steps base .. base + DEPTH - 1: a step is multiplied as soon as ITS loads
    // have landed (loads return in order), and its place is refilled at once.
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) load(d, min(d, steps - 1));    // beyond the segment: a valid step again
    int base = 0;
    for (; base + 2 * DEPTH <= steps; base += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        multiply(d);
        load(d, base + DEPTH + d);
      }
    }
    // the tail: what the ring holds, refilled only where a step is left, then those
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (base + d < steps) multiply(d);
      if (base + DEPTH + d < steps) load(d, base + DEPTH + d);
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (base + DEPTH + d < steps) multiply(d);
  }

  if (SEGS > 1) {
#pragma unroll
    for (int j = 0; j < MT32; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g)
        sums[((wave * MT32 + j) * 4 + g) * 64 + lane] =
            make_float4(acc[j][4 * g], acc[j][4 * g + 1], acc[j][4 * g + 2], acc[j][4 * g + 3]);
    __syncthreads();
  }
  if (!live) return;

  // Units of work: 4 registers (4 consecutive W rows 8 g + 4 half ..) of one 32-row part of X;
  // the paired epilogues take group g (rows of A0) together with group g + 2 (the same rows of A1).
  // The tile's waves share the units out; each adds the segments' sums in segment order.
  constexpr int GROUPS = EPI == EPI_PLAIN ? 4 : 2;
  const int first_wave = (wave / SEGS) * SEGS;
  auto summed = [&](int j, int g) {
    if (SEGS == 1) return make_float4(acc[j][4 * g], acc[j][4 * g + 1], acc[j][4 * g + 2], acc[j][4 * g + 3]);
    float4 v = sums[(((first_wave + 0) * MT32 + j) * 4 + g) * 64 + lane];
#pragma unroll
    for (int s = 1; s < SEGS; ++s) {
      const float4 p = sums[(((first_wave + s) * MT32 + j) * 4 + g) * 64 + lane];
      v.x += p.x; v.y += p.y; v.z += p.z; v.w += p.w;
    }
    return v;
  };
#pragma unroll
  for (int u0 = 0; u0 < MT32 * GROUPS; u0 += SEGS) {
    const int u = u0 + seg;
    if (u >= MT32 * GROUPS) break;
    // SEGS == 1: u is a compile-time constant, so the registers are indexed statically
    const int j = u / GROUPS, g = u % GROUPS;
    const int m = j * 32 + l32;
    const int r = 8 * g + 4 * half;               // first of the 4 rows, within the 32 of the tile (or the 16 of A0)
    if (m >= M) continue;
    if (ROPE) {
      const int hd = rope.head_dim, hh = hd / 2, per_head = hd / 32;
      const int slot = tile / per_head;             // q heads, then k heads, then v heads
      const int d = (tile % per_head) * 16 + r;
      const float4 lo4 = summed(j, g), hi4 = summed(j, g + 2);
      const float lo_s[4] = {lo4.x, lo4.y, lo4.z, lo4.w}, hi_s[4] = {hi4.x, hi4.y, hi4.z, hi4.w};
      float a[4], b[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float lo = lo_s[e], hi = hi_s[e];
        if (bias) {
          lo += load_vec(bias, bias_is_f32, slot * hd + d + e);
          hi += load_vec(bias, bias_is_f32, slot * hd + hh + d + e);
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
            vdst[(size_t)(hh + d + e) * rope.page_size] = float_to_bf16(b[e]);
          }
          continue;
        }
        const int kvh = slot - rope.n_heads;
        dst = rope.k_cache + (((size_t)page * rope.n_kv_heads + kvh) * rope.page_size + in_page) * hd;
      }
      const float4* tab = reinterpret_cast<const float4*>(rope.table + ((size_t)m * hh + d) * 2);
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
      *reinterpret_cast<uint2*>(dst + hh + d) = pk;
      continue;
    }
    if (GLU) {
      const int n = tile * 16 + r;                  // N is a multiple of 16: the unit's 4 columns exist
      const float4 g4 = summed(j, g), u4 = summed(j, g + 2);
      uint2 pk;
      pk.x = pack2_bf16(swiglu1(g4.x, u4.x), swiglu1(g4.y, u4.y));
      pk.y = pack2_bf16(swiglu1(g4.z, u4.z), swiglu1(g4.w, u4.w));
      bf16_t* dst = reinterpret_cast<bf16_t*>(out) + (size_t)m * out_stride + n;
      if (out_stride % 4 == 0 && ((uintptr_t)out & 7) == 0) *reinterpret_cast<uint2*>(dst) = pk;
      else {
        dst[0].bits = (uint16_t)pk.x; dst[1].bits = (uint16_t)(pk.x >> 16);
        dst[2].bits = (uint16_t)pk.y; dst[3].bits = (uint16_t)(pk.y >> 16);
      }
      continue;
    }
    const int n = tile * 32 + r;
    if (n >= N) continue;
    const float4 v4 = summed(j, g);
    float v[4] = {v4.x, v4.y, v4.z, v4.w};
    if (bias) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < N) v[e] += load_vec(bias, bias_is_f32, n + e);
    }
    const size_t at = (size_t)m * out_stride + n;
    const bool whole = n + 3 < N && out_stride % 4 == 0;
    if (mode == MODE_STORE) {
      bf16_t* dst = reinterpret_cast<bf16_t*>(out) + at;
      if (whole && ((uintptr_t)out & 7) == 0) {
        uint2 pk;
        pk.x = pack2_bf16(v[0], v[1]);
        pk.y = pack2_bf16(v[2], v[3]);
        *reinterpret_cast<uint2*>(dst) = pk;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) dst[e] = float_to_bf16(v[e]);
      }
    } else {
      float* dst = reinterpret_cast<float*>(out) + at;
      if (whole && ((uintptr_t)out & 15) == 0) {
        float4 o = make_float4(v[0], v[1], v[2], v[3]);
        if (mode == MODE_ADD_F32) {
          const float4 old = *reinterpret_cast<const float4*>(dst);
          o.x = old.x + v[0]; o.y = old.y + v[1]; o.z = old.z + v[2]; o.w = old.w + v[3];
        }
        *reinterpret_cast<float4*>(dst) = o;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) dst[e] = mode == MODE_ADD_F32 ? dst[e] + v[e] : v[e];
      }
    }
  }
}

template <int MT32, int SEGS, int EPI>
static int launch_stream(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                         int out_stride, int m, int n, int k, int mode, hipStream_t stream, int n_tiles,
                         const RopeStore& rope) {
  // eight waves a block where the segments allow it; the ring as deep as the registers allow
  constexpr int TILES = SEGS >= 8 ? 1 : SEGS == 4 ? 2 : 4;
  constexpr int DEPTH = MT32 == 1 ? 16 : 10;
  gemm_stream_kernel<MT32, SEGS, TILES, DEPTH, EPI><<<ceil_div(n_tiles, TILES), SEGS * TILES * 64, 0, stream>>>(
      x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, n_tiles, rope);
  AXK_LAUNCH_CHECK("gemm_stream");
  return 0;
}

template <int EPI>
static int launch_stream_any(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                             int out_stride, int m, int n, int k, int mode, hipStream_t stream, int n_tiles, int segs,
                             const RopeStore& rope) {
#define ARGS x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream, n_tiles, rope
  if (m <= 32) {
    switch (segs) {
      case 1: return launch_stream<1, 1, EPI>(ARGS);
      case 2: return launch_stream<1, 2, EPI>(ARGS);
      case 4: return launch_stream<1, 4, EPI>(ARGS);
      case 8: return launch_stream<1, 8, EPI>(ARGS);
    }
  } else {
    switch (segs) {
      case 1: return launch_stream<2, 1, EPI>(ARGS);
      case 2: return launch_stream<2, 2, EPI>(ARGS);
      case 4: return launch_stream<2, 4, EPI>(ARGS);
      case 8: return launch_stream<2, 8, EPI>(ARGS);
    }
  }
#undef ARGS
  axk_set_error("gemm_stream: %d segments", segs);
  return -1;
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


// ---------------------------------------------------------------------------- the order and the dispatch
// The number of segments K is cut into for a matrix of `tiles32` tiles of 32 rows (as gemm_stream
// counts them: ceil(N / 32); N / 16 for a [gate; up] matrix of 2 N rows) and K columns: a power
// of two up to 8, so that a step of few rows still gives some 768 waves a chain of their own,
// with at least 4 K tiles (256 k) a segment.  It is a property of the matrix: it fixes the order
// of addition of every product with it.
int gemm_segments(int tiles32, int k) {
  const int nk = k / 64;
  int s = 1;
  while (s < 8 && tiles32 * s < 768 && nk / (2 * s) >= 4) s *= 2;
  return s;
}

static int tiles32_of(int n, int mode) { return mode == MODE_SWIGLU ? n / 16 : (n + 31) / 32; }

// M > 64 with S > 1 segments: kept apart in registers by blocks that walk all of K where the output
// alone gives enough tiles of 128 x 128 (or 128 x 256) to occupy the chip, else a block a segment
// and the sums through a workspace.  Decided by the sizes alone.
static bool segments_across_blocks(int m, int n, int k, int mode, int segs) {
  if (segs <= 1 || n % 4 != 0) return false;
  const long blocks = (long)ceil_div(m, 128) * ceil_div(n, mode == MODE_SWIGLU ? 64 : 128);
  return blocks < 100;
}

size_t gemm_workspace_bytes(int m, int n, int k, int mode) {
  if (k % 64 != 0 || m <= 64) return 0;
  const int s = gemm_segments(tiles32_of(n, mode), k);
  if (!segments_across_blocks(m, n, k, mode, s)) return 0;
  return (size_t)s * (mode == MODE_SWIGLU ? 2 : 1) * m * n * sizeof(float);
}

// Whether the product that adds into the rows runs with a block a segment, so that the kernel that
// adds the segments' sums can also norm the finished rows (gemm_split_reduce_norm_kernel: rows of
// up to SRN_MAX_N columns).
int gemm_then_norm_ok(int m, int n, int k) {
  return gemm_pack_ok(n, k, 0) && m > 64 && n <= SRN_MAX_N &&
         segments_across_blocks(m, n, k, MODE_ADD_F32, gemm_segments(tiles32_of(n, MODE_ADD_F32), k));
}

static int gemm_mfma_dispatch(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                              int out_stride, int m, int n, int k, int mode, hipStream_t stream,
                              const SplitNorm* norm, void* workspace, size_t workspace_bytes,
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
  const int tiles32 = tiles32_of(n, mode);
  const int segs = gemm_segments(tiles32, k);
#define ARGS x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream
  if (m <= 64) {
    if (norm || rope_after) {
      axk_set_error("gemm: M=%d goes to the streaming kernel, which has these epilogues of its own", m);
      return -1;
    }
    if (mode == MODE_SWIGLU) return launch_stream_any<EPI_GLU>(ARGS, tiles32, segs, RopeStore());
    return launch_stream_any<EPI_PLAIN>(ARGS, tiles32, segs, RopeStore());
  }
  const bool across = segments_across_blocks(m, n, k, mode, segs);
  if ((norm || rope_after) && (!across || mode != (norm ? MODE_ADD_F32 : MODE_STORE))) {
    axk_set_error("gemm: M=%d N=%d K=%d mode %d does not run with a block a segment: no kernel adds sums after it", m, n,
                  k, mode);
    return -1;
  }
  const size_t need = gemm_workspace_bytes(m, n, k, mode);
  if (need > workspace_bytes || (need > 0 && (workspace == nullptr || ((uintptr_t)workspace & 15)))) {
    axk_set_error("gemm: M=%d N=%d K=%d needs a workspace of %zu bytes, 16-byte aligned (got %zu)", m, n, k, need,
                  workspace_bytes);
    return -1;
  }
  float* ws = (float*)workspace;
  const bool glu = mode == MODE_SWIGLU;
  if (segs > 1 && !across) {
    // the segments in registers: 128 x 256 tiles (8 waves) where they occupy the chip, else 128 x 128
    const long wide = (long)ceil_div(m, 128) * ceil_div(n, glu ? 128 : 256);
    if (wide >= 200) {
      if (glu) return launch_tile<128, 256, 2, 4, true, true>(ARGS, segs);
      return launch_tile<128, 256, 2, 4, false, true>(ARGS, segs);
    }
    if (glu) return launch_tile<128, 128, 2, 2, true, true>(ARGS, segs);
    return launch_tile<128, 128, 2, 2, false, true>(ARGS, segs);
  }
  if (m <= 256) {
    if (glu) return launch_tile<128, 128, 2, 2, true>(ARGS, segs, ws);
    return launch_tile<128, 128, 2, 2, false>(ARGS, segs, ws, norm, rope_after);
  }
  // 256 x 256 tiles (8 waves) where they fill the chip: one round of at least 140 blocks (on 256
  // CUs), or several rounds of which the last is not mostly idle; else 128 x 128 tiles, four times
  // as many blocks at twice the traffic from L2 per product.  Thresholds are measured ones.
  const int splits = across ? segs : 1;
  const int n_per_block = glu ? 128 : 256;
  const long big = (long)ceil_div(m, 256) * ceil_div(n, n_per_block) * splits;
  const long rounds = (big + 255) / 256;
  const bool use_big = big <= 256 ? big >= 140 : big * 10 >= rounds * 256 * 7;
  if (glu) {
    if (use_big) return launch_tile<256, 256, 4, 2, true>(ARGS, segs, ws);
    return launch_tile<128, 128, 2, 2, true>(ARGS, segs, ws);
  }
  // one round of 256 x 256 tiles that leaves a quarter of the CUs idle, and N in whole tiles of
  // 192 columns that still fit one round: the narrower tile (measured 1.1 times the cost per
  // product, three quarters of the products per block).
  if (use_big && splits == 1 && big <= 192 && n % 192 == 0 && (long)ceil_div(m, 256) * (n / 192) <= 256)
    return launch_tile<256, 192, 4, 2, false>(ARGS, segs, ws, norm);
  if (use_big) return launch_tile<256, 256, 4, 2, false>(ARGS, segs, ws, norm, rope_after);
  return launch_tile<128, 128, 2, 2, false>(ARGS, segs, ws, norm, rope_after);
#undef ARGS
}

int launch_gemm_mfma(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                     int out_stride, int m, int n, int k, int mode, hipStream_t stream, const GemmNormFold* then_norm,
                     void* workspace, size_t workspace_bytes) {
  SplitNorm after = {nullptr, 0, 0.0f, nullptr};
  if (then_norm)
    after = SplitNorm{then_norm->norm_gain, then_norm->norm_gain_is_f32, then_norm->norm_eps, (bf16_t*)then_norm->norm_values};
  return gemm_mfma_dispatch(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream,
                            then_norm ? &after : nullptr, workspace, workspace_bytes, nullptr);
}

// The [q; k; v] product with rotary encoding and cache store (see RopeStore): up to 64 rows in
// the epilogue of gemm_stream, more rows where the product runs with a block a segment (then the
// kernel that adds the segments' sums rotates and stores); every head rotated over its whole
// width, halves of a head a multiple of 16 wide.
int gemm_qkv_rope_ok(int m, int n, int k, int head_dim, int rotary_dim) {
  if (m < 1 || k % 64 != 0 || rotary_dim != head_dim || head_dim % 32 != 0 || n % head_dim != 0) return 0;
  if (!gemm_pack_ok(n, k, 0)) return 0;
  if (m <= 64) return 1;
  return segments_across_blocks(m, n, k, MODE_STORE, gemm_segments(tiles32_of(n, MODE_STORE), k));
}

int launch_gemm_qkv_rope(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, bf16_t* out,
                         int out_stride, int m, int n, int k, const float* table, const int32_t* positions,
                         const int32_t* seq_rows, const int32_t* block_table, int table_stride, bf16_t* k_cache,
                         bf16_t* v_cache, int n_heads, int n_kv_heads, int head_dim, int page_size, void* workspace,
                         size_t workspace_bytes, hipStream_t stream) {
  const RopeStore rope = {table, positions, seq_rows, block_table, table_stride, k_cache, v_cache,
                          n_heads, n_kv_heads, head_dim, page_size};
  if (m > 64)
    return gemm_mfma_dispatch(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, MODE_STORE, stream, nullptr,
                              workspace, workspace_bytes, &rope);
  const int tiles32 = n / 32;
  return launch_stream_any<EPI_ROPE>(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, MODE_STORE, stream,
                                     tiles32, gemm_segments(tiles32, k), rope);
}

#endif  // AXON_BF16
