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
// * gemm_stream (M <= 16): bound by reading W once.  A wave owns one or two tiles of 16 rows of W
//   and one segment of K and streams its share from memory straight into 16x16x32 MFMA operands
//   (one such MFMA gives the bits of two chained 32x32x16 ones over the same k), keeping a ring
//   of steps in flight; W is the A operand, the rows of X the B operand.  The waves of a block
//   are the segments of its tiles; their sums are added in segment order through LDS.
//   Epilogues: bias / residual add / SwiGLU, and the attention's qkv product with the rotary
//   encoding and the store into the paged cache.
//
// * gemm_normed (M <= 16, the operand an RMS norm of float32 rows): gemm_stream's product with the
//   norm inside; waves of their own norm the rows into LDS while the streaming waves fill their
//   rings, so the norm is no launch of its own in a decoding step.
//
// * gemm_rows (17 <= M <= 128): W still streams into registers, but the waves of a block walk the
//   same segment of K and share X through LDS; a block a segment, the sums of several segments
//   through a workspace.
//
// * gemm_tile (M > 128): a block of 4 or 8 waves owns a BM x BN tile of the output, walks K in
//   steps of 64 through LDS stages filled by direct global -> LDS loads (the next step's loads
//   in flight while this one multiplies), and each wave keeps a tile of 32x32x16 MFMA
//   accumulators.  With S > 1 segments each goes to blocks of its own (gridDim.y = S), whose sums
//   go through a workspace and are added in segment order by gemm_split_reduce, which also
//   applies the epilogue.  X rows land in LDS with their 16-byte slots permuted so that fragment reads of
//   neighbouring rows fall into different banks; W blocks land as they are.  Blocks are numbered
//   so that the blocks of one XCD (every eighth block) share weight tiles in that XCD's L2.
#include "api.h"
#include "common.h"
#include "instances.h"

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
  static_assert(BK == 64 || BK == 32, "segments of K are counted in steps of 64: whole K tiles");
  constexpr int PER64 = 64 / BK;                       // K tiles in a step of 64
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

  // Block numbering: every eighth block runs on the same XCD, 32 of them at a time.  An XCD takes
  // every eighth n block and walks its share in squares of up to 8 m blocks x 4 n blocks, so that
  // the 32 blocks at work share 12 tiles of operands in that XCD's L2 (with many m blocks, all m
  // blocks of one n block in a row would share 33), the squares of the same four n blocks one
  // after the other.
  const int bid = blockIdx.x;
  int mb, nb;
  if (bid < (n_blocks / 8) * 8 * m_blocks) {
    constexpr int GM = 8, GN = 4;
    const int xcd = bid & 7, j = bid >> 3, mine = n_blocks / 8;       // this XCD's n blocks: xcd, xcd + 8, ...
    const int whole_groups = mine / GN;
    int g = j / (GN * m_blocks), rest = j % (GN * m_blocks), gn = GN;
    if (g >= whole_groups) {                                          // the last, narrower group of n blocks
      g = whole_groups;
      rest = j - whole_groups * GN * m_blocks;
      gn = mine - whole_groups * GN;
    }
    const int whole_rows = m_blocks / GM;
    int ms = rest / (gn * GM), r = rest % (gn * GM), gm = GM;
    if (ms >= whole_rows) {                                           // the last, shorter square
      ms = whole_rows;
      r = rest - whole_rows * gn * GM;
      gm = m_blocks - whole_rows * GM;
    }
    mb = ms * GM + r % gm;
    nb = (g * GN + r / gm) * 8 + xcd;
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
  const int kt_begin = (int)((long)blockIdx.y * (K / 64) / gridDim.y) * PER64;
  const int nk = (int)((long)(blockIdx.y + 1) * (K / 64) / gridDim.y) * PER64 - kt_begin;
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

// The same for a width that is no multiple of 4 (rows of the workspace are then not 16-byte
// aligned): a thread an element, the same additions in the same order.  No gated epilogue here: a
// [gate; up] matrix has whole row tiles.
__global__ void __launch_bounds__(256)
gemm_split_reduce_any_kernel(const float* __restrict__ partial, int splits, int M, int N, const void* __restrict__ bias,
                             int bias_is_f32, void* __restrict__ out, int out_stride, int mode) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)M * N) return;
  const int m = (int)(idx / N), n = (int)(idx % N);
  const size_t plane = (size_t)M * N;
  float v = partial[idx];
  for (int z = 1; z < splits; ++z) v += partial[(size_t)z * plane + idx];
  if (bias) v += load_vec(bias, bias_is_f32, n);
  const size_t at = (size_t)m * out_stride + n;
  if (mode == MODE_STORE) reinterpret_cast<bf16_t*>(out)[at] = float_to_bf16(v);
  else if (mode == MODE_ADD_F32) reinterpret_cast<float*>(out)[at] += v;
  else reinterpret_cast<float*>(out)[at] = v;
}

// The sums of the split-K blocks, added in block order, then the epilogue of the product.
// One thread per 4 consecutive columns of a row (N a multiple of 4).
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

// The second launch of a product whose blocks left a segment's sums each: the sums in segment
// order, then the epilogue (with the rotary store, or the norm of the new rows, where asked).
static int add_split_sums(const float* partial, int splits, int m, int n, const void* bias, int bias_is_f32, void* out,
                          int out_stride, int mode, const SplitNorm* norm, const RopeStore* rope, hipStream_t stream) {
  if (rope != nullptr) {
    AXK_INSTANCE(INST_GEMM_SPLIT_REDUCE, 2);
    return launch_split_reduce_rope(partial, splits, m, n, bias, bias_is_f32, out, out_stride, *rope, stream);
  }
  if (norm != nullptr) {
    AXK_INSTANCE(INST_GEMM_SPLIT_REDUCE, 1);
    gemm_split_reduce_norm_kernel<<<m, SRN_THREADS, 0, stream>>>(partial, splits, m, n, bias, bias_is_f32, (float*)out,
                                                                 out_stride, *norm);
    AXK_LAUNCH_CHECK("gemm_split_reduce_norm");
    return 0;
  }
  if (n % 4 != 0) {
    AXK_INSTANCE(INST_GEMM_SPLIT_REDUCE, 3);
    gemm_split_reduce_any_kernel<<<(unsigned)(((size_t)m * n + 255) / 256), 256, 0, stream>>>(partial, splits, m, n, bias,
                                                                                             bias_is_f32, out, out_stride, mode);
    AXK_LAUNCH_CHECK("gemm_split_reduce");
    return 0;
  }
  AXK_INSTANCE(INST_GEMM_SPLIT_REDUCE, 0);
  gemm_split_reduce_kernel<<<ceil_div(m * (n / 4), 256), 256, 0, stream>>>(partial, splits, m, n, bias, bias_is_f32, out,
                                                                          out_stride, mode);
  AXK_LAUNCH_CHECK("gemm_split_reduce");
  return 0;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool GLU, int BK = 64, int STAGES = 2>
static int launch_tile(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                       int out_stride, int m, int n, int k, int mode, hipStream_t stream, int segs = 1,
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
  // a block a segment (gridDim.y), the sums through `partial`
  const int splits = segs;
  const int m_blocks = ceil_div(m, BM), n_blocks = ceil_div(n, GLU ? BN / 2 : BN);
  AXK_INSTANCE(INST_GEMM_TILE, BM, BN, WAVES_M, WAVES_N, GLU, STAGES);
  kernel<<<dim3(m_blocks * n_blocks, splits), WAVES_M * WAVES_N * 64, lds_bytes, stream>>>(
      x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, m_blocks, n_blocks, splits > 1 ? partial : nullptr);
  AXK_LAUNCH_CHECK("gemm_tile");
  return splits > 1 ? add_split_sums(partial, splits, m, n, bias, bias_is_f32, out, out_stride, mode, norm, rope, stream) : 0;
}

// ---------------------------------------------------------------------------- gemm_stream
// Up to 16 rows of X: the product is bound by reading W once.  A block owns NT16 row tiles (of
// 16) of W; its waves are the S segments of K, each streaming its share of the tiles from memory
// straight into 16x16x32 MFMA operands (a packed block as it lies in memory, 1 KB an
// instruction), keeping a ring of steps in flight so that the memory pipe never drains, and
// multiplying with the rows of X (the B operand: lane l holds row l % 16, 8 consecutive k
// from (l / 16) * 8).  C[n][m] tiles of 16 x 16: a lane ends with 4 consecutive n of one m, one
// vector store.  The segments' sums meet in LDS and are added in segment order.  A 16x16x32 MFMA
// gives the bits of two chained 32x32x16 MFMAs over the same 32 k (measured over wide ranges of
// exponents; the tests compare the kernels bit for bit), so the chain is the tile kernel's.
// * GLU (NT16 = 2): the block's two tiles are the gate rows n0 .. n0 + 15 and the up rows of the
//   same columns (W holds 2 N rows), and the output is silu(gate) * up.
// * ROPE (NT16 = 2; the attention's fused [q; k; v] matrix, W's rows are heads of head_dim): a
//   block owns dims d0 .. d0 + 15 of one head and their rotation partners d0 + half .., so that a
//   lane ends with both values of a pair.  q heads go rotated to `out`, k heads rotated into the
//   request's page of keys, v heads as they are into its page of values (kept
//   position-contiguous, [dim][slot]).  The arithmetic is that of the rotary kernel after a
//   plain product: the sums are rounded to bfloat16 first, and each product and sum of the
//   rotation is rounded on its own.
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
// other, bit for bit.  A block per token and group of head slots; a thread takes 4 consecutive dims
// of a head's lower half and their partners in the upper half (every load a float4, all of a
// thread's loads independent of each other); q heads go rotated to `out`, k heads rotated into the
// request's page of keys, v heads as they are into its page of values.  Every head is rotated
// over its whole width.
__global__ void __launch_bounds__(256)
gemm_split_reduce_rope_kernel(const float* __restrict__ partial, int splits, int M, int N, const void* __restrict__ bias,
                              int bias_is_f32, bf16_t* __restrict__ out, int out_stride, RopeStore rope) {
  const int hd = rope.head_dim, half = hd / 2, per_head = half / 4;     // threads a head
  const int heads_a_block = 256 / per_head;
  const int m = blockIdx.x, within = threadIdx.x / per_head, slot = blockIdx.y * heads_a_block + within;
  const int d = (threadIdx.x % per_head) * 4;
  if (within >= heads_a_block || slot * hd >= N) return;
  const size_t plane = (size_t)M * N;
  // four columns' sums, rounded as the product's own store rounds them
  auto values = [&](int col, float (&v)[4]) {
    const float* src = partial + (size_t)m * N + col;
    float4 g = *reinterpret_cast<const float4*>(src);
    for (int z = 1; z < splits; ++z) {
      const float4 a = *reinterpret_cast<const float4*>(src + (size_t)z * plane);
      g.x += a.x; g.y += a.y; g.z += a.z; g.w += a.w;
    }
    v[0] = g.x; v[1] = g.y; v[2] = g.z; v[3] = g.w;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (bias) v[e] += load_vec(bias, bias_is_f32, col + e);
      v[e] = bf16_to_float(float_to_bf16(v[e]));
    }
  };
  float a[4], b[4];
  values(slot * hd + d, a);
  values(slot * hd + half + d, b);
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
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        vdst[(size_t)(d + e) * rope.page_size] = float_to_bf16(a[e]);
        vdst[(size_t)(half + d + e) * rope.page_size] = float_to_bf16(b[e]);
      }
      return;
    }
    dst = rope.k_cache + (((size_t)page * rope.n_kv_heads + (slot - rope.n_heads)) * rope.page_size + in_page) * hd;
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

static int launch_split_reduce_rope(const float* partial, int splits, int m, int n, const void* bias, int bias_is_f32,
                                    void* out, int out_stride, const RopeStore& rope, hipStream_t stream) {
  const int heads_a_block = 256 / (rope.head_dim / 8);
  const dim3 grid(m, ceil_div(n / rope.head_dim, heads_a_block));
  gemm_split_reduce_rope_kernel<<<grid, 256, 0, stream>>>(partial, splits, m, n, bias, bias_is_f32, (bf16_t*)out, out_stride,
                                                          rope);
  AXK_LAUNCH_CHECK("gemm_split_reduce_rope");
  return 0;
}

// What the rotary epilogue reads besides the sums (a token's position, the page it is stored in,
// its sines and cosines): a chain of dependent loads that can start before the product does.
template <int MT16>
struct RopeAhead {
  int pos[MT16], page[MT16];
  float4 t0[MT16], t1[MT16];
};

// First the loads that depend on nothing (issued before the product's own first loads), then,
// once those are under way, the page, which needs the position.
template <int MT16, int SHARE>
__device__ inline RopeAhead<MT16> rope_look_ahead(const RopeStore& rope, int share, int unit, int lane, int M) {
  RopeAhead<MT16> ahead;
  const int half = rope.head_dim / 2, per_head = half / 16;
  const int slot = unit / per_head, d = (unit % per_head) * 16 + (lane >> 4) * 4;
#pragma unroll
  for (int j = 0; j < MT16; ++j) {
    ahead.pos[j] = ahead.page[j] = 0;
    ahead.t0[j] = ahead.t1[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    const int m = j * 16 + (lane & 15);
    if (j % SHARE != share || m >= M) continue;
    if (slot >= rope.n_heads) {
      ahead.pos[j] = rope.positions[m];
      ahead.page[j] = rope.seq_rows[m];                 // the row of the block table, until rope_look_ahead_page
    }
    if (slot < rope.n_heads + rope.n_kv_heads) {
      const float4* tab = reinterpret_cast<const float4*>(rope.table + ((size_t)m * half + d) * 2);
      ahead.t0[j] = tab[0];
      ahead.t1[j] = tab[1];
    }
  }
  return ahead;
}

template <int MT16, int SHARE>
__device__ inline void rope_look_ahead_page(RopeAhead<MT16>& ahead, const RopeStore& rope, int share, int unit, int lane, int M) {
  const int slot = unit / (rope.head_dim / 32);
#pragma unroll
  for (int j = 0; j < MT16; ++j) {
    if (j % SHARE != share || j * 16 + (lane & 15) >= M || slot < rope.n_heads) continue;
    ahead.page[j] = rope.block_table[(size_t)ahead.page[j] * rope.table_stride + ahead.pos[j] / rope.page_size];
  }
}

// What a wave does with finished sums (`summed(t, e)`: tile t = i * MT16 + j, element e; a lane
// holds X row 16 j + lane % 16 and W rows 4 (lane / 16) .. + 3 of tile i): the epilogue of the
// product.  `unit` names the tiles: for PLAIN the columns from unit * NT16 * 16, for GLU gate and
// up rows of columns unit * 16 .., for ROPE the half-pair `unit` of the [q; k; v] heads.  SHARE
// waves (`share` = which one) divide the tiles among themselves.
template <int NT16, int MT16, int EPI, int SHARE, class Summed>
__device__ inline void rows_epilogue(Summed summed, int share, int unit, int lane, const void* __restrict__ bias,
                                     int bias_is_f32, void* __restrict__ out, int out_stride, int M, int N, int mode,
                                     const RopeStore& rope, const RopeAhead<MT16>& ahead) {
  constexpr bool GLU = EPI == EPI_GLU, ROPE = EPI == EPI_ROPE;
  const int r16 = lane & 15;
  const int n0 = unit * (GLU ? 16 : NT16 * 16);
  if (ROPE) {
    const int hd = rope.head_dim, half = hd / 2, per_head = half / 16;
    const int slot = unit / per_head;                  // q heads, then k heads, then v heads
    const int d = (unit % per_head) * 16 + (lane >> 4) * 4;
#pragma unroll
    for (int j0 = 0; j0 < MT16; j0 += SHARE) {
      const int j = j0 + share;
      if (j >= MT16) break;
      const int m = j * 16 + r16;
      if (m >= M) continue;
      float a[4], b[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float lo = summed(j, e), hi = summed(MT16 + j, e);
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
        const int pos = ahead.pos[j], page = ahead.page[j];
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
      const float4 t0 = ahead.t0[j], t1 = ahead.t1[j];
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
#pragma unroll
    for (int j0 = 0; j0 < MT16; j0 += SHARE) {
      const int j = j0 + share;
      if (j >= MT16) break;
      const int m = j * 16 + r16;
      const int n = n0 + (lane >> 4) * 4;
      if (m >= M) continue;
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = swiglu1(summed(j, e), summed(MT16 + j, e));
      bf16_t* dst = reinterpret_cast<bf16_t*>(out) + (size_t)m * out_stride + n;
      if (n + 3 < N && out_stride % 4 == 0 && ((uintptr_t)out & 7) == 0) {
        uint2 pk;
        pk.x = pack2_bf16(v[0], v[1]);
        pk.y = pack2_bf16(v[2], v[3]);
        *reinterpret_cast<uint2*>(dst) = pk;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) dst[e] = float_to_bf16(v[e]);
      }
    }
    return;
  }
  // tiles are shared out between the waves
#pragma unroll
  for (int t0 = 0; t0 < NT16 * MT16; t0 += SHARE) {
    const int t = t0 + share;
    if (t >= NT16 * MT16) break;
    const int i = t / MT16, j = t % MT16;
    const int m = j * 16 + r16;
    const int n = n0 + i * 16 + (lane >> 4) * 4;
    if (m >= M || n >= N) continue;
    float v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      v[e] = summed(t, e);
      if (bias && n + e < N) v[e] += load_vec(bias, bias_is_f32, n + e);
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

template <int NT16, int MT16, int SEGS, int DEPTH, int EPI>
__global__ void __launch_bounds__(SEGS * 64)
gemm_stream_kernel(const bf16_t* __restrict__ x, int x_stride, const bf16_t* __restrict__ w,
                   const void* __restrict__ bias, int bias_is_f32, void* __restrict__ out, int out_stride, int M, int N,
                   int K, int mode, RopeStore rope) {
  constexpr bool GLU = EPI == EPI_GLU, ROPE = EPI == EPI_ROPE;
  static_assert(EPI == EPI_PLAIN || NT16 == 2, "the paired epilogues own two tiles of W rows");
  __shared__ float partial[SEGS > 1 ? SEGS : 1][NT16 * MT16][64][4];
  const int tid = threadIdx.x, lane = tid & 63, seg = tid >> 6;
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

  // This wave's segment: the K tiles (of 64) nk seg / SEGS .. nk (seg + 1) / SEGS - 1, one chain
  // in ascending k.  A ring of DEPTH steps (of 64 k) is kept in flight: a step is multiplied as
  // soon as ITS loads have landed (loads return in order), and its place in the ring is refilled
  // at once, so the memory pipe never drains.
  const int nk = K / 64;
  const int first = (int)((long)seg * nk / SEGS);
  const int mine = (int)((long)(seg + 1) * nk / SEGS) - first;
  uint4 wf[DEPTH][NT16][2], xf[DEPTH][MT16][2];
  auto load = [&](int slot, int local) {
    const int k0 = (first + local) * 64;
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
  // one 16x16x32 MFMA is two chained 32x32x16 ones over the same k, bit for bit (the tile kernel's)
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
  RopeAhead<MT16> ahead;
  if (ROPE) ahead = rope_look_ahead<MT16, SEGS>(rope, seg, blockIdx.x, lane, M);
  if (mine > 0) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) load(d, min(d, mine - 1));   // beyond this wave's steps: a valid step again
    if (ROPE) rope_look_ahead_page<MT16, SEGS>(ahead, rope, seg, blockIdx.x, lane, M);
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

  if (SEGS > 1) {
#pragma unroll
    for (int i = 0; i < NT16; ++i)
#pragma unroll
      for (int j = 0; j < MT16; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) partial[seg][i * MT16 + j][lane][e] = acc[i][j][e];
    __syncthreads();
  }
  // the segments' sums in segment order; lane: X row 16 j + r16, W rows 4 (lane / 16) .. + 3 of tile i
  auto summed = [&](int t, int e) {
    if (SEGS == 1) return acc[t / MT16][t % MT16][e];
    float sum = partial[0][t][lane][e];
#pragma unroll
    for (int q = 1; q < SEGS; ++q) sum += partial[q][t][lane][e];
    return sum;
  };

  rows_epilogue<NT16, MT16, EPI, SEGS>(summed, seg, blockIdx.x, lane, bias, bias_is_f32, out, out_stride, M, N, mode, rope,
                                       ahead);
}

// ---------------------------------------------------------------------------- gemm_normed
// The product of few rows with the RMS norm before it inside: X never exists in memory.  A block
// has waves of two kinds.  NORMED_NORM_WAVES waves read the float32 rows, norm them and leave
// X = bf16((row * inv) * gain) in LDS, in the blocks of MPAD rows x 32 k that one LDS read of a
// wave takes as an MFMA operand.  The others stream W as gemm_stream does (G groups of tiles times
// the S segments of K, a wave each; every block needs all of X, so G is such that each CU has
// about one block): their ring of loads is filled while the rows are normed (behind the loads
// of the rows themselves), and they start to multiply when X is there.  The gain is bfloat16 and
// K a multiple of 256.  The norm is the norm kernel's, bit for bit: a wave takes a row, lane l
// stands for that kernel's threads l, 64 + l, 128 + l and 192 + l (four chains over the float4
// l + 64 j, j = v, v + 4, ...), the four butterflies are added in order.  Takes the norm's launch
// out of a decoding step.
struct NormedRows {
  const float* rows;       // [M, K], rows_stride apart
  int rows_stride;
  const bf16_t* gain;      // [K]
  float eps;
};

#define NORMED_MAX_LDS (152 * 1024)
#define NORMED_STREAM_WAVES 4   // at most
#define NORMED_NORM_WAVES 4
#define NORMED_MAX_KC 20        // float4 of a row a lane holds at most: K <= 256 * 20

// UNITS: pairs of row tiles a streaming wave
#define NORMED_MAX_M 16

template <int UNITS, int SEGS, int DEPTH, int EPI, int MPAD, int KC>
__global__ void __launch_bounds__((NORMED_STREAM_WAVES + NORMED_NORM_WAVES) * 64, 1)
gemm_normed_kernel(NormedRows in, const bf16_t* __restrict__ w, const void* __restrict__ bias, int bias_is_f32,
                   void* __restrict__ out, int out_stride, int M, int N, int K, int mode, RopeStore rope, int n_units) {
  constexpr bool GLU = EPI == EPI_GLU, ROPE = EPI == EPI_ROPE;
  constexpr int NT = 2 * UNITS, XBLOCK = MPAD * 64;             // XBLOCK: bytes of MPAD rows x 32 k of X
  static_assert(GLU || ROPE, "the paired epilogues");
  static_assert(!ROPE || UNITS == 1, "one head half-pair a wave");
  static_assert(MPAD == 8 || MPAD == 16, "rows of X in LDS: a tile of 16, or half of one (lanes of rows 8 .. 15 then read rows 0 .. 7 again)");
  extern __shared__ __align__(16) unsigned char x_lds[];        // X, then the segments' sums [wave][tile][lane][4]
  // the norming waves are the block's first: they are at work before the others have started
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) - NORMED_NORM_WAVES;
  const int nw = (blockDim.x >> 6) - NORMED_NORM_WAVES;         // streaming waves: 0 .. nw - 1
  const int KB = K / 32;

  if (wave < 0) {
    // ------------------------------------------------------------------ a norming wave: rows w, w + 4, ..., two at a time
    // A row is `full` rounds of 64 float4 (K a multiple of 256); lane l holds the float4 l + 64 j.
    // In LDS that is block (l >> 3) + 8 j of X, chunk (l & 7) >> 1, half l & 1: one address a lane
    // and row, 8 blocks further for every j.
    const int full = K >> 8, first_row = wave + NORMED_NORM_WAVES;
    int ln = lane;
    asm volatile("" : "+v"(ln));        // what follows from the lane is worked out here, not kept in registers from the start
    uint2 gain_bf[KC];                                          // the gain (bfloat16): the lane's share, asked for behind the rows
    const int q = (ln & 7) >> 1;
    const unsigned swz = (q + 4 * ((ln >> 3) & 1)) & 7;           // slots of 16 bytes (a row's 8 k) are permuted within
    unsigned char* at0 = x_lds + (ln >> 3) * XBLOCK + (ln & 1) * 8;   // eights, by chunk and block parity: these stores,
                                                                  // which walk along a row, spread over the banks
    if (first_row >= M) __builtin_amdgcn_s_barrier();           // a wave without rows: the barrier of those with
    for (int m0 = first_row; m0 < M; m0 += 2 * NORMED_NORM_WAVES) {
      const int m1 = m0 + NORMED_NORM_WAVES;
      float4 kept[2][KC];
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const int m = min(r ? m1 : m0, M - 1);                   // no second row: the first again, not stored
        const float4* row = reinterpret_cast<const float4*>(in.rows + (size_t)m * in.rows_stride) + ln;
#pragma unroll
        for (int j = 0; j < KC; ++j)
          kept[r][j] = j < full ? row[64 * j] : make_float4(0.0f, 0.0f, 0.0f, 0.0f);     // (the same for every lane)
      }
      if (m0 == first_row) {
        // the rows are asked for: only now do the streaming waves ask for their W (the barrier alone,
        // which waits for no load; nothing moves across it)
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int j = 0; j < KC; ++j)
          if (j < full) gain_bf[j] = *reinterpret_cast<const uint2*>((const bf16_t*)in.gain + 4 * (ln + 64 * j));
      }
      // four chains a row as the norm kernel's four waves have them, then their butterflies, all
      // eight side by side
      float ss[2][4];
#pragma unroll
      for (int r = 0; r < 2; ++r) {
#pragma unroll
        for (int v = 0; v < 4; ++v) ss[r][v] = 0.0f;
#pragma unroll
        for (int j = 0; j < KC; ++j) {
          const float4 x = kept[r][j];
          ss[r][j & 3] = fmaf(x.x, x.x, ss[r][j & 3]);
          ss[r][j & 3] = fmaf(x.y, x.y, ss[r][j & 3]);
          ss[r][j & 3] = fmaf(x.z, x.z, ss[r][j & 3]);
          ss[r][j & 3] = fmaf(x.w, x.w, ss[r][j & 3]);
        }
      }
      // wave_sum's butterfly (lane l adds lane l ^ off, off = 32, 16, 8, 4, 2, 1): the same pairs, so
      // the same bits.  The steps across rows of 16 lanes go through the LDS crossbar, those within a
      // row through the adder's lane permutations, which cost an instruction and no round trip.
#define NORMED_DPP(val, old, ctrl, banks) \
  __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, val), ctrl, 0xf, banks, false))
#pragma unroll
      for (int off = 32; off >= 16; off >>= 1) {
        float other[2][4];
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
          for (int v = 0; v < 4; ++v) other[r][v] = __shfl_xor(ss[r][v], off, AXON_WAVE);
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
          for (int v = 0; v < 4; ++v) ss[r][v] += other[r][v];
      }
#pragma unroll
      for (int r = 0; r < 2; ++r)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          float x = ss[r][v];
          x += NORMED_DPP(x, 0.0f, 0x128, 0xf);                              // row_ror:8: lane l ^ 8
          const float up = NORMED_DPP(x, 0.0f, 0x104, 0x5);                  // row_shl:4 in lanes 0-3, 8-11: lane l + 4
          x += NORMED_DPP(x, up, 0x114, 0xa);                                // row_shr:4 in lanes 4-7, 12-15: lane l - 4
          x += NORMED_DPP(x, 0.0f, 0x4e, 0xf);                               // quad_perm [2, 3, 0, 1]: lane l ^ 2
          x += NORMED_DPP(x, 0.0f, 0xb1, 0xf);                               // quad_perm [1, 0, 3, 2]: lane l ^ 1
          ss[r][v] = x;
        }
#undef NORMED_DPP
      float inv[2];
      unsigned char* at[2];
#pragma unroll
      for (int r = 0; r < 2; ++r) {
        const float total = ((ss[r][0] + ss[r][1]) + ss[r][2]) + ss[r][3];
        inv[r] = 1.0f / sqrtf(total / (float)K + in.eps);
        at[r] = at0 + (((unsigned)(r ? m1 : m0) + MPAD * q) ^ swz) * 16;
      }
      const bool second = m1 < M;
      // a chunk of the gain at a time, for both rows
#pragma unroll
      for (int j = 0; j < KC; ++j) {
        if (j >= full) continue;                                 // (the same for every lane)
        const uint2 gb = gain_bf[j];
        const float4 gn = make_float4(__uint_as_float(gb.x << 16), __uint_as_float(gb.x & 0xffff0000u),
                                      __uint_as_float(gb.y << 16), __uint_as_float(gb.y & 0xffff0000u));
#pragma unroll
        for (int r = 0; r < 2; ++r) {
          if (r && !second) continue;
          const float4 x = kept[r][j];
          uint2 pk;
          pk.x = pack2_bf16((x.x * inv[r]) * gn.x, (x.y * inv[r]) * gn.y);
          pk.y = pack2_bf16((x.z * inv[r]) * gn.z, (x.w * inv[r]) * gn.w);
          *reinterpret_cast<uint2*>(at[r] + j * 8 * XBLOCK) = pk;
        }
      }
    }
    __syncthreads();                     // X is there
    if (SEGS > 1) __syncthreads();       // (the streaming waves exchange their sums)
    return;
  }

  // -------------------------------------------------------------------- a streaming wave
  const int seg = wave % SEGS, g = wave / SEGS, groups = nw / SEGS;
  const int r16 = lane & 15;
  float* partial = reinterpret_cast<float*>(x_lds + (size_t)KB * XBLOCK);
  int unit[UNITS];
  bool live[UNITS];
  const bf16_t* wtile[NT];
#pragma unroll
  for (int u = 0; u < UNITS; ++u) {
    const int at = ((int)blockIdx.x * groups + g) * UNITS + u;
    live[u] = at < n_units;
    unit[u] = min(at, n_units - 1);                             // past the last: the last again, nothing stored
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      int tile;
      if (GLU) tile = i * (N / 16) + unit[u];                    // gate rows, then the up rows of the same columns
      else {
        const int half = rope.head_dim / 2, per_head = half / 16;
        tile = ((unit[u] / per_head) * rope.head_dim + i * half) / 16 + unit[u] % per_head;
      }
      wtile[u * 2 + i] = w + (size_t)tile * KB * 512 + lane * 8;
    }
  }
  f32x4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

  const int nk = K / 64;
  const int first = (int)((long)seg * nk / SEGS);
  const int mine = (int)((long)(seg + 1) * nk / SEGS) - first;
  uint4 wf[DEPTH][NT][2];
  auto load = [&](int slot, int local) {
    const int k0 = (first + local) * 64;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      wf[slot][t][0] = *reinterpret_cast<const uint4*>(wtile[t] + k0 * 16);
      wf[slot][t][1] = *reinterpret_cast<const uint4*>(wtile[t] + k0 * 16 + 512);
    }
  };
  // X of a step: lane (row r16, chunk q of 8 k) reads the slot of (row, chunk) in the step's two blocks
  const int q4 = lane >> 4;
  const unsigned xslot = (r16 % MPAD) + MPAD * q4;
  const unsigned xoff0 = (xslot ^ (q4 & 7)) * 16, xoff1 = (xslot ^ ((q4 + 4) & 7)) * 16;
  auto multiply = [&](int slot, int local) {
    const unsigned char* xs = x_lds + (size_t)(first + local) * 2 * XBLOCK;
    const uint4 x0 = *reinterpret_cast<const uint4*>(xs + xoff0);
    const uint4 x1 = *reinterpret_cast<const uint4*>(xs + XBLOCK + xoff1);
#pragma unroll
    for (int t = 0; t < NT; ++t)
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(wf[slot][t][0]), as_frag(x0), acc[t], 0, 0, 0);
#pragma unroll
    for (int t = 0; t < NT; ++t)
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(wf[slot][t][1]), as_frag(x1), acc[t], 0, 0, 0);
  };
  RopeAhead<1> ahead;
  if (ROPE) ahead = rope_look_ahead<1, SEGS>(rope, seg, unit[0], lane, M);
  // The ring is filled once the norming waves have asked for their rows: the rings of every wave of
  // the chip at once are tens of megabytes, and rows asked for among them arrive last.
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
  if (ROPE) rope_look_ahead_page<1, SEGS>(ahead, rope, seg, unit[0], lane, M);
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) load(d, min(d, mine - 1));     // beyond this wave's steps: a valid step again
  __syncthreads();                                               // X is there

  {
    int base = 0;  // the ring holds local steps base .. base + DEPTH - 1
    for (; base + 2 * DEPTH <= mine; base += DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        multiply(d, base + d);
        load(d, base + DEPTH + d);
      }
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (base + d < mine) multiply(d, base + d);
      if (base + DEPTH + d < mine) load(d, base + DEPTH + d);
    }
#pragma unroll
    for (int d = 0; d < DEPTH; ++d)
      if (base + DEPTH + d < mine) multiply(d, base + DEPTH + d);
  }

  if (SEGS > 1) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
      *reinterpret_cast<f32x4*>(partial + (((size_t)wave * NT + t) * 64 + lane) * 4) = acc[t];
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < UNITS; ++u) {
    if (!live[u]) continue;
    // the segments' sums in segment order; lane: X row r16, W rows 4 (lane / 16) .. + 3 of tile t
    auto summed = [&](int t, int e) {
      if (SEGS == 1) return acc[u * 2 + t][e];
      float sum = partial[(((size_t)(g * SEGS) * NT + u * 2 + t) * 64 + lane) * 4 + e];
#pragma unroll
      for (int q = 1; q < SEGS; ++q) sum += partial[(((size_t)(g * SEGS + q) * NT + u * 2 + t) * 64 + lane) * 4 + e];
      return sum;
    };
    rows_epilogue<2, 1, EPI, SEGS>(summed, seg, unit[u], lane, bias, bias_is_f32, out, out_stride, M, N, mode, rope, ahead);
  }
}

// How a product with n / 16 (gated) or n / 32 pairs of row tiles is laid over blocks: streaming
// waves = groups x segs <= 4, a wave `per_wave` pairs, about one block a CU.  0 groups: not taken.
struct NormedShape {
  int groups, per_wave, blocks;
};

static NormedShape normed_shape(int units, int segs, bool gated) {
  const int most = NORMED_STREAM_WAVES / segs;                   // groups a block can hold
  const int per_block = ceil_div(units, 256);
  int per_wave = gated ? ceil_div(per_block, most) : 1;          // the rotary epilogue: one pair a wave
  if (per_wave > 3) per_wave = 3;
  int groups = ceil_div(per_block, per_wave);
  groups = groups < 1 ? 1 : groups > most ? most : groups;
  return NormedShape{groups, per_wave, ceil_div(units, groups * per_wave)};
}

// Whether a product of m rows of width k takes the norm inside: X (and the segments' sums) fit LDS,
// a lane holds a row's share in registers.
int gemm_normed_ok(int m, int k) {
  if (m < 1 || m > NORMED_MAX_M || k % 256 != 0 || k > 256 * NORMED_MAX_KC) return 0;     // whole rounds of 64 float4 a row
  if (k > 256 * 16 && m > 8) return 0;
  return (size_t)(k / 32) * (m <= 8 ? 8 : 16) * 64 + NORMED_STREAM_WAVES * 6 * 1024 <= NORMED_MAX_LDS;
}

template <int UNITS, int SEGS, int EPI>
static int launch_normed_of(const NormedRows& in, const bf16_t* w, const void* bias, int bias_is_f32, void* out, int out_stride,
                            int m, int n, int k, int mode, hipStream_t stream, const RopeStore& rope, int units,
                            const NormedShape& shape) {
  const int nw = shape.groups * SEGS;
  const size_t lds = (size_t)(k / 32) * (m <= 8 ? 8 : 16) * 64 + (SEGS > 1 ? (size_t)nw * 2 * UNITS * 1024 : 0);
#define NORMED_LAUNCH(MPAD, KCV)                                                                                         \
  {                                                                                                                   \
    auto kernel = &gemm_normed_kernel<UNITS, SEGS, UNITS == 1 ? 8 : UNITS == 2 ? 4 : 3, EPI, MPAD, KCV>;              \
    static bool configured = false;                                                                                   \
    if (!configured) {                                                                                                \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                         NORMED_MAX_LDS);                                                             \
      if (e != hipSuccess) {                                                                                          \
        axk_set_error("gemm_normed: cannot reserve %d bytes of LDS: %s", NORMED_MAX_LDS, hipGetErrorString(e));       \
        return -2;                                                                                                    \
      }                                                                                                               \
      configured = true;                                                                                              \
    }                                                                                                                 \
    AXK_INSTANCE(INST_GEMM_NORMED, UNITS, SEGS, EPI, MPAD, KCV);                                                      \
    kernel<<<shape.blocks, (nw + NORMED_NORM_WAVES) * 64, lds, stream>>>(in, w, bias, bias_is_f32, out, out_stride, m, n, k, \
                                                                         mode, rope, units);                          \
  }
  if (k > 256 * 16) NORMED_LAUNCH(8, NORMED_MAX_KC) else if (m <= 8) NORMED_LAUNCH(8, 16) else NORMED_LAUNCH(16, 16)
#undef NORMED_LAUNCH
  AXK_LAUNCH_CHECK("gemm_normed");
  return 0;
}

template <int EPI>
static int launch_normed(const NormedRows& in, const bf16_t* w, const void* bias, int bias_is_f32, void* out, int out_stride,
                         int m, int n, int k, int mode, hipStream_t stream, int segs, const RopeStore& rope) {
  const int units = EPI == EPI_GLU ? n / 16 : n / 32;
  const NormedShape shape = normed_shape(units, segs, EPI == EPI_GLU);
#define ARGS_NORMED in, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream, rope, units, shape
#define BY_SEGS(U)                                                    \
  switch (segs) {                                                     \
    case 1: return launch_normed_of<U, 1, EPI>(ARGS_NORMED);          \
    case 2: return launch_normed_of<U, 2, EPI>(ARGS_NORMED);          \
    case 4: return launch_normed_of<U, 4, EPI>(ARGS_NORMED);          \
  }
  if (shape.per_wave == 1) BY_SEGS(1)
  if constexpr (EPI == EPI_GLU) {
    if (shape.per_wave == 2) BY_SEGS(2)
    // three pairs a wave: only matrices so large that K is one segment (normed_shape, gemm_segments)
    if (shape.per_wave == 3 && segs == 1) return launch_normed_of<3, 1, EPI>(ARGS_NORMED);
  }
#undef BY_SEGS
#undef ARGS_NORMED
  axk_set_error("gemm_normed: %d segments, %d pairs of tiles a wave", segs, shape.per_wave);
  return -1;
}

// ---------------------------------------------------------------------------- gemm_rows
// 17 to 128 rows of X: still bound by reading W once, but X is now as large as a tile of W, and a
// wave that fetched its own X for every step (as gemm_stream does) would ask the caches for as
// many bytes of X as of W.  Here the WAVES waves of a block walk the same K together, each
// with its own NT16 row tiles of W streamed from memory straight into MFMA operands (a ring of
// NS - 1 steps of 64 k in flight), and share X: a step's X (16 MT16 rows x 64 k, 8 or 16 KB) goes straight
// into LDS once a block, in the blocks of 1 KB that one LDS read of a wave takes (16 rows x 32 k,
// lane l: row l % 16, 8 k from 8 (l / 16)), each wave fetching its share.  One barrier a step:
// behind it the step's X is there for everyone and the step before is read by everyone, so its
// place can be filled again.  A block works on one segment of K (blockIdx.y): with one segment
// it ends with the product's epilogue, with more it leaves its sums in `partial`
// [segment][gate | up][M][N] and the kernels that add such sums in segment order finish the
// product.  The chain of an output element is the same as in every other kernel: 16x16x32
// MFMAs in ascending k from zero over its segment.
template <int NT16, int MT16, int WAVES, int NS, int EPI>
__global__ void __launch_bounds__(WAVES * 64, 2)      // two waves a SIMD: 256 registers each
gemm_rows_kernel(const bf16_t* __restrict__ x, int x_stride, const bf16_t* __restrict__ w, const void* __restrict__ bias,
                 int bias_is_f32, void* __restrict__ out, int out_stride, int M, int N, int K, int mode,
                 float* __restrict__ partial, int n_units) {
  constexpr bool GLU = EPI == EPI_GLU;
  // every wave fetches XI blocks of X a step (where the waves do not divide the blocks, some
  // twice: the same bytes to the same place), so that every wave counts the same loads
  constexpr int XB = MT16 * 2, XI = (XB + WAVES - 1) / WAVES, WI = NT16 * 2, LOADS = XI + WI;
  static_assert(EPI == EPI_PLAIN || (EPI == EPI_GLU && NT16 == 2), "plain tiles, or gate and up tiles of the same columns");
  static_assert((NS - 2) * LOADS < 64, "the counter of loads in flight has six bits");
  extern __shared__ __align__(16) unsigned char x_ring[];      // [NS][XB][1 KB]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int unit = min((int)blockIdx.x * WAVES + wave, n_units - 1);     // past the last: the last again, nothing stored
  const bool live = (int)blockIdx.x * WAVES + wave < n_units;
  const int segs = gridDim.y, seg = blockIdx.y;
  const int KB = K / 32;
  const bf16_t* wtile[NT16];
#pragma unroll
  for (int i = 0; i < NT16; ++i) {
    int tile;
    if (GLU) tile = i * (N / 16) + unit;
    else tile = min(unit * NT16 + i, (N + 15) / 16 - 1);
    wtile[i] = w + (size_t)tile * KB * 512 + lane * 8;
  }
  // this wave's blocks of X: block b = (16 rows j, 32 k h), lane: row 16 j + lane % 16, 8 k from 8 (lane / 16)
  const bf16_t* xsrc[XI];
  int xdst[XI];
#pragma unroll
  for (int q = 0; q < XI; ++q) {
    const int b = (wave * XI + q) % XB;
    xsrc[q] = x + (size_t)min((b >> 1) * 16 + (lane & 15), M - 1) * x_stride + (b & 1) * 32 + (lane >> 4) * 8;
    xdst[q] = b * 1024;
  }
  const int nk = K / 64;
  const int first = (int)((long)seg * nk / segs);
  const int mine = (int)((long)(seg + 1) * nk / segs) - first;      // the same for every wave of the block
  const unsigned ring0 = (unsigned)(size_t)(lds_ptr_t)x_ring;

  f32x4 acc[NT16][MT16];
#pragma unroll
  for (int i = 0; i < NT16; ++i)
#pragma unroll
    for (int j = 0; j < MT16; ++j) acc[i][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  // In whole rounds of the ring every step issues the loads of the step NS - 1 ahead, also past
  // the segment's end (then its last step again, which the cache still holds, into places nobody
  // reads); the steps left after the last whole round issue nothing.  So the number of loads in
  // flight at every wait is fixed by the code alone, for the kernel's count and for the compiler's.
  uint4 wf[NS][NT16][2];
  auto issue = [&](int slot, int local) {
    const int k0 = (first + min(local, mine - 1)) * 64;
    // X straight into LDS, written as an instruction (M0: where the wave's 1 KB goes): the compiler,
    // seeing such a load in a loop, would wait for every load in flight once a round of the ring.
    // It then counts the loads of W alone and waits a little earlier than it must: never too late.
#pragma unroll
    for (int q = 0; q < XI; ++q) {
      const bf16_t* src = xsrc[q] + k0;
      const unsigned dst = __builtin_amdgcn_readfirstlane(ring0 + slot * XB * 1024 + xdst[q]);
      unsigned kept;                                      // M0 goes back as it was: the compiler counts on it
      asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
                   : "=&s"(kept)
                   : "v"(src), "s"(dst)
                   : "memory");
    }
#pragma unroll
    for (int i = 0; i < NT16; ++i) {
      wf[slot][i][0] = *reinterpret_cast<const uint4*>(wtile[i] + k0 * 16);          // k block k0 / 32: 512 elements each
      wf[slot][i][1] = *reinterpret_cast<const uint4*>(wtile[i] + k0 * 16 + 512);
    }
  };
  // one step: behind the barrier its X is in LDS for every wave and nobody reads the step before
  // any more (the bare barrier: the fence of __syncthreads would wait for every load under way)
  // (the second half of the step's k is read while the first is multiplied)
  auto multiply = [&](int d) {
    u32x4 xf[2][MT16];
    read_frags<MT16, 2048>(xf[0], ring0 + d * (XB * 1024) + lane * 16);
    read_frags<MT16, 2048>(xf[1], ring0 + d * (XB * 1024) + 1024 + lane * 16);
    wait_lgkmcnt<MT16>();
    use_frags<MT16>(xf[0]);
#pragma unroll
    for (int i = 0; i < NT16; ++i)
#pragma unroll
      for (int j = 0; j < MT16; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(wf[d][i][0]), as_frag(xf[0][j]), acc[i][j], 0, 0, 0);
    wait_lgkmcnt<0>();
    use_frags<MT16>(xf[1]);
#pragma unroll
    for (int i = 0; i < NT16; ++i)
#pragma unroll
      for (int j = 0; j < MT16; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(wf[d][i][1]), as_frag(xf[1][j]), acc[i][j], 0, 0, 0);
  };
  static_assert(NS >= 4 && NS <= 8, "the ring of steps");
#pragma unroll
  for (int d = 0; d < NS - 1; ++d) issue(d, d);
  int base = 0;
  for (; base + NS <= mine; base += NS) {
#pragma unroll
    for (int d = 0; d < NS; ++d) {
      wait_vmcnt<(NS - 2) * LOADS>();      // this step's loads have landed (loads return in order)
      __builtin_amdgcn_s_barrier();
      issue((d + NS - 1) % NS, base + d + NS - 1);
      multiply(d);
    }
  }
  const int left = mine - base;            // 0 .. NS - 1 steps, their loads under way already; the same for every wave
#define ROWS_LAST(T)                                                \
  if (T < NS - 1 && left > T) {                                     \
    wait_vmcnt<(NS - 2 - (T < NS - 2 ? T : NS - 2)) * LOADS>();     \
    __builtin_amdgcn_s_barrier();                                   \
    multiply(T);                                                    \
  }
  ROWS_LAST(0) ROWS_LAST(1) ROWS_LAST(2) ROWS_LAST(3) ROWS_LAST(4) ROWS_LAST(5) ROWS_LAST(6)
#undef ROWS_LAST
  wait_vmcnt<0>();                         // the loads past the end: nothing of this block is in flight when it leaves
  if (!live) return;
  if (partial) {
    // [segment][gate | up][M][N], 32-bit sums as they are; a lane: 4 consecutive columns of a row
    constexpr int PARTS = GLU ? 2 : 1;
#pragma unroll
    for (int i = 0; i < NT16; ++i) {
      const int part = GLU ? i : 0;
      const int n = (GLU ? unit : unit * NT16 + i) * 16 + (lane >> 4) * 4;
      if (n >= N) continue;
      float* dst = partial + ((size_t)seg * PARTS + part) * M * N + n;
#pragma unroll
      for (int j = 0; j < MT16; ++j) {
        const int m = j * 16 + (lane & 15);
        if (m >= M) continue;
        if (N % 4 == 0) {
          *reinterpret_cast<float4*>(dst + (size_t)m * N) = make_float4(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
        } else {                                                   // rows of the workspace that are not 16-byte aligned
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) dst[(size_t)m * N + e] = acc[i][j][e];
        }
      }
    }
    return;
  }
  auto summed = [&](int t, int e) { return acc[t / MT16][t % MT16][e]; };
  rows_epilogue<NT16, MT16, EPI, 1>(summed, 0, unit, lane, bias, bias_is_f32, out, out_stride, M, N, mode, RopeStore(),
                                    RopeAhead<MT16>());
}

// The ring of steps: eight for up to 64 rows; with 128 rows a step's X is 16 KB and the sums take
// twice the registers, so four steps (two row tiles a wave: 12 KB of W in flight a wave) or six.
template <int NT16, int MT16>
struct RowsRing {
  static constexpr int NS = MT16 <= 4 ? 8 : NT16 == 2 ? 4 : 6;
};

template <int NT16, int MT16, int WAVES, int EPI>
static int launch_rows_of(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                          int out_stride, int m, int n, int k, int mode, hipStream_t stream, int segs, float* partial, int units) {
  constexpr int NS = RowsRing<NT16, MT16>::NS, lds_bytes = NS * MT16 * 2 * 1024;
  static_assert(lds_bytes <= 160 * 1024, "the ring does not fit the LDS of a CU");
  auto kernel = &gemm_rows_kernel<NT16, MT16, WAVES, NS, EPI>;
  static bool configured = lds_bytes <= 64 * 1024;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                       lds_bytes);
    if (e != hipSuccess) {
      axk_set_error("gemm_rows: cannot reserve %d bytes of LDS: %s", lds_bytes, hipGetErrorString(e));
      return -2;
    }
    configured = true;
  }
  AXK_INSTANCE(INST_GEMM_ROWS, NT16, MT16, WAVES, EPI);
  kernel<<<dim3(ceil_div(units, WAVES), segs), WAVES * 64, lds_bytes, stream>>>(
      x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, segs > 1 ? partial : nullptr, units);
  AXK_LAUNCH_CHECK("gemm_rows");
  return 0;
}

// A CU streams at its own pace however many blocks it holds, so the waves of a block are as many
// as it takes to give each of the chip's 256 CUs one block (at most eight: two a SIMD).
template <int NT16, int MT16, int EPI>
static int launch_rows(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                       int out_stride, int m, int n, int k, int mode, hipStream_t stream, int segs, float* partial,
                       const SplitNorm* norm, const RopeStore* rope) {
  const int units = EPI == EPI_GLU ? n / 16 : ceil_div(ceil_div(n, 16), NT16);
  constexpr int LEAST = MT16 <= 4 ? 2 : 3;      // 128 rows with two waves: each would fetch half of X and spill
  int waves = ceil_div(units * segs, 256);
  waves = waves < LEAST ? LEAST : waves > 8 ? 8 : waves;
#define ARGS_ROWS x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream, segs, partial, units
  int rc = -1;
  switch (waves) {
    case 2:
      if constexpr (LEAST <= 2) rc = launch_rows_of<NT16, MT16, 2, EPI>(ARGS_ROWS);
      break;
    case 3: rc = launch_rows_of<NT16, MT16, 3, EPI>(ARGS_ROWS); break;
    case 4: rc = launch_rows_of<NT16, MT16, 4, EPI>(ARGS_ROWS); break;
    case 5: rc = launch_rows_of<NT16, MT16, 5, EPI>(ARGS_ROWS); break;
    case 6: rc = launch_rows_of<NT16, MT16, 6, EPI>(ARGS_ROWS); break;
    case 7: rc = launch_rows_of<NT16, MT16, 7, EPI>(ARGS_ROWS); break;
    default: rc = launch_rows_of<NT16, MT16, 8, EPI>(ARGS_ROWS); break;
  }
#undef ARGS_ROWS
  if (rc != 0) return rc;
  return segs > 1 ? add_split_sums(partial, segs, m, n, bias, bias_is_f32, out, out_stride, mode, norm, rope, stream) : 0;
}

template <int NT16, int MT16, int SEGS, int EPI>
static int launch_stream(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                         int out_stride, int m, int n, int k, int mode, hipStream_t stream, const RopeStore& rope) {
  // the ring as deep as the registers allow: (NT16 + MT16) 8 registers a step
  constexpr int FIT = 384 / ((NT16 + MT16) * 8), DEPTH = FIT < 8 ? FIT : 8;
  AXK_INSTANCE(INST_GEMM_STREAM, NT16, MT16, SEGS, EPI);
  gemm_stream_kernel<NT16, MT16, SEGS, DEPTH, EPI><<<ceil_div(n, EPI == EPI_GLU ? 16 : NT16 * 16), SEGS * 64, 0, stream>>>(
      x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, rope);
  AXK_LAUNCH_CHECK("gemm_stream");
  return 0;
}

template <int NT16, int EPI>
static int launch_stream_rows(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                              int out_stride, int m, int n, int k, int mode, hipStream_t stream, int segs,
                              const RopeStore& rope) {
#define ARGS x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream, rope
#define BY_SEGS(MT16)                                                   \
  switch (segs) {                                                       \
    case 1: return launch_stream<NT16, MT16, 1, EPI>(ARGS);             \
    case 2: return launch_stream<NT16, MT16, 2, EPI>(ARGS);             \
    case 4: return launch_stream<NT16, MT16, 4, EPI>(ARGS);             \
  }
  // two row tiles a block without a paired epilogue: matrices of 16,384 rows or more, which have
  // one or two segments, never four (gemm_segments)
  if constexpr (NT16 == 2 && EPI == EPI_PLAIN) {
    if (segs == 1) return launch_stream<NT16, 1, 1, EPI>(ARGS);
    if (segs == 2) return launch_stream<NT16, 1, 2, EPI>(ARGS);
  } else {
    BY_SEGS(1)
  }
#undef BY_SEGS
#undef ARGS
  axk_set_error("gemm_stream: %d segments", segs);
  return -1;
}

// Two row tiles a block where the matrix is large (the paired epilogues always), one where that
// gives the chip more blocks.
template <int EPI>
static int launch_stream_any(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                             int out_stride, int m, int n, int k, int mode, hipStream_t stream, int segs,
                             const RopeStore& rope) {
  if (EPI != EPI_PLAIN || n >= 32 * 512)
    return launch_stream_rows<2, EPI>(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream, segs, rope);
  return launch_stream_rows<EPI == EPI_PLAIN ? 1 : 2, EPI>(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode,
                                                           stream, segs, rope);
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
// The number of segments K is cut into for a matrix of `tiles32` tiles of 32 rows (ceil(N / 32);
// N / 16 for a [gate; up] matrix of 2 N rows) and K columns: 1, 2 or 4, so that a step of few rows
// still gives some 768 waves a chain of their own, with at least 4 K tiles (256 k) a segment.
// It is a property of the matrix: it fixes the order of addition of every product with it.
// Measured on the 7B and 14B widths: more segments help steps of 33 to 256 rows (more blocks)
// and cost long prompts (more sums through the workspace); 4 is the balance.
int gemm_segments(int tiles32, int k) {
  const int nk = k / 64;
  int s = 1;
  while (s < 4 && tiles32 * s < 768 && nk / (2 * s) >= 4) s *= 2;
  return s;
}

static int tiles32_of(int n, int mode) { return mode == MODE_SWIGLU ? n / 16 : (n + 31) / 32; }

// The most rows the streaming kernel takes: with more, its waves, which fetch X each for itself,
// ask the caches for as much of X as of W, and the kernel that shares X within a block is faster
// (measured on the products of a 7B layer: from 17 rows on, by 10 to 30 %).
#define AXON_STREAM_MAX_M 16

// More rows than the streaming kernel takes, S > 1 segments: a block a segment; the blocks' sums
// go through a workspace and are added in segment order by a second kernel (measured faster for
// every product of the 7B and 14B layers up to 8,192 rows than keeping the segments apart in one
// block's registers, and the only way to occupy the chip when the output is small).  The
// workspace holds the sums of at most GEMM_PASS_BYTES: a product of more rows runs in passes of
// `rows_a_pass` rows, one after the other (a row's bits do not depend on the rows beside it).
#define GEMM_PASS_BYTES ((size_t)2048 << 20)

static int rows_a_pass(int n, int mode, int segs) {
  const size_t row_bytes = (size_t)segs * (mode == MODE_SWIGLU ? 2 : 1) * n * sizeof(float);
  const size_t rows = GEMM_PASS_BYTES / row_bytes / 256 * 256;       // whole tiles of 256 rows
  return (int)(rows < 256 ? 256 : rows > (1u << 30) ? (1u << 30) : rows);
}

size_t gemm_workspace_bytes(int m, int n, int k, int mode) {
  if (k % 64 != 0 || m <= AXON_STREAM_MAX_M) return 0;
  const int s = gemm_segments(tiles32_of(n, mode), k);
  if (s <= 1) return 0;
  const int rows = m < rows_a_pass(n, mode, s) ? m : rows_a_pass(n, mode, s);
  return (size_t)s * (mode == MODE_SWIGLU ? 2 : 1) * rows * n * sizeof(float);
}

// Whether the product that adds into the rows runs with a block a segment, so that the kernel that
// adds the segments' sums can also norm the finished rows (gemm_split_reduce_norm_kernel: rows of
// up to SRN_MAX_N columns, in whole float4).
int gemm_then_norm_ok(int m, int n, int k) {
  return gemm_pack_ok(n, k, 0) && m > AXON_STREAM_MAX_M && n <= SRN_MAX_N && n % 4 == 0 &&
         gemm_segments(tiles32_of(n, MODE_ADD_F32), k) > 1;
}

static int gemm_mfma_pass(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                          int out_stride, int m, int n, int k, int mode, hipStream_t stream, int segs, const SplitNorm* norm,
                          float* ws, const RopeStore* rope_after);

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
  const int segs = gemm_segments(tiles32_of(n, mode), k);
  if (m <= AXON_STREAM_MAX_M) {
    if (norm || rope_after) {
      axk_set_error("gemm: M=%d goes to the streaming kernel, which has these epilogues of its own", m);
      return -1;
    }
    if (mode == MODE_SWIGLU)
      return launch_stream_any<EPI_GLU>(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream, segs, RopeStore());
    return launch_stream_any<EPI_PLAIN>(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream, segs, RopeStore());
  }
  if ((norm || rope_after) && (segs <= 1 || mode != (norm ? MODE_ADD_F32 : MODE_STORE))) {
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
  const int pass = segs > 1 ? rows_a_pass(n, mode, segs) : m;
  if (m <= pass)
    return gemm_mfma_pass(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream, segs, norm,
                          (float*)workspace, rope_after);
  // in passes: every operand that has a row per row of X moves on with it
  const size_t out_elem = mode == MODE_STORE || mode == MODE_SWIGLU ? sizeof(bf16_t) : sizeof(float);
  for (int m0 = 0; m0 < m; m0 += pass) {
    const int rows = m - m0 < pass ? m - m0 : pass;
    SplitNorm norm_at;
    RopeStore rope_at;
    if (norm) {
      norm_at = *norm;
      norm_at.values += (size_t)m0 * n;
    }
    if (rope_after) {
      rope_at = *rope_after;
      rope_at.table += (size_t)m0 * (rope_at.head_dim / 2) * 2;
      rope_at.positions += m0;
      rope_at.seq_rows += m0;
    }
    const int rc = gemm_mfma_pass(x + (size_t)m0 * x_stride, x_stride, w, bias, bias_is_f32,
                                  (char*)out + (size_t)m0 * out_stride * out_elem, out_stride, rows, n, k, mode, stream, segs,
                                  norm ? &norm_at : nullptr, (float*)workspace, rope_after ? &rope_at : nullptr);
    if (rc != 0) return rc;
  }
  return 0;
}

// One pass: more than AXON_STREAM_MAX_M rows whose segments' sums (if S > 1) fit the workspace.
static int gemm_mfma_pass(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, void* out,
                          int out_stride, int m, int n, int k, int mode, hipStream_t stream, int segs, const SplitNorm* norm,
                          float* ws, const RopeStore* rope_after) {
#define ARGS x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, mode, stream
  const bool glu = mode == MODE_SWIGLU;
  if (m <= 64) {
    // W streamed, X shared through LDS; a block a segment.  Two row tiles a wave where the matrix is large.
    if (glu) return launch_rows<2, 4, EPI_GLU>(ARGS, segs, ws, nullptr, nullptr);
    if (n >= 32 * 512) return launch_rows<2, 4, EPI_PLAIN>(ARGS, segs, ws, norm, rope_after);
    return launch_rows<1, 4, EPI_PLAIN>(ARGS, segs, ws, norm, rope_after);
  }
  if (m <= 128) {
    // the same with 128 rows of X a step: still bound by reading W (a tile kernel's blocks are too few here)
    if (glu) return launch_rows<2, 8, EPI_GLU>(ARGS, segs, ws, nullptr, nullptr);
    if (n >= 32 * 512) return launch_rows<2, 8, EPI_PLAIN>(ARGS, segs, ws, norm, rope_after);
    return launch_rows<1, 8, EPI_PLAIN>(ARGS, segs, ws, norm, rope_after);
  }
  // 256 x 256 tiles (8 waves, a block a CU) or 128 x 128 tiles (4 waves, two blocks a CU, four
  // times as many blocks at twice the traffic from L2 per product): whichever takes the chip's 256
  // CUs fewer rounds, a round of the small tiles counted as 0.65 of a round of the large ones
  // (measured on the four products of the 7B and 14B layers at 200 to 2,048 rows: the rule picks
  // the faster tile in 66 of 70 cases and loses 7 % at most in the others).
  const long big = (long)ceil_div(m, 256) * ceil_div(n, glu ? 128 : 256) * segs;
  const long small = (long)ceil_div(m, 128) * ceil_div(n, glu ? 64 : 128) * segs;
  const long rounds_big = (big + 255) / 256, rounds_small = (small + 511) / 512;
  const bool use_big = rounds_big * 100 <= rounds_small * 65;
  if (!use_big) {
    // Up to 256 rows still wait for W more than for the matrix cores.  Where the small tiles are no
    // more blocks than CUs, a block has its CU's LDS to itself: four stages instead of two, three
    // steps of loads in flight (the down projection of a 7B layer at 256 rows 79 -> 64 us); with
    // more blocks two of them share a CU and cover each other's waits (four stages there: slower).
    const bool deep = m <= 256 && small <= 256;
    if (glu) {
      if (deep) return launch_tile<128, 128, 2, 2, true, 64, 4>(ARGS, segs, ws);
      return launch_tile<128, 128, 2, 2, true>(ARGS, segs, ws);
    }
    if (deep) return launch_tile<128, 128, 2, 2, false, 64, 4>(ARGS, segs, ws, norm, rope_after);
    return launch_tile<128, 128, 2, 2, false>(ARGS, segs, ws, norm, rope_after);
  }
  if (glu) return launch_tile<256, 256, 4, 2, true>(ARGS, segs, ws);
  // one round of 256 x 256 tiles that leaves a quarter of the CUs idle, and N in whole tiles of
  // 192 columns that still fit one round: the narrower tile (measured 1.1 times the cost per
  // product, three quarters of the products per block).
  if (segs == 1 && big <= 192 && n % 192 == 0 && (long)ceil_div(m, 256) * (n / 192) <= 256)
    return launch_tile<256, 192, 4, 2, false>(ARGS, segs, ws, norm);
  return launch_tile<256, 256, 4, 2, false>(ARGS, segs, ws, norm, rope_after);
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

// The [q; k; v] product with rotary encoding and cache store (see RopeStore): up to 16 rows in
// the epilogue of gemm_stream, more rows where the product runs with a block a segment (then the
// kernel that adds the segments' sums rotates and stores); every head rotated over its whole
// width, halves of a head a multiple of 16 wide.
int gemm_qkv_rope_ok(int m, int n, int k, int head_dim, int rotary_dim) {
  if (m < 1 || k % 64 != 0 || rotary_dim != head_dim || head_dim % 32 != 0 || n % head_dim != 0) return 0;
  if (!gemm_pack_ok(n, k, 0)) return 0;
  if (m <= AXON_STREAM_MAX_M) return 1;
  return gemm_segments(tiles32_of(n, MODE_STORE), k) > 1;
}

int launch_gemm_qkv_rope(const bf16_t* x, int x_stride, const bf16_t* w, const void* bias, int bias_is_f32, bf16_t* out,
                         int out_stride, int m, int n, int k, const float* table, const int32_t* positions,
                         const int32_t* seq_rows, const int32_t* block_table, int table_stride, bf16_t* k_cache,
                         bf16_t* v_cache, int n_heads, int n_kv_heads, int head_dim, int page_size, void* workspace,
                         size_t workspace_bytes, hipStream_t stream) {
  const RopeStore rope = {table, positions, seq_rows, block_table, table_stride, k_cache, v_cache,
                          n_heads, n_kv_heads, head_dim, page_size};
  if (m > AXON_STREAM_MAX_M)
    return gemm_mfma_dispatch(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, MODE_STORE, stream, nullptr,
                              workspace, workspace_bytes, &rope);
  return launch_stream_any<EPI_ROPE>(x, x_stride, w, bias, bias_is_f32, out, out_stride, m, n, k, MODE_STORE, stream,
                                     gemm_segments(n / 32, k), rope);
}

// The gated product and the [q; k; v] product of few rows with the RMS norm of their operand
// inside (gemm_normed_kernel): rows are the float32 rows the norm would read.
int launch_gemm_normed_glu(const float* rows, int rows_stride, const bf16_t* gain, float eps, const bf16_t* w, bf16_t* out,
                           int out_stride, int m, int n, int k, hipStream_t stream) {
  const NormedRows in = {rows, rows_stride, gain, eps};
  return launch_normed<EPI_GLU>(in, w, nullptr, 0, out, out_stride, m, n, k, MODE_SWIGLU, stream,
                                gemm_segments(tiles32_of(n, MODE_SWIGLU), k), RopeStore());
}

int launch_gemm_normed_qkv_rope(const float* rows, int rows_stride, const bf16_t* gain, float eps,
                                const bf16_t* w, const void* bias, int bias_is_f32, bf16_t* out, int out_stride, int m, int n,
                                int k, const float* table, const int32_t* positions, const int32_t* seq_rows,
                                const int32_t* block_table, int table_stride, bf16_t* k_cache, bf16_t* v_cache, int n_heads,
                                int n_kv_heads, int head_dim, int page_size, hipStream_t stream) {
  const NormedRows in = {rows, rows_stride, gain, eps};
  const RopeStore rope = {table, positions, seq_rows, block_table, table_stride, k_cache, v_cache,
                          n_heads, n_kv_heads, head_dim, page_size};
  return launch_normed<EPI_ROPE>(in, w, bias, bias_is_f32, out, out_stride, m, n, k, MODE_STORE, stream,
                                 gemm_segments(n / 32, k), rope);
}

#endif  // AXON_BF16
