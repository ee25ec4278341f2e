// Paged causal attention on the matrix cores (bfloat16 build only): one kernel for prompt
// portions, one for decoding tokens.  Both keep the order of attention.hip: positions in
// blocks of 64 aligned to absolute position, folded in ascending order with running
// (max, sum, output); the decoding kernel gives every block of 64 positions to a wave of its
// own, folds the four waves of a chunk of 256 positions in wave order (sizes that depend on
// nothing) and a second kernel folds the chunks' partial results in ascending order.  No atomics.  Scores, softmax and all sums are 32-bit; q, k, v and the
// softmax weights enter the MFMAs as bfloat16.
//
// Both compute the TRANSPOSED products, S^T = K Q^T and O^T = V^T P^T, so that what one MFMA
// leaves in a lane's registers is what the next one wants there, without a trip through LDS:
// after S^T a lane holds, for ONE query, several key positions; the softmax over positions is
// then a loop over the lane's registers plus one or two exchanges between lane groups, and the
// rounded weights are already laid out as the B operand of O^T.  The MFMA's k slots are
// matched to the positions a lane holds by reading V^T accordingly (values are cached
// position-contiguous: [page][kv head][dim][slot]).
#include <math.h>

#include "api.h"
#include "common.h"

#define DC_CHUNK 256          // positions of one chunk of a decoding token's range
#define CMB_MAX_CHUNKS 1024   // the most chunks of a token; the factor of the token's slot in a work item

#if AXON_BF16

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef const __attribute__((address_space(1))) void* global_ptr_t;
typedef __attribute__((address_space(3))) void* lds_ptr_t;

#define LOG2E 1.4426950408889634f

__device__ inline bf16x8 frag_of(uint4 v) {
  union { uint4 u; bf16x8 f; } c;
  c.u = v;
  return c.f;
}

__device__ inline bf16x8 frag_of2(uint2 lo, uint2 hi) {
  union { uint2 u[2]; bf16x8 f; } c;
  c.u[0] = lo;
  c.u[1] = hi;
  return c.f;
}

__device__ inline uint32_t pack_bf16(float a, float b) { return pack2_bf16(a, b); }

// ============================================================================ prompt portions
// grid (tiles, kv heads x groups of HPB query heads); a tile is up to 128 consecutive tokens of
// one request.  4 waves per query head, each owning 32 query rows; with HPB = 2 two query heads of
// the same kv head share every K and V^T block in LDS (the path from L2 into LDS carries about 32
// bytes a cycle and CU, which is what one head's products use up).  Per block of 64 key positions the waves bring K [64][HD] and
// V^T [HD][64] into LDS with direct global -> LDS loads (two stages: the next block's loads are
// in flight while this one is multiplied).  16-byte slots of an LDS row are permuted
// (slot ^ row & 7) so that fragment reads of neighbouring rows fall into different banks.
#define PF_TOKENS 128
#define PF_BLOCK 64

template <int HD, int HPB>
__device__ __forceinline__ void
attention_prefill_tile(unsigned char* smem, int t0, int count, const bf16_t* __restrict__ q, int q_stride,
                       const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                       const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ positions,
                       const int32_t* __restrict__ seq_rows, bf16_t* __restrict__ out, int n_heads, int n_kv_heads,
                       int page_size, int window, float scale) {
  constexpr int K_BYTES = PF_BLOCK * HD * 2;      // K tile: 64 rows of HD
  constexpr int V_BYTES = HD * PF_BLOCK * 2;      // V^T tile: HD rows of 64 positions
  constexpr int STAGE = K_BYTES + V_BYTES;
  constexpr int KROW = HD * 2;                    // bytes per K row
  constexpr int KCH = HD / 8;                     // 16-byte slots per K row
  constexpr int K_ROWS_PER_INSTR = 1024 / KROW;
  constexpr int NW = 4 * HPB;                               // waves of the block
  constexpr int K_INSTR = PF_BLOCK / K_ROWS_PER_INSTR / NW;  // per wave
  constexpr int V_INSTR = HD / 8 / NW;                       // V^T: 8 rows per instruction
  static_assert(K_INSTR >= 1 && V_INSTR >= 1, "more waves than load instructions");
  constexpr int DT = HD / 32;                     // output tiles (32 dims each)
  constexpr int KS = HD / 16;                     // k steps of S^T

  const int tid = threadIdx.x, lane = tid & 63, block_wave = tid >> 6;
  const int wave = block_wave & 3;                 // which 32 query rows of the tile
  const int group = n_heads / n_kv_heads, sets = (group + HPB - 1) / HPB;   // sets of HPB query heads per kv head
  const int kvh = blockIdx.y / sets;
  const int in_group = (blockIdx.y % sets) * HPB + (block_wave >> 2);
  const bool head_live = in_group < group;         // an odd group leaves the last set's second half idle
  const int head = kvh * group + min(in_group, group - 1);
  const int pos0 = positions[t0];
  const int32_t* table_row = block_table + (size_t)seq_rows[t0] * table_stride;
  const int hi = pos0 + count - 1;                               // last position any row of the tile sees
  const int lo = window > 0 ? max(0, pos0 + 1 - window) : 0;     // first position any row sees
  const int first_block = (lo / PF_BLOCK) * PF_BLOCK;
  const int n_blocks = (hi - first_block) / PF_BLOCK + 1;

  const int l32 = lane & 31, half = lane >> 5;
  const int my_row = wave * 32 + l32;                            // this lane's query row in the tile
  const int my_pos = pos0 + min(my_row, count - 1);
  const int my_lo = window > 0 ? max(0, my_pos + 1 - window) : 0;
  const int wave_hi = pos0 + min(wave * 32 + 31, count - 1);     // last position this wave's rows see
  const int wave_lo = window > 0 ? max(0, wave_hi + 1 - window) : 0;  // the latest window start among them
  const bool wave_live = head_live && wave * 32 < count;

  // Q^T fragments (B operand): column = query row, 8 consecutive dims from 16 ks + 8 half
  bf16x8 qf[KS];
  {
    const bf16_t* qrow = q + (size_t)(t0 + min(my_row, count - 1)) * q_stride + (size_t)head * HD + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qf[ks] = frag_of(*reinterpret_cast<const uint4*>(qrow + ks * 16));
  }

  const size_t kv_head_stride = (size_t)HD * page_size;           // elements of one (page, kv head)
  // The pages a block of positions lies in are looked up one block ahead of the loads that use
  // them, so that no load waits for a table entry behind the loads issued just before it.
  int k_page[K_INSTR], v_page[V_INSTR];
  auto lookup = [&](int b) {
    const int p0 = first_block + b * PF_BLOCK;
#pragma unroll
    for (int n = 0; n < K_INSTR; ++n) {
      const int row = (n * NW + block_wave) * K_ROWS_PER_INSTR + lane / KCH;
      k_page[n] = table_row[min(p0 + row, hi) / page_size];       // rows past the tile's last position: any valid row
    }
#pragma unroll
    for (int n = 0; n < V_INSTR; ++n) {
      const int d = (n * NW + block_wave) * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ (d & 7);
      v_page[n] = table_row[min(p0 + chunk * 8, hi) / page_size];
    }
  };
  auto issue = [&](int b) {
    unsigned char* stage = smem + (b & 1) * STAGE;
    const int p0 = first_block + b * PF_BLOCK;
    // K: lane i of an instruction brings row i / KCH, slot i % KCH holding chunk slot ^ (row & 7)
#pragma unroll
    for (int n = 0; n < K_INSTR; ++n) {
      const int instr = n * NW + block_wave;
      const int row = instr * K_ROWS_PER_INSTR + lane / KCH;
      const int chunk = (lane % KCH) ^ (row & 7);
      const int p = min(p0 + row, hi);
      const bf16_t* src = k_cache + ((size_t)k_page[n] * n_kv_heads + kvh) * kv_head_stride +
                          (size_t)(p % page_size) * HD + chunk * 8;
      __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + instr * 1024), 16, 0, 0);
    }
    // V^T: lane i brings row (dim) i / 8, slot i % 8 holding the 8 positions of chunk slot ^ (row & 7)
#pragma unroll
    for (int n = 0; n < V_INSTR; ++n) {
      const int instr = n * NW + block_wave;
      const int d = instr * 8 + (lane >> 3);
      const int chunk = (lane & 7) ^ (d & 7);
      const int p = min(p0 + chunk * 8, hi);
      const bf16_t* src = v_cache + ((size_t)v_page[n] * n_kv_heads + kvh) * kv_head_stride +
                          (size_t)d * page_size + ((p % page_size) & ~7);
      __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + K_BYTES + instr * 1024), 16, 0, 0);
    }
  };

  f32x16 o_acc[DT];
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  const float c = scale * LOG2E;

  // Fragment reads are written as instructions (see common.h).  Row r of an S^T tile is key
  // position pi(r) of the tile, pi swapping bits 2 and 3 of r: a lane then ends with weights of
  // 8 CONSECUTIVE positions per k step of O^T, which are one 16-byte read of a V^T row.
  const unsigned lds0 = (unsigned)(size_t)(lds_ptr_t)smem;
  const int k_row = (l32 & 0x13) | ((l32 & 4) << 1) | ((l32 & 8) >> 1);
  const unsigned k_at = lds0 + k_row * KROW, k_swz = k_row & 7;
  const unsigned v_at = lds0 + K_BYTES + l32 * 128, v_swz = l32 & 7;

  lookup(0);
  issue(0);
  if (n_blocks > 1) lookup(1);
  for (int b = 0; b < n_blocks; ++b) {
    wait_vmcnt<0>();                  // this wave's part of block b has landed
    __builtin_amdgcn_s_barrier();     // so has everyone's, and everyone is done with block b - 1
    if (b + 1 < n_blocks) {
      issue(b + 1);                   // into the stage block b - 1 has left, under way during block b's products
      if (b + 2 < n_blocks) lookup(b + 2);
    }
    unsigned char* stage = smem + (b & 1) * STAGE;
    const unsigned st = (b & 1) * STAGE;
    const int p0 = first_block + b * PF_BLOCK;
    if (p0 + PF_BLOCK - 1 > hi) {
      // the last block: positions past `hi` were never written for this request.  Their
      // weights are zero, but zero times whatever the page holds must stay zero: clear them.
      const int first_bad = hi - p0 + 1;
      for (int idx = tid; idx < HD * PF_BLOCK; idx += 64 * NW) {
        const int d = idx / PF_BLOCK, col = idx % PF_BLOCK;
        if (col >= first_bad) {
          const int slot = (col >> 3) ^ (d & 7);
          *reinterpret_cast<uint16_t*>(stage + K_BYTES + d * 128 + slot * 16 + (col & 7) * 2) = 0;
        }
      }
      __syncthreads();
    }
    if (!wave_live || p0 > wave_hi) continue;  // nothing for this wave's rows in this block (all waves reach the barriers)

    // S^T [64 positions][32 queries] = K Q^T: two tiles of 32 positions, two k steps a group
    f32x16 s_acc[2];
#pragma unroll
    for (int pt = 0; pt < 2; ++pt)
#pragma unroll
      for (int e = 0; e < 16; ++e) s_acc[pt][e] = 0.0f;
    u32x4 kf[2][4];
    auto read_k = [&](u32x4 (&dst)[4], int ks0) {
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        const unsigned at = k_at + st + ((((ks0 + kk) * 2 + half) ^ k_swz) << 4);
        lds_read16<0>(dst[kk * 2 + 0], at);
        lds_read16<32 * KROW>(dst[kk * 2 + 1], at);
      }
    };
    read_k(kf[0], 0);
#pragma unroll
    for (int g = 0; g < KS / 2; ++g) {
      if (g + 1 < KS / 2) {
        read_k(kf[(g + 1) & 1], 2 * (g + 1));
        wait_lgkmcnt<4>();
      } else {
        wait_lgkmcnt<0>();
      }
      use_frags<4>(kf[g & 1]);
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int pt = 0; pt < 2; ++pt)
          s_acc[pt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, kf[g & 1][kk * 2 + pt]),
                                                              qf[2 * g + kk], s_acc[pt], 0, 0, 0);
    }
    // V^T fragments of the first k step of O^T: on their way during the softmax
    u32x4 vf[2][DT];
    auto read_v = [&](u32x4 (&dst)[DT], int s2) {
      const unsigned chunk = (s2 >> 1) * 4 + (s2 & 1) * 2 + half;
      read_frags<DT, 32 * 128>(dst, v_at + st + ((chunk ^ v_swz) << 4));
    };
    read_v(vf[0], 0);

    // this lane: query my_row; register e of tile pt is position
    // p0 + 32 pt + 16 (e / 8) + 8 half + (e % 8).  A block that every row of the wave sees whole
    // needs no mask (all but the blocks on the diagonal and at the window's edge).
    const bool whole = p0 + PF_BLOCK - 1 <= pos0 + wave * 32 && p0 >= wave_lo;
    // the largest raw score first (the scale is positive), then exp2(score * c - max * c) in one
    // multiply-add each
    float mloc = -INFINITY;
    if (whole) {
#pragma unroll
      for (int pt = 0; pt < 2; ++pt)
#pragma unroll
        for (int e = 0; e < 16; ++e) mloc = fmaxf(mloc, s_acc[pt][e]);
    } else {
#pragma unroll
      for (int pt = 0; pt < 2; ++pt)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int p = p0 + pt * 32 + (e >> 3) * 16 + half * 8 + (e & 7);
          const bool seen = p <= my_pos && p >= my_lo;
          const float v = seen ? s_acc[pt][e] : -INFINITY;
          s_acc[pt][e] = v;
          mloc = fmaxf(mloc, v);
        }
    }
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, AXON_WAVE));
    const float mn = fmaxf(m_run, mloc * c);
    const float mref = mn == -INFINITY ? 0.0f : mn;     // a row that has seen nothing yet
    const float alpha = __builtin_amdgcn_exp2f(m_run - mref);
    float lsum = 0.0f;
#pragma unroll
    for (int pt = 0; pt < 2; ++pt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float pv = __builtin_amdgcn_exp2f(fmaf(s_acc[pt][e], c, -mref));
        s_acc[pt][e] = pv;
        lsum += pv;
      }
    lsum += __shfl_xor(lsum, 32, AXON_WAVE);
    l_run = l_run * alpha + lsum;
    m_run = mn;
    if (__any(alpha != 1.0f)) {  // the running maximum moved for some row: rescale what is summed so far
#pragma unroll
      for (int i = 0; i < DT; ++i)
#pragma unroll
        for (int e = 0; e < 16; ++e) o_acc[i][e] *= alpha;
    }

    // O^T [HD][32 queries] += V^T P^T.  k step s2 (16 positions) takes registers 8 (s2 % 2) .. + 7
    // of tile s2 / 2: the 8 consecutive positions 32 (s2 / 2) + 16 (s2 % 2) + 8 half + {0..7}.
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) {
      if (s2 + 1 < 4) {
        read_v(vf[(s2 + 1) & 1], s2 + 1);
        wait_lgkmcnt<DT>();
      } else {
        wait_lgkmcnt<0>();
      }
      use_frags<DT>(vf[s2 & 1]);
      const int pt = s2 >> 1, e0 = (s2 & 1) * 8;
      union { uint32_t u[4]; bf16x8 f; } pf;
#pragma unroll
      for (int j = 0; j < 4; ++j) pf.u[j] = pack_bf16(s_acc[pt][e0 + 2 * j], s_acc[pt][e0 + 2 * j + 1]);
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf[s2 & 1][dt]), pf.f, o_acc[dt], 0,
                                                            0, 0);
    }
  }

  if (!wave_live || my_row >= count) return;
  const float inv = 1.0f / l_run;
  bf16_t* orow = out + (size_t)(t0 + my_row) * n_heads * HD + (size_t)head * HD;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = dt * 32 + g * 8 + half * 4;
      uint2 pk;
      pk.x = pack_bf16(o_acc[dt][g * 4 + 0] * inv, o_acc[dt][g * 4 + 1] * inv);
      pk.y = pack_bf16(o_acc[dt][g * 4 + 2] * inv, o_acc[dt][g * 4 + 3] * inv);
      *reinterpret_cast<uint2*>(orow + d) = pk;
    }
}

// A block takes one tile or two, one after the other: tiles [n][4] = (first token, count) twice,
// the second count 0 if there is none.  The caller pairs a tile that sees many positions with
// one that sees few, so that every block has about the same work (a causal prompt's tiles see
// 1, 2, 3 ... blocks of positions).
template <int HD, int HPB>
__global__ void __launch_bounds__(256 * HPB, 2)
attention_prefill_kernel(const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_cache,
                         const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_table, int table_stride,
                         const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                         bf16_t* __restrict__ out, const int32_t* __restrict__ tiles, int n_heads, int n_kv_heads,
                         int page_size, int window, float scale) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int32_t* mine = tiles + 4 * blockIdx.x;
  for (int part = 0; part < 2; ++part) {
    const int t0 = mine[2 * part], count = mine[2 * part + 1];
    if (count <= 0) break;                        // the same for the whole block
    if (part) __syncthreads();                    // everyone has read the first tile's last stage
    attention_prefill_tile<HD, HPB>(smem, t0, count, q, q_stride, k_cache, v_cache, block_table, table_stride, positions,
                                    seq_rows, out, n_heads, n_kv_heads, page_size, window, scale);
  }
}

// ============================================================================ decoding tokens
// grid (work items x kv heads): a block of four waves per (token, kv head, chunk of 256
// positions); a wave takes 64 of them.  The work list names the chunks that exist, token by
// token (item = token slot * CMB_MAX_CHUNKS + chunk, -1: nothing), so that a batch of short and
// long contexts launches no block without work: a block that only finds out that it has none
// still holds its place on a CU for a good part of a working block's time.  The wave issues
// every load of its positions at once (K rows and V^T rows go straight from the pages into
// 16x16x32 MFMA operands, 32 KB in flight per wave), then multiplies; the query heads of the
// group are the 16 columns (a group of up to 16 heads).  The four waves' results are folded in
// LDS, in wave order.  Output: if the token's whole range is one chunk, the normalised result;
// else the chunk's (max, sum, unnormalised output) into `partial`, folded by
// attention_combine_kernel.  How a token's range is cut depends on its own position and the
// window alone, never on the rest of the batch.
#define DC_WAVE 64

template <int HD>
__global__ void __launch_bounds__(256)
attention_decode_kernel(const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_cache,
                        const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_table, int table_stride,
                        const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                        bf16_t* __restrict__ out, const int32_t* __restrict__ token_index,
                        int n_tokens, const int32_t* __restrict__ work, float* __restrict__ partial, int max_chunks,
                        int n_heads, int n_kv_heads, int page_size, int window, float scale) {
  constexpr int KS = HD / 32;   // k steps of S^T (32 dims each)
  constexpr int DT = HD / 16;   // output tiles (16 dims each)
  constexpr int ROW = HD + 4;   // floats of a head's row in LDS (padded: rows start in different banks)
  extern __shared__ float fold_lds[];                // [4 waves][group][ROW] outputs, then [4][group][2] max and sum
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int item = work[blockIdx.x / n_kv_heads];    // the kv heads of a chunk side by side: they share its pages
  if (item < 0) return;                              // padding of the list
  const int slot = item / CMB_MAX_CHUNKS, chunk = item % CMB_MAX_CHUNKS;
  if (slot >= n_tokens || chunk >= max_chunks) return;   // no item of this launch
  const int t = token_index ? token_index[slot] : slot;
  const int kvh = blockIdx.x % n_kv_heads;
  const int group = n_heads / n_kv_heads;
  float* fold_o = fold_lds;
  float* fold_ml = fold_lds + 4 * group * ROW;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
  const int first = (lo / DC_CHUNK) * DC_CHUNK;
  const int n_chunks = (pos - first) / DC_CHUNK + 1;
  if (chunk >= n_chunks) return;                     // the whole block: no wave of it waits below
  const int p0 = first + chunk * DC_CHUNK + wave * DC_WAVE;
  const int c1 = min(p0 + DC_WAVE - 1, pos);         // last position of this wave
  const int r16 = lane & 15, q4 = lane >> 4;
  // a wave with no position at all (past the token, or wholly before the window): nothing to add
  const bool wave_live = p0 <= pos && c1 >= lo;
  if (wave_live) {
  const int32_t* table_row = block_table + (size_t)seq_rows[t] * table_stride;
  const size_t kv_head_stride = (size_t)HD * page_size;

  // ---- every load first.  K (A operand of S^T): 4 tiles of 16 positions.  Row r of tile pt is
  // position p0 + 32 (pt / 2) + 8 (r / 4) + 4 (pt % 2) + r % 4, so that what S^T leaves in a
  // lane's registers (rows 4 q4 .. 4 q4 + 3 of every tile) are, over a pair of tiles, 8
  // consecutive positions: the V^T operand below is then one 16-byte read.  8 consecutive dims
  // from 32 ks + 8 q4.  Rows past the chunk's end: any valid row (masked below).
  uint4 kf[4][KS];
#pragma unroll
  for (int pt = 0; pt < 4; ++pt) {
    const int p = min(p0 + 32 * (pt >> 1) + 8 * (r16 >> 2) + 4 * (pt & 1) + (r16 & 3), c1);
    const bf16_t* krow = k_cache + ((size_t)table_row[p / page_size] * n_kv_heads + kvh) * kv_head_stride +
                         (size_t)(p % page_size) * HD + q4 * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) kf[pt][ks] = *reinterpret_cast<const uint4*>(krow + ks * 32);
  }
  // V^T (A operand of O^T): k step u takes the lane's positions p0 + 32 u + 8 q4 + {0..7} of dim
  // 16 dt + r16: 16 bytes of one page (a page holds a multiple of 8 positions).
  uint4 vf[2][DT];
  int keep[2];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    const int pa = p0 + 32 * u + 8 * q4;
    keep[u] = max(0, min(c1 - pa + 1, 8));
    const int pa_c = min(pa, c1);
    const bf16_t* va = v_cache + ((size_t)table_row[pa_c / page_size] * n_kv_heads + kvh) * kv_head_stride +
                       ((pa_c % page_size) & ~7);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vf[u][dt] = *reinterpret_cast<const uint4*>(va + (size_t)(dt * 16 + r16) * page_size);
  }
  // Q^T (B operand): column = head of the group (zero beyond it), 8 consecutive dims
  bf16x8 qf[KS];
  {
    const bf16_t* qrow = q + (size_t)t * q_stride + (size_t)(kvh * group + min(r16, group - 1)) * HD + q4 * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 v = *reinterpret_cast<const uint4*>(qrow + ks * 32);
      if (r16 >= group) v = uint4{0, 0, 0, 0};
      qf[ks] = frag_of(v);
    }
  }

  // ---- S^T [64 positions][16 heads]
  f32x4 s_acc[4];
#pragma unroll
  for (int pt = 0; pt < 4; ++pt) {
    s_acc[pt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks)
      s_acc[pt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(frag_of(kf[pt][ks]), qf[ks], s_acc[pt], 0, 0, 0);
  }
  // this lane: head r16; positions p0 + 32 (pt / 2) + 8 q4 + 4 (pt % 2) + e
  const float c = scale * LOG2E;
  float m = -INFINITY;
#pragma unroll
  for (int pt = 0; pt < 4; ++pt)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int p = p0 + 32 * (pt >> 1) + 8 * q4 + 4 * (pt & 1) + e;
      const float v = (p <= c1 && p >= lo) ? s_acc[pt][e] * c : -INFINITY;
      s_acc[pt][e] = v;
      m = fmaxf(m, v);
    }
  m = fmaxf(m, __shfl_xor(m, 16, AXON_WAVE));
  m = fmaxf(m, __shfl_xor(m, 32, AXON_WAVE));
  const float mref = m == -INFINITY ? 0.0f : m;
  float l = 0.0f;
#pragma unroll
  for (int pt = 0; pt < 4; ++pt)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float pv = __builtin_amdgcn_exp2f(s_acc[pt][e] - mref);
      s_acc[pt][e] = pv;
      l += pv;
    }
  l += __shfl_xor(l, 16, AXON_WAVE);
  l += __shfl_xor(l, 32, AXON_WAVE);

  // ---- O^T [HD][16 heads] = V^T P^T.  Positions past the chunk's end were never written: their
  // weights are zero, and the values read for them are replaced by zero so that zero times
  // anything stays zero.
  f32x4 o_acc[DT];
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    union { uint32_t w[4]; bf16x8 f; } pf;
    pf.w[0] = pack_bf16(s_acc[2 * u][0], s_acc[2 * u][1]);
    pf.w[1] = pack_bf16(s_acc[2 * u][2], s_acc[2 * u][3]);
    pf.w[2] = pack_bf16(s_acc[2 * u + 1][0], s_acc[2 * u + 1][1]);
    pf.w[3] = pack_bf16(s_acc[2 * u + 1][2], s_acc[2 * u + 1][3]);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      uint4 v = vf[u][dt];
      if (keep[u] < 8) {
        uint32_t* w = reinterpret_cast<uint32_t*>(&v);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (keep[u] <= 2 * i) w[i] = 0;
          else if (keep[u] == 2 * i + 1) w[i] &= 0xffffu;
        }
      }
      if (u == 0) o_acc[dt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
      o_acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(frag_of(v), pf.f, o_acc[dt], 0, 0, 0);
    }
  }

  if (r16 < group) {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
      *reinterpret_cast<f32x4*>(&fold_o[(wave * group + r16) * ROW + dt * 16 + q4 * 4]) = o_acc[dt];
    if (q4 == 0) {
      fold_ml[(wave * group + r16) * 2] = m;
      fold_ml[(wave * group + r16) * 2 + 1] = l;
    }
  }
  } else if (lane < group) {
    fold_ml[(wave * group + lane) * 2] = -INFINITY;
    fold_ml[(wave * group + lane) * 2 + 1] = 0.0f;
  }
  __syncthreads();

  // ---- the four waves' results into one, in wave order: a thread takes 4 dims of a head
  for (int task = threadIdx.x; task < group * (HD / 4); task += 256) {
    const int hg = task / (HD / 4), d = (task % (HD / 4)) * 4;
    float M = fold_ml[hg * 2];
#pragma unroll
    for (int w = 1; w < 4; ++w) M = fmaxf(M, fold_ml[(w * group + hg) * 2]);
    const float mref = M == -INFINITY ? 0.0f : M;
    float L = 0.0f;
    f32x4 O = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = fold_ml[(w * group + hg) * 2];
      if (mw == -INFINITY) continue;                 // a wave without positions wrote no output
      const float weight = __builtin_amdgcn_exp2f(mw - mref);
      L = fmaf(fold_ml[(w * group + hg) * 2 + 1], weight, L);
      const f32x4 o = *reinterpret_cast<const f32x4*>(&fold_o[(w * group + hg) * ROW + d]);
#pragma unroll
      for (int e = 0; e < 4; ++e) O[e] = fmaf(o[e], weight, O[e]);
    }
    const int head = kvh * group + hg;
    if (n_chunks == 1) {
      const float inv = 1.0f / L;
      uint2 pk;
      pk.x = pack_bf16(O[0] * inv, O[1] * inv);
      pk.y = pack_bf16(O[2] * inv, O[3] * inv);
      *reinterpret_cast<uint2*>(out + (size_t)t * n_heads * HD + (size_t)head * HD + d) = pk;
    } else {
      // partial [token slot][head][chunk][HD + 2]: output, then max (log2 domain) and sum
      float* dst = partial + (((size_t)slot * n_heads + head) * max_chunks + chunk) * (HD + 2);
      *reinterpret_cast<float2*>(dst + d) = make_float2(O[0], O[1]);
      *reinterpret_cast<float2*>(dst + d + 2) = make_float2(O[2], O[3]);
      if (d == 0) {
        dst[HD] = M;
        dst[HD + 1] = L;
      }
    }
  }
}

// Fold a token's chunks: M = max of the chunks' maxima (exact in any order), then
// L = sum l_c 2^(m_c - M) and O = sum o_c 2^(m_c - M); out = O / L.  The sums run in a fixed
// order (the chunks' weights by a butterfly over lanes, the outputs chunk by chunk ascending).
// grid (tokens, heads), HD threads.

template <int HD>
__global__ void __launch_bounds__(HD)
attention_combine_kernel(const float* __restrict__ partial, const int32_t* __restrict__ positions,
                         const int32_t* __restrict__ token_index, bf16_t* __restrict__ out, int max_chunks, int n_heads,
                         int window) {
  __shared__ float weight[CMB_MAX_CHUNKS];
  __shared__ float red[2][HD / 64];
  const int t = token_index ? token_index[blockIdx.x] : blockIdx.x, head = blockIdx.y, d = threadIdx.x;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
  const int n_chunks = (pos - (lo / DC_CHUNK) * DC_CHUNK) / DC_CHUNK + 1;
  if (n_chunks == 1) return;  // the decoding kernel wrote the result itself
  const float* src = partial + ((size_t)blockIdx.x * n_heads + head) * max_chunks * (HD + 2);
  // the maximum: every thread takes chunks d, d + HD, ...
  float mloc = -INFINITY;
  for (int cidx = d; cidx < n_chunks; cidx += HD) mloc = fmaxf(mloc, src[(size_t)cidx * (HD + 2) + HD]);
  mloc = wave_max(mloc);
  if ((d & 63) == 0) red[0][d >> 6] = mloc;
  __syncthreads();
  float M = red[0][0];
#pragma unroll
  for (int i = 1; i < HD / 64; ++i) M = fmaxf(M, red[0][i]);
  const float mref = M == -INFINITY ? 0.0f : M;
  float lloc = 0.0f;
  for (int cidx = d; cidx < n_chunks; cidx += HD) {
    const float* p = src + (size_t)cidx * (HD + 2);
    const float w = __builtin_amdgcn_exp2f(p[HD] - mref);
    weight[cidx] = w;
    lloc = fmaf(p[HD + 1], w, lloc);
  }
  lloc = wave_sum(lloc);
  if ((d & 63) == 0) red[1][d >> 6] = lloc;
  __syncthreads();
  float L = red[1][0];
#pragma unroll
  for (int i = 1; i < HD / 64; ++i) L += red[1][i];
  float O = 0.0f;
#pragma unroll 8
  for (int cidx = 0; cidx < n_chunks; ++cidx) O = fmaf(src[(size_t)cidx * (HD + 2) + d], weight[cidx], O);
  out[(size_t)t * n_heads * HD + (size_t)head * HD + d] = float_to_bf16(O / L);
}

#endif  // AXON_BF16

// ============================================================================ entry points
// 1 if the MFMA attention kernels take this head size, page size and group of heads.
extern "C" int axk_attention_fast_ok(int head_dim, int page_size, int n_heads, int n_kv_heads) {
#if AXON_BF16
  const bool hd_ok = head_dim == 64 || head_dim == 128;
  const bool page_ok = page_size >= 8 && page_size <= 64 && (page_size & (page_size - 1)) == 0;
  return hd_ok && page_ok && n_kv_heads > 0 && n_heads % n_kv_heads == 0 && n_heads / n_kv_heads <= 16;
#else
  return 0;
#endif
}

extern "C" int axk_attention_prefill(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                     const int32_t* block_table, int table_stride, const int32_t* positions,
                                     const int32_t* seq_rows, void* out, const int32_t* tiles, int n_tiles, int n_heads,
                                     int n_kv_heads, int head_dim, int page_size, int window, float scale, void* stream) {
#if AXON_BF16
  AXK_REQUIRE(axk_attention_fast_ok(head_dim, page_size, n_heads, n_kv_heads),
              "attention_prefill: head_dim %d, page size %d, %d/%d heads are not taken by this kernel", head_dim,
              page_size, n_heads, n_kv_heads);
  AXK_REQUIRE(n_tiles >= 0 && n_heads <= 65535 && window >= 0 && q_stride % 8 == 0 && ((uintptr_t)q & 15) == 0,
              "attention_prefill: bad arguments (tiles %d, heads %d, window %d, q stride %d)", n_tiles, n_heads, window,
              q_stride);
  if (n_tiles == 0) return 0;
  const int group = n_heads / n_kv_heads;
#define LAUNCH(HD, HPB)                                                                                             \
  {                                                                                                                 \
    static bool configured = false;                                                                                 \
    constexpr int lds = 2 * (PF_BLOCK * HD * 2 + HD * PF_BLOCK * 2);                                                \
    const dim3 grid(n_tiles, n_kv_heads * ((group + HPB - 1) / HPB));                                               \
    if (!configured) {                                                                                              \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_prefill_kernel<HD, HPB>),         \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);                          \
      if (e != hipSuccess) {                                                                                        \
        axk_set_error("attention_prefill: cannot reserve %d bytes of LDS: %s", lds, hipGetErrorString(e));          \
        return -2;                                                                                                  \
      }                                                                                                             \
      configured = true;                                                                                            \
    }                                                                                                               \
    attention_prefill_kernel<HD, HPB><<<grid, 256 * HPB, lds, (hipStream_t)stream>>>(                               \
        (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_stride,      \
        positions, seq_rows, (bf16_t*)out, tiles, n_heads, n_kv_heads, page_size, window, scale);                   \
  }
  // two query heads of a kv head a block (they share each K and V block in LDS) where that still
  // gives the chip's 256 CUs about a block each; else one head a block
  const int blocks_of_pairs = n_tiles * n_kv_heads * ((group + 1) / 2);
  if (group >= 2 && blocks_of_pairs >= 200) {
    if (head_dim == 64) LAUNCH(64, 2) else LAUNCH(128, 2)
  } else {
    if (head_dim == 64) LAUNCH(64, 1) else LAUNCH(128, 1)
  }
#undef LAUNCH
  AXK_LAUNCH_CHECK("attention_prefill");
  return 0;
#else
  axk_set_error("attention_prefill: only in the bfloat16 build");
  return -1;
#endif
}

// Positions of one chunk of a decoding token's range, and the factor of the token's slot in an
// item of the work list (item = slot * factor + chunk).
extern "C" int axk_attention_decode_chunk(void) { return DC_CHUNK; }
extern "C" int axk_attention_decode_item_factor(void) { return CMB_MAX_CHUNKS; }

// Floats of `partial` that n_tokens decoding tokens with up to max_chunks chunks need.
extern "C" long axk_attention_decode_workspace(int n_tokens, int n_heads, int head_dim, int max_chunks) {
  return (long)n_tokens * n_heads * max_chunks * (head_dim + 2);
}

extern "C" int axk_attention_decode(const void* q, int q_stride, const void* k_cache, const void* v_cache,
                                    const int32_t* block_table, int table_stride, const int32_t* positions,
                                    const int32_t* seq_rows, void* out, const int32_t* token_index, int n_tokens,
                                    const int32_t* work, int n_work, float* partial, int max_chunks, int n_heads,
                                    int n_kv_heads, int head_dim, int page_size, int window, float scale,
                                    void* stream) {
#if AXON_BF16
  AXK_REQUIRE(axk_attention_fast_ok(head_dim, page_size, n_heads, n_kv_heads),
              "attention_decode: head_dim %d, page size %d, %d/%d heads are not taken by this kernel", head_dim,
              page_size, n_heads, n_kv_heads);
  AXK_REQUIRE(max_chunks <= CMB_MAX_CHUNKS, "attention_decode: %d chunks of %d positions (at most %d: %d positions)",
              max_chunks, DC_CHUNK, CMB_MAX_CHUNKS, CMB_MAX_CHUNKS * DC_CHUNK);
  AXK_REQUIRE(n_tokens >= 0 && n_tokens <= 65535 && max_chunks >= 1 && n_kv_heads <= 65535 && window >= 0 &&
                  q_stride % 8 == 0 && ((uintptr_t)q & 15) == 0,
              "attention_decode: bad arguments (tokens %d, chunks %d, window %d, q stride %d)", n_tokens, max_chunks,
              window, q_stride);
  AXK_REQUIRE(max_chunks == 1 || partial != nullptr, "attention_decode: %d chunks need a workspace", max_chunks);
  AXK_REQUIRE(n_work >= 0 && (n_work == 0 || work != nullptr) && (long)n_work * n_kv_heads < (1l << 31),
              "attention_decode: a work list of %d items", n_work);
  if (n_tokens == 0 || n_work == 0) return 0;
  const int group = n_heads / n_kv_heads;
  dim3 grid((unsigned)n_work * n_kv_heads), cgrid(n_tokens, n_heads);
#define LAUNCH(HD)                                                                                                   \
  {                                                                                                                  \
    attention_decode_kernel<HD><<<grid, 256, 4 * group * (HD + 4 + 2) * sizeof(float), (hipStream_t)stream>>>(      \
        (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_stride,       \
        positions, seq_rows, (bf16_t*)out, token_index, n_tokens, work, partial, max_chunks, n_heads, n_kv_heads,    \
        page_size, window, scale);                                                                                   \
    if (max_chunks > 1)                                                                                              \
      attention_combine_kernel<HD><<<cgrid, HD, 0, (hipStream_t)stream>>>(partial, positions, token_index,          \
                                                                         (bf16_t*)out, max_chunks, n_heads, window); \
  }
  if (head_dim == 64) LAUNCH(64) else LAUNCH(128)
#undef LAUNCH
  AXK_LAUNCH_CHECK("attention_decode");
  return 0;
#else
  axk_set_error("attention_decode: only in the bfloat16 build");
  return -1;
#endif
}
