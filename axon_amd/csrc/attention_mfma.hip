// Paged causal attention on the matrix cores (bfloat16 build only): one kernel for prompt
// portions, one for decoding tokens, and ONE arithmetic for both, so that a position's result
// does not depend on whether it was computed in a prompt portion or as a decoded token, alone
// or in a batch (src/lm.rs:272-278; docs/determinism.md:53-57 of the reference: 64-position
// blocks folded ascending "in prefill and decode alike").
//
// The arithmetic, for one query vector q of a head at position pos (window start lo):
// * Positions are taken in blocks of 64 aligned to absolute position.  For a block b,
//     s_p = K_p . q            one chain of 32x32x16 MFMAs over the head's dims in steps of 16
//     m_b = (max_p s_p) c      over the positions the query sees; c = scale log2(e)
//     w_p = 2^(s_p c - m_b)    one multiply-add and one exp2 each; 0 for unseen positions
//     l_b = sum_p w_p          32-bit, in a fixed order of the block's 64 places
//     o_b = sum_p bf16(w_p) V_p   one chain of 32x32x16 MFMAs over the 64 positions, from zero
//   (attention_block below: the same instructions in both kernels).
// * The blocks are folded in ascending order into a running (m, l, o), starting from
//   (-inf, 0, 0): mn = max(m, m_b); a = 2^(m - mn); b = 2^(m_b - mn); l = l a + l_b b;
//   o = o a + o_b b (attention_fold).  The result is o (1 / l).
// The prompt kernel folds as it walks the blocks; the decoding kernel gives every block of a
// token's range to a wave of its own, which leaves (m_b, l_b, o_b) in a workspace, and a second
// kernel folds them in the same order with the same instructions.  No atomics.
//
// Both compute the TRANSPOSED products, S^T = K Q^T and O^T = V^T P^T, so that what one MFMA
// leaves in a lane's registers is what the next one wants there, without a trip through LDS:
// after S^T a lane holds, for ONE query, several key positions; the softmax over positions is
// then a loop over the lane's registers plus one exchange between the two halves of the wave,
// and the rounded weights are already laid out as the B operand of O^T.  The MFMA's k slots are
// matched to the positions a lane holds by reading V^T accordingly (values are cached
// position-contiguous: [page][kv head][dim][slot]).
#include <math.h>

#include <type_traits>

#include "api.h"
#include "common.h"
#include "instances.h"

#define ATT_BLOCK 64          // positions of a block: the unit of the fold
#define DC_CHUNK 256          // positions of one work item of the decoding kernel: four blocks, a wave each
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

__device__ inline uint32_t pack_bf16(float a, float b) { return pack2_bf16(a, b); }

// ============================================================================ one block of 64 positions
// A stage of LDS holds a block's K [64][HD] and V^T [HD][64], brought by direct global -> LDS
// loads of 16 bytes a lane (an instruction fills 1 KB: 1024 / (2 HD) rows of K, or 8 rows of
// V^T).  16-byte slots of a row are permuted so that the fragment reads of 16 neighbouring rows
// fall into 16 different slots of the 256 bytes (64 banks) that LDS serves in a cycle: rows of
// 256 bytes (K at head size 128) by slot ^ (row & 15), rows of 128 bytes (K at head size 64, V^T),
// of which two lie side by side, by slot ^ ((row >> 1) & 7).  (With slot ^ (row & 7) for both, two
// of every 16 rows met in a slot: the counters showed more cycles of bank conflicts than of reads.)
#define ATT_ZERO16 (f32x16{0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f})

template <int HD>
struct AttStage {
  static constexpr int K_BYTES = ATT_BLOCK * HD * 2;
  static constexpr int V_BYTES = HD * ATT_BLOCK * 2;
  static constexpr int BYTES = K_BYTES + V_BYTES;
  static constexpr int KROW = HD * 2;                       // bytes of a K row
  static constexpr int KCH = HD / 8;                        // 16-byte slots of a K row
  static constexpr int K_ROWS_PER_INSTR = 1024 / KROW;
  static constexpr int K_INSTR = ATT_BLOCK / K_ROWS_PER_INSTR;   // load instructions of a block's K
  static constexpr int V_INSTR = HD / 8;                         // and of its V^T
  // the permutation of a row's slots (see above)
  __device__ static __forceinline__ int k_swizzle(int row) { return KROW == 256 ? (row & 15) : ((row >> 1) & 7); }
  __device__ static __forceinline__ int v_swizzle(int dim) { return (dim >> 1) & 7; }
};

// Pages hold a power of two of positions (axk_attention_fast_ok): the page of a position and its
// place in it by a shift and a mask, not by a division (which costs some twenty instructions).
__device__ __forceinline__ int page_index(int p, int page_size) { return p >> (31 - __builtin_clz(page_size)); }
__device__ __forceinline__ int page_offset(int p, int page_size) { return p & (page_size - 1); }

// The page a lane's piece of load instruction `instr` lies in (looked up ahead of the load that
// uses it).  Positions past `hi` (never written for this request): any valid row.
// (K: an instruction's 4 or 8 rows lie in one page, pages holding at least 8 positions, and rows
// past `hi` read row `hi`, which lies in the page of the instruction's first row or before every
// row of it: the page is the wave's, looked up once, and the address a scalar base plus an offset.)
template <int HD>
__device__ __forceinline__ int att_k_page(int instr, int lane, int p0, int hi, const int32_t* table_row, int page_size) {
  const int row0 = instr * AttStage<HD>::K_ROWS_PER_INSTR;
  return table_row[page_index(min(p0 + row0, hi), page_size)];
}

template <int HD>
__device__ __forceinline__ int att_v_page(int instr, int lane, int p0, int hi, const int32_t* table_row, int page_size) {
  const int d = instr * 8 + (lane >> 3);
  const int chunk = (lane & 7) ^ AttStage<HD>::v_swizzle(d);
  return table_row[page_index(min(p0 + chunk * 8, hi), page_size)];
}

// K: lane i of instruction `instr` brings row i / KCH of the instruction's rows, into slot i % KCH,
// which holds the row's chunk slot ^ k_swizzle(row).
template <int HD>
__device__ __forceinline__ void att_issue_k(unsigned char* stage, int instr, int lane, int page, int p0, int hi,
                                            const bf16_t* k_head, size_t page_stride, int page_size) {
  using S = AttStage<HD>;
  const int row = instr * S::K_ROWS_PER_INSTR + lane / S::KCH;
  const int chunk = (lane % S::KCH) ^ S::k_swizzle(row);
  const int p = min(p0 + row, hi);
  const bf16_t* base = k_head + (size_t)page * page_stride;          // scalar arithmetic where the page is the wave's
  const bf16_t* src = base + (unsigned)(page_offset(p, page_size) * HD + chunk * 8);
  __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + instr * 1024), 16, 0, 0);
}

// V^T: lane i brings row (dim) i / 8 of the instruction's 8 dims, into slot i % 8, which holds the
// 8 positions of chunk slot ^ v_swizzle(dim).
template <int HD>
__device__ __forceinline__ void att_issue_v(unsigned char* stage, int instr, int lane, int page, int p0, int hi,
                                            const bf16_t* v_head, size_t page_stride, int page_size) {
  using S = AttStage<HD>;
  const int d = instr * 8 + (lane >> 3);
  const int chunk = (lane & 7) ^ S::v_swizzle(d);
  const int p = min(p0 + chunk * 8, hi);
  const bf16_t* base = v_head + (size_t)page * page_stride;
  const bf16_t* src = base + (unsigned)(d * page_size + (page_offset(p, page_size) & ~7));
  __builtin_amdgcn_global_load_lds((global_ptr_t)src, (lds_ptr_t)(stage + S::K_BYTES + instr * 1024), 16, 0, 0);
}

// Positions past `hi` in the last block of a request were never written.  Their weights are
// zero, but zero times whatever the page holds must stay zero: clear those columns of V^T.
// Thread `t` of `n_threads` that share the stage; the caller orders this against the reads.
template <int HD>
__device__ __forceinline__ void att_clear_unwritten(unsigned char* stage, int p0, int hi, int t, int n_threads) {
  const int first_bad = hi - p0 + 1;
  for (int idx = t; idx < HD * ATT_BLOCK; idx += n_threads) {
    const int d = idx / ATT_BLOCK, col = idx % ATT_BLOCK;
    if (col >= first_bad) {
      const int slot = (col >> 3) ^ AttStage<HD>::v_swizzle(d);
      *reinterpret_cast<uint16_t*>(stage + AttStage<HD>::K_BYTES + d * 128 + slot * 16 + (col & 7) * 2) = 0;
    }
  }
}

// The block in the stage at LDS address `st`, for the 32 queries (columns) of this wave: lane
// (l32, half) belongs to column l32; qf are its Q^T fragments (B operand: 8 consecutive dims
// from 16 ks + 8 half).  Register e of tile pt of S^T is position
// p0 + 32 pt + 16 (e / 8) + 8 half + (e % 8): row r of an S^T tile is key position pi(r) of the
// tile, pi swapping bits 2 and 3 of r, so that a lane ends with weights of 8 CONSECUTIVE
// positions per k step of O^T, which are one 16-byte read of a V^T row.
// `whole`: every column of the wave sees every position of the block (no mask needed);
// else column l32 sees the positions my_lo .. my_pos.
// attention_scores leaves m_b (log2 domain), l_b and the rounded weights as the four B operands
// of O^T (k step s2: the positions 32 (s2 / 2) + 16 (s2 % 2) + 8 half + {0..7}).  It is two
// halves, the products (attention_raw_scores: the matrix cores) and what follows
// (attention_weights: the vector unit), which the prompt kernel runs apart.
// Fragment reads are written as instructions (see common.h): the stage may be one that direct
// loads of a later block are filling elsewhere in LDS.

// The K row of the stage that lane l32 reads as row l32 of an S^T tile (pi above).
__device__ __forceinline__ int att_k_row(int l32) { return (l32 & 0x13) | ((l32 & 4) << 1) | ((l32 & 8) >> 1); }

// S^T [64 positions][32 queries] = K Q^T: two tiles of 32 positions, each one chain over the k
// steps ascending, from the constant zero.
template <int HD>
__device__ __forceinline__ void attention_raw_scores(unsigned st, const bf16x8 (&qf)[HD / 16], int lane, f32x16 (&s_acc)[2]) {
  using S = AttStage<HD>;
  constexpr int KS = HD / 16;
  const int l32 = lane & 31, half = lane >> 5;
  const int k_row = att_k_row(l32);
  const unsigned k_at = st + k_row * S::KROW, k_swz = S::k_swizzle(k_row);
  u32x4 kf[2][4];
  auto read_k = [&](u32x4 (&dst)[4], int ks0) {
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      const unsigned at = k_at + ((((ks0 + kk) * 2 + half) ^ k_swz) << 4);
      lds_read16<0>(dst[kk * 2 + 0], at);
      lds_read16<32 * S::KROW>(dst[kk * 2 + 1], at);
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
                                                            qf[2 * g + kk], g + kk == 0 ? ATT_ZERO16 : s_acc[pt], 0, 0, 0);
  }
}

// From the raw scores (which it uses up): the largest first (the scale is positive), then
// exp2(score * c - max * c) in one multiply-add each.
__device__ __forceinline__ void attention_weights(f32x16 (&s_acc)[2], int p0, bool whole, int my_pos, int my_lo, float c,
                                                  int lane, float& m_b, float& l_b, bf16x8 (&pf)[4]) {
  const int half = lane >> 5;
  if (!whole) {
    asm volatile("" ::: "memory");      // a branch of its own: the blocks every column sees whole pay nothing for the mask
#pragma unroll
    for (int pt = 0; pt < 2; ++pt)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int p = p0 + pt * 32 + (e >> 3) * 16 + half * 8 + (e & 7);
        const bool seen = p <= my_pos && p >= my_lo;
        s_acc[pt][e] = seen ? s_acc[pt][e] : -INFINITY;
      }
  }
  float mpt[2] = {-INFINITY, -INFINITY};      // a chain a tile: the maximum does not depend on the order
#pragma unroll
  for (int pt = 0; pt < 2; ++pt)
#pragma unroll
    for (int e = 0; e < 16; ++e) mpt[pt] = fmaxf(mpt[pt], s_acc[pt][e]);
  float mloc = fmaxf(mpt[0], mpt[1]);
  mloc = fmaxf(mloc, __shfl_xor(mloc, 32, AXON_WAVE));
  m_b = __fmul_rn(mloc, c);
  const float mref = m_b == -INFINITY ? 0.0f : m_b;     // a column that sees nothing of this block
  float lsum = 0.0f;
#pragma unroll
  for (int pt = 0; pt < 2; ++pt)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const float pv = __builtin_amdgcn_exp2f(__builtin_fmaf(s_acc[pt][e], c, -mref));
      s_acc[pt][e] = pv;
      lsum = __fadd_rn(lsum, pv);
    }
  l_b = __fadd_rn(lsum, __shfl_xor(lsum, 32, AXON_WAVE));
#pragma unroll
  for (int s2 = 0; s2 < 4; ++s2) {
    const int pt = s2 >> 1, e0 = (s2 & 1) * 8;
    union { uint32_t u[4]; bf16x8 f; } w;
#pragma unroll
    for (int j = 0; j < 4; ++j) w.u[j] = pack_bf16(s_acc[pt][e0 + 2 * j], s_acc[pt][e0 + 2 * j + 1]);
    pf[s2] = w.f;
  }
}

template <int HD>
__device__ __forceinline__ void attention_scores(unsigned st, const bf16x8 (&qf)[HD / 16], int p0, bool whole, int my_pos,
                                                 int my_lo, float c, int lane, float& m_b, float& l_b, bf16x8 (&pf)[4]) {
  f32x16 s_acc[2];
  attention_raw_scores<HD>(st, qf, lane, s_acc);
  attention_weights(s_acc, p0, whole, my_pos, my_lo, c, lane, m_b, l_b, pf);
}

// o_b = V^T P^T [HD][32 queries], one tile of 32 dims after the other: each is one chain of four
// MFMAs over the block's positions in ascending steps of 16, from zero, handed to `consume(dt,
// tile)` (dt a constant after unrolling).  Of tile dt a lane holds, in register e, dim
// 32 dt + 8 (e / 4) + 4 half + e % 4 of its column.  The next tile's V^T fragments are on their
// way while this one is multiplied.
template <int HD, typename Consume>
__device__ __forceinline__ void attention_values(unsigned st, const bf16x8 (&pf)[4], int lane, Consume consume) {
  using S = AttStage<HD>;
  constexpr int DT = HD / 32;
  const int l32 = lane & 31, half = lane >> 5;
  const unsigned v_at = st + S::K_BYTES + l32 * 128, v_swz = S::v_swizzle(l32);      // the same for every tile of 32 dims
  u32x4 vf[2][4];
  auto read_v = [&](u32x4 (&dst)[4], int dt) {
    const unsigned row = v_at + dt * 32 * 128;
    lds_read16<0>(dst[0], row + (((0 + half) ^ v_swz) << 4));      // k step s2: chunk 4 (s2 / 2) + 2 (s2 % 2) + half
    lds_read16<0>(dst[1], row + (((2 + half) ^ v_swz) << 4));
    lds_read16<0>(dst[2], row + (((4 + half) ^ v_swz) << 4));
    lds_read16<0>(dst[3], row + (((6 + half) ^ v_swz) << 4));
  };
  read_v(vf[0], 0);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    if (dt + 1 < DT) {
      read_v(vf[(dt + 1) & 1], dt + 1);
      wait_lgkmcnt<4>();
    } else {
      wait_lgkmcnt<0>();
    }
    use_frags<4>(vf[dt & 1]);
    // the chain starts from the constant zero (an operand of the instruction, not sixteen registers to clear)
    f32x16 tile = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf[dt & 1][0]), pf[0], ATT_ZERO16, 0, 0, 0);
#pragma unroll
    for (int s2 = 1; s2 < 4; ++s2)
      tile = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, vf[dt & 1][s2]), pf[s2], tile, 0, 0, 0);
    consume(dt, tile);
  }
}

// A block's o_b and the NEXT block's raw scores in one stretch of matrix products, with the fold
// of o_b into the running output between them: the vector unit works beside the matrix cores only
// on what the same wave issues between two products or what the SIMD's other wave has to do, so
// the prompt kernel keeps its two long vector stretches (the weights of a block, the fold) apart
// from each other and lays the products of two blocks over one of them.  The chains are those of
// attention_values (stage st_v, this block) and of attention_raw_scores (stage st_k, the next
// block), instruction for instruction; only their order among each other is new.
// For a tile dt of 32 dims: V^T k steps 0-1, V^T k steps 2-3, K k step 2 dt, K k step 2 dt + 1,
// two products each, their fragments read a unit ahead; consume(dt, e0, tile) is called
// for a half of the tile (eight registers from e0) after each of its two units of K: by then the
// tile's chain has left the matrix cores, and the products issued just before run meanwhile.
template <int HD, typename Consume>
__device__ __forceinline__ void attention_values_and_next_scores(unsigned st_v, const bf16x8 (&pf)[4], unsigned st_k,
                                                                 const bf16x8 (&qf)[HD / 16], int lane, f32x16 (&s_acc)[2],
                                                                 Consume consume) {
  using S = AttStage<HD>;
  constexpr int DT = HD / 32, UNITS = 4 * DT;
  static_assert(HD / 16 == 2 * DT, "two k steps of S^T for every tile of o");
  const int l32 = lane & 31, half = lane >> 5;
  const int k_row = att_k_row(l32);
  // A row of the stage starts at a multiple of its size, and an even chunk number c plus `half` is
  // c ^ half, so the address of chunk (c + half) ^ swizzle of a row is that of chunk half ^ swizzle
  // with c exclusive-ored in: one instruction from a base each.  The bases are made opaque, or the
  // compiler keeps every address in a register of its own across the whole loop of blocks and
  // runs out of registers.
  unsigned v_base = st_v + S::K_BYTES + l32 * 128 + ((half ^ S::v_swizzle(l32)) << 4);
  unsigned k_base = st_k + k_row * S::KROW + ((half ^ S::k_swizzle(k_row)) << 4);
  asm volatile("" : "+v"(v_base), "+v"(k_base));
  u32x4 fr[2][2];
  auto read_unit = [&](u32x4 (&dst)[2], int u) {
    const int dt = u >> 2, w = u & 3;
    if (w < 2) {                        // V^T k steps 2 w and 2 w + 1 of tile dt: chunks 4 w + half and 4 w + 2 + half
      lds_read16_step<32 * 128, DT>(dst[0], v_base ^ ((4 * w) << 4), dt);
      lds_read16_step<32 * 128, DT>(dst[1], v_base ^ ((4 * w + 2) << 4), dt);
    } else {                            // K k step ks, the two tiles of 32 positions
      const int ks = 2 * dt + (w - 2);
      const unsigned at = k_base ^ (ks << 5);
      lds_read16<0>(dst[0], at);
      lds_read16<32 * S::KROW>(dst[1], at);
    }
  };
  f32x16 tile;
  read_unit(fr[0], 0);
#pragma unroll
  for (int u = 0; u < UNITS; ++u) {
    const int dt = u >> 2, w = u & 3;
    if (u + 1 < UNITS) {
      read_unit(fr[(u + 1) & 1], u + 1);
      wait_lgkmcnt<2>();
    } else {
      wait_lgkmcnt<0>();
    }
    use_frags<2>(fr[u & 1]);
    if (w < 2) {
      tile = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fr[u & 1][0]), pf[2 * w],
                                                     w == 0 ? ATT_ZERO16 : tile, 0, 0, 0);
      tile = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fr[u & 1][1]), pf[2 * w + 1], tile, 0, 0, 0);
    } else {
      const int ks = 2 * dt + (w - 2);
#pragma unroll
      for (int pt = 0; pt < 2; ++pt)
        s_acc[pt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fr[u & 1][pt]), qf[ks],
                                                            ks == 0 ? ATT_ZERO16 : s_acc[pt], 0, 0, 0);
      consume(dt, 8 * (w - 2), tile);
    }
  }
}

// The same chains with the V^T fragments in registers (the decoding kernel loads them straight
// from the pages): vf[dt][s2] is what attention_values reads from the stage for tile dt, k step s2.
template <int HD, typename Consume>
__device__ __forceinline__ void attention_values_of(const uint4 (&vf)[HD / 32][4], const bf16x8 (&pf)[4], Consume consume) {
  constexpr int DT = HD / 32;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    f32x16 tile = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_of(vf[dt][0]), pf[0], ATT_ZERO16, 0, 0, 0);
#pragma unroll
    for (int s2 = 1; s2 < 4; ++s2)
      tile = __builtin_amdgcn_mfma_f32_32x32x16_bf16(frag_of(vf[dt][s2]), pf[s2], tile, 0, 0, 0);
    consume(dt, tile);
  }
}

// The fold of a block into the running state: the factors of the old state and of the block.
__device__ __forceinline__ void attention_fold(float& m, float& l, float m_b, float l_b, float& a, float& b) {
  const float mn = fmaxf(m, m_b);
  const float mref = mn == -INFINITY ? 0.0f : mn;     // nothing seen yet, here or before
  a = __builtin_amdgcn_exp2f(__fsub_rn(m, mref));
  b = __builtin_amdgcn_exp2f(__fsub_rn(m_b, mref));
  l = __builtin_fmaf(l, a, __fmul_rn(l_b, b));
  m = mn;
}

// o = fma(o, a, o_b b), written as the instruction with o's register as its result: left to itself
// the compiler puts the result where the product was and moves every value back into the loop's
// own register afterwards (64 moves a block of positions, and as many registers held twice).
__device__ __forceinline__ void attention_fold_into(float& o, float a, float o_b, float b) {
  const float t = __fmul_rn(o_b, b);
  asm("v_fma_f32 %0, %0, %1, %2" : "+v"(o) : "v"(a), "v"(t));
}

__device__ __forceinline__ float attention_inverse(float l) { return __fdiv_rn(1.0f, l); }

// ============================================================================ prompt portions
// grid (tiles, kv heads x groups of HPB query heads); a tile is up to 128 consecutive tokens of
// one request.  4 waves per query head, each owning 32 query rows; with HPB = 2 two query heads of
// the same kv head share every K and V^T block in LDS (the path from L2 into LDS carries about 32
// bytes a cycle and CU, which is what one head's products use up).  Two stages: the next block's
// loads are in flight while this one is multiplied.
#define PF_TOKENS 128     // (axk_attention_prefill_tile says so to the caller)
#ifndef ATT_LATE_WAVE
#define ATT_LATE_WAVE(w) (((w) >> 2) & 1)
#endif

template <int HD, int HPB, bool ONE_PAGE, bool LATE>
__device__ __forceinline__ void
attention_prefill_tile(unsigned char* smem, int t0, int count, const bf16_t* __restrict__ q, int q_stride,
                       const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
                       const int32_t* __restrict__ block_table, int table_stride, const int32_t* __restrict__ positions,
                       const int32_t* __restrict__ seq_rows, bf16_t* __restrict__ out, int n_heads, int n_kv_heads,
                       int page_size, int window, float scale) {
  using S = AttStage<HD>;
  constexpr int NW = 4 * HPB;                               // waves of the block
  constexpr int K_INSTR = S::K_INSTR / NW;                  // load instructions per wave
  constexpr int V_INSTR = S::V_INSTR / NW;
  static_assert(K_INSTR >= 1 && V_INSTR >= 1, "more waves than load instructions");
  constexpr int DT = HD / 32;                     // output tiles (32 dims each)
  constexpr int KS = HD / 16;                     // k steps of S^T

  const int tid = threadIdx.x, lane = tid & 63;
  const int block_wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // a scalar: what depends on it alone branches, not masks
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
  const int first_block = (lo / ATT_BLOCK) * ATT_BLOCK;
  const int n_blocks = (hi - first_block) / ATT_BLOCK + 1;

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

  const size_t page_stride = (size_t)n_kv_heads * HD * page_size;    // elements of one page (all kv heads)
  const bf16_t* k_head = k_cache + (size_t)kvh * HD * page_size;
  const bf16_t* v_head = v_cache + (size_t)kvh * HD * page_size;
  // The pages a block of positions lies in are looked up one block ahead of the loads that use
  // them, so that no load waits for a table entry behind the loads issued just before it.
  // ONE_PAGE (pages of 64 positions or more): a block lies in one page, known to the whole wave,
  // and the addresses are a scalar base plus a lane's 32-bit offset.
  int k_page[K_INSTR], v_page[1];
  auto lookup_k = [&](int b) {
    const int p0 = first_block + b * ATT_BLOCK;
    if (ONE_PAGE) {
      k_page[0] = table_row[page_index(p0, page_size)];
      return;
    }
#pragma unroll
    for (int n = 0; n < K_INSTR; ++n) k_page[n] = att_k_page<HD>(n * NW + block_wave, lane, p0, hi, table_row, page_size);
  };
  auto lookup_v = [&](int b) {
    const int p0 = first_block + b * ATT_BLOCK;
    if (ONE_PAGE) {
      v_page[0] = table_row[page_index(p0, page_size)];
      return;
    }
    // the 8 positions a lane brings depend on the instruction through its parity alone (the
    // permutation of a V^T row's slots), and a wave's instructions are NW apart: one page for all
    static_assert(NW % 2 == 0, "a wave's load instructions have one parity");
    v_page[0] = att_v_page<HD>(block_wave, lane, p0, hi, table_row, page_size);
  };
  auto issue_k = [&](int b) {
    unsigned char* stage = smem + (b & 1) * S::BYTES;
    const int p0 = first_block + b * ATT_BLOCK;
#pragma unroll
    for (int n = 0; n < K_INSTR; ++n)
      att_issue_k<HD>(stage, n * NW + block_wave, lane, ONE_PAGE ? k_page[0] : k_page[n], p0, hi, k_head, page_stride,
                      page_size);
  };
  auto issue_v = [&](int b) {
    unsigned char* stage = smem + (b & 1) * S::BYTES;
    const int p0 = first_block + b * ATT_BLOCK;
#pragma unroll
    for (int n = 0; n < V_INSTR; ++n)
      att_issue_v<HD>(stage, n * NW + block_wave, lane, v_page[0], p0, hi, v_head, page_stride, page_size);
  };

  float o_acc[DT][16];              // (plain registers: the fold below names each as an instruction's operand)
#pragma unroll
  for (int i = 0; i < DT; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) o_acc[i][e] = 0.0f;
  float m_run = -INFINITY, l_run = 0.0f;
  const float c = scale * LOG2E;
  const unsigned lds0 = (unsigned)(size_t)(lds_ptr_t)smem;
  // the blocks of which this wave's rows see anything: the first my_blocks of the tile's
  const int my_blocks = wave_live ? min(n_blocks, (wave_hi - first_block) / ATT_BLOCK + 1) : 0;

  // A wave's work on block b is three stretches: the raw scores (matrix cores), the weights (vector
  // unit), and the block's o_b with its fold (both).  The raw scores of block b + 1 are laid over
  // the third stretch of block b, so K runs a block ahead of V^T: at the barrier of block b the
  // keys of block b + 1 and the values of block b have landed, everyone has left the keys of block
  // b and the values of block b - 1, and their stages take the keys of block b + 2 and the values
  // of block b + 1.
  f32x16 s_acc[2];
  lookup_k(0);
  lookup_v(0);
  issue_k(0);
  issue_v(0);
  if (n_blocks > 1) {
    lookup_k(1);
    lookup_v(1);
    issue_k(1);
    if (n_blocks > 2) lookup_k(2);
  }
  wait_vmcnt<0>();
  __builtin_amdgcn_s_barrier();
  // what every wave does between the weights of block b and its products, whether it has any or not
  auto turn_stages = [&](int b) {
    const int p0 = first_block + b * ATT_BLOCK;
    wait_vmcnt<0>();                  // this wave's part of the keys of block b + 1 and the values of block b has landed
    __builtin_amdgcn_s_barrier();     // so has everyone's
    if (b + 2 < n_blocks) {
      issue_k(b + 2);
      if (b + 3 < n_blocks) lookup_k(b + 3);
    }
    if (b + 1 < n_blocks) {
      issue_v(b + 1);
      if (b + 2 < n_blocks) lookup_v(b + 2);
    }
    if (p0 + ATT_BLOCK - 1 > hi) {
      att_clear_unwritten<HD>(smem + (b & 1) * S::BYTES, p0, hi, tid, 64 * NW);
      __syncthreads();
    }
  };
  if (my_blocks > 0) attention_raw_scores<HD>(lds0, qf, lane, s_acc);
  int b = 0;
  // One path through the body, whatever the block: after the wave's last block the products of
  // "the next block's scores" run on whatever the other stage holds and are dropped (sixteen
  // products a tile).  A second path would have the compiler copy the running output between the
  // registers of the two, and branches around those products alone cost more than the products.
  for (; b < my_blocks; ++b) {
    const int p0 = first_block + b * ATT_BLOCK;
    // A block that every row of the wave sees whole needs no mask (all but the blocks on the
    // diagonal and at the window's edge).
    const bool whole = p0 + ATT_BLOCK - 1 <= pos0 + wave * 32 && p0 >= wave_lo;
    float m_b, l_b, a, bb;
    bf16x8 pf[4];
    // The two waves of a SIMD take turns: one has its weights done before the barrier and starts
    // with the products, the other (LATE) starts with its weights, which the first one's
    // products leave the vector unit free for; and so on, half a block apart.
    if (!LATE) {
      attention_weights(s_acc, p0, whole, my_pos, my_lo, c, lane, m_b, l_b, pf);
      attention_fold(m_run, l_run, m_b, l_b, a, bb);
    }
    turn_stages(b);
    if (LATE) {
      attention_weights(s_acc, p0, whole, my_pos, my_lo, c, lane, m_b, l_b, pf);
      attention_fold(m_run, l_run, m_b, l_b, a, bb);
    }
    attention_values_and_next_scores<HD>(lds0 + (b & 1) * S::BYTES, pf, lds0 + ((b + 1) & 1) * S::BYTES, qf, lane, s_acc,
                                         [&](int dt, int e0, const f32x16& tile) {
#pragma unroll
      for (int e = e0; e < e0 + 8; ++e) attention_fold_into(o_acc[dt][e], a, tile[e], bb);
    });
  }
  for (; b < n_blocks; ++b) turn_stages(b);   // (all waves reach the barriers)

  if (!wave_live || my_row >= count) return;
  const float inv = attention_inverse(l_run);
  bf16_t* orow = out + (size_t)(t0 + my_row) * n_heads * HD + (size_t)head * HD;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = dt * 32 + g * 8 + half * 4;
      uint2 pk;
      pk.x = pack_bf16(__fmul_rn(o_acc[dt][g * 4 + 0], inv), __fmul_rn(o_acc[dt][g * 4 + 1], inv));
      pk.y = pack_bf16(__fmul_rn(o_acc[dt][g * 4 + 2], inv), __fmul_rn(o_acc[dt][g * 4 + 3], inv));
      *reinterpret_cast<uint2*>(orow + d) = pk;
    }
}

// A block takes one tile or two, one after the other: tiles [n][4] = (first token, count) twice,
// the second count 0 if there is none.  The caller pairs a tile that sees many positions with
// one that sees few, so that every block has about the same work (a causal prompt's tiles see
// 1, 2, 3 ... blocks of positions).
// ONE_PAGE (pages of 64 positions or more, the launch's choice): each has its own addressing, and a
// kernel that held both would keep the lane's constants of both in registers.
template <int HD, int HPB, bool ONE_PAGE>
__global__ void __launch_bounds__(256 * HPB, 2)
attention_prefill_kernel(const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_cache,
                         const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_table, int table_stride,
                         const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                         bf16_t* __restrict__ out, const int32_t* __restrict__ tiles, int n_heads, int n_kv_heads,
                         int page_size, int window, float scale) {
  extern __shared__ __align__(256) unsigned char smem[];       // (a stage's rows start at multiples of their size)
  const int32_t* mine = tiles + 4 * blockIdx.x;
  for (int part = 0; part < 2; ++part) {
    const int t0 = mine[2 * part], count = mine[2 * part + 1];
    if (count <= 0) break;                        // the same for the whole block
    if (part) __syncthreads();                    // everyone has read the first tile's last stage
    // waves w and w + 4 of a block share a SIMD: with two heads a block, the second head's waves are the late ones
    if (HPB == 2 && ATT_LATE_WAVE(__builtin_amdgcn_readfirstlane(threadIdx.x >> 6)))
      attention_prefill_tile<HD, HPB, ONE_PAGE, true>(smem, t0, count, q, q_stride, k_cache, v_cache, block_table,
                                                      table_stride, positions, seq_rows, out, n_heads, n_kv_heads, page_size,
                                                      window, scale);
    else
      attention_prefill_tile<HD, HPB, ONE_PAGE, false>(smem, t0, count, q, q_stride, k_cache, v_cache, block_table,
                                                       table_stride, positions, seq_rows, out, n_heads, n_kv_heads, page_size,
                                                       window, scale);
  }
}

// ============================================================================ decoding tokens
// A wave takes one block of 64 positions of a (token, kv head): the range of a token is cut into
// chunks of 256 positions, four such blocks each (grid: work items x kv heads, in blocks of four
// waves or of one).  A wave is on its own from start to end: it brings the block's K into a stage of LDS (16 KB at head
// size 128: ten waves fit a CU) and its V^T straight into registers as MFMA operands (every load
// issued at once, 32 KB in flight per wave), runs attention_scores and the chains of
// attention_values with the query heads of the group as the columns (a group of up to 32 heads)
// and leaves (o_b, m_b, l_b) of every head in `partial`.  The work list names the chunks that
// exist, token by token (item = token slot * CMB_MAX_CHUNKS + chunk, -1: nothing), so that a
// batch of short and long contexts launches few blocks without work.  How a token's range is cut
// depends on its own position and the window alone, never on the rest of the batch.
// partial [token slot][head][block][HD + 2]: o_b, then m_b and l_b; blocks counted from the
// chunk that holds the window's first position (or 0).
template <int HD, int BW>
__global__ void __launch_bounds__(BW * 64, BW == 1 ? 3 : 2)      // waves a SIMD: three leave each 168 registers
attention_decode_kernel(const bf16_t* __restrict__ q, int q_stride, const bf16_t* __restrict__ k_cache,
                        const bf16_t* __restrict__ v_cache, const int32_t* __restrict__ block_table, int table_stride,
                        const int32_t* __restrict__ positions, const int32_t* __restrict__ seq_rows,
                        const int32_t* __restrict__ token_index, int n_tokens, const int32_t* __restrict__ work,
                        float* __restrict__ partial, int max_chunks, int n_heads, int n_kv_heads, int page_size,
                        int window, float scale) {
  using S = AttStage<HD>;
  constexpr int KS = HD / 16, DT = HD / 32;
  extern __shared__ __align__(16) unsigned char smem[];
  static_assert(DC_CHUNK / ATT_BLOCK == 4 && (BW == 1 || BW == 4), "four blocks of positions a chunk");
  const int lane = threadIdx.x & 63;
  const int wave = BW == 1 ? blockIdx.x & 3 : __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // which 64 positions of the chunk (a scalar)
  const int unit = BW == 1 ? blockIdx.x >> 2 : blockIdx.x;
  const int item = work[unit / n_kv_heads];          // the kv heads of a chunk side by side: they share its pages
  if (item < 0) return;                              // padding of the list
  const int slot = item / CMB_MAX_CHUNKS, chunk = item % CMB_MAX_CHUNKS;
  if (slot >= n_tokens || chunk >= max_chunks) return;   // no item of this launch
  const int t = token_index ? token_index[slot] : slot;
  const int kvh = unit % n_kv_heads;
  const int group = n_heads / n_kv_heads;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
  const int first = (lo / DC_CHUNK) * DC_CHUNK;
  const int p0 = first + chunk * DC_CHUNK + wave * ATT_BLOCK;
  // a wave with no position at all (past the token, or wholly before the window): nothing to leave
  if (p0 > pos || p0 + ATT_BLOCK - 1 < lo) return;   // no barrier below: every wave is on its own
  const int l32 = lane & 31, half = lane >> 5;
  const int32_t* table_row = block_table + (size_t)seq_rows[t] * table_stride;
  const size_t page_stride = (size_t)n_kv_heads * HD * page_size;
  const bf16_t* k_head = k_cache + (size_t)kvh * HD * page_size;
  const bf16_t* v_head = v_cache + (size_t)kvh * HD * page_size;
  unsigned char* stage = smem + (BW == 1 ? 0 : wave) * S::K_BYTES;   // keys only

  // every page first, then every load: nothing waits behind a table entry.  V^T: k step s2 takes
  // the lane's positions p0 + 8 c .. + 7, c = 4 (s2 / 2) + 2 (s2 % 2) + half, of dim 32 dt + l32:
  // 16 bytes of one page (a page holds a multiple of 8 positions); the two halves of a wave read
  // neighbouring chunks, so an instruction reads whole rows of a page of 16 positions.
  int keep[4];
  uint4 vf[DT][4];
#pragma unroll
  for (int s2 = 0; s2 < 4; ++s2) keep[s2] = max(0, min(pos - (p0 + 8 * (4 * (s2 >> 1) + 2 * (s2 & 1) + half)) + 1, 8));
  if (page_size >= ATT_BLOCK) {
    // the block lies in one page, known to the whole wave: a scalar base and 32-bit offsets
    const int page = table_row[page_index(p0, page_size)];
#pragma unroll
    for (int n = 0; n < S::K_INSTR; ++n) att_issue_k<HD>(stage, n, lane, page, p0, pos, k_head, page_stride, page_size);
    const bf16_t* base = v_head + (size_t)page * page_stride;
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) {
      const int pa_c = min(p0 + 8 * (4 * (s2 >> 1) + 2 * (s2 & 1) + half), pos);
      const unsigned at = page_offset(pa_c, page_size) & ~7;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt)
        vf[dt][s2] = *reinterpret_cast<const uint4*>(base + (unsigned)((dt * 32 + l32) * page_size + at));
    }
  } else {
    int k_page[S::K_INSTR], v_page[4], v_at[4];
#pragma unroll
    for (int n = 0; n < S::K_INSTR; ++n) k_page[n] = att_k_page<HD>(n, lane, p0, pos, table_row, page_size);
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) {
      const int pa_c = min(p0 + 8 * (4 * (s2 >> 1) + 2 * (s2 & 1) + half), pos);   // positions past the token were never written
      v_page[s2] = table_row[page_index(pa_c, page_size)];
      v_at[s2] = page_offset(pa_c, page_size) & ~7;
    }
#pragma unroll
    for (int n = 0; n < S::K_INSTR; ++n) att_issue_k<HD>(stage, n, lane, k_page[n], p0, pos, k_head, page_stride, page_size);
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2) {
      const bf16_t* va = v_head + (size_t)v_page[s2] * page_stride + v_at[s2];
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) vf[dt][s2] = *reinterpret_cast<const uint4*>(va + (size_t)(dt * 32 + l32) * page_size);
    }
  }

  // Q^T (B operand): column = head of the group (zero beyond it), 8 consecutive dims from 16 ks + 8 half
  bf16x8 qf[KS];
  {
    const bf16_t* qrow = q + (size_t)t * q_stride + (size_t)(kvh * group + min(l32, group - 1)) * HD + half * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      uint4 v = *reinterpret_cast<const uint4*>(qrow + ks * 16);
      if (l32 >= group) v = uint4{0, 0, 0, 0};
      qf[ks] = frag_of(v);
    }
  }
  wait_vmcnt<0>();                    // the stage is this wave's alone: what it loaded is what it reads
  // weights of unwritten positions are zero, and zero times whatever a page holds must stay zero:
  // only the block that holds the token's own position has any (one branch for the wave), and
  // there a word of two positions keeps both, the first or none of them
  if (p0 + ATT_BLOCK - 1 > pos) {
#pragma unroll
    for (int s2 = 0; s2 < 4; ++s2)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int kept = keep[s2] - 2 * i;                          // positions of word i that were written
        const uint32_t mask = kept >= 2 ? 0xffffffffu : kept == 1 ? 0x0000ffffu : 0u;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) reinterpret_cast<uint32_t*>(&vf[dt][s2])[i] &= mask;
      }
  }
  const bool whole = p0 + ATT_BLOCK - 1 <= pos && p0 >= lo;
  float m_b, l_b;
  bf16x8 pf[4];
  const unsigned st = (unsigned)(size_t)(lds_ptr_t)stage;
  attention_scores<HD>(st, qf, p0, whole, pos, lo, scale * LOG2E, lane, m_b, l_b, pf);
  const int block = chunk * (DC_CHUNK / ATT_BLOCK) + wave;
  float* dst = partial + (((size_t)slot * n_heads + kvh * group + min(l32, group - 1)) *
                              (max_chunks * (DC_CHUNK / ATT_BLOCK)) + block) * (HD + 2);
  const bool head_live = l32 < group;
  attention_values_of<HD>(vf, pf, [&](int dt, const f32x16& tile) {
    if (!head_live) return;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      const int d = dt * 32 + g * 8 + half * 4;
      *reinterpret_cast<float2*>(dst + d) = make_float2(tile[g * 4 + 0], tile[g * 4 + 1]);
      *reinterpret_cast<float2*>(dst + d + 2) = make_float2(tile[g * 4 + 2], tile[g * 4 + 3]);
    }
  });
  if (head_live && half == 0) {
    dst[HD] = m_b;
    dst[HD + 1] = l_b;
  }
}

// The fold of a token's blocks, in ascending order, with the prompt kernel's own arithmetic
// (attention_fold: the factors a = 2^(m - m'), b = 2^(m_b - m') of the old state and of the
// block, m' the new maximum; l' = fma(l, a, l_b b), o' = fma(o, a, o_b b)).
// grid (tokens, heads), HD threads.  The factors depend on the blocks' maxima alone, so they are
// worked out for HD blocks at once, thread i those of block i (the running maximum before a block
// is the largest of the maxima before it: no rounding, any order), and only the two multiply-adds
// a block remain a chain: thread d folds dim d, every thread folds l for itself.
template <int HD>
__global__ void __launch_bounds__(HD)
attention_combine_kernel(const float* __restrict__ partial, const int32_t* __restrict__ positions,
                         const int32_t* __restrict__ token_index, bf16_t* __restrict__ out, int max_chunks, int n_heads,
                         int window) {
  __shared__ float block_max[HD], block_sum[HD], wave_max[HD / 64];
  __shared__ __align__(16) float old_factor[HD], new_factor[HD], scaled_sum[HD];   // a, b, and l_b b, of the group's blocks
  const int t = token_index ? token_index[blockIdx.x] : blockIdx.x, head = blockIdx.y, d = threadIdx.x;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos + 1 - window) : 0;
  const int first = (lo / DC_CHUNK) * DC_CHUNK;
  const int b0 = (lo - first) / ATT_BLOCK, b1 = (pos - first) / ATT_BLOCK;     // the blocks that hold seen positions
  const float* src = partial + ((size_t)blockIdx.x * n_heads + head) * (max_chunks * (DC_CHUNK / ATT_BLOCK)) * (HD + 2);
  float m = -INFINITY, l = 0.0f, o = 0.0f;     // m: the maximum of all blocks before this group
  for (int g0 = b0; g0 <= b1; g0 += HD) {
    const int n = min(HD, b1 - g0 + 1);        // blocks of this group
    if (g0 > b0) __syncthreads();              // everyone has read the group before
    if (d < n) {
      const float* p = src + (size_t)(g0 + d) * (HD + 2);
      block_max[d] = p[HD];
      block_sum[d] = p[HD + 1];
    }
    __syncthreads();
    {
      // the running maximum before block d: a scan over the lanes of each wave, then the waves before
      const int lane = d & 63, wave = d >> 6;
      const float mine = d < n ? block_max[d] : -INFINITY;
      float upto = mine;                       // the largest of this wave's blocks up to d
#pragma unroll
      for (int off = 1; off < 64; off <<= 1) {
        const float other = __shfl_up(upto, off, AXON_WAVE);
        if (lane >= off) upto = fmaxf(upto, other);
      }
      float before = __shfl_up(upto, 1, AXON_WAVE);
      if (lane == 0) before = -INFINITY;
      if (lane == 63) wave_max[wave] = upto;
      __syncthreads();
      before = fmaxf(before, m);
      for (int w = 0; w < wave; ++w) before = fmaxf(before, wave_max[w]);
      if (d < n) {
        float fa, fb, unused = 0.0f;
        attention_fold(before, unused, mine, 0.0f, fa, fb);
        old_factor[d] = fa;
        new_factor[d] = fb;
        scaled_sum[d] = __fmul_rn(block_sum[d], fb);
      }
    }
    __syncthreads();
    // the fold is a chain, the loads are not: thirty-two blocks' values under way at a time where
    // that many are left, then sixteen; the blocks' factors come from LDS four at a time
    int i = 0;
    auto fold_batch = [&](auto count) {
      constexpr int COUNT = decltype(count)::value;
      for (; i + COUNT - 1 < n; i += COUNT) {
        float ob[COUNT];
#pragma unroll
        for (int j = 0; j < COUNT; ++j) ob[j] = src[(size_t)(g0 + i + j) * (HD + 2) + d];
#pragma unroll
        for (int q = 0; q < COUNT / 4; ++q) {
          const float4 fa = *reinterpret_cast<const float4*>(&old_factor[i + 4 * q]);
          const float4 fb = *reinterpret_cast<const float4*>(&new_factor[i + 4 * q]);
          const float4 ls = *reinterpret_cast<const float4*>(&scaled_sum[i + 4 * q]);
          const float a4[4] = {fa.x, fa.y, fa.z, fa.w}, b4[4] = {fb.x, fb.y, fb.z, fb.w}, l4[4] = {ls.x, ls.y, ls.z, ls.w};
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            l = __builtin_fmaf(l, a4[e], l4[e]);
            attention_fold_into(o, a4[e], ob[4 * q + e], b4[e]);
          }
        }
      }
    };
    fold_batch(std::integral_constant<int, 32>());
    fold_batch(std::integral_constant<int, 16>());
    for (; i < n; ++i) {
      const float fa = old_factor[i], fb = new_factor[i];
      l = __builtin_fmaf(l, fa, scaled_sum[i]);
      attention_fold_into(o, fa, src[(size_t)(g0 + i) * (HD + 2) + d], fb);
    }
    for (int w = 0; w < HD / 64; ++w) m = fmaxf(m, wave_max[w]);     // blocks past n count as -inf
  }
  out[(size_t)t * n_heads * HD + (size_t)head * HD + d] = float_to_bf16(__fmul_rn(o, attention_inverse(l)));
}

#endif  // AXON_BF16

// ============================================================================ entry points
// 1 if the MFMA attention kernels take this head size, page size and group of heads.
extern "C" int axk_attention_fast_ok(int head_dim, int page_size, int n_heads, int n_kv_heads) {
#if AXON_BF16
  const bool hd_ok = head_dim == 64 || head_dim == 128;
  const bool page_ok = page_size >= 8 && page_size <= 1024 && (page_size & (page_size - 1)) == 0;
  return hd_ok && page_ok && n_kv_heads > 0 && n_heads % n_kv_heads == 0 && n_heads / n_kv_heads <= 32;
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
#define LAUNCH_PAGED(HD, HPB, ONE_PAGE)                                                                             \
  {                                                                                                                 \
    static bool configured = false;                                                                                 \
    constexpr int lds = 2 * (ATT_BLOCK * HD * 2 + HD * ATT_BLOCK * 2);                                                \
    const dim3 grid(n_tiles, n_kv_heads * ((group + HPB - 1) / HPB));                                               \
    if (!configured) {                                                                                              \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_prefill_kernel<HD, HPB, ONE_PAGE>), \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);                          \
      if (e != hipSuccess) {                                                                                        \
        axk_set_error("attention_prefill: cannot reserve %d bytes of LDS: %s", lds, hipGetErrorString(e));          \
        return -2;                                                                                                  \
      }                                                                                                             \
      configured = true;                                                                                            \
    }                                                                                                               \
    AXK_INSTANCE(INST_ATTENTION_PREFILL, HD, HPB, ONE_PAGE);                                                        \
    attention_prefill_kernel<HD, HPB, ONE_PAGE><<<grid, 256 * HPB, lds, (hipStream_t)stream>>>(                     \
        (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_stride,      \
        positions, seq_rows, (bf16_t*)out, tiles, n_heads, n_kv_heads, page_size, window, scale);                   \
  }
#define LAUNCH(HD, HPB) \
  if (page_size >= ATT_BLOCK) LAUNCH_PAGED(HD, HPB, 1) else LAUNCH_PAGED(HD, HPB, 0)
  // one query head a block while such blocks find a CU each (256 of them); beyond that two query
  // heads of a kv head a block, which share each K and V block in LDS and whose waves fill each
  // other's waits (7B sizes: 2,304 tokens 88 against 101 us with one head, 2,560 tokens 123 against
  // 109 us with two; 14B sizes at 2,048 tokens 101 against 88 us)
  if (group >= 2 && (long)n_tiles * n_heads > 256) {
    if (head_dim == 64) LAUNCH(64, 2) else LAUNCH(128, 2)
  } else {
    if (head_dim == 64) LAUNCH(64, 1) else LAUNCH(128, 1)
  }
#undef LAUNCH
#undef LAUNCH_PAGED
  AXK_LAUNCH_CHECK("attention_prefill");
  return 0;
#else
  axk_set_error("attention_prefill: only in the bfloat16 build");
  return -1;
#endif
}

// The most consecutive tokens of one request that a run of axk_attention_prefill's tiles holds.
extern "C" int axk_attention_prefill_tile(void) { return 128; }

// Positions of one chunk of a decoding token's range, and the factor of the token's slot in an
// item of the work list (item = slot * factor + chunk).
extern "C" int axk_attention_decode_chunk(void) { return DC_CHUNK; }
extern "C" int axk_attention_decode_item_factor(void) { return CMB_MAX_CHUNKS; }

// Floats of `partial` that n_tokens decoding tokens with up to max_chunks chunks need.
extern "C" long axk_attention_decode_workspace(int n_tokens, int n_heads, int head_dim, int max_chunks) {
  return (long)n_tokens * n_heads * max_chunks * (DC_CHUNK / ATT_BLOCK) * (head_dim + 2);
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
  AXK_REQUIRE(partial != nullptr && ((uintptr_t)partial & 7) == 0, "attention_decode: needs its workspace, 8-byte aligned");
  AXK_REQUIRE(n_work >= 0 && (n_work == 0 || work != nullptr) && (long)n_work * n_kv_heads * 4 < (1l << 31),
              "attention_decode: a work list of %d items", n_work);
  if (n_tokens == 0 || n_work == 0) return 0;
  // A wave a block where every wave finds a place on the chip at once (ten a CU): an even spread
  // over the CUs; blocks of four waves where there are more, which are launched faster.
  const bool single = (long)n_work * n_kv_heads * 4 <= 2560;
  dim3 cgrid(n_tokens, n_heads);
#define LAUNCH(HD, BW)                                                                                               \
  {                                                                                                                  \
    static bool configured = false;                                                                                  \
    constexpr int lds = BW * ATT_BLOCK * HD * 2;                             /* a wave its block's keys */        \
    if (!configured) {                                                                                               \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attention_decode_kernel<HD, BW>),            \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, lds);                           \
      if (e != hipSuccess) {                                                                                         \
        axk_set_error("attention_decode: cannot reserve %d bytes of LDS: %s", lds, hipGetErrorString(e));            \
        return -2;                                                                                                   \
      }                                                                                                              \
      configured = true;                                                                                             \
    }                                                                                                                \
    AXK_INSTANCE(INST_ATTENTION_DECODE, HD, BW);                                                                     \
    attention_decode_kernel<HD, BW><<<(unsigned)n_work * n_kv_heads * (4 / BW), BW * 64, lds, (hipStream_t)stream>>>( \
        (const bf16_t*)q, q_stride, (const bf16_t*)k_cache, (const bf16_t*)v_cache, block_table, table_stride,       \
        positions, seq_rows, token_index, n_tokens, work, partial, max_chunks, n_heads, n_kv_heads, page_size,       \
        window, scale);                                                                                              \
    attention_combine_kernel<HD><<<cgrid, HD, 0, (hipStream_t)stream>>>(partial, positions, token_index,            \
                                                                       (bf16_t*)out, max_chunks, n_heads, window);   \
  }
  if (head_dim == 64) { if (single) LAUNCH(64, 1) else LAUNCH(64, 4) }
  else { if (single) LAUNCH(128, 1) else LAUNCH(128, 4) }
#undef LAUNCH
  AXK_LAUNCH_CHECK("attention_decode");
  return 0;
#else
  axk_set_error("attention_decode: only in the bfloat16 build");
  return -1;
#endif
}
