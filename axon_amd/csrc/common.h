// Shared by every kernel file: the element type of this build, conversions, wave-level
// reductions with a fixed order, and the error channel of the C interface.
//
// The library is compiled once per compute dtype: -DAXON_BF16=1 gives the bfloat16 build
// (what serving uses: bf16 operands, every sum in 32-bit), -DAXON_BF16=0 the float32 build
// (true 32-bit products and sums everywhere).  Both export the same C symbols.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#ifndef AXON_BF16
#error "compile with -DAXON_BF16=0 or -DAXON_BF16=1"
#endif

#define AXON_WAVE 64

// ---------------------------------------------------------------------------- bf16
struct bf16_t {
  uint16_t bits;
};

__host__ __device__ inline float bf16_to_float(bf16_t v) {
  union { uint32_t u; float f; } c;
  c.u = ((uint32_t)v.bits) << 16;
  return c.f;
}

// Round to nearest, ties to even; NaN stays NaN (quiet).  On the device this is the hardware's
// conversion (one instruction on gfx950); the host version does the same in integer arithmetic.
__host__ __device__ inline bf16_t float_to_bf16(float f) {
  bf16_t r;
#if defined(__HIP_DEVICE_COMPILE__)
  const __bf16 h = (__bf16)f;
  __builtin_memcpy(&r.bits, &h, sizeof r.bits);
#else
  union { uint32_t u; float f; } c;
  c.f = f;
  if ((c.u & 0x7fffffffu) > 0x7f800000u) {
    r.bits = (uint16_t)((c.u >> 16) | 0x0040u);
    return r;
  }
  uint32_t lsb = (c.u >> 16) & 1u;
  c.u += 0x7fffu + lsb;
  r.bits = (uint16_t)(c.u >> 16);
#endif
  return r;
}

// Two floats to a packed pair of bfloat16 (low half first).
__device__ inline uint32_t pack2_bf16(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  const f32x2_t v = {a, b};
  const bf16x2_t h = __builtin_convertvector(v, bf16x2_t);
  uint32_t r;
  __builtin_memcpy(&r, &h, sizeof r);
  return r;
}

#if AXON_BF16
typedef bf16_t elem_t;
__host__ __device__ inline float to_float(elem_t v) { return bf16_to_float(v); }
__host__ __device__ inline elem_t from_float(float f) { return float_to_bf16(f); }
#else
typedef float elem_t;
__host__ __device__ inline float to_float(elem_t v) { return v; }
__host__ __device__ inline elem_t from_float(float f) { return f; }
#endif

// A vector (gain or bias) keeps the precision it was stored in: the caller says which.
__device__ inline float load_vec(const void* p, int is_f32, int i) {
  return is_f32 ? ((const float*)p)[i] : bf16_to_float(((const bf16_t*)p)[i]);
}

// Four consecutive elements as floats: one 8- or 16-byte load where `vec` says the address is
// aligned for it and all four exist, else the `valid` first ones singly and zeros behind them.
__device__ inline void load4_guarded(const elem_t* __restrict__ p, int valid, bool vec, float out[4]) {
  if (vec && valid >= 4) {
#if AXON_BF16
    const uint2 raw = *reinterpret_cast<const uint2*>(p);
    union { uint32_t u; float f; } c;
    c.u = raw.x << 16; out[0] = c.f;
    c.u = raw.x & 0xffff0000u; out[1] = c.f;
    c.u = raw.y << 16; out[2] = c.f;
    c.u = raw.y & 0xffff0000u; out[3] = c.f;
#else
    const float4 raw = *reinterpret_cast<const float4*>(p);
    out[0] = raw.x; out[1] = raw.y; out[2] = raw.z; out[3] = raw.w;
#endif
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = i < valid ? to_float(p[i]) : 0.0f;
  }
}

// ---------------------------------------------------------------------------- reductions
// Butterfly over the 64 lanes of a wave: every lane ends with the same value, and the order
// of the additions is fixed by the lane numbers alone.
__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, AXON_WAVE);
  return v;
}

// The sum of the 64 lanes in lane 63 alone (other lanes end with partial sums), through the
// lane-permuting forms of the adder instead of the LDS crossbar: a few cycles a step where the
// butterfly above takes an LDS round trip.  Pairs, quads, halves of a row of 16, the row, then
// rows 0+1 and 2+3, then both: the order is fixed.
__device__ inline float wave_sum_to_last(float v) {
#define AXON_DPP(val, ctrl, rows) \
  __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, val), ctrl, rows, 0xf, false))
  v += AXON_DPP(v, 0xb1, 0xf);    // quad_perm [1, 0, 3, 2]
  v += AXON_DPP(v, 0x4e, 0xf);    // quad_perm [2, 3, 0, 1]
  v += AXON_DPP(v, 0x141, 0xf);   // row_half_mirror
  v += AXON_DPP(v, 0x140, 0xf);   // row_mirror
  v += AXON_DPP(v, 0x142, 0xa);   // lane 15 of rows 0 and 2 to the rows after them
  v += AXON_DPP(v, 0x143, 0xc);   // lane 31 to rows 2 and 3
#undef AXON_DPP
  return v;
}

// The sum over a block of 256 threads: within each wave (butterfly), then the four waves' sums
// in wave order.  `partial` is 4 floats of LDS; every thread returns the same value.
__device__ inline float block_sum_256(float v, float* partial) {
  v = wave_sum(v);
  if ((threadIdx.x & (AXON_WAVE - 1)) == 0) partial[threadIdx.x / AXON_WAVE] = v;
  __syncthreads();
  float total = partial[0];
#pragma unroll
  for (int w = 1; w < 256 / AXON_WAVE; ++w) total += partial[w];
  return total;
}

__device__ inline float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, AXON_WAVE));
  return v;
}

// ---------------------------------------------------------------------------- LDS reads as instructions
// A kernel that fills LDS with direct global -> LDS loads while it reads other parts of LDS has
// to write those reads as instructions: the compiler cannot tell the part being read from the
// part a load is filling, and would wait for every load in flight before each read of its own,
// so that loads never overlap the work on what has landed.  The kernel then counts its reads
// itself: wait_lgkmcnt<N> returns when at most N of them are outstanding (they return in
// order), and use_frags ties registers to that point, so that what uses them stays behind it.
template <int N>
__device__ inline void wait_vmcnt() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int N>
__device__ inline void wait_lgkmcnt() {
  asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(N) : "memory");
}

typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

// 16 bytes a lane from LDS byte address `lds_address` + OFFSET.
template <int OFFSET>
__device__ inline void lds_read16(u32x4& dst, unsigned lds_address) {
  static_assert(OFFSET >= 0 && OFFSET < 65536, "the offset field of an LDS read");
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(lds_address), "n"(OFFSET));
}

// The same at OFFSET = i STEP, i < MAX a constant once the caller's loop is unrolled.
template <int STEP, int MAX>
__device__ __forceinline__ void lds_read16_step(u32x4& dst, unsigned lds_address, int i) {
  if constexpr (MAX > 0) {
    if (i == MAX - 1)
      lds_read16<(MAX - 1) * STEP>(dst, lds_address);
    else
      lds_read16_step<STEP, MAX - 1>(dst, lds_address, i);
  }
}

// COUNT such reads, STEP bytes apart.
template <int COUNT, int STEP, int I = 0>
__device__ inline void read_frags(u32x4 (&dst)[COUNT], unsigned lds_address) {
  if constexpr (I < COUNT) {
    lds_read16<I * STEP>(dst[I], lds_address);
    read_frags<COUNT, STEP, I + 1>(dst, lds_address);
  }
}

template <int COUNT>
__device__ inline void use_frags(u32x4 (&regs)[COUNT]) {
#pragma unroll
  for (int i = 0; i < COUNT; ++i) asm volatile("" : "+v"(regs[i]));
}

// ---------------------------------------------------------------------------- errors
// Every entry point returns 0, or a negative code after recording a message that
// axk_last_error() returns.  Shapes are checked on the host before anything is launched.
void axk_set_error(const char* fmt, ...);

#define AXK_REQUIRE(cond, ...)        \
  do {                                \
    if (!(cond)) {                    \
      axk_set_error(__VA_ARGS__);     \
      return -1;                      \
    }                                 \
  } while (0)

#define AXK_LAUNCH_CHECK(name)                                              \
  do {                                                                      \
    hipError_t e_ = hipGetLastError();                                      \
    if (e_ != hipSuccess) {                                                 \
      axk_set_error("%s: launch failed: %s", name, hipGetErrorString(e_));  \
      return -2;                                                            \
    }                                                                       \
  } while (0)

static inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Epilogues of a matrix product (see axk_gemm).
enum { MODE_STORE = 0, MODE_ADD_F32 = 1, MODE_STORE_F32 = 2, MODE_SWIGLU = 3 };

// act = (g / (1 + exp(-g))) * u: divide, then multiply (src/vmath.rs:128-132;
// src/cuda/prefill.cu:109-123).
__device__ inline float swiglu1(float g, float u) { return __fmul_rn(__fdiv_rn(g, 1.0f + expf(-g)), u); }
