// Which kernel instance a launch chose.
//
// The products and the attention are templates with many instances (tile shapes, waves a block,
// segments, epilogues), one of which a dispatch picks from the sizes of a call.  An instance that
// no test ever launches is unverified arithmetic: so every launch site names its instance here,
// the library knows every instance that was compiled into it (they register themselves when the
// library is loaded) and which of them have been launched since the last reset, and a test
// asserts that the two lists are the same (the reference tests its products at the sizes of its
// models for the same reason: src/cuda/prefill.cu:1100, src/model.rs:6238-6319).
//
//   AXK_INSTANCE(INST_GEMM_TILE, BM, BN, ...);     // at the launch, inside the launching template
//
// Host code only; costs one store a launch.
#pragma once

#include <initializer_list>

enum {
  INST_GEMM_FMA = 0,
  INST_GEMM_TILE,            // BM, BN, waves m, waves n, gated, stages
  INST_GEMM_STREAM,          // row tiles, tiles of X rows, segments, epilogue
  INST_GEMM_NORMED,          // tile pairs a wave, segments, epilogue, rows of X in LDS, float4 a lane
  INST_GEMM_ROWS,            // row tiles of W a wave, tiles of 16 rows of X, waves, epilogue
  INST_GEMM_SPLIT_REDUCE,    // 0 plain, 1 with the norm, 2 with the rotary store
  INST_ATTENTION_ROWS,       // bfloat16 build, waves a (token, head)
  INST_ATTENTION_PREFILL,    // head_dim, query heads a block, pages of 64 positions or more
  INST_ATTENTION_DECODE,     // head_dim, waves a block
  INST_RMSNORM,              // 1: rows read as float4
  INST_KINDS
};

int axk_register_instance(int kind, std::initializer_list<int> params);
void axk_note_instance(int id);

template <int KIND, int... P>
struct KernelInstance {
  static const int id;
};
template <int KIND, int... P>
const int KernelInstance<KIND, P...>::id = axk_register_instance(KIND, {P...});

#define AXK_INSTANCE(...) axk_note_instance(KernelInstance<__VA_ARGS__>::id)
