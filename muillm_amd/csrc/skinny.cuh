// Interface between the single-token GEMV entry points and the small-batch MFMA kernel.
#pragma once

#include "common.cuh"

namespace mui {

enum { WF_16BIT = 0, WF_I8_CHANNEL = 1, WF_U8_GROUP = 2 };
enum { SK_LINEAR = 0, SK_GATEUP = 1 };

struct SkinnyParams {
  const void* w0;       // linear: matrix; gate/up: gate rows
  const void* w1;       // gate/up: up rows
  long pitch;           // row pitch in weight elements
  const uint16_t* s0;   // I8_CHANNEL: scale of row n at s0[n*s_pitch]; U8_GROUP: pairs at s0 + n*s_pitch + 2g
  const uint16_t* s1;
  long s_pitch;
  int group_shift;
  const uint16_t* x;    // [tokens, k]
  const uint16_t* gamma;
  const uint16_t* mul_bias;
  const uint16_t* add_bias;
  const uint16_t* residual;  // [tokens, n]
  uint16_t* y;               // [tokens, n]
  int n;       // outputs (weight rows, or gate/up pairs)
  int k;
  int tokens;  // 2..8 (1 works too)
  float eps;
};

// launches gemm_skinny_kernel<dtype, weight format, epilogue>; returns a MUI_* status
int launch_skinny(hipStream_t s, int dtype, int weight_format, int epilogue, const SkinnyParams& p);
// experiments: 0 disables the B-stationary persistent variant
void skinny_set_bstat(int on);

}  // namespace mui
