// Shared helpers of the sequence-mixer kernels (gfx950, wave64).
//
// Activations are either fp32 or bf16 (raw u16 bits); statistics, the
// residual stream, rotary angles, softmax and recurrent state are fp32
// in both modes. Kernels are templated on the activation type `A`.
#pragma once

#include "common.h"

namespace fi {

template <typename A>
struct Act;

template <>
struct Act<float> {
  static FI_DEV float ld(const float* p) { return *p; }
  static FI_DEV void st(float* p, float v) { *p = v; }
};

template <>
struct Act<u16> {
  static FI_DEV float ld(const u16* p) { return bf16_to_f32(*p); }
  static FI_DEV void st(u16* p, float v) { *p = f32_to_bf16(v); }
};

// VW consecutive activations (VW = 1, or 4 with one 16-/8-byte access)
template <typename A, int VW>
FI_DEV void ldv(const A* p, float* v);
template <typename A, int VW>
FI_DEV void stv(A* p, const float* v);

template <>
FI_DEV void ldv<float, 1>(const float* p, float* v) { v[0] = *p; }
template <>
FI_DEV void ldv<u16, 1>(const u16* p, float* v) { v[0] = bf16_to_f32(*p); }
template <>
FI_DEV void ldv<float, 4>(const float* p, float* v) {
  const float4 x = *reinterpret_cast<const float4*>(p);
  v[0] = x.x; v[1] = x.y; v[2] = x.z; v[3] = x.w;
}
template <>
FI_DEV void ldv<u16, 4>(const u16* p, float* v) {
  const bf16x4 x = *reinterpret_cast<const bf16x4*>(p);
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = bf16_to_f32(x.h[i]);
}
template <>
FI_DEV void ldv<u16, 8>(const u16* p, float* v) {
  const bf16x4 x = *reinterpret_cast<const bf16x4*>(p);
  const bf16x4 y = *reinterpret_cast<const bf16x4*>(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    v[i] = bf16_to_f32(x.h[i]);
    v[4 + i] = bf16_to_f32(y.h[i]);
  }
}
template <>
FI_DEV void stv<float, 1>(float* p, const float* v) { *p = v[0]; }
template <>
FI_DEV void stv<u16, 1>(u16* p, const float* v) { *p = f32_to_bf16(v[0]); }
template <>
FI_DEV void stv<float, 4>(float* p, const float* v) {
  *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
}
template <>
FI_DEV void stv<u16, 4>(u16* p, const float* v) {
  bf16x4 x;
#pragma unroll
  for (int i = 0; i < 4; ++i) x.h[i] = f32_to_bf16(v[i]);
  *reinterpret_cast<bf16x4*>(p) = x;
}

// Sum of two values over a 256-thread block at once (one barrier pair).
// scratch: 8 floats. Safe to call repeatedly with the same scratch.
FI_DEV void block_reduce_sum2_256(float& a, float& b, float* scratch) {
  a = wave_reduce_sum(a);
  b = wave_reduce_sum(b);
  const int wave = threadIdx.x / kWaveSize;
  const int lane = threadIdx.x % kWaveSize;
  __syncthreads();  // previous readers of scratch are done
  if (lane == 0) {
    scratch[wave] = a;
    scratch[4 + wave] = b;
  }
  __syncthreads();
  a = scratch[0] + scratch[1] + scratch[2] + scratch[3];
  b = scratch[4] + scratch[5] + scratch[6] + scratch[7];
}

FI_DEV float sigmoidf_acc(float x) { return 1.0f / (1.0f + expf(-x)); }

}  // namespace fi
