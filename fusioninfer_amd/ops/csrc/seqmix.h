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
