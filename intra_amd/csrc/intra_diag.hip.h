// Measurement kernel: what the matrix cores of the board sustain when they do nothing else.
//
// Every wavefront of every workgroup (8 per CU) issues back-to-back bf16 MFMAs into independent
// accumulators, v_mfma_f32_16x16x32_bf16 (SHAPE16: the instruction of the forward and backward kernels, 8 accumulators)
// or v_mfma_f32_32x32x16_bf16 (the shape these kernels used before, 4 accumulators), the same flop count per
// iteration either way, on operands taken once from a caller-filled table, so the same launch can
// be timed with constant and with random operand bits: on a power-limited board the sustained
// clock, and with it the attainable fraction of the nominal peak, depends on how many operand and
// accumulator bits toggle, and on the instruction shape.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace intra {

constexpr int CEILING_TABLE_BYTES = 8192 * 16;  // operand table: 8192 entries of 16 bytes
constexpr int CEILING_FLOP_PER_ITER = 16 * 32768;  // per wavefront: 16 MFMAs of 32x32x16 or 32 of 16x16x32

// sink: grid * 512 floats (keeps the accumulators alive); clocks: per workgroup {shader cycles,
// 100 MHz wall-clock ticks} of the loop
template <bool SHAPE16>
__global__ __launch_bounds__(512) void mfma_ceiling_kernel(const uint4* table, float* sink, int iters, long long* clocks) {
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  typedef float floatx16 __attribute__((ext_vector_type(16)));
  typedef float floatx4 __attribute__((ext_vector_type(4)));
  const int l = threadIdx.x;
  bf16x8 a[8], b[8];
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    a[r] = __builtin_bit_cast(bf16x8, table[(l * 16 + r) & 8191]);
    b[r] = __builtin_bit_cast(bf16x8, table[(l * 16 + 8 + r) & 8191]);
  }
  floatx16 acc[4];
  floatx4 acc4[8];
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[r][e] = 0.f;
#pragma unroll
  for (int r = 0; r < 8; ++r) acc4[r] = floatx4{0.f, 0.f, 0.f, 0.f};
  const long long c0 = __builtin_readcyclecounter(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
    if (SHAPE16) {
#pragma unroll
      for (int r = 0; r < 32; ++r)
        acc4[r & 7] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[r & 7], b[(r * 3) & 7], acc4[r & 7], 0, 0, 0);
    } else {
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[r & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[r & 7], b[(r * 3) & 7], acc[r & 3], 0, 0, 0);
    }
  }
  const long long c1 = __builtin_readcyclecounter(), w1 = wall_clock64();
  float s = 0.f;
#pragma unroll
  for (int r = 0; r < 4; ++r)
#pragma unroll
    for (int e = 0; e < 16; ++e) s += acc[r][e];
#pragma unroll
  for (int r = 0; r < 8; ++r) s += acc4[r][0] + acc4[r][1] + acc4[r][2] + acc4[r][3];
  sink[(size_t)blockIdx.x * 512 + l] = s;
  if (l == 0) {
    clocks[2 * blockIdx.x] = c1 - c0;
    clocks[2 * blockIdx.x + 1] = w1 - w0;
  }
}

}  // namespace intra
