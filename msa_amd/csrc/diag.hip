// Diagnostics that back the roofline figures: what the matrix cores of this GPU sustain when nothing but MFMAs runs.
// The published dense bf16 peak assumes the boost clock; under MFMA load with operands that toggle, the shader clock
// falls with power, and the rate a register-only loop reaches is the ceiling any kernel of the library can be held to.
#include "common.h"

namespace {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float floatx16_t __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kThreads = 512;          // 8 wavefronts, two per SIMD: the scoring kernel's occupancy
constexpr int kMfmasPerIter = 8;       // a 4 x 2 grid of 32 x 32 accumulators per wavefront, as in the scoring kernel

// mode 0: zero operands; 1: all ones (the result is known exactly: 16 per MFMA); 2: operands whose mantissas and signs
// change from one iteration to the next (what a GEMM on real data presents to the multipliers)
__global__ __launch_bounds__(kThreads) void mfma_loop_kernel(int32_t iters, int32_t mode, float* __restrict__ sink) {
  const uint32_t tid = blockIdx.x * kThreads + threadIdx.x;
  u32x4_t a[4], b[2];
  uint32_t seed = tid * 2654435761u + 12345u;
  auto word = [&]() -> uint32_t {
    if (mode == 0) return 0u;
    if (mode == 1) return 0x3f803f80u;                       // two bf16 ones
    seed = seed * 1664525u + 1013904223u;
    return (seed & 0x807f807fu) | 0x3f803f80u;               // random sign and mantissa, exponent of 1.0
  };
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = u32x4_t{word(), word(), word(), word()};
#pragma unroll
  for (int j = 0; j < 2; ++j) b[j] = u32x4_t{word(), word(), word(), word()};
  const uint32_t flip = mode == 2 ? 0x00550055u : 0u;        // mantissa bits that toggle every iteration
  floatx16_t acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[i]),
                                                            __builtin_bit_cast(bf16x8_t, b[j]), acc[i][j], 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] ^= flip;
#pragma unroll
    for (int j = 0; j < 2; ++j) b[j] ^= flip;
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) s += acc[i][j][0];
  sink[tid] = s;
}

}  // namespace

extern "C" int msa_diag_mfma_loop(int32_t workgroups, int32_t iters, int32_t mode, float* sink, double* flops_out,
                                  void* stream) {
  MSA_REQUIRE(workgroups > 0 && workgroups <= 65536 && iters > 0 && iters <= (1 << 24), "msa_diag_mfma_loop: bad sizes");
  MSA_REQUIRE(mode >= 0 && mode <= 2 && sink != nullptr, "msa_diag_mfma_loop: bad mode / null sink");
  mfma_loop_kernel<<<workgroups, kThreads, 0, as_stream(stream)>>>(iters, mode, sink);
  MSA_LAUNCH_CHECK();
  if (flops_out)
    *flops_out = (double)workgroups * (kThreads / 64) * (double)iters * kMfmasPerIter * (2.0 * 32 * 32 * 16);
  return MSA_OK;
}
