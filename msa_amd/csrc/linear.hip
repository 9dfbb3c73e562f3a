// Weight-streaming linear layer for a handful of rows (the decode step of the host model):
//   y[M, N] = x[M, K] . w[N, K]^T   (+ residual, or silu(gate) * up over interleaved row groups)
// with M <= 16.  The weight matrix is read from HBM exactly once, which is the whole cost: per
// decode step of a 36-layer model the projections stream ~8 GB.  The 16 rows of x are exactly one
// 16x16x32 MFMA operand, so a wavefront multiplies 16 weight rows (one row group) at a time:
//   lane (n = lane % 16, g = lane / 16), vector j = 0..J-1, loads the 16 bytes of weight row n at
//   k = unit * 32 J + 32 j + 8 g   (one load instruction covers 64 contiguous bytes of each of 16 rows),
// and the same bytes of x row n (J = 4, or 2 when the RMSNorm is folded in).  The contraction order
// inside a unit is permuted the same way on both operands, which a dot product does not see.  A workgroup owns R row groups and splits
// K over its wavefronts; partial sums meet in LDS and are added in wavefront order (deterministic).
#include <algorithm>

#include "common.h"

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4_t;
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kUnit = 128;           // K must be a multiple of this; a wavefront steps through K in units of 32 J
constexpr int kMaxWaves = 16;

enum { kEpiPlain = 0, kEpiResidual = 1, kEpiSiluMul = 2 };

// two floats -> packed bf16 pair, round to nearest even in hardware (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_rne(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  union { bf16x2_t b; uint32_t u; } c;
  c.b = __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t);
  return c.u;
}

__device__ __forceinline__ bf16x8_t as_frag(u32x4_t v) {
  union { u32x4_t u; bf16x8_t b; } c;
  c.u = v;
  return c.b;
}

template <int R, int kEpi, bool kNorm, int J>
__global__ __launch_bounds__(kMaxWaves * 64) void skinny_linear_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const bf16_t* __restrict__ residual,
    const bf16_t* __restrict__ norm_w, float eps, bf16_t* __restrict__ y, int32_t M, int32_t N, int32_t K,
    int64_t y_row_stride) {
  constexpr int kUnitBytes = 64 * J;   // one unit = J vectors of 16 bytes per lane = 32 J elements of a row
  const int units = K / (32 * J);
  extern __shared__ __align__(16) float part[];   // [waves][R][64][4], then [waves][16] row sums of squares
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
  const int n_l = lane & 15, g = lane >> 4;
  const int n_base = blockIdx.x * (16 * R);
  const int64_t row_bytes = (int64_t)K * 2;

  // rows past N (weights) and past M (activations) read as zero through the buffer bounds
  const int rows_w = min(16 * R, N - n_base);
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(reinterpret_cast<const char*>(w)) + (int64_t)n_base * row_bytes, 0, (int)(rows_w * row_bytes),
      0x00020000);
  const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(reinterpret_cast<const char*>(x)), 0, (int)(M * row_bytes), 0x00020000);
  const int voff = n_l * (int)row_bytes + g * 16;

  // this wavefront's share of the K units
  const int u0 = (int)((int64_t)units * wave / waves), u1 = (int)((int64_t)units * (wave + 1) / waves);

  floatx4_t acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = floatx4_t{0.f, 0.f, 0.f, 0.f};

  const __amdgpu_buffer_rsrc_t rs_g = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(reinterpret_cast<const char*>(kNorm ? norm_w : x)), 0, (int)row_bytes, 0x00020000);
  float ssq = 0.f;                      // this lane's share of sum(x^2) of row n_l
  u32x4_t fw[2][R][J];
  auto load_w = [&](int slot, int u) {
    const int k_off = u * kUnitBytes;
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < J; ++j)
        fw[slot][r][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, voff + r * 16 * (int)row_bytes, k_off + j * 64, 0);
  };

  {
    u32x4_t fx[2][J];
    u32x4_t fg[kNorm ? 2 : 1][J];     // norm weights of the unit (every row group shares them; they hit L1 / L2)
    auto load_unit = [&](int slot, int u) {
      const int k_off = u * kUnitBytes;
#pragma unroll
      for (int j = 0; j < J; ++j) fx[slot][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, voff, k_off + j * 64, 0);
      if constexpr (kNorm) {
#pragma unroll
        for (int j = 0; j < J; ++j) fg[slot][j] = __builtin_amdgcn_raw_buffer_load_b128(rs_g, g * 16, k_off + j * 64, 0);
      }
      load_w(slot, u);
    };
    auto mul_unit = [&](int slot) {
      if constexpr (kNorm) {
        // RMSNorm folded in: the operand is bf16(x * norm_w); the row scale rsqrt(mean(x^2) + eps) commutes
        // with the product and is applied to the fp32 sums in the epilogue, so nothing here waits for it.
#pragma unroll
        for (int j = 0; j < J; ++j)
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const float lo = bf16lo(fx[slot][j][c]), hi = bf16hi(fx[slot][j][c]);
            ssq += lo * lo + hi * hi;
            fx[slot][j][c] = pack_rne(lo * bf16lo(fg[slot][j][c]), hi * bf16hi(fg[slot][j][c]));
          }
      }
#pragma unroll
      for (int j = 0; j < J; ++j)
#pragma unroll
        for (int r = 0; r < R; ++r)
          acc[r] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(fx[slot][j]), as_frag(fw[slot][r][j]), acc[r], 0, 0, 0);
    };
    // two register stages, one unit each: the loads of unit u+1 are in flight under the MFMAs of u
    if (u0 < u1) load_unit(0, u0);
    int u = u0;
    for (; u + 2 <= u1; u += 2) {
      load_unit(1, u + 1);
      mul_unit(0);
      if (u + 2 < u1) load_unit(0, u + 2);
      mul_unit(1);
    }
    if (u < u1) mul_unit(0);
  }

  // partial sums -> LDS; acc[r][e] is y[m = 4 g + e][n_base + 16 r + n_l]
#pragma unroll
  for (int r = 0; r < R; ++r) *reinterpret_cast<floatx4_t*>(&part[((wave * R + r) * 64 + lane) * 4]) = acc[r];
  float* row_ssq = part + waves * R * 256;
  if constexpr (kNorm) {
    ssq += __shfl_xor(ssq, 16);
    ssq += __shfl_xor(ssq, 32);
    if (g == 0) row_ssq[wave * 16 + n_l] = ssq;
  }
  __syncthreads();
  floatx4_t inv = floatx4_t{1.f, 1.f, 1.f, 1.f};   // row scales of this lane's four output rows
  if constexpr (kNorm) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      float tot = 0.f;
      for (int wv = 0; wv < waves; ++wv) tot += row_ssq[wv * 16 + 4 * g + e];
      inv[e] = rsqrtf(tot / (float)K + eps);
    }
  }
  if (kEpi == kEpiSiluMul) {
    // row groups alternate gate, up: group 2i holds gate rows [16 i, 16 i + 16), group 2i+1 the same up rows
    for (int r = 2 * wave; r < R; r += 2 * waves) {
      floatx4_t gate = floatx4_t{0.f, 0.f, 0.f, 0.f}, up = gate;
      for (int wv = 0; wv < waves; ++wv) {
        gate += *reinterpret_cast<const floatx4_t*>(&part[((wv * R + r) * 64 + lane) * 4]);
        up += *reinterpret_cast<const floatx4_t*>(&part[((wv * R + r + 1) * 64 + lane) * 4]);
      }
      const int n = ((n_base + 16 * r) >> 1) + n_l;    // output column: a pair of groups folds into one
      if (n_base + 16 * (r + 1) + n_l >= N) continue;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = 4 * g + e;
        if (m >= M) continue;
        const float a = bf16_to_f32(f32_to_bf16(gate[e] * inv[e])), b = bf16_to_f32(f32_to_bf16(up[e] * inv[e]));
        y[(int64_t)m * y_row_stride + n] = f32_to_bf16(a / (1.f + __expf(-a)) * b);
      }
    }
    return;
  }
  for (int r = wave; r < R; r += waves) {
    floatx4_t sum = floatx4_t{0.f, 0.f, 0.f, 0.f};
    for (int wv = 0; wv < waves; ++wv) sum += *reinterpret_cast<const floatx4_t*>(&part[((wv * R + r) * 64 + lane) * 4]);
    const int n = n_base + 16 * r + n_l;
    if (n >= N) continue;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int m = 4 * g + e;
      if (m >= M) continue;
      float v = sum[e] * inv[e];
      if (kEpi == kEpiResidual) v = bf16_to_f32(f32_to_bf16(v)) + bf16_to_f32(residual[(int64_t)m * y_row_stride + n]);
      y[(int64_t)m * y_row_stride + n] = f32_to_bf16(v);
    }
  }
}

template <int R, int kEpi, bool kNorm>
int launch(const void* x, const void* w, const void* residual, const void* norm_w, float eps, void* y, int32_t M,
           int32_t N, int32_t K, int waves, hipStream_t st) {
  const int groups = (N + 16 * R - 1) / (16 * R);
  const size_t lds = (size_t)waves * (R * 256 + 16) * sizeof(float);
  const int64_t y_stride = kEpi == kEpiSiluMul ? N / 2 : N;
  // with the norm folded in a unit is 64 elements instead of 128: the extra fragments then fit 128 VGPRs
  skinny_linear_kernel<R, kEpi, kNorm, kNorm ? 2 : 4><<<groups, waves * 64, lds, st>>>(
      static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<const bf16_t*>(residual),
      static_cast<const bf16_t*>(norm_w), eps, static_cast<bf16_t*>(y), M, N, K, y_stride);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

}  // namespace

extern "C" int msa_skinny_linear(const void* x, const void* w, const void* residual, const void* norm_w, float eps,
                                 int32_t epilogue, int32_t dtype, int32_t M, int32_t N, int32_t K, void* y,
                                 void* stream) {
  MSA_REQUIRE(x && w && y, "msa_skinny_linear: null pointer");
  MSA_REQUIRE(dtype == MSA_BF16, "msa_skinny_linear: bf16 only");
  MSA_REQUIRE(M > 0 && M <= 16, "msa_skinny_linear: M=%d (1..16 rows)", M);
  MSA_REQUIRE(N > 0 && K > 0 && K % kUnit == 0, "msa_skinny_linear: N=%d K=%d (K must be a multiple of %d)", N, K, kUnit);
  MSA_REQUIRE((int64_t)32 * K * 2 < ((int64_t)1 << 31) && (int64_t)M * K * 2 < ((int64_t)1 << 31),
              "msa_skinny_linear: K=%d too large", K);
  MSA_REQUIRE(epilogue >= kEpiPlain && epilogue <= kEpiSiluMul, "msa_skinny_linear: epilogue %d", epilogue);
  MSA_REQUIRE((epilogue == kEpiResidual) == (residual != nullptr), "msa_skinny_linear: residual pointer and epilogue disagree");
  MSA_REQUIRE(epilogue != kEpiSiluMul || N % 32 == 0, "msa_skinny_linear: silu-mul needs N %% 32 == 0");
  MSA_REQUIRE((((uintptr_t)x | (uintptr_t)w | (uintptr_t)norm_w) & 15) == 0, "msa_skinny_linear: x / w / norm_w must be 16-byte aligned");
  const int units = K / kUnit;
  MSA_REQUIRE(norm_w == nullptr || eps > 0.f, "msa_skinny_linear: folded RMSNorm needs eps > 0");
  hipStream_t st = as_stream(stream);

  // Wavefronts per workgroup: split K far enough that the launch has a few thousand wavefronts, and
  // prefer a count that divides the K units so every wavefront streams the same number of bytes.
  static const int env_waves = [] { const char* e = getenv("MSA_LINEAR_WAVES"); return e ? atoi(e) : 0; }();
  static const int env_r = [] { const char* e = getenv("MSA_LINEAR_R"); return e ? atoi(e) : 0; }();
  // Row groups per wavefront: two share one load of x (every workgroup re-reads x from L2) when N is large
  // enough to still fill the chip with workgroups.
  int R = ((int64_t)N / 32 * kMaxWaves >= 3072 || epilogue == kEpiSiluMul) ? 2 : 1;
  if (env_r == 1 && epilogue != kEpiSiluMul) R = 1;
  if (env_r == 2) R = 2;
  const int groups = (N + 16 * R - 1) / (16 * R);
  int want = (int)std::min<int64_t>(kMaxWaves, std::max<int64_t>(1, (4096 + groups - 1) / groups));
  want = std::max(1, std::min(want, units));
  int waves = want;
  for (int cand = want; cand >= std::max(1, want / 2); --cand)
    if (units % cand == 0) { waves = cand; break; }
  if (env_waves > 0) waves = std::max(1, std::min(std::min(env_waves, kMaxWaves), units));

#define MSA_LIN(R_, E_)                                                                              \
  (norm_w ? launch<R_, E_, true>(x, w, residual, norm_w, eps, y, M, N, K, waves, st)                 \
          : launch<R_, E_, false>(x, w, residual, norm_w, eps, y, M, N, K, waves, st))
  switch (epilogue * 8 + R) {
    case kEpiPlain * 8 + 1: return MSA_LIN(1, kEpiPlain);
    case kEpiPlain * 8 + 2: return MSA_LIN(2, kEpiPlain);
    case kEpiResidual * 8 + 1: return MSA_LIN(1, kEpiResidual);
    case kEpiResidual * 8 + 2: return MSA_LIN(2, kEpiResidual);
    case kEpiSiluMul * 8 + 2: return MSA_LIN(2, kEpiSiluMul);
  }
#undef MSA_LIN
  msa_set_error("msa_skinny_linear: no kernel for epilogue %d with %d row groups", epilogue, R);
  return MSA_EINVAL;
}
