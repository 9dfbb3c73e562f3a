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
#include <type_traits>

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
    int64_t y_row_stride, int32_t rows_per_wg) {
  constexpr int kUnitBytes = 64 * J;   // one unit = J vectors of 16 bytes per lane = 32 J elements of a row
  const int units = K / (32 * J);
  extern __shared__ __align__(16) float part[];   // [waves][R][64][4], then [waves][16] row sums of squares
  const int tid = threadIdx.x, lane = tid & 63, waves = blockDim.x >> 6;
  // the wavefront index as a scalar: every K offset below derives from it and rides in the scalar offset of the
  // buffer loads, which must be provably uniform (a value the compiler takes for divergent costs a
  // read-first-lane loop around every load)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_l = lane & 15, g = lane >> 4;
  // a workgroup owns rows [n_base, n_base + rows_per_wg) of w, rows_per_wg <= 16 R (fewer than 16 R when the matrix
  // has too few rows to give every compute unit a full set: the rows past it read as zero and are not stored)
  const int n_base = blockIdx.x * rows_per_wg;
  const int64_t row_bytes = (int64_t)K * 2;

  // rows past N (weights) and past M (activations) read as zero through the buffer bounds
  const int rows_w = min(rows_per_wg, N - n_base);
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(reinterpret_cast<const char*>(w)) + (int64_t)n_base * row_bytes, 0, (int)(rows_w * row_bytes),
      0x00020000);
  const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(reinterpret_cast<const char*>(x)), 0, (int)(M * row_bytes), 0x00020000);
  const int voff = n_l * (int)row_bytes + g * 16;

  // this wavefront's share of the K units
  const int u0 = (int)((uint32_t)units * (uint32_t)wave / (uint32_t)waves);        // units * waves < 2^31: K is bounded by the host
  const int u1 = (int)((uint32_t)units * (uint32_t)(wave + 1) / (uint32_t)waves);

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
    // every 16-row group holds gate rows [8 i, 8 i + 8) in its first half and the same up rows in its second: a
    // lane with n_l < 8 has the gate sum and takes the up sum from the lane 8 further on
    for (int r = wave; r < R; r += waves) {
      floatx4_t sum = floatx4_t{0.f, 0.f, 0.f, 0.f};
      for (int wv = 0; wv < waves; ++wv) sum += *reinterpret_cast<const floatx4_t*>(&part[((wv * R + r) * 64 + lane) * 4]);
      floatx4_t up;
#pragma unroll
      for (int e = 0; e < 4; ++e) up[e] = __shfl_xor(sum[e], 8);
      const int n = ((n_base + 16 * r) >> 1) + n_l;    // output column: a group of 16 rows folds into 8 outputs
      if (n_l >= 8 || n_base + 16 * r + 8 + n_l >= N) continue;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int m = 4 * g + e;
        if (m >= M) continue;
        const float a = bf16_to_f32(f32_to_bf16(sum[e] * inv[e])), b = bf16_to_f32(f32_to_bf16(up[e] * inv[e]));
        y[(int64_t)m * y_row_stride + n] = f32_to_bf16(a / (1.f + __expf(-a)) * b);
      }
    }
    return;
  }
  for (int r = wave; r < R; r += waves) {
    floatx4_t sum = floatx4_t{0.f, 0.f, 0.f, 0.f};
    for (int wv = 0; wv < waves; ++wv) sum += *reinterpret_cast<const floatx4_t*>(&part[((wv * R + r) * 64 + lane) * 4]);
    const int n = n_base + 16 * r + n_l;
    if (n >= N || 16 * r + n_l >= rows_per_wg) continue;
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

// Streaming form for matrices with many row groups per compute unit (gate/up, LM head): a workgroup stays for the
// whole launch.  Wavefront w owns the K slice [32 F w, 32 F (w + 1)) for every row group the workgroup visits and
// keeps its x operands for that slice (with the RMSNorm weight folded in) in registers, so the activations are read
// once per workgroup instead of once per row group, and far fewer workgroups have to be dispatched.  Work items are
// pairs of row groups (32 weight rows), or single row groups for the silu epilogue (8 gate rows and the same 8 up
// rows: the finer grain matters because a launch lasts as long as its busiest compute unit), dealt round robin;
// a step is one row group: its F weight vectors per lane are prefetched one step ahead, the partial sums meet in
// a ring of four LDS buffers behind one barrier per step, and all threads share the work of adding them up (a fixed
// tree) and storing the row group.  Launched with 16 wavefronts.
template <int F, int kEpi, bool kNorm>
__global__ __launch_bounds__(kMaxWaves * 64) void skinny_stream_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, const bf16_t* __restrict__ residual,
    const bf16_t* __restrict__ norm_w, float eps, bf16_t* __restrict__ y, int32_t M, int32_t N, int32_t K,
    int64_t y_row_stride, int32_t n_items) {
  extern __shared__ __align__(16) float part[];   // [4][waves][64][4] partial sums, then [waves][16] sums of squares
  const int tid = threadIdx.x, lane = tid & 63, waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_l = lane & 15, g = lane >> 4;
  const int row_bytes = K * 2;
  const int slice_off = wave * (F * 64);           // byte offset of this wavefront's K slice inside a row
  const int voff = n_l * row_bytes + g * 16;
  float* row_ssq = part + 4 * waves * 256;

  // activations of the slice, once
  const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(reinterpret_cast<const char*>(x)), 0, M * row_bytes, 0x00020000);
  u32x4_t xf[F];
#pragma unroll
  for (int f = 0; f < F; ++f) xf[f] = __builtin_amdgcn_raw_buffer_load_b128(rs_x, voff, slice_off + f * 64, 0);

  // this workgroup's items: blockIdx.x, blockIdx.x + gridDim.x, ...; an item is a pair of row groups (two steps), or
  // a single row group for the silu epilogue, whose groups are complete in themselves (8 gate rows + 8 up rows)
  constexpr int kPer = kEpi == kEpiSiluMul ? 1 : 2;
  const int my_items = n_items > (int)blockIdx.x ? (n_items - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x : 0;
  const int n_steps = kPer * my_items;
  auto group_of = [&](int s) {
    return kPer == 1 ? (int)blockIdx.x + s * (int)gridDim.x : 2 * ((int)blockIdx.x + (s >> 1) * (int)gridDim.x) + (s & 1);
  };
  // Three register stages of weight operands, always indexed by compile-time constants: a step's loads are issued
  // two steps ahead.  Every step issues its prefetch (an empty one past the end) and the step count is padded to a
  // multiple of three, so the loop body is straight-line as far as memory instructions go and the wait counts the
  // compiler derives are exact; with one stage less, the wait for a step's operands also covered the output store
  // of the step before, i.e. a store round trip per step.
  constexpr int kStages = 3;
  u32x4_t fw[kStages][F];
  auto load_w = [&](auto slot_tag, int s) {
    constexpr int slot = decltype(slot_tag)::value;
    const int gid = group_of(s);
    // rows <= 0 for the missing second group of an odd tail and for the step past the last one (the prefetch is
    // issued unconditionally so that the wait counts in the loop stay exact): an empty extent reads zeros and
    // touches no memory.  The clamp compiles to a vector instruction; read-first-lane brings the extent back into a
    // scalar register so that the descriptor stays scalar and the loads need no per-lane descriptor loop.
    const int rows = s < n_steps ? min(16, N - gid * 16) : 0;
    const int extent = __builtin_amdgcn_readfirstlane(max(0, rows) * row_bytes);
    const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(reinterpret_cast<const char*>(w)) + (int64_t)gid * 16 * row_bytes, 0, extent, 0x00020000);
#pragma unroll
    for (int f = 0; f < F; ++f) fw[slot][f] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, voff, slice_off + f * 64, 0);
  };
  load_w(std::integral_constant<int, 0>{}, 0);
  load_w(std::integral_constant<int, 1>{}, 1);

  if constexpr (kNorm) {
    // RMSNorm folded in: the operand is bf16(x * norm_w); the row scale rsqrt(mean(x^2) + eps) commutes with the
    // product and is applied to the fp32 sums when a row group is stored
    const __amdgpu_buffer_rsrc_t rs_g = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(reinterpret_cast<const char*>(norm_w)), 0, row_bytes, 0x00020000);
    float ssq = 0.f;
#pragma unroll
    for (int f = 0; f < F; ++f) {
      const u32x4_t gf = __builtin_amdgcn_raw_buffer_load_b128(rs_g, g * 16, slice_off + f * 64, 0);
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const float lo = bf16lo(xf[f][c]), hi = bf16hi(xf[f][c]);
        ssq += lo * lo + hi * hi;
        xf[f][c] = pack_rne(lo * bf16lo(gf[c]), hi * bf16hi(gf[c]));
      }
    }
    ssq += __shfl_xor(ssq, 16);
    ssq += __shfl_xor(ssq, 32);
    if (g == 0) row_ssq[wave * 16 + n_l] = ssq;       // visible to everyone behind the first step's barrier
  }

  // Adding up a step's partial sums is shared by all 1024 threads, so that no wavefront falls behind the others at
  // the next barrier: eight threads own a pair of neighbouring outputs (row o_m of x, columns o_n, o_n + 1 of the
  // row group); each adds the partials of two wavefronts and the eight meet by three DPP exchanges (a fixed tree:
  // results are reproducible).  A wavefront thus holds one output row of the group, and its store covers the row's
  // 32 contiguous bytes in one instruction (a full memory sector; narrower pieces cost a read-modify-write).
  const int pair = tid >> 3, sub = tid & 7;
  const int o_m = pair >> 3, o_n = (pair & 7) * 2;
  const int o_idx = ((o_m >> 2) * 16 + o_n) * 4 + (o_m & 3);          // float index of (o_m, o_n) in a partial row
  float inv = 1.f;                                                  // RMSNorm scale of row o_m
  bool have_inv = !kNorm;
  auto sum_parts = [&](int s, float& v0, float& v1) {
    const float* base = part + ((s & 3) * waves + 2 * sub) * 256 + o_idx;
    v0 = base[0] + base[256];
    v1 = base[4] + base[256 + 4];
#pragma unroll
    for (int x = 1; x < 8; x <<= 1) {
      v0 += __shfl_xor(v0, x);
      v1 += __shfl_xor(v1, x);
    }
  };
  const bool pair_store = ((y_row_stride & 1) == 0) && ((reinterpret_cast<uintptr_t>(y) & 3) == 0);
  auto store_pair = [&](int n, float a, float b) {          // columns n, n + 1 of row o_m
    bf16_t* at = y + (int64_t)o_m * y_row_stride + n;
    const int n_end = kEpi == kEpiSiluMul ? N / 2 : N;
    if (pair_store && n + 1 < n_end) {
      *reinterpret_cast<uint32_t*>(at) = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
    } else {
      if (n < n_end) at[0] = f32_to_bf16(a);
      if (n + 1 < n_end) at[1] = f32_to_bf16(b);
    }
  };

  auto step = [&](int s, auto slot_tag) {
    constexpr int slot = decltype(slot_tag)::value;
    load_w(std::integral_constant<int, (slot + 2) % kStages>{}, s + 2);
    floatx4_t acc = floatx4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int f = 0; f < F; ++f)
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(xf[f]), as_frag(fw[slot][f]), acc, 0, 0, 0);
    // acc[e] is y[m = 4 g + e][16 gid + n_l] over this wavefront's K slice
    *reinterpret_cast<floatx4_t*>(part + ((s & 3) * waves + wave) * 256 + lane * 4) = acc;
    __syncthreads();
    if (s >= n_steps) return;                        // padding step
    if (!have_inv) {
      float tot = 0.f;
      for (int wv = 0; wv < waves; ++wv) tot += row_ssq[wv * 16 + o_m];
      inv = rsqrtf(tot / (float)K + eps);
      have_inv = true;
    }
    const int gid = group_of(s);
    if constexpr (kEpi == kEpiSiluMul) {
      // columns 0..7 of the group are gate rows, 8..15 the same up rows: the lanes 32 further on hold the up pair
      float g0, g1;
      sum_parts(s, g0, g1);
      const float u0 = __shfl_xor(g0, 32), u1 = __shfl_xor(g1, 32);
      if (sub != 0 || o_m >= M || o_n >= 8) return;
      const float a0 = bf16_to_f32(f32_to_bf16(g0 * inv)), b0 = bf16_to_f32(f32_to_bf16(u0 * inv));
      const float a1 = bf16_to_f32(f32_to_bf16(g1 * inv)), b1 = bf16_to_f32(f32_to_bf16(u1 * inv));
      store_pair(gid * 8 + o_n, a0 / (1.f + __expf(-a0)) * b0, a1 / (1.f + __expf(-a1)) * b1);
    } else {
      float v0, v1;
      sum_parts(s, v0, v1);
      const int n = gid * 16 + o_n;
      if (sub != 0 || o_m >= M) return;
      v0 *= inv;
      v1 *= inv;
      if (kEpi == kEpiResidual) {
        const bf16_t* r = residual + (int64_t)o_m * y_row_stride + n;
        if (n < N) v0 = bf16_to_f32(f32_to_bf16(v0)) + bf16_to_f32(r[0]);
        if (n + 1 < N) v1 = bf16_to_f32(f32_to_bf16(v1)) + bf16_to_f32(r[1]);
      }
      store_pair(n, v0, v1);
    }
  };
  for (int s = 0; s < n_steps; s += kStages) {
    step(s, std::integral_constant<int, 0>{});
    step(s + 1, std::integral_constant<int, 1>{});
    step(s + 2, std::integral_constant<int, 2>{});
  }
}

template <int F, int kEpi, bool kNorm>
int launch_stream(const void* x, const void* w, const void* residual, const void* norm_w, float eps, void* y, int32_t M,
                  int32_t N, int32_t K, int waves, int grid, int n_items, hipStream_t st) {
  const size_t lds = (size_t)waves * (4 * 256 + 16) * sizeof(float);
  const int64_t y_stride = kEpi == kEpiSiluMul ? N / 2 : N;
  static std::atomic<int> lds_limit_raised{0};   // 16 wavefronts need 65 KB, just past the default dynamic LDS limit
  MSA_HIP(raise_dynamic_lds_limit(lds_limit_raised, reinterpret_cast<const void*>(skinny_stream_kernel<F, kEpi, kNorm>),
                                  kMaxWaves * (4 * 256 + 16) * (int)sizeof(float)));
  skinny_stream_kernel<F, kEpi, kNorm><<<grid, waves * 64, lds, st>>>(
      static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<const bf16_t*>(residual),
      static_cast<const bf16_t*>(norm_w), eps, static_cast<bf16_t*>(y), M, N, K, y_stride, n_items);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

// ------------------------------------------------------------------------------------------------
// Tiled form for matrices with few rows and a long K (down_proj: 2560 x 9728): the matrix is cut both ways,
// workgroup (row block, K slice) owns `gpw` row groups (one per wavefront) over a slice of K.  A compute unit moves
// only about 34 GB/s whatever the source, so what counts is the weight plus activation bytes per compute unit and
// that all compute units take part: with one 16-row group per workgroup every workgroup re-reads all of x, as many
// bytes as its weights, and 160 row groups leave 96 compute units idle; a tile of ten row groups over a sixteenth of
// K reads a tenth of its weight bytes in activations and there are 256 of them.  The x slice is staged once in LDS
// in operand order; a wavefront streams its 16 weight rows of the slice (up to twenty loads in flight per lane) and
// stores its fp32 partial block; `skinny_tile_reduce_kernel` adds the K slices in order and applies the epilogue.
// K slices are runs of 32-element MFMA steps, as even as the step count allows.  (The same cut measured slower than
// the other forms for the gate/up and q/k/v matrices, which have rows enough: 29.7 vs 28.0 and 15.7 vs 12.8 us.)
// ------------------------------------------------------------------------------------------------
constexpr int kTileDepth = 20;      // weight vectors in flight per lane
constexpr int kTileMaxSlices = 16;

__global__ __launch_bounds__(kMaxWaves * 64) void skinny_tile_partial_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ w, float* __restrict__ part, int32_t M, int32_t N, int32_t K,
    int32_t gpw) {
  extern __shared__ __align__(16) u32x4_t xs[];     // [steps padded to kTileDepth][64] x operands of the K slice
  const int tid = threadIdx.x, lane = tid & 63, waves = blockDim.x >> 6;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int n_l = lane & 15, g = lane >> 4;
  const int row_bytes = K * 2;
  const int rb = blockIdx.x, ks = blockIdx.y, n_slices = gridDim.y;
  const int steps_total = K / 32;
  const int s0 = (int)((int64_t)steps_total * ks / n_slices), s1 = (int)((int64_t)steps_total * (ks + 1) / n_slices);
  const int steps = s1 - s0;
  const int steps_max = (steps_total + n_slices - 1) / n_slices;
  const int steps_pad = (steps_max + kTileDepth - 1) / kTileDepth * kTileDepth;    // the host sizes LDS with this
  const int slice_off = s0 * 64;
  const int voff = n_l * row_bytes + g * 16;
  const int groups = (N + 15) >> 4;

  const __amdgpu_buffer_rsrc_t rs_x = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(reinterpret_cast<const char*>(x)), 0, M * row_bytes, 0x00020000);
  for (int f = wave; f < steps_pad; f += waves)      // padding steps hold zeros: their products must not be NaN
    xs[f * 64 + lane] = f < steps ? __builtin_amdgcn_raw_buffer_load_b128(rs_x, voff, slice_off + f * 64, 0)
                                  : u32x4_t{0u, 0u, 0u, 0u};
  __syncthreads();

  const int gid = rb * gpw + wave;                   // this wavefront's row group
  if (wave >= gpw || gid >= groups) return;
  const int extent = __builtin_amdgcn_readfirstlane(min(16, N - gid * 16) * row_bytes);
  const __amdgpu_buffer_rsrc_t rs_w = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(reinterpret_cast<const char*>(w)) + (int64_t)gid * 16 * row_bytes, 0, extent, 0x00020000);
  floatx4_t acc = floatx4_t{0.f, 0.f, 0.f, 0.f};
  for (int f0 = 0; f0 < steps; f0 += kTileDepth) {
    u32x4_t fw[kTileDepth];
#pragma unroll
    for (int i = 0; i < kTileDepth; ++i) {
      // steps past the slice read through an offset beyond the extent: zeros, no memory access, no branch
      const int vo = f0 + i < steps ? voff : 0x7fffffff - 4096;
      fw[i] = __builtin_amdgcn_raw_buffer_load_b128(rs_w, vo, slice_off + (f0 + i) * 64, 0);
    }
#pragma unroll
    for (int i = 0; i < kTileDepth; ++i)
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_frag(xs[(f0 + i) * 64 + lane]), as_frag(fw[i]), acc, 0, 0, 0);
  }
  // acc[e] is the partial of y[m = 4 g + e][16 gid + n_l] over this K slice
  *reinterpret_cast<floatx4_t*>(part + (((int64_t)ks * groups + gid) * 64 + lane) * 4) = acc;
}

// One thread per output element in the order the partial blocks are stored (row group, lane, accumulator element),
// so the reads of every K slice are contiguous; all slices are loaded first and added in K order.
template <int kEpi>
__global__ __launch_bounds__(256) void skinny_tile_reduce_kernel(const float* __restrict__ part,
                                                                 const bf16_t* __restrict__ residual,
                                                                 bf16_t* __restrict__ y, int32_t M, int32_t N,
                                                                 int32_t n_slices) {
  const int groups = (N + 15) >> 4;
  const int t = blockIdx.x * blockDim.x + threadIdx.x;       // (row group, lane, element)
  if (t >= groups * 256) return;
  float v[kTileMaxSlices];
#pragma unroll
  for (int s = 0; s < kTileMaxSlices; ++s) v[s] = s < n_slices ? part[(int64_t)s * groups * 256 + t] : 0.f;
  float sum = 0.f;
#pragma unroll
  for (int s = 0; s < kTileMaxSlices; ++s) sum += v[s];
  const int lane = (t >> 2) & 63;
  const int m = 4 * (lane >> 4) + (t & 3), n = 16 * (t >> 8) + (lane & 15);
  if (m >= M || n >= N) return;
  if (kEpi == kEpiResidual) sum = bf16_to_f32(f32_to_bf16(sum)) + bf16_to_f32(residual[(int64_t)m * N + n]);
  y[(int64_t)m * N + n] = f32_to_bf16(sum);
}

// The cut of the tiled form: up to 16 row groups per row block (fewer when the matrix has fewer than 256 groups), as
// many K slices as keep the launch within one workgroup per compute unit (at most 16); used when it takes at least
// 8 us less per compute unit than the plain form at ~34 GB/s (the second launch costs ~4 us).
struct TilePlan {
  int n_slices, gpw, row_blocks;
  bool use;
};
TilePlan plan_tile(int32_t N, int32_t K) {
  TilePlan t{0, 0, 0, false};
  const int groups = (N + 15) / 16;
  const int steps = K / 32;
  if (K % 32 != 0 || groups > 256) return t;
  t.gpw = std::min(kMaxWaves, (groups + 15) / 16);
  t.row_blocks = (groups + t.gpw - 1) / t.gpw;
  t.n_slices = std::min(std::min(kTileMaxSlices, steps), 256 / std::max(1, t.row_blocks));
  if (t.n_slices < 2) return t;
  const double plain_bytes = (16.0 + 16.0) * K * 2;                             // one row group + all of x
  const double tiled_bytes = (16.0 * t.gpw + 16.0) * ((double)K / t.n_slices) * 2;
  t.use = (plain_bytes - tiled_bytes) / 34e3 > 8.0;                             // bytes / (34 GB/s) in us
  return t;
}

size_t tile_workspace_bytes(const TilePlan& t, int32_t N) {
  return (size_t)t.n_slices * ((N + 15) / 16) * 256 * sizeof(float);
}

template <int R, int kEpi, bool kNorm>
int launch(const void* x, const void* w, const void* residual, const void* norm_w, float eps, void* y, int32_t M,
           int32_t N, int32_t K, int waves, int rows_per_wg, hipStream_t st) {
  const int groups = (N + rows_per_wg - 1) / rows_per_wg;
  const size_t lds = (size_t)waves * (R * 256 + 16) * sizeof(float);
  const int64_t y_stride = kEpi == kEpiSiluMul ? N / 2 : N;
  // with the norm folded in a unit is 64 elements instead of 128: the extra fragments then fit 128 VGPRs
  skinny_linear_kernel<R, kEpi, kNorm, kNorm ? 2 : 4><<<groups, waves * 64, lds, st>>>(
      static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), static_cast<const bf16_t*>(residual),
      static_cast<const bf16_t*>(norm_w), eps, static_cast<bf16_t*>(y), M, N, K, y_stride, rows_per_wg);
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
  MSA_REQUIRE(epilogue != kEpiSiluMul || N % 16 == 0, "msa_skinny_linear: silu-mul needs N %% 16 == 0");
  MSA_REQUIRE((((uintptr_t)x | (uintptr_t)w | (uintptr_t)norm_w) & 15) == 0, "msa_skinny_linear: x / w / norm_w must be 16-byte aligned");
  const int units = K / kUnit;
  MSA_REQUIRE(norm_w == nullptr || eps > 0.f, "msa_skinny_linear: folded RMSNorm needs eps > 0");
  hipStream_t st = as_stream(stream);

  // Many row groups per compute unit and a K that 16 wavefronts split into 5 MFMA steps each (K = 2560): the
  // streaming kernel, one workgroup per compute unit at most, an equal number of items (32 rows) each.
  if (K == 16 * 5 * 32) {
    const int n_items = epilogue == kEpiSiluMul ? N / 16 : (N + 31) / 32;
    const int iters = (n_items + 255) / 256;
    const int grid = (n_items + iters - 1) / iters;
    if (iters >= 2) {                                // with one item per workgroup the plain kernel does the same work
#define MSA_STREAM(E_)                                                                                              \
  (norm_w ? launch_stream<5, E_, true>(x, w, residual, norm_w, eps, y, M, N, K, kMaxWaves, grid, n_items, st)       \
          : launch_stream<5, E_, false>(x, w, residual, norm_w, eps, y, M, N, K, kMaxWaves, grid, n_items, st))
      switch (epilogue) {
        case kEpiPlain: return MSA_STREAM(kEpiPlain);
        case kEpiResidual: return MSA_STREAM(kEpiResidual);
        case kEpiSiluMul: return MSA_STREAM(kEpiSiluMul);
      }
#undef MSA_STREAM
    }
  }

  // Wavefronts per workgroup: split K far enough that the launch has a few thousand wavefronts, and
  // prefer a count that divides the K units so every wavefront streams the same number of bytes.
  // Row groups per wavefront: two share one load of x (every workgroup re-reads x from L2) when N is large
  // enough to still fill the chip with workgroups.
  int R = ((int64_t)N / 32 * kMaxWaves >= 3072 || epilogue == kEpiSiluMul) ? 2 : 1;
  // Rows per workgroup: 16 R, or fewer when that leaves compute units without a workgroup (a compute unit moves
  // only ~34 GB/s, so 256 workgroups of 10 rows beat 160 of 16 on a 2560-row matrix); the silu epilogue needs whole
  // gate / up groups.
  int rows_per_wg = 16 * R;
  if (epilogue != kEpiSiluMul && (N + 16 * R - 1) / (16 * R) < 256) {
    const int spread = std::max(8, (N + 255) / 256);
    if (spread > 16 * (R - 1) && spread < 16 * R) rows_per_wg = spread;
  }
  const int groups = (N + rows_per_wg - 1) / rows_per_wg;
  int want = (int)std::min<int64_t>(kMaxWaves, std::max<int64_t>(1, (4096 + groups - 1) / groups));
  want = std::max(1, std::min(want, units));
  int waves = want;
  for (int cand = want; cand >= std::max(1, want / 2); --cand)
    if (units % cand == 0) { waves = cand; break; }

#define MSA_LIN(R_, E_)                                                                              \
  (norm_w ? launch<R_, E_, true>(x, w, residual, norm_w, eps, y, M, N, K, waves, rows_per_wg, st)    \
          : launch<R_, E_, false>(x, w, residual, norm_w, eps, y, M, N, K, waves, rows_per_wg, st))
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

extern "C" size_t msa_skinny_linear_workspace_bytes(int32_t M, int32_t N, int32_t K) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const TilePlan t = plan_tile(N, K);
  return t.use ? tile_workspace_bytes(t, N) : 0;
}

extern "C" int msa_skinny_linear_ws(const void* x, const void* w, const void* residual, const void* norm_w, float eps,
                                    int32_t epilogue, int32_t dtype, int32_t M, int32_t N, int32_t K, void* y,
                                    void* workspace, size_t workspace_bytes, void* stream) {
  const bool fits = x && w && y && dtype == MSA_BF16 && M > 0 && M <= 16 && N > 0 && K > 0 && K % kUnit == 0 &&
                    norm_w == nullptr && (epilogue == kEpiPlain || epilogue == kEpiResidual) &&
                    (epilogue == kEpiResidual) == (residual != nullptr) && (int64_t)M * K * 2 < ((int64_t)1 << 31) &&
                    (int64_t)32 * K * 2 < ((int64_t)1 << 31) &&
                    (((uintptr_t)x | (uintptr_t)w | (uintptr_t)workspace) & 15) == 0;
  const TilePlan t = fits ? plan_tile(N, K) : TilePlan{0, 0, 0, false};
  if (!fits || !t.use || workspace == nullptr || workspace_bytes < tile_workspace_bytes(t, N))
    return msa_skinny_linear(x, w, residual, norm_w, eps, epilogue, dtype, M, N, K, y, stream);   // it reports bad arguments
  hipStream_t st = as_stream(stream);
  const int groups = (N + 15) / 16;
  const int steps_max = (K / 32 + t.n_slices - 1) / t.n_slices;
  const int steps_pad = (steps_max + kTileDepth - 1) / kTileDepth * kTileDepth;
  const size_t lds = (size_t)steps_pad * 64 * 16;
  MSA_REQUIRE(lds <= 64 * 1024, "msa_skinny_linear_ws: a K slice of %d steps does not fit LDS", steps_max);
  float* part = static_cast<float*>(workspace);
  skinny_tile_partial_kernel<<<dim3(t.row_blocks, t.n_slices), t.gpw * 64, lds, st>>>(
      static_cast<const bf16_t*>(x), static_cast<const bf16_t*>(w), part, M, N, K, t.gpw);
  MSA_LAUNCH_CHECK();
  if (epilogue == kEpiResidual)
    skinny_tile_reduce_kernel<kEpiResidual><<<groups, 256, 0, st>>>(part, static_cast<const bf16_t*>(residual),
                                                                   static_cast<bf16_t*>(y), M, N, t.n_slices);
  else
    skinny_tile_reduce_kernel<kEpiPlain><<<groups, 256, 0, st>>>(part, nullptr, static_cast<bf16_t*>(y), M, N, t.n_slices);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}
