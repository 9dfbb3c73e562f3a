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
// change from one iteration to the next (what a GEMM on real data presents to the multipliers).
// kExtra: other VALU work per iteration of 8 MFMAs, on registers of its own (what a kernel that does arithmetic on its
// accumulators between the products, such as the softmax of an attention kernel, asks of the SIMD's issue port):
// 0 none; 1 / 2: 24 / 48 v_fma_f32; 3 / 4: 24 / 48 v_exp_f32; 5: 24 v_cvt_pk_bf16_f32; 6: 24 v_dot2c_f32_bf16; 7: 24 v_max3_f32.
template <int kExtra>
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
  typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
  typedef float floatx2_t __attribute__((ext_vector_type(2)));
  float x[24];
#pragma unroll
  for (int i = 0; i < 24; ++i) x[i] = (float)(tid & 7) * 0.125f - (float)i;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[i]),
                                                            __builtin_bit_cast(bf16x8_t, b[j]), acc[i][j], 0, 0, 0);
    if constexpr (kExtra != 0) {
#pragma unroll
      for (int rep = 0; rep < ((kExtra == 2 || kExtra == 4) ? 2 : 1); ++rep)
#pragma unroll
        for (int i = 0; i < 24; ++i) {
          if constexpr (kExtra == 1 || kExtra == 2) x[i] = fmaf(x[i], 1.0001f, 0.5f);
          if constexpr (kExtra == 3 || kExtra == 4) x[i] = __builtin_amdgcn_exp2f(x[i]);
          if constexpr (kExtra == 5) {
            const floatx2_t f = {x[i], x[i]};
            x[i] = __builtin_bit_cast(float, __builtin_convertvector(f, bf16x2_t));
          }
          if constexpr (kExtra == 6)
            x[i] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, 0x3f803f80u),
                                                   __builtin_bit_cast(bf16x2_t, __float_as_uint(x[(i + 1) % 24])), x[i], false);
          if constexpr (kExtra == 7) x[i] = fmaxf(fmaxf(x[i], x[(i + 1) % 24]), x[(i + 2) % 24]);
        }
    }
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
  if constexpr (kExtra != 0) {          // keeps the extra work alive; sink values are only defined for kExtra == 0
#pragma unroll
    for (int i = 0; i < 24; ++i) s += x[i] * 1e-30f;
  }
  sink[tid] = s;
}

// What the memory system delivers to loops that only read, in the access patterns of the library's HBM-bound kernels.
// `src` is taken as rows of 2 KB (a token's or a cache row's 8 heads x 128 bf16).  The loaded words are folded with
// xor so that the loads cannot be dropped.
// kMode 0: 64 consecutive rows (128 KB) per workgroup of 256 threads, non-temporal 16-byte buffer loads, four per
//          lane in flight - the pooling kernel's reads.  The fold is stored only if it equals a value it cannot take.
// kMode 1: the same, and lanes 0 - 127 store their fold: one non-temporal 2 KB row per 128 KB read - pooling's writes.
template <int kMode>
__global__ __launch_bounds__(256) void read_rows_kernel(const char* __restrict__ src, char* __restrict__ dst) {
  const int64_t wg = blockIdx.x;
  const __amdgpu_buffer_rsrc_t rs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(src) + wg * (64 * 2048), 0, 64 * 2048, 0x00020000);
  u32x4_t acc = {0u, 0u, 0u, 0u};
  for (int i = threadIdx.x * 16; i < 64 * 2048; i += 256 * 16 * 4) {
    u32x4_t v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = __builtin_amdgcn_raw_buffer_load_b128(rs, i + u * 4096, 0, 2);
#pragma unroll
    for (int u = 0; u < 4; ++u) acc ^= v[u];
  }
  if constexpr (kMode == 1) {
    if (threadIdx.x < 128) __builtin_nontemporal_store(acc, reinterpret_cast<u32x4_t*>(dst + wg * 2048) + threadIdx.x);
  } else {
    if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u && (acc.x | acc.y) == 0u) *reinterpret_cast<u32x4_t*>(dst) = acc;
  }
}

// One KV head's 256-byte piece of every row, 2 KB apart: the decode attention's reads.  Workgroup (head, range) of 512
// threads, 16 lanes per piece, 32 rows per step and four steps in flight, as in that kernel.
__global__ __launch_bounds__(512) void read_head_pieces_kernel(const char* __restrict__ src, int64_t rows, int32_t ranges,
                                                               char* __restrict__ dst) {
  const int head = blockIdx.x & 7, range = blockIdx.x >> 3;
  const int64_t per = (rows + ranges - 1) / ranges;
  const int64_t row0 = range * per, row1 = min(rows, row0 + per);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const char* base = src + head * 256 + (lane & 15) * 16;
  u32x4_t acc = {0u, 0u, 0u, 0u};
  for (int64_t r = row0 + wave * 4 + (lane >> 4); r < row1; r += 32 * 4) {
    u32x4_t v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int64_t rr = r + 32 * u;
      v[u] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(base + (rr < row1 ? rr : r) * 2048));
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) acc ^= v[u];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x9e3779b9u && (acc.x | acc.y) == 0u) *reinterpret_cast<u32x4_t*>(dst) = acc;
}

// fills the workgroup's dynamic LDS with `word`
__global__ __launch_bounds__(256) void fill_lds_kernel(uint32_t word, int32_t words, uint32_t* __restrict__ check) {
  extern __shared__ uint32_t lds_words[];
  for (int i = threadIdx.x; i < words; i += 256) lds_words[i] = word;
  __syncthreads();
  // read one word back so that the stores cannot be dropped
  if (threadIdx.x == 0 && check != nullptr) check[blockIdx.x] = lds_words[(blockIdx.x * 61) % words];
}

}  // namespace

extern "C" int msa_diag_fill_lds(uint32_t word, uint32_t* check, int32_t workgroups, void* stream) {
  MSA_REQUIRE(workgroups > 0 && workgroups <= 65536, "msa_diag_fill_lds: bad workgroup count %d", workgroups);
  constexpr int kBytes = 160 * 1024;                       // a compute unit's whole LDS: one workgroup per unit at a time
  static std::atomic<int> lds_limit_raised{0};
  MSA_HIP(raise_dynamic_lds_limit(lds_limit_raised, reinterpret_cast<const void*>(fill_lds_kernel), kBytes));
  fill_lds_kernel<<<workgroups, 256, kBytes, as_stream(stream)>>>(word, kBytes / 4, check);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

extern "C" int msa_diag_read_stream(const void* src, int64_t bytes, void* dst, int32_t mode, void* stream) {
  MSA_REQUIRE(src != nullptr && dst != nullptr, "msa_diag_read_stream: null pointer");
  MSA_REQUIRE(mode >= 0 && mode <= 2, "msa_diag_read_stream: mode %d (0 rows, 1 rows + stores, 2 head pieces)", mode);
  MSA_REQUIRE(bytes > 0 && bytes % (64 * 2048) == 0 && bytes / (64 * 2048) <= 0x7fffffff,
              "msa_diag_read_stream: bytes must be a positive multiple of 128 KB");
  MSA_REQUIRE((((uintptr_t)src | (uintptr_t)dst) & 15) == 0, "msa_diag_read_stream: pointers must be 16-byte aligned");
  hipStream_t st = as_stream(stream);
  const unsigned groups = (unsigned)(bytes / (64 * 2048));
  if (mode == 0) {
    read_rows_kernel<0><<<groups, 256, 0, st>>>(static_cast<const char*>(src), static_cast<char*>(dst));
  } else if (mode == 1) {
    read_rows_kernel<1><<<groups, 256, 0, st>>>(static_cast<const char*>(src), static_cast<char*>(dst));
  } else {
    const int ranges = std::max(1, device_compute_units() / 8);       // one workgroup per compute unit
    read_head_pieces_kernel<<<8 * ranges, 512, 0, st>>>(static_cast<const char*>(src), bytes / 2048, ranges,
                                                        static_cast<char*>(dst));
  }
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

extern "C" int msa_diag_mfma_loop(int32_t workgroups, int32_t iters, int32_t mode, float* sink, double* flops_out,
                                  void* stream) {
  MSA_REQUIRE(workgroups > 0 && workgroups <= 65536 && iters > 0 && iters <= (1 << 24), "msa_diag_mfma_loop: bad sizes");
  const int operands = mode & 15, extra = mode >> 4;          // mode = operands + 16 * extra VALU work
  MSA_REQUIRE(mode >= 0 && operands <= 2 && extra <= 7 && sink != nullptr, "msa_diag_mfma_loop: bad mode / null sink");
  hipStream_t st = as_stream(stream);
  switch (extra) {
    case 0: mfma_loop_kernel<0><<<workgroups, kThreads, 0, st>>>(iters, operands, sink); break;
    case 1: mfma_loop_kernel<1><<<workgroups, kThreads, 0, st>>>(iters, operands, sink); break;
    case 2: mfma_loop_kernel<2><<<workgroups, kThreads, 0, st>>>(iters, operands, sink); break;
    case 3: mfma_loop_kernel<3><<<workgroups, kThreads, 0, st>>>(iters, operands, sink); break;
    case 4: mfma_loop_kernel<4><<<workgroups, kThreads, 0, st>>>(iters, operands, sink); break;
    case 5: mfma_loop_kernel<5><<<workgroups, kThreads, 0, st>>>(iters, operands, sink); break;
    case 6: mfma_loop_kernel<6><<<workgroups, kThreads, 0, st>>>(iters, operands, sink); break;
    default: mfma_loop_kernel<7><<<workgroups, kThreads, 0, st>>>(iters, operands, sink); break;
  }
  MSA_LAUNCH_CHECK();
  if (flops_out)
    *flops_out = (double)workgroups * (kThreads / 64) * (double)iters * kMfmasPerIter * (2.0 * 32 * 32 * 16);
  return MSA_OK;
}
