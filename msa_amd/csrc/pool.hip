// Chunk-mean pooling of K / V / K_r over ragged documents (HBM-bound streaming kernel).
//
// One workgroup per (chunk, tensor).  A token row [H, 128] is covered by H*8 lanes; lane (h, j)
// owns d in [8j, 8j+8) and [64+8j, 64+8j+8) — the two halves the half-split rotary pairs — so the
// optional RoPE on K needs no cross-lane traffic.  256 threads cover R = 256 / (H*8) token rows
// per step, accumulate in fp32 registers, and fold the R partial rows through LDS at the end.
// Each lane keeps two groups of rows in flight as raw 16-byte loads (16 KB per wavefront in bf16):
// with one row per wait the kernel was bound by load latency at 0.65-0.68 of the HBM rate; the
// two-group pipeline reaches 0.76, and 0.79 with non-temporal stores of the pooled rows (see store8).
#include <type_traits>

#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kStreamHint = 2;   // non-temporal: every input row is read once

struct PoolArgs {
  const void* in[3];
  void* out[3];
  int rope[3];       // rotate this tensor while reading
  int normalize[3];  // L2-normalise this tensor's pooled rows
  int n_tensors;
  int64_t T;
  int32_t H;
  const int32_t* chunk_start;
  const int32_t* chunk_len;
  const int32_t* chunk_doc;
  const int32_t* doc_start;
  const float* rope_cos;
  const float* rope_sin;
  int32_t rope_rows;
};

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// Eight consecutive elements of a row as they come from memory; converted to fp32 only when consumed,
// so a wavefront can keep two groups of rows in flight without holding them as floats.
template <typename T>
struct Raw8;
template <>
struct Raw8<bf16_t> {
  u32x4_t w;
  __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t rs, int voff, int soff) {
    w = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, soff, kStreamHint);
  }
  __device__ __forceinline__ void unpack(float (&x)[8]) const {
    x[0] = bf16lo(w.x); x[1] = bf16hi(w.x); x[2] = bf16lo(w.y); x[3] = bf16hi(w.y);
    x[4] = bf16lo(w.z); x[5] = bf16hi(w.z); x[6] = bf16lo(w.w); x[7] = bf16hi(w.w);
  }
};
template <>
struct Raw8<float> {
  u32x4_t a, b;
  __device__ __forceinline__ void load(__amdgpu_buffer_rsrc_t rs, int voff, int soff) {
    a = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, soff, kStreamHint);
    b = __builtin_amdgcn_raw_buffer_load_b128(rs, voff + 16, soff, kStreamHint);
  }
  __device__ __forceinline__ void unpack(float (&x)[8]) const {
    x[0] = __uint_as_float(a.x); x[1] = __uint_as_float(a.y); x[2] = __uint_as_float(a.z); x[3] = __uint_as_float(a.w);
    x[4] = __uint_as_float(b.x); x[5] = __uint_as_float(b.y); x[6] = __uint_as_float(b.z); x[7] = __uint_as_float(b.w);
  }
};

template <typename T>
__device__ __forceinline__ void store8(T* p, const float (&x)[8]);
template <>
__device__ __forceinline__ void store8<bf16_t>(bf16_t* p, const float (&x)[8]) {
  uint4 w;
  w.x = pack_bf16x2(x[0], x[1]); w.y = pack_bf16x2(x[2], x[3]);
  w.z = pack_bf16x2(x[4], x[5]); w.w = pack_bf16x2(x[6], x[7]);
  // Non-temporal: a write among the saturated read stream is what holds this kernel below the rate of its loads (a
  // bare loop of the same loads streams at 0.90 of the HBM rate, at 0.75 once every workgroup ends with a plain 2 KB
  // store and at 0.79 with a non-temporal one; 512 bytes per workgroup already cost 0.10).  Writing the pooled rows
  // eight at a time from LDS, from threads that take no part in the loads, or from a persistent workgroup whose next
  // loads are in flight changed nothing: the cost is the memory system's, per write and per byte.
  const u32x4_t ww = {w.x, w.y, w.z, w.w};
  __builtin_nontemporal_store(ww, reinterpret_cast<u32x4_t*>(p));
}
template <>
__device__ __forceinline__ void store8<float>(float* p, const float (&x)[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(x[4], x[5], x[6], x[7]);
}

// kRope: the launch's tensors are rotated while read (a launch holds tensors of one kind, so the plain kind does not
// carry the rotary state's registers: 3 - 4 workgroups per compute unit instead of 2).
template <typename T, bool kRope>
__global__ __launch_bounds__(kThreads, 2) void pool_chunks_kernel(PoolArgs a) {
  __shared__ float fold[kThreads * 16];

  const int c = blockIdx.x;
  const int slot = blockIdx.y;
  const T* __restrict__ in = static_cast<const T*>(a.in[slot]);
  T* __restrict__ out = static_cast<T*>(a.out[slot]);
  constexpr bool rope = kRope;

  const int U = a.H * 8;          // lanes per token row
  const int R = kThreads / U;     // token rows per step (the host checks that U divides the workgroup)
  const int tid = threadIdx.x;
  const int r = tid / U, u = tid % U;
  const int h = u >> 3, j = u & 7;
  const int row_elems = a.H * kHeadDim;
  const int col_lo = h * kHeadDim + 8 * j, col_hi = col_lo + 64;

  const int32_t t0 = __builtin_amdgcn_readfirstlane(a.chunk_start[c]);
  const int32_t len = __builtin_amdgcn_readfirstlane(a.chunk_len[c]);

  // Rows are fetched in groups of R * kRows through a buffer resource that spans exactly the group's
  // valid rows: a row past the chunk's end (or past T) reads as zero without touching memory and adds
  // nothing to the sums, so the loop needs no per-row predicate.  Two groups (A, B) alternate; the
  // loads of one are in flight while the other is consumed.
  constexpr int kRows = sizeof(T) == 2 ? 4 : 2;
  const int row_bytes = row_elems * (int)sizeof(T);
  const int group_rows = R * kRows;
  const int voff = r * row_bytes + col_lo * (int)sizeof(T);
  const int q_stride = R * row_bytes;
  const int32_t rows_valid = (int32_t)min((int64_t)len, a.T - (int64_t)t0);
  const char* chunk_base = reinterpret_cast<const char*>(in) + (int64_t)t0 * row_bytes;
  Raw8<T> lo_a[kRows], hi_a[kRows], lo_b[kRows], hi_b[kRows];
  auto issue = [&](Raw8<T>(&lo)[kRows], Raw8<T>(&hi)[kRows], int base) {
    const int rows = max(0, min(rows_valid - base, group_rows));
    const __amdgpu_buffer_rsrc_t group = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(chunk_base) + (int64_t)base * row_bytes, 0, rows * row_bytes, 0x00020000);
#pragma unroll
    for (int q = 0; q < kRows; ++q) {
      // the row displacement rides in the vector offset, the operand the range check is defined on
      lo[q].load(group, voff + q * q_stride, 0);
      hi[q].load(group, voff + q * q_stride + 64 * (int)sizeof(T), 0);
    }
  };
  // (loads are issued at raised priority: a wavefront that has requests to make goes ahead of those that are summing,
  // which keeps more bytes in flight per compute unit: 0.9 %)
  __builtin_amdgcn_s_setprio(3);
  issue(lo_a, hi_a, 0);
  __builtin_amdgcn_s_setprio(0);

  float acc_lo[8], acc_hi[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc_lo[i] = acc_hi[i] = 0.f;

  // rotary state of this lane's 8 frequencies at its current token, advanced by R positions per step
  float rc[8], rs[8], sc[8], ss[8];
  if constexpr (rope) {
    const int32_t pos0 = t0 - a.doc_start[a.chunk_doc[c]] + r;
    const int32_t p = min(pos0, a.rope_rows - 1), st = min(R, a.rope_rows - 1);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      rc[i] = a.rope_cos[(int64_t)p * 64 + 8 * j + i];
      rs[i] = a.rope_sin[(int64_t)p * 64 + 8 * j + i];
      sc[i] = a.rope_cos[(int64_t)st * 64 + 8 * j + i];
      ss[i] = a.rope_sin[(int64_t)st * 64 + 8 * j + i];
    }
  }

  auto consume = [&](auto rope_tag, const Raw8<T>(&lo)[kRows], const Raw8<T>(&hi)[kRows]) {
    constexpr bool kRotate = decltype(rope_tag)::value;
#pragma unroll
    for (int q = 0; q < kRows; ++q) {
      float xl[8], xh[8];
      lo[q].unpack(xl);
      hi[q].unpack(xh);
      if constexpr (kRotate) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          acc_lo[i] += xl[i] * rc[i] - xh[i] * rs[i];
          acc_hi[i] += xh[i] * rc[i] + xl[i] * rs[i];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {   // advance the angle by R positions
          const float nc = rc[i] * sc[i] - rs[i] * ss[i];
          rs[i] = rs[i] * sc[i] + rc[i] * ss[i];
          rc[i] = nc;
        }
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          acc_lo[i] += xl[i];
          acc_hi[i] += xh[i];
        }
      }
    }
  };
  auto stream = [&](auto rope_tag) {
    for (int base = 0; base < rows_valid; base += 2 * group_rows) {
      __builtin_amdgcn_s_setprio(3);
      issue(lo_b, hi_b, base + group_rows);
      __builtin_amdgcn_s_setprio(0);
      consume(rope_tag, lo_a, hi_a);
      __builtin_amdgcn_s_setprio(3);
      issue(lo_a, hi_a, base + 2 * group_rows);   // empty once past the end
      __builtin_amdgcn_s_setprio(0);
      consume(rope_tag, lo_b, hi_b);
    }
  };
  stream(std::integral_constant<bool, kRope>{});

  // fold the R partial rows through LDS: value i of thread t at fold[i * kThreads + t] (consecutive lanes hit
  // consecutive banks on the way in and on the way out)
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    fold[i * kThreads + tid] = acc_lo[i];
    fold[(8 + i) * kThreads + tid] = acc_hi[i];
  }
  __syncthreads();
  if (tid < U) {
    const float inv = 1.0f / (float)len;
    float lo[8], hi[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) lo[i] = hi[i] = 0.f;
    for (int rr = 0; rr < R; ++rr) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        lo[i] += fold[i * kThreads + rr * U + tid];
        hi[i] += fold[(8 + i) * kThreads + rr * U + tid];
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) { lo[i] *= inv; hi[i] *= inv; }
    if (a.normalize[slot]) {
      float ssq = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) ssq += lo[i] * lo[i] + hi[i] * hi[i];
      // the 8 lanes of one head are consecutive: butterfly over the low 3 lane bits
      ssq += __shfl_xor(ssq, 1);
      ssq += __shfl_xor(ssq, 2);
      ssq += __shfl_xor(ssq, 4);
      const float sc2 = 1.0f / fmaxf(sqrtf(ssq), 1e-12f);
#pragma unroll
      for (int i = 0; i < 8; ++i) { lo[i] *= sc2; hi[i] *= sc2; }
    }
    T* o = out + (int64_t)c * row_elems;
    store8<T>(o + col_lo, lo);
    store8<T>(o + col_hi, hi);
  }
}

}  // namespace

extern "C" int msa_pool_chunks(const void* k, const void* v, const void* kr, int32_t dtype, int64_t T, int32_t H,
                               int32_t D, const int32_t* chunk_start, const int32_t* chunk_len,
                               const int32_t* chunk_doc, int64_t C, const int32_t* doc_start, const float* rope_cos,
                               const float* rope_sin, int32_t rope_rows, int32_t max_doc_len, int32_t normalize_kr,
                               void* k_out, void* v_out, void* kr_out, void* stream) {
  MSA_REQUIRE(D == kHeadDim, "msa_pool_chunks: head dim %d unsupported (need %d)", D, kHeadDim);
  MSA_REQUIRE(H > 0 && H <= 32 && (kThreads % (H * 8)) == 0, "msa_pool_chunks: H=%d must divide 32", H);
  MSA_REQUIRE(dtype == MSA_BF16 || dtype == MSA_F32, "msa_pool_chunks: bad dtype %d", dtype);
  MSA_REQUIRE(T > 0 && T < (int64_t)1 << 31, "msa_pool_chunks: T=%lld out of range", (long long)T);
  MSA_REQUIRE(C >= 0 && C < (int64_t)1 << 31, "msa_pool_chunks: C=%lld out of range", (long long)C);
  MSA_REQUIRE(chunk_start && chunk_len && chunk_doc, "msa_pool_chunks: null chunk table");
  MSA_REQUIRE((k == nullptr) == (k_out == nullptr) && (v == nullptr) == (v_out == nullptr) &&
                  (kr == nullptr) == (kr_out == nullptr),
              "msa_pool_chunks: each input needs its output and vice versa");
  const bool rope = rope_cos != nullptr || rope_sin != nullptr;
  if (rope) {
    MSA_REQUIRE(rope_cos && rope_sin && doc_start, "msa_pool_chunks: rotary needs cos, sin and doc_start");
    MSA_REQUIRE(k != nullptr, "msa_pool_chunks: rotary requested without K");
    MSA_REQUIRE(max_doc_len > 0 && max_doc_len <= rope_rows,
                "msa_pool_chunks: max_doc_len=%d exceeds the rotary table (%d rows)", max_doc_len, rope_rows);
    MSA_REQUIRE(rope_rows > kThreads / (H * 8), "msa_pool_chunks: rotary table too short (%d rows)", rope_rows);
  }
  if (C == 0) return MSA_OK;

  // two launches at most: the tensors read plain, and the one rotated while read
  PoolArgs plain{}, rotated{};
  auto add = [&](PoolArgs& a, const void* in, void* out, int nm) {
    if (!in) return;
    const int n = a.n_tensors++;
    a.in[n] = in; a.out[n] = out; a.rope[n] = &a == &rotated; a.normalize[n] = nm;
  };
  add(rope ? rotated : plain, k, k_out, 0);
  add(plain, v, v_out, 0);
  add(plain, kr, kr_out, normalize_kr ? 1 : 0);
  MSA_REQUIRE(plain.n_tensors + rotated.n_tensors > 0, "msa_pool_chunks: nothing to pool");
  for (PoolArgs* a : {&plain, &rotated}) {
    for (int i = 0; i < a->n_tensors; ++i)
      MSA_REQUIRE(((uintptr_t)a->in[i] & 15) == 0 && ((uintptr_t)a->out[i] & 15) == 0,
                  "msa_pool_chunks: tensors must be 16-byte aligned");
    a->T = T; a->H = H;
    a->chunk_start = chunk_start; a->chunk_len = chunk_len; a->chunk_doc = chunk_doc; a->doc_start = doc_start;
    a->rope_cos = rope_cos; a->rope_sin = rope_sin; a->rope_rows = rope_rows;
  }
  if (plain.n_tensors > 0) {
    const dim3 grid((unsigned)C, (unsigned)plain.n_tensors);
    if (dtype == MSA_BF16)
      pool_chunks_kernel<bf16_t, false><<<grid, kThreads, 0, as_stream(stream)>>>(plain);
    else
      pool_chunks_kernel<float, false><<<grid, kThreads, 0, as_stream(stream)>>>(plain);
    MSA_LAUNCH_CHECK();
  }
  if (rotated.n_tensors > 0) {
    const dim3 grid((unsigned)C, (unsigned)rotated.n_tensors);
    if (dtype == MSA_BF16)
      pool_chunks_kernel<bf16_t, true><<<grid, kThreads, 0, as_stream(stream)>>>(rotated);
    else
      pool_chunks_kernel<float, true><<<grid, kThreads, 0, as_stream(stream)>>>(rotated);
    MSA_LAUNCH_CHECK();
  }
  return MSA_OK;
}
