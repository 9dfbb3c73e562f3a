// Small fused kernels around the attention call of a decoder layer: per-head q/k RMSNorm + rotary
// in one pass, row RMSNorm with the residual add folded in, and SiLU(gate) * up.  All are a few
// bytes per FLOP: one read of the input, one write of the output.
#include <algorithm>

#include "common.h"

namespace {

template <typename T>
__device__ __forceinline__ void load8g(const T* p, float (&x)[8]) {
  if constexpr (sizeof(T) == 2) {
    const uint4 w = *reinterpret_cast<const uint4*>(p);
    x[0] = bf16lo(w.x); x[1] = bf16hi(w.x); x[2] = bf16lo(w.y); x[3] = bf16hi(w.y);
    x[4] = bf16lo(w.z); x[5] = bf16hi(w.z); x[6] = bf16lo(w.w); x[7] = bf16hi(w.w);
  } else {
    const float4 a = *reinterpret_cast<const float4*>(p);
    const float4 b = *reinterpret_cast<const float4*>(p + 4);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w; x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
  }
}
template <typename T>
__device__ __forceinline__ void store8g(T* p, const float (&x)[8]) {
  if constexpr (sizeof(T) == 2) {
    uint4 w;
    w.x = pack_bf16x2(x[0], x[1]); w.y = pack_bf16x2(x[2], x[3]);
    w.z = pack_bf16x2(x[4], x[5]); w.w = pack_bf16x2(x[6], x[7]);
    *reinterpret_cast<uint4*>(p) = w;
  } else {
    *reinterpret_cast<float4*>(p) = make_float4(x[0], x[1], x[2], x[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(x[4], x[5], x[6], x[7]);
  }
}

// One workgroup per token; 16 lanes per head (8 dims each): heads 0..Hq-1 are q, the rest k.
// RMSNorm over the head's 128 dims (fp32), times the norm weight, then half-split rotary at the
// token's position: lane j pairs with lane j^8 of its row (dims d and d +- 64).
template <typename T>
__global__ void qk_norm_rope_kernel(const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                    int64_t q_stride, int64_t k_stride, int64_t v_stride,
                                    const int64_t* __restrict__ pos, const T* __restrict__ qw,
                                    const T* __restrict__ kw, float eps, const float* __restrict__ cos_t,
                                    const float* __restrict__ sin_t, int32_t rope_rows, int32_t Hq, int32_t Hkv,
                                    T* __restrict__ q_out, T* __restrict__ k_out, T* __restrict__ v_out,
                                    int32_t Lcap, int32_t* __restrict__ kv_len) {
  const int64_t n = blockIdx.x;
  const int head = threadIdx.x >> 4, j = threadIdx.x & 15;
  // Append mode (kv_len given; token n is the one new token of sample n): k / v rows go straight into the
  // sample's cache [n][kv_len[n]] and the length is bumped; a full cache drops the row.
  int64_t kv_row = n;
  bool keep_kv = true;
  if (kv_len != nullptr) {
    const int at = kv_len[n];
    __syncthreads();                     // every lane has read the old length before lane 0 bumps it
    keep_kv = at < Lcap;
    kv_row = n * Lcap + at;
    if (threadIdx.x == 0 && keep_kv) kv_len[n] = at + 1;
  }
  if (head >= Hq + Hkv) {                       // optional V heads: a straight copy into a dense row
    const int hv = head - Hq - Hkv;
    if (v != nullptr && hv < Hkv && keep_kv) {
      float t[8];
      load8g<T>(v + n * v_stride + hv * kHeadDim + 8 * j, t);
      store8g<T>(v_out + (kv_row * Hkv + hv) * kHeadDim + 8 * j, t);
    }
    return;
  }
  const bool is_q = head < Hq;
  const int h = is_q ? head : head - Hq;
  const T* src = is_q ? q + n * q_stride + h * kHeadDim : k + n * k_stride + h * kHeadDim;
  T* dst = is_q ? q_out + (n * Hq + h) * kHeadDim : k_out + (kv_row * Hkv + h) * kHeadDim;
  float x[8], w[8];
  load8g<T>(src + 8 * j, x);
  load8g<T>((is_q ? qw : kw) + 8 * j, w);
  float ssq = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) ssq += x[i] * x[i];
  const float inv = rsqrtf(row16_sum(ssq) * (1.0f / kHeadDim) + eps);
  const int64_t p = min((int64_t)max((int64_t)0, pos[n]), (int64_t)rope_rows - 1);
  const int f = 8 * (j & 7);                    // frequency index of this lane's first element
  // lanes j and j ^ 8 need the same eight cosines and sines: the lower lane fetches the cosines, the upper one the
  // sines, and they swap (the table reads were four of a lane's seven memory instructions)
  const float* tab = (j < 8 ? cos_t : sin_t) + p * 64 + f;
  const float4 t0 = *reinterpret_cast<const float4*>(tab), t1 = *reinterpret_cast<const float4*>(tab + 4);
  const float mine[8] = {t0.x, t0.y, t0.z, t0.w, t1.x, t1.y, t1.z, t1.w};
  float out[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float y = x[i] * inv * w[i];
    const float other = row16_ror8(y);          // the paired dim (d + 64 for j < 8, d - 64 for j >= 8)
    const float theirs = row16_ror8(mine[i]);
    const float c = j < 8 ? mine[i] : theirs, s = j < 8 ? theirs : mine[i];
    out[i] = j < 8 ? y * c - other * s : y * c + other * s;
  }
  if (is_q || keep_kv) store8g<T>(dst + 8 * j, out);
}

// One workgroup per row.  With `residual`: residual <- residual + x (stored in T), then normalised.
// Eight elements per lane per step (16-byte accesses for bf16) when H is a multiple of 8 and every tensor is
// 16-byte aligned (`vec`); the summed row is kept in registers between
// the two passes when it fits (H <= 256 * 8 * kKeep), otherwise it is re-read from `residual` / `x`.
template <typename T>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const T* __restrict__ x, T* __restrict__ residual,
                                                      const T* __restrict__ w, int32_t H, float eps,
                                                      T* __restrict__ out, int32_t vec) {
  constexpr int kKeep = 2;                       // steps of a row held in registers (H <= 4096)
  __shared__ float part[4];
  const int64_t row = blockIdx.x;
  const T* xr = x + row * H;
  T* rr = residual ? residual + row * H : nullptr;
  T* orow = out + row * H;
  float keep[kKeep][8];
  float ssq = 0.f;
  if (vec) {
    int step = 0;
    for (int i = threadIdx.x * 8; i < H; i += 256 * 8, ++step) {
      float v[8];
      load8g<T>(xr + i, v);
      if (rr) {
        float r[8];
        load8g<T>(rr + i, r);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          v[e] += r[e];
          if constexpr (sizeof(T) == 2) v[e] = bf16_to_f32(f32_to_bf16(v[e]));     // the residual stream is stored in T
        }
        store8g<T>(rr + i, v);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ssq += v[e] * v[e];
      if (step < kKeep) {
#pragma unroll
        for (int e = 0; e < 8; ++e) keep[step][e] = v[e];
      }
    }
  } else {
    for (int i = threadIdx.x; i < H; i += 256) {
      float v;
      if constexpr (sizeof(T) == 2) v = bf16_to_f32(xr[i]); else v = xr[i];
      if (rr) {
        if constexpr (sizeof(T) == 2) { v = bf16_to_f32(f32_to_bf16(v + bf16_to_f32(rr[i]))); rr[i] = f32_to_bf16(v); }
        else { v = v + rr[i]; rr[i] = v; }
      }
      ssq += v * v;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) ssq += __shfl_xor(ssq, o);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ssq;
  __syncthreads();
  const float inv = rsqrtf((part[0] + part[1] + part[2] + part[3]) / (float)H + eps);
  const T* src = rr ? rr : xr;      // rr was written by this same thread for the same indices
  if (vec) {
    int step = 0;
    for (int i = threadIdx.x * 8; i < H; i += 256 * 8, ++step) {
      float v[8], g[8];
      if (step < kKeep) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = keep[step][e];
      } else {
        load8g<T>(src + i, v);
      }
      load8g<T>(w + i, g);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = v[e] * inv * g[e];
      store8g<T>(orow + i, v);
    }
  } else {
    for (int i = threadIdx.x; i < H; i += 256) {
      float v, g;
      if constexpr (sizeof(T) == 2) { v = bf16_to_f32(src[i]); g = bf16_to_f32(w[i]); orow[i] = f32_to_bf16(v * inv * g); }
      else { v = src[i]; g = w[i]; orow[i] = v * inv * g; }
    }
  }
}

// out[n, i] = silu(gate_up[n, i]) * gate_up[n, I + i]; eight elements per lane (16-byte accesses for bf16)
// when I is a multiple of 8 and the tensors are 16-byte aligned (`vec`).
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate_up, int64_t N, int32_t I, T* __restrict__ out, int32_t vec) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  if (vec) {
    const int64_t per_row = I / 8, total = N * per_row;
    for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
      const int64_t n = idx / per_row, i = (idx % per_row) * 8;
      float g[8], u[8];
      load8g<T>(gate_up + n * 2 * I + i, g);
      load8g<T>(gate_up + n * 2 * I + I + i, u);
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = g[e] / (1.0f + __expf(-g[e])) * u[e];
      store8g<T>(out + n * I + i, g);
    }
    return;
  }
  const int64_t total = N * I;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += stride) {
    const int64_t n = idx / I, i = idx % I;
    float g, u;
    if constexpr (sizeof(T) == 2) { g = bf16_to_f32(gate_up[n * 2 * I + i]); u = bf16_to_f32(gate_up[n * 2 * I + I + i]); }
    else { g = gate_up[n * 2 * I + i]; u = gate_up[n * 2 * I + I + i]; }
    const float y = g / (1.0f + __expf(-g)) * u;
    if constexpr (sizeof(T) == 2) out[idx] = f32_to_bf16(y); else out[idx] = y;
  }
}

// ------------------------------------------------------------------------------------------------
// Greedy sampling of a decode step: row-wise argmax of the logits and the token bookkeeping around it in two
// launches (partial maxima over slices of a row, then one thread per row).  A candidate is the 64-bit key
// (order-preserving bits of the value) << 32 | (0xffffffff - index): the largest key is the largest value and,
// among equal values, the smallest index.
// ------------------------------------------------------------------------------------------------
constexpr int kArgmaxSplits = 32;

template <typename T>
__device__ __forceinline__ uint32_t sortable_bits(T v);
template <>
__device__ __forceinline__ uint32_t sortable_bits<bf16_t>(bf16_t v) {
  const uint32_t b = (uint32_t)v << 16;
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
template <>
__device__ __forceinline__ uint32_t sortable_bits<float>(float v) {
  const uint32_t b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

template <typename T>
__global__ __launch_bounds__(256) void argmax_partial_kernel(const T* __restrict__ logits, int64_t V,
                                                             unsigned long long* __restrict__ partial) {
  const int row = blockIdx.x, split = blockIdx.y;
  const int64_t per = (V + kArgmaxSplits - 1) / kArgmaxSplits;
  const int64_t lo = split * per, hi = min(V, lo + per);
  const T* x = logits + (int64_t)row * V;
  unsigned long long best = 0;
  for (int64_t i = lo + threadIdx.x; i < hi; i += blockDim.x) {
    const unsigned long long cand = ((unsigned long long)sortable_bits<T>(x[i]) << 32) | (0xffffffffu - (uint32_t)i);
    best = cand > best ? cand : best;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const unsigned long long other = __shfl_xor(best, off);
    best = other > best ? other : best;
  }
  __shared__ unsigned long long wave_best[4];
  if ((threadIdx.x & 63) == 0) wave_best[threadIdx.x >> 6] = best;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) best = wave_best[w] > best ? wave_best[w] : best;
    partial[(int64_t)row * kArgmaxSplits + split] = best;
  }
}

__global__ void greedy_commit_kernel(const unsigned long long* __restrict__ partial, int32_t B, int64_t* __restrict__ tok,
                                     int64_t* __restrict__ pos, int64_t* __restrict__ out, int64_t out_stride,
                                     int64_t* __restrict__ col, int32_t max_new) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  unsigned long long best = 0;
  for (int s = 0; s < kArgmaxSplits; ++s) {
    const unsigned long long c = partial[(int64_t)b * kArgmaxSplits + s];
    best = c > best ? c : best;
  }
  const int64_t idx = (int64_t)(0xffffffffu - (uint32_t)(best & 0xffffffffu));
  tok[b] = idx;
  if (pos) pos[b] += 1;
  if (out) {
    const int64_t c = col[b];
    if (c >= 0 && c < max_new) out[(int64_t)b * out_stride + c] = idx;
    col[b] = c + 1;
  }
}

}  // namespace

static int qk_norm_rope_launch(const char* who, const void* q, const void* k, const void* v, int64_t q_row_stride,
                               int64_t k_row_stride, int64_t v_row_stride, const int64_t* positions,
                               const void* q_norm_w, const void* k_norm_w, float eps, const float* rope_cos,
                               const float* rope_sin, int32_t rope_rows, int32_t dtype, int64_t N, int32_t Hq,
                               int32_t Hkv, int32_t D, void* q_out, void* k_out, void* v_out, int32_t Lcap,
                               int32_t* kv_len, void* stream) {
  MSA_REQUIRE(q && k && positions && q_norm_w && k_norm_w && rope_cos && rope_sin && q_out && k_out,
              "%s: null pointer", who);
  MSA_REQUIRE(D == kHeadDim, "%s: head dim %d unsupported (need %d)", who, D, kHeadDim);
  MSA_REQUIRE(dtype == MSA_BF16 || dtype == MSA_F32, "%s: bad dtype %d", who, dtype);
  MSA_REQUIRE(N > 0 && N < (int64_t)1 << 31, "%s: N=%lld out of range", who, (long long)N);
  MSA_REQUIRE((((uintptr_t)rope_cos | (uintptr_t)rope_sin) & 15) == 0, "%s: rotary tables must be 16-byte aligned", who);
  MSA_REQUIRE((v == nullptr) == (v_out == nullptr), "%s: v and v_out go together", who);
  const int heads = Hq + Hkv + (v ? Hkv : 0);
  MSA_REQUIRE(Hq > 0 && Hkv > 0 && heads * 16 <= 1024, "%s: Hq=%d Hkv=%d unsupported", who, Hq, Hkv);
  MSA_REQUIRE(v == nullptr || (v_row_stride >= (int64_t)Hkv * D && v_row_stride % 8 == 0), "%s: bad V row stride", who);
  MSA_REQUIRE(rope_rows > 0, "%s: empty rotary table", who);
  MSA_REQUIRE(q_row_stride >= (int64_t)Hq * D && k_row_stride >= (int64_t)Hkv * D && q_row_stride % 8 == 0 &&
                  k_row_stride % 8 == 0, "%s: bad row strides", who);
  const int threads = (heads * 16 + 63) / 64 * 64;
  if (dtype == MSA_BF16)
    qk_norm_rope_kernel<bf16_t><<<(unsigned)N, threads, 0, as_stream(stream)>>>(
        (const bf16_t*)q, (const bf16_t*)k, (const bf16_t*)v, q_row_stride, k_row_stride, v_row_stride, positions,
        (const bf16_t*)q_norm_w, (const bf16_t*)k_norm_w, eps, rope_cos, rope_sin, rope_rows, Hq, Hkv,
        (bf16_t*)q_out, (bf16_t*)k_out, (bf16_t*)v_out, Lcap, kv_len);
  else
    qk_norm_rope_kernel<float><<<(unsigned)N, threads, 0, as_stream(stream)>>>(
        (const float*)q, (const float*)k, (const float*)v, q_row_stride, k_row_stride, v_row_stride, positions,
        (const float*)q_norm_w, (const float*)k_norm_w, eps, rope_cos, rope_sin, rope_rows, Hq, Hkv, (float*)q_out,
        (float*)k_out, (float*)v_out, Lcap, kv_len);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

extern "C" int msa_qk_norm_rope(const void* q, const void* k, const void* v, int64_t q_row_stride,
                                int64_t k_row_stride, int64_t v_row_stride, const int64_t* positions,
                                const void* q_norm_w, const void* k_norm_w, float eps, const float* rope_cos,
                                const float* rope_sin, int32_t rope_rows, int32_t dtype, int64_t N, int32_t Hq,
                                int32_t Hkv, int32_t D, void* q_out, void* k_out, void* v_out, void* stream) {
  return qk_norm_rope_launch("msa_qk_norm_rope", q, k, v, q_row_stride, k_row_stride, v_row_stride, positions, q_norm_w,
                             k_norm_w, eps, rope_cos, rope_sin, rope_rows, dtype, N, Hq, Hkv, D, q_out, k_out, v_out, 0,
                             nullptr, stream);
}

extern "C" int msa_qk_norm_rope_append(const void* q, const void* k, const void* v, int64_t q_row_stride,
                                       int64_t k_row_stride, int64_t v_row_stride, const int64_t* positions,
                                       const void* q_norm_w, const void* k_norm_w, float eps, const float* rope_cos,
                                       const float* rope_sin, int32_t rope_rows, int32_t dtype, int32_t B, int32_t Hq,
                                       int32_t Hkv, int32_t D, void* q_out, void* kcache, void* vcache, int32_t Lcap,
                                       int32_t* kv_len, void* stream) {
  MSA_REQUIRE(v && kcache && vcache && kv_len && Lcap > 0, "msa_qk_norm_rope_append: null cache pointer or Lcap <= 0");
  return qk_norm_rope_launch("msa_qk_norm_rope_append", q, k, v, q_row_stride, k_row_stride, v_row_stride, positions,
                             q_norm_w, k_norm_w, eps, rope_cos, rope_sin, rope_rows, dtype, B, Hq, Hkv, D, q_out, kcache,
                             vcache, Lcap, kv_len, stream);
}

extern "C" int msa_rmsnorm(const void* x, void* residual, const void* weight, int32_t dtype, int64_t N, int32_t H,
                           float eps, void* out, void* stream) {
  MSA_REQUIRE(x && weight && out, "msa_rmsnorm: null pointer");
  MSA_REQUIRE(dtype == MSA_BF16 || dtype == MSA_F32, "msa_rmsnorm: bad dtype %d", dtype);
  MSA_REQUIRE(N > 0 && N < (int64_t)1 << 31 && H > 0, "msa_rmsnorm: bad shape");
  const int vec = (H & 7) == 0 && (((uintptr_t)x | (uintptr_t)residual | (uintptr_t)weight | (uintptr_t)out) & 15) == 0;
  if (dtype == MSA_BF16)
    rmsnorm_kernel<bf16_t><<<(unsigned)N, 256, 0, as_stream(stream)>>>((const bf16_t*)x, (bf16_t*)residual,
                                                                       (const bf16_t*)weight, H, eps, (bf16_t*)out, vec);
  else
    rmsnorm_kernel<float><<<(unsigned)N, 256, 0, as_stream(stream)>>>((const float*)x, (float*)residual,
                                                                      (const float*)weight, H, eps, (float*)out, vec);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

extern "C" int msa_silu_mul(const void* gate_up, int32_t dtype, int64_t N, int32_t I, void* out, void* stream) {
  MSA_REQUIRE(gate_up && out, "msa_silu_mul: null pointer");
  MSA_REQUIRE(dtype == MSA_BF16 || dtype == MSA_F32, "msa_silu_mul: bad dtype %d", dtype);
  MSA_REQUIRE(N > 0 && I > 0, "msa_silu_mul: bad shape");
  const int64_t total = N * I;
  const int vec = (I & 7) == 0 && (((uintptr_t)gate_up | (uintptr_t)out) & 15) == 0;
  const int64_t items = vec ? total / 8 : total;
  const int grid = (int)std::min<int64_t>((items + 255) / 256, 16384);
  if (dtype == MSA_BF16)
    silu_mul_kernel<bf16_t><<<grid, 256, 0, as_stream(stream)>>>((const bf16_t*)gate_up, N, I, (bf16_t*)out, vec);
  else
    silu_mul_kernel<float><<<grid, 256, 0, as_stream(stream)>>>((const float*)gate_up, N, I, (float*)out, vec);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

extern "C" int msa_greedy_sample(const void* logits, int32_t dtype, int32_t B, int64_t V, void* scratch, int64_t* tok,
                                 int64_t* pos, int64_t* out, int64_t out_stride, int64_t* col, int32_t max_new,
                                 void* stream) {
  MSA_REQUIRE(logits && scratch && tok, "msa_greedy_sample: null pointer");
  MSA_REQUIRE(dtype == MSA_BF16 || dtype == MSA_F32, "msa_greedy_sample: dtype %d", dtype);
  MSA_REQUIRE(B > 0 && B <= 65535 && V > 0 && V < ((int64_t)1 << 32), "msa_greedy_sample: B=%d V=%lld", B, (long long)V);
  MSA_REQUIRE((out == nullptr) == (col == nullptr), "msa_greedy_sample: out and col go together");
  hipStream_t st = as_stream(stream);
  dim3 grid((unsigned)B, kArgmaxSplits);
  if (dtype == MSA_BF16) {
    argmax_partial_kernel<bf16_t><<<grid, 256, 0, st>>>(static_cast<const bf16_t*>(logits), V,
                                                        static_cast<unsigned long long*>(scratch));
  } else {
    argmax_partial_kernel<float><<<grid, 256, 0, st>>>(static_cast<const float*>(logits), V,
                                                       static_cast<unsigned long long*>(scratch));
  }
  MSA_LAUNCH_CHECK();
  greedy_commit_kernel<<<(B + 63) / 64, 64, 0, st>>>(static_cast<const unsigned long long*>(scratch), B, tok, pos, out,
                                                     out_stride, col, max_new);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}
