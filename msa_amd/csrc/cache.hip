// Context assembly and in-place cache append: plain 16-byte row copies.
#include <algorithm>

#include "common.h"

namespace {

// One workgroup per (destination row, sample); rows are Hkv*D elements copied as uint4.
__global__ void assemble_kernel(const uint4* __restrict__ prefix_k, const uint4* __restrict__ prefix_v,
                                int32_t n_prefix, const uint4* __restrict__ mem_k, const uint4* __restrict__ mem_v,
                                const int32_t* __restrict__ cu_sel, const uint4* __restrict__ local_k,
                                const uint4* __restrict__ local_v, const int32_t* __restrict__ cu_local,
                                int32_t row_vecs, uint4* __restrict__ kcache, uint4* __restrict__ vcache,
                                int32_t Lcap, int32_t* __restrict__ kv_len) {
  const int b = blockIdx.y;
  const int n_mem = cu_sel ? cu_sel[b + 1] - cu_sel[b] : 0;
  const int n_loc = cu_local ? cu_local[b + 1] - cu_local[b] : 0;
  const int total = min(n_prefix + n_mem + n_loc, Lcap);
  if (blockIdx.x == 0 && threadIdx.x == 0) kv_len[b] = total;
  for (int row = blockIdx.x; row < total; row += gridDim.x) {
    const uint4 *sk, *sv;
    if (row < n_prefix) {
      sk = prefix_k + (int64_t)row * row_vecs; sv = prefix_v + (int64_t)row * row_vecs;
    } else if (row < n_prefix + n_mem) {
      const int64_t r = (int64_t)cu_sel[b] + (row - n_prefix);
      sk = mem_k + r * row_vecs; sv = mem_v + r * row_vecs;
    } else {
      const int64_t r = (int64_t)cu_local[b] + (row - n_prefix - n_mem);
      sk = local_k + r * row_vecs; sv = local_v + r * row_vecs;
    }
    uint4* dk = kcache + ((int64_t)b * Lcap + row) * row_vecs;
    uint4* dv = vcache + ((int64_t)b * Lcap + row) * row_vecs;
    for (int i = threadIdx.x; i < row_vecs; i += blockDim.x) { dk[i] = sk[i]; dv[i] = sv[i]; }
  }
}

__global__ void append_kernel(const uint4* __restrict__ k_new, const uint4* __restrict__ v_new, int32_t row_vecs,
                              uint4* __restrict__ kcache, uint4* __restrict__ vcache, int32_t Lcap,
                              int32_t* __restrict__ kv_len) {
  const int b = blockIdx.x;
  const int at = kv_len[b];
  __syncthreads();                       // every lane has read the old length before lane 0 bumps it
  if (at >= Lcap) return;                // full: drop the row rather than write out of bounds
  uint4* dk = kcache + ((int64_t)b * Lcap + at) * row_vecs;
  uint4* dv = vcache + ((int64_t)b * Lcap + at) * row_vecs;
  for (int i = threadIdx.x; i < row_vecs; i += blockDim.x) {
    dk[i] = k_new[(int64_t)b * row_vecs + i];
    dv[i] = v_new[(int64_t)b * row_vecs + i];
  }
  if (threadIdx.x == 0) kv_len[b] = at + 1;
}

// Ragged form: sample b appends rows cu_new[b] .. cu_new[b+1] of k_new / v_new; rows that do not fit are dropped.
__global__ void append_rows_kernel(const uint4* __restrict__ k_new, const uint4* __restrict__ v_new,
                                   const int32_t* __restrict__ cu_new, int32_t row_vecs, uint4* __restrict__ kcache,
                                   uint4* __restrict__ vcache, int32_t Lcap, int32_t* __restrict__ kv_len) {
  const int b = blockIdx.y;
  const int at = kv_len[b];
  const int first = cu_new[b], n = min(cu_new[b + 1] - first, Lcap - at);
  // the length is bumped by a second tiny launch (bump_len_kernel): other workgroups of this launch still read it
  for (int r = blockIdx.x; r < n; r += gridDim.x) {
    const uint4* sk = k_new + (int64_t)(first + r) * row_vecs;
    const uint4* sv = v_new + (int64_t)(first + r) * row_vecs;
    uint4* dk = kcache + ((int64_t)b * Lcap + at + r) * row_vecs;
    uint4* dv = vcache + ((int64_t)b * Lcap + at + r) * row_vecs;
    for (int i = threadIdx.x; i < row_vecs; i += blockDim.x) {
      dk[i] = sk[i];
      dv[i] = sv[i];
    }
  }
}

__global__ void bump_len_kernel(const int32_t* __restrict__ cu_new, int32_t B, int32_t Lcap, int32_t* __restrict__ kv_len) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b < B) kv_len[b] = min(Lcap, kv_len[b] + max(0, cu_new[b + 1] - cu_new[b]));
}

}  // namespace

extern "C" int msa_assemble_context(const void* prefix_k, const void* prefix_v, int32_t n_prefix, const void* mem_k,
                                    const void* mem_v, const int32_t* cu_sel, const void* local_k, const void* local_v,
                                    const int32_t* cu_local, int32_t B, int32_t Hkv, int32_t D, int32_t dtype,
                                    void* kcache, void* vcache, int32_t Lcap, int32_t* kv_len, void* stream) {
  MSA_REQUIRE(B > 0 && Hkv > 0 && D == kHeadDim && Lcap > 0, "msa_assemble_context: bad shape");
  MSA_REQUIRE(dtype == MSA_BF16 || dtype == MSA_F32, "msa_assemble_context: bad dtype %d", dtype);
  MSA_REQUIRE(kcache && vcache && kv_len, "msa_assemble_context: null output");
  MSA_REQUIRE(n_prefix >= 0 && (n_prefix == 0 || (prefix_k && prefix_v)), "msa_assemble_context: prefix missing");
  MSA_REQUIRE((cu_sel == nullptr) || (mem_k && mem_v), "msa_assemble_context: cu_sel without memory rows");
  MSA_REQUIRE((cu_local == nullptr) || (local_k && local_v), "msa_assemble_context: cu_local without local rows");
  const int32_t row_vecs = (int32_t)((size_t)Hkv * D * elem_bytes(dtype) / 16);
  dim3 grid((unsigned)std::min(Lcap, 2048), (unsigned)B);
  assemble_kernel<<<grid, 128, 0, as_stream(stream)>>>(
      (const uint4*)prefix_k, (const uint4*)prefix_v, n_prefix, (const uint4*)mem_k, (const uint4*)mem_v, cu_sel,
      (const uint4*)local_k, (const uint4*)local_v, cu_local, row_vecs, (uint4*)kcache, (uint4*)vcache, Lcap, kv_len);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

extern "C" int msa_cache_append(const void* k_new, const void* v_new, int32_t B, int32_t Hkv, int32_t D,
                                int32_t dtype, void* kcache, void* vcache, int32_t Lcap, int32_t* kv_len,
                                void* stream) {
  MSA_REQUIRE(B > 0 && Hkv > 0 && D == kHeadDim && Lcap > 0, "msa_cache_append: bad shape");
  MSA_REQUIRE(dtype == MSA_BF16 || dtype == MSA_F32, "msa_cache_append: bad dtype %d", dtype);
  MSA_REQUIRE(k_new && v_new && kcache && vcache && kv_len, "msa_cache_append: null pointer");
  const int32_t row_vecs = (int32_t)((size_t)Hkv * D * elem_bytes(dtype) / 16);
  append_kernel<<<B, 128, 0, as_stream(stream)>>>((const uint4*)k_new, (const uint4*)v_new, row_vecs, (uint4*)kcache,
                                                  (uint4*)vcache, Lcap, kv_len);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

extern "C" int msa_cache_append_rows(const void* k_new, const void* v_new, const int32_t* cu_new, int32_t max_new,
                                     int32_t B, int32_t Hkv, int32_t D, int32_t dtype, void* kcache, void* vcache,
                                     int32_t Lcap, int32_t* kv_len, void* stream) {
  MSA_REQUIRE(B > 0 && B <= 65535 && Hkv > 0 && D == kHeadDim && Lcap > 0 && max_new > 0, "msa_cache_append_rows: bad shape");
  MSA_REQUIRE(dtype == MSA_BF16 || dtype == MSA_F32, "msa_cache_append_rows: bad dtype %d", dtype);
  MSA_REQUIRE(k_new && v_new && cu_new && kcache && vcache && kv_len, "msa_cache_append_rows: null pointer");
  const int32_t row_vecs = (int32_t)((size_t)Hkv * D * elem_bytes(dtype) / 16);
  dim3 grid((unsigned)std::min(max_new, 1024), (unsigned)B);
  append_rows_kernel<<<grid, 128, 0, as_stream(stream)>>>((const uint4*)k_new, (const uint4*)v_new, cu_new, row_vecs,
                                                          (uint4*)kcache, (uint4*)vcache, Lcap, kv_len);
  MSA_LAUNCH_CHECK();
  bump_len_kernel<<<(B + 255) / 256, 256, 0, as_stream(stream)>>>(cu_new, B, Lcap, kv_len);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}
