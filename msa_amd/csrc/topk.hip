// Streaming document top-k: segmented max over each document's chunk keys fused with a
// wavefront-level bitonic select, an LDS merge across the workgroup's wavefronts, and a final
// per-query merge of the per-workgroup candidate lists.
//
// Candidates are 64-bit composites (score key << 32 | ~doc) so one unsigned compare orders by
// score descending, then document index ascending; 0 is the empty slot.
#include "route_internal.h"

namespace {

constexpr int kWaves = 4;

__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int m) {
  return (uint64_t)__shfl_xor((unsigned long long)v, m);
}
__device__ __forceinline__ uint64_t shfl_u64(uint64_t v, int src) {
  return (uint64_t)__shfl((unsigned long long)v, src);
}
__device__ __forceinline__ uint64_t umax64(uint64_t a, uint64_t b) { return a > b ? a : b; }
__device__ __forceinline__ uint64_t umin64(uint64_t a, uint64_t b) { return a < b ? a : b; }

// Full bitonic sort of one value per lane, descending by lane index.
__device__ __forceinline__ uint64_t wave_sort_desc(uint64_t v, int lane) {
#pragma unroll
  for (int k = 2; k <= 64; k <<= 1) {
#pragma unroll
    for (int j = k >> 1; j > 0; j >>= 1) {
      const uint64_t o = shfl_xor_u64(v, j);
      const bool desc_block = (lane & k) == 0;
      const bool lower = (lane & j) == 0;
      v = (lower == desc_block) ? umax64(v, o) : umin64(v, o);
    }
  }
  return v;
}

// best (sorted descending) <- top 64 of best U batch (sorted descending)
__device__ __forceinline__ uint64_t wave_merge_desc(uint64_t best, uint64_t batch, int lane) {
  uint64_t v = umax64(best, shfl_u64(batch, 63 - lane));   // bitonic, holds the 64 largest of the union
#pragma unroll
  for (int j = 32; j > 0; j >>= 1) {
    const uint64_t o = shfl_xor_u64(v, j);
    v = (lane & j) == 0 ? umax64(v, o) : umin64(v, o);
  }
  return v;
}

__global__ __launch_bounds__(kWaves * 64) void doc_topk_kernel(const uint32_t* __restrict__ chunk_key,
                                                               const int32_t* __restrict__ doc_chunk_off,
                                                               int64_t C, int32_t n_docs,
                                                               uint64_t* __restrict__ cand) {
  __shared__ uint64_t lists[kWaves][64];
  const int b = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t* key = chunk_key + (int64_t)b * C;
  const int d_begin = blockIdx.x * kTopkDocsPerBlock;
  const int d_end = min(d_begin + kTopkDocsPerBlock, n_docs);

  uint64_t best = 0;
  for (int base = d_begin + wave * 64; base < d_end; base += kWaves * 64) {   // wave-uniform trip count
    const int d = base + lane;
    uint64_t v = 0;
    if (d < d_end) {
      const int c0 = doc_chunk_off[d], c1 = doc_chunk_off[d + 1];
      uint32_t m = 0;
      for (int c = c0; c < c1; c += 16) {          // 16 independent loads in flight per lane (clamped: duplicates are harmless)
        uint32_t kv[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) kv[u] = key[min(c + u, c1 - 1)];
#pragma unroll
        for (int u = 0; u < 16; ++u) m = max(m, kv[u]);
      }
      v = ((uint64_t)m << 32) | (uint64_t)(0xffffffffu - (uint32_t)d);
    }
    v = wave_sort_desc(v, lane);
    best = wave_merge_desc(best, v, lane);
  }
  lists[wave][lane] = best;
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int w = 1; w < kWaves; ++w) best = wave_merge_desc(best, lists[w][lane], lane);
    cand[((int64_t)b * gridDim.x + blockIdx.x) * kTopkMax + lane] = best;
  }
}

__global__ __launch_bounds__(64) void merge_topk_kernel(const uint64_t* __restrict__ cand, int32_t blocks,
                                                        const int64_t* __restrict__ doc_global_id, float mul,
                                                        int32_t topk, float* __restrict__ scores_out,
                                                        int32_t* __restrict__ doc_out,
                                                        int64_t* __restrict__ doc_global_out) {
  const int b = blockIdx.x, lane = threadIdx.x;
  uint64_t best = 0;
  for (int i = 0; i < blocks; ++i) best = wave_merge_desc(best, cand[((int64_t)b * blocks + i) * kTopkMax + lane], lane);
  if (lane < topk) {
    const int64_t o = (int64_t)b * topk + lane;
    if (best == 0) {
      scores_out[o] = -INFINITY;
      doc_out[o] = -1;
      if (doc_global_out) doc_global_out[o] = -1;
    } else {
      const uint32_t k = (uint32_t)(best >> 32);
      const int32_t d = (int32_t)(0xffffffffu - (uint32_t)best);
      scores_out[o] = k == 0 ? -INFINITY : key_to_f32(k) * mul;
      doc_out[o] = d;
      if (doc_global_out) doc_global_out[o] = doc_global_id[d];
    }
  }
}

}  // namespace

extern "C" int msa_route_topk(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B,
                              int32_t S, int32_t Hq, int32_t mode, float scale, int32_t topk, float* scores_out,
                              int32_t* doc_out, int64_t* doc_global_out, void* workspace, size_t workspace_bytes,
                              void* stream) {
  MSA_REQUIRE(scores_out && doc_out, "msa_route_topk: null output");
  MSA_REQUIRE(topk > 0 && topk <= kTopkMax, "msa_route_topk: topk=%d out of range (1..%d)", topk, kTopkMax);
  RouteWorkspace w;
  float mul;
  hipStream_t st = as_stream(stream);
  int rc = route_scores_to_keys(bank, layer, q, qmask_u8, B, S, Hq, mode, scale, workspace, workspace_bytes, st, &w,
                                &mul, "msa_route_topk");
  if (rc != MSA_OK) return rc;
  char* ws = static_cast<char*>(workspace);
  const uint32_t* key = reinterpret_cast<const uint32_t*>(ws + w.off_chunk_key);
  uint64_t* cand = reinterpret_cast<uint64_t*>(ws + w.off_cand);
  dim3 grid((unsigned)w.topk_blocks, (unsigned)B);
  doc_topk_kernel<<<grid, kWaves * 64, 0, st>>>(key, bank->doc_chunk_off_dev, bank->C, (int32_t)bank->n_docs, cand);
  MSA_LAUNCH_CHECK();
  merge_topk_kernel<<<B, 64, 0, st>>>(cand, w.topk_blocks, bank->doc_global_id_dev, mul, topk, scores_out, doc_out,
                                      doc_global_out);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}
