// Streaming document top-k over the per-document keys the scoring kernel's epilogue leaves: a
// wavefront-level bitonic select, an LDS merge across the workgroup's wavefronts, and a final
// per-query merge of the per-workgroup candidate lists.
//
// Candidates are 64-bit composites (score key << 32 | ~doc) so one unsigned compare orders by
// score descending, then document index ascending; 0 is the empty slot.
#include <mutex>

#include "gather_device.h"
#include "route_internal.h"

namespace {

constexpr int kWaves = 4;

// Lane i receives the value of lane i ^ m.  Masks up to 8 stay inside a row of 16 lanes and are data-parallel
// moves (a few cycles); 16 and 32 cross rows and go through the LDS crossbar.  The sort networks below are chains of
// dependent exchanges, so this latency is what the top-k kernels spend their time on.
__device__ __forceinline__ uint32_t xor_lanes_u32(uint32_t v, int m) {
  const int x = (int)v;
  switch (m) {
    case 1: return (uint32_t)__builtin_amdgcn_update_dpp(x, x, 0xB1, 0xF, 0xF, false);    // quad_perm [1,0,3,2]
    case 2: return (uint32_t)__builtin_amdgcn_update_dpp(x, x, 0x4E, 0xF, 0xF, false);    // quad_perm [2,3,0,1]
    case 4: {
      // lanes 0-3 and 8-11 of a row read four lanes up (row_shl:4), the others four lanes down (row_shr:4)
      const int t = __builtin_amdgcn_update_dpp(x, x, 0x104, 0xF, 0x5, false);
      return (uint32_t)__builtin_amdgcn_update_dpp(t, x, 0x114, 0xF, 0xA, false);
    }
    case 8: return (uint32_t)__builtin_amdgcn_update_dpp(x, x, 0x128, 0xF, 0xF, false);   // row_ror:8
    default: return (uint32_t)__shfl_xor(x, m);
  }
}
__device__ __forceinline__ uint64_t shfl_xor_u64(uint64_t v, int m) {
  return ((uint64_t)xor_lanes_u32((uint32_t)(v >> 32), m) << 32) | xor_lanes_u32((uint32_t)v, m);
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

// The scoring kernel leaves one key per (query, document).  A wavefront walks its share of a workgroup's
// documents 256 at a time (four coalesced loads in flight per lane).  Documents that cannot enter the wavefront's
// top-k (composite not above the k-th best so far) are dropped by a ballot; the rest queue in LDS and are
// sorted and merged 64 at a time, so the bitonic network runs a few times per wavefront, not once per batch.
constexpr int kLoadsPerLane = 4;

__global__ __launch_bounds__(kWaves * 64) void doc_topk_kernel(const uint32_t* __restrict__ doc_key, int32_t n_docs,
                                                               int32_t topk, uint64_t* __restrict__ cand) {
  __shared__ uint64_t pend[kWaves][128];
  __shared__ uint64_t lists[kWaves][64];
  const int b = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t* key = doc_key + (int64_t)b * n_docs;
  const int d_begin = blockIdx.x * kTopkDocsPerBlock;
  const int d_end = min(d_begin + kTopkDocsPerBlock, n_docs);
  uint64_t* queue = pend[wave];

  uint64_t best = 0, thr = 0;
  int n_pend = 0;
  auto flush = [&](int take_from, int count) {      // sort `count` (<= 64) queued composites and merge them
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    uint64_t x = lane < count ? queue[take_from + lane] : 0;
    x = wave_sort_desc(x, lane);
    best = wave_merge_desc(best, x, lane);
    thr = shfl_u64(best, topk - 1);
  };

  for (int base = d_begin + wave * 64 * kLoadsPerLane; base < d_end; base += kWaves * 64 * kLoadsPerLane) {   // wave-uniform
    uint32_t kv[kLoadsPerLane];
#pragma unroll
    for (int u = 0; u < kLoadsPerLane; ++u) {
      const int d = base + u * 64 + lane;
      kv[u] = d < d_end ? __builtin_nontemporal_load(key + d) : 0u;
    }
#pragma unroll
    for (int u = 0; u < kLoadsPerLane; ++u) {
      const int d = base + u * 64 + lane;
      const uint64_t v = d < d_end ? ((uint64_t)kv[u] << 32) | (uint64_t)(0xffffffffu - (uint32_t)d) : 0;
      const bool in = v > thr;
      const uint64_t mask = __ballot(in);
      if (mask != 0) {
        const int pos = n_pend + __builtin_amdgcn_mbcnt_hi((uint32_t)(mask >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)mask, 0));
        if (in) queue[pos] = v;
        n_pend += __builtin_popcountll(mask);
        if (n_pend >= 64) {
          n_pend -= 64;
          flush(n_pend, 64);
        }
      }
    }
  }
  flush(0, n_pend);
  lists[wave][lane] = best;
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int w = 1; w < kWaves; ++w) best = wave_merge_desc(best, lists[w][lane], lane);
    cand[((int64_t)b * gridDim.x + blockIdx.x) * kTopkMax + lane] = best;
  }
}

constexpr int kMergeWaves = 4;

__global__ __launch_bounds__(kMergeWaves * 64) void merge_topk_kernel(const uint64_t* __restrict__ cand, int32_t blocks,
                                                                      const int64_t* __restrict__ doc_global_id, float mul,
                                                                      int32_t topk, float* __restrict__ scores_out,
                                                                      int32_t* __restrict__ doc_out,
                                                                      int64_t* __restrict__ doc_global_out) {
  __shared__ uint64_t lists[kMergeWaves][64];
  const int b = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  uint64_t best = 0;
  const uint64_t* mine = cand + (int64_t)b * blocks * kTopkMax + lane;
  for (int i = wave; i < blocks; i += 4 * kMergeWaves) {   // four lists in flight: the loads do not wait on the merges
    uint64_t x[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) x[u] = i + u * kMergeWaves < blocks ? mine[(int64_t)(i + u * kMergeWaves) * kTopkMax] : 0;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + u * kMergeWaves < blocks) best = wave_merge_desc(best, x[u], lane);
  }
  lists[wave][lane] = best;
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int w = 1; w < kMergeWaves; ++w) best = wave_merge_desc(best, lists[w][lane], lane);
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

namespace {

int route_topk_impl(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B, int32_t S,
                    int32_t Hq, int32_t mode, float scale, int32_t topk, float* scores_out, int32_t* doc_out,
                    int64_t* doc_global_out, void* workspace, size_t workspace_bytes, void* stream, const char* who,
                    const GatherJob* job, bool* job_taken) {
  MSA_REQUIRE(scores_out && doc_out, "%s: null output", who);
  MSA_REQUIRE(topk > 0 && topk <= kTopkMax, "%s: topk=%d out of range (1..%d)", who, topk, kTopkMax);
  RouteWorkspace w;
  float mul;
  hipStream_t st = as_stream(stream);
  int rc = route_scores_to_keys(bank, layer, q, qmask_u8, B, S, Hq, mode, scale, true, workspace, workspace_bytes, st, &w,
                                &mul, who, job, job_taken);
  if (rc != MSA_OK) return rc;
  char* ws = static_cast<char*>(workspace);
  const uint32_t* key = reinterpret_cast<const uint32_t*>(ws + w.off_key);
  uint64_t* cand = reinterpret_cast<uint64_t*>(ws + w.off_cand);
  dim3 grid((unsigned)w.topk_blocks, (unsigned)B);
  doc_topk_kernel<<<grid, kWaves * 64, 0, st>>>(key, (int32_t)bank->n_docs, topk, cand);
  MSA_LAUNCH_CHECK();
  merge_topk_kernel<<<B, kMergeWaves * 64, 0, st>>>(cand, w.topk_blocks, bank->doc_global_id_dev, mul, topk, scores_out, doc_out,
                                      doc_global_out);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

// keys of the per-chunk scores [B, C] -> keys of each document's mean over its chunks [B, n_docs]; a query whose
// chunk keys are 0 (no scored token) keeps 0.  One thread per (query, document).
__global__ void doc_mean_kernel(const uint32_t* __restrict__ chunk_key, const int32_t* __restrict__ doc_chunk_off,
                                int64_t C, int32_t n_docs, uint32_t* __restrict__ doc_key) {
  const int d = blockIdx.x * blockDim.x + threadIdx.x, b = blockIdx.y;
  if (d >= n_docs) return;
  const int c0 = doc_chunk_off[d], c1 = doc_chunk_off[d + 1];
  float sum = 0.f;
  bool none = c1 <= c0;
  for (int c = c0; c < c1; ++c) {
    const uint32_t k = chunk_key[(int64_t)b * C + c];
    if (k == 0) none = true;
    else sum += key_to_f32(k);
  }
  doc_key[(int64_t)b * n_docs + d] = none ? 0u : f32_to_key(sum / (float)(c1 - c0));
}

}  // namespace

extern "C" int msa_route_topk_reduce(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B,
                                     int32_t S, int32_t Hq, int32_t mode, float scale, int32_t query_reduce,
                                     int32_t chunk_reduce, int32_t topk, float* scores_out, int32_t* doc_out,
                                     int64_t* doc_global_out, void* workspace, size_t workspace_bytes, void* stream) {
  const char* who = "msa_route_topk_reduce";
  MSA_REQUIRE(chunk_reduce == MSA_CHUNK_MAX || chunk_reduce == MSA_CHUNK_MEAN, "%s: bad chunk reduction %d", who, chunk_reduce);
  MSA_REQUIRE(scores_out && doc_out, "%s: null output", who);
  MSA_REQUIRE(topk > 0 && topk <= kTopkMax, "%s: topk=%d out of range (1..%d)", who, topk, kTopkMax);
  MSA_REQUIRE(bank != nullptr, "%s: null bank", who);
  RouteWorkspace w;
  float mul;
  hipStream_t st = as_stream(stream);
  const bool doc_max = chunk_reduce == MSA_CHUNK_MAX;
  // (chunk mean: the scan leaves one key per (query, chunk); the per-document keys go behind that plane)
  int rc = route_scores_to_keys(bank, layer, q, qmask_u8, B, S, Hq, mode, scale, doc_max, workspace, workspace_bytes, st, &w,
                                &mul, who, nullptr, nullptr, query_reduce, doc_max ? 0 : bank->n_docs);
  if (rc != MSA_OK) return rc;
  char* ws = static_cast<char*>(workspace);
  const uint32_t* key = reinterpret_cast<const uint32_t*>(ws + w.off_key);
  if (!doc_max) {
    uint32_t* doc_key = reinterpret_cast<uint32_t*>(ws + w.off_key) + (size_t)B * bank->C;
    const dim3 mgrid((unsigned)((bank->n_docs + 255) / 256), (unsigned)B);
    doc_mean_kernel<<<mgrid, 256, 0, st>>>(key, bank->doc_chunk_off_dev, bank->C, (int32_t)bank->n_docs, doc_key);
    MSA_LAUNCH_CHECK();
    key = doc_key;
  }
  uint64_t* cand = reinterpret_cast<uint64_t*>(ws + w.off_cand);
  dim3 grid((unsigned)w.topk_blocks, (unsigned)B);
  doc_topk_kernel<<<grid, kWaves * 64, 0, st>>>(key, (int32_t)bank->n_docs, topk, cand);
  MSA_LAUNCH_CHECK();
  merge_topk_kernel<<<B, kMergeWaves * 64, 0, st>>>(cand, w.topk_blocks, bank->doc_global_id_dev, mul, topk, scores_out, doc_out,
                                      doc_global_out);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

extern "C" int msa_route_topk(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B,
                              int32_t S, int32_t Hq, int32_t mode, float scale, int32_t topk, float* scores_out,
                              int32_t* doc_out, int64_t* doc_global_out, void* workspace, size_t workspace_bytes,
                              void* stream) {
  return route_topk_impl(bank, layer, q, qmask_u8, B, S, Hq, mode, scale, topk, scores_out, doc_out, doc_global_out,
                         workspace, workspace_bytes, stream, "msa_route_topk", nullptr, nullptr);
}

// Routing of one layer with the K / V gather of an earlier selection inside the same launch: one workgroup of the
// scan copies while the others score.  When the scan's form cannot carry the copy (few query rows, fp32) the gather's
// own kernels run on the same stream first; the results are the same either way.
extern "C" int msa_route_topk_gather(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B,
                                     int32_t S, int32_t Hq, int32_t mode, float scale, int32_t topk, float* scores_out,
                                     int32_t* doc_out, int64_t* doc_global_out, void* workspace,
                                     size_t workspace_bytes, int32_t gather_layer, const int32_t* gather_doc_sel,
                                     int32_t gather_B, int32_t gather_k, void* k_out, void* v_out,
                                     int64_t out_capacity_chunks, int32_t* cu_sel, void* gather_workspace,
                                     size_t gather_workspace_bytes, void* stream) {
  const char* who = "msa_route_topk_gather";
  MSA_REQUIRE(bank && gather_doc_sel && k_out && v_out && cu_sel && gather_workspace, "%s: null pointer", who);
  MSA_REQUIRE(gather_B > 0 && gather_B <= 8192 && gather_k > 0 && gather_k <= 64, "%s: gather B=%d k=%d out of range", who,
              gather_B, gather_k);
  MSA_REQUIRE(gather_layer >= 0 && gather_layer < bank->n_layers, "%s: gather layer %d out of range", who, gather_layer);
  MSA_REQUIRE(out_capacity_chunks > 0, "%s: empty gather output", who);
  if (!bank->k_host[gather_layer] || !bank->v_host[gather_layer]) {
    msa_set_error("%s: layer %d has no host K / V set", who, gather_layer);
    return MSA_ESTATE;
  }
  if (gather_workspace_bytes < msa_gather_device_workspace_bytes(gather_B, gather_k)) {
    msa_set_error("%s: gather workspace of %zu bytes, need %zu", who, gather_workspace_bytes,
                  msa_gather_device_workspace_bytes(gather_B, gather_k));
    return MSA_ESIZE;
  }
  GatherJob job{};
  job.doc_sel = gather_doc_sel;
  job.doc_chunk_off = bank->doc_chunk_off_dev;
  job.cu_sel = cu_sel;
  job.plan = static_cast<int32_t*>(gather_workspace);
  job.k_src = static_cast<const uint4*>(bank->k_host[gather_layer]);
  job.v_src = static_cast<const uint4*>(bank->v_host[gather_layer]);
  job.k_dst = static_cast<uint4*>(k_out);
  job.v_dst = static_cast<uint4*>(v_out);
  job.capacity_rows = out_capacity_chunks;
  job.n_docs = (int32_t)bank->n_docs;
  job.B = gather_B;
  job.k = gather_k;
  job.dedup = gather_B > 1 && gather_B * gather_k <= msa_gather::kDedupMaxEntries ? 1 : 0;
  job.row_vecs = (int32_t)((size_t)bank->Hkv * bank->D * elem_bytes(bank->dtype) / 16);
  job.active = 1;
  bool taken = false;
  // the scan's form is known only inside; if it cannot carry the job the gather runs by itself, in front of the scan
  // (probed with the same routing arguments: the decision depends on the query rows and the dtype alone)
  const bool fused = bank->dtype == MSA_BF16 && (int64_t)B * ((S + 31) / 32 * 32) > 128;
  if (!fused) {
    int rc = msa_gather_kv_device(bank, gather_layer, gather_doc_sel, gather_B, gather_k, k_out, v_out, out_capacity_chunks,
                                  cu_sel, gather_workspace, gather_workspace_bytes, stream);
    if (rc != MSA_OK) return rc;
  }
  int rc = route_topk_impl(bank, layer, q, qmask_u8, B, S, Hq, mode, scale, topk, scores_out, doc_out, doc_global_out,
                           workspace, workspace_bytes, stream, who, fused ? &job : nullptr, &taken);
  if (rc != MSA_OK) return rc;
  if (fused && !taken) {
    msa_set_error("%s: internal: the scan did not take the gather", who);
    return MSA_ESTATE;
  }
  return MSA_OK;
}

// ------------------------------------------------------------------------------------------
// msa_route_topk without a workspace argument and without any allocation: the scratch (pre-summed queries, row
// masks, one key per (query, document), candidate lists) lives in a device array of this code object.  Every
// device the library runs on holds its own copy of the array at its own address, looked up once per device.
// ------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[MSA_ROUTE_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
void* g_scratch_ptr[kMaxDevices] = {};

// Address of the current device's copy of `scratch` (the array's name is only a host-side handle).
int scratch_of_current_device(void** out) {
  int dev = -1;
  MSA_HIP(hipGetDevice(&dev));
  MSA_REQUIRE(dev >= 0 && dev < kMaxDevices, "msa_route_topk_static: device %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    MSA_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    MSA_REQUIRE(p != nullptr && ((uintptr_t)p & 255) == 0, "msa_route_topk_static: bad scratch address");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return MSA_OK;
}

}  // namespace

extern "C" int msa_route_topk_static(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8,
                                     int32_t B, int32_t S, int32_t Hq, int32_t mode, float scale, int32_t topk,
                                     float* scores_out, int32_t* doc_out, int64_t* doc_global_out, void* stream) {
  MSA_REQUIRE(bank != nullptr, "msa_route_topk_static: null bank");
  MSA_REQUIRE(B > 0 && S > 0 && Hq > 0, "msa_route_topk_static: B=%d S=%d Hq=%d", B, S, Hq);
  const size_t need = route_workspace_layout(B, S, bank->Hkv, bank->D, bank->n_docs, bank->n_docs, bank->dtype).bytes;
  if (need > (size_t)MSA_ROUTE_STATIC_SCRATCH_BYTES) {
    msa_set_error("msa_route_topk_static: B=%d x S=%d queries over %lld documents need %zu bytes of scratch, the "
                  "built-in buffer holds %d; use msa_route_topk with a workspace", B, S, (long long)bank->n_docs,
                  need, MSA_ROUTE_STATIC_SCRATCH_BYTES);
    return MSA_ESIZE;
  }
  int dev = -1;
  MSA_HIP(hipGetDevice(&dev));
  MSA_REQUIRE(dev == bank->device, "msa_route_topk_static: bank lives on device %d, current device is %d", bank->device, dev);
  void* ws = nullptr;
  const int rc = scratch_of_current_device(&ws);
  if (rc != MSA_OK) return rc;
  // every byte of the scratch a call reads is written by that call's own kernels first (the prologue writes the
  // queries and all mask words and clears the key plane; the select kernel writes every candidate list)
  return msa_route_topk(bank, layer, q, qmask_u8, B, S, Hq, mode, scale, topk, scores_out, doc_out, doc_global_out, ws,
                        MSA_ROUTE_STATIC_SCRATCH_BYTES, stream);
}
