// Gather of the selected documents' pooled K / V from pinned host memory.
// A document's chunks are contiguous rows of the chunk-major bank, so every document — and every
// run of bank-adjacent documents — is one hipMemcpyAsync per tensor on the caller's copy stream.
// A document picked by several samples of the batch crosses the host link once: later samples copy its
// rows from the first sample's segment on the device (the batch-wide unique() of src/msa_service.py:1214).
#include <algorithm>
#include <unordered_map>
#include <vector>

#include "gather_device.h"

namespace {

// Sorted unique valid documents of sample b; returns false on an out-of-range index.
bool sample_docs(const msa_bank* bank, const int32_t* sel, int32_t k, std::vector<int32_t>& docs) {
  docs.clear();
  for (int32_t j = 0; j < k; ++j) {
    const int32_t d = sel[j];
    if (d < 0) continue;
    if (d >= bank->n_docs) return false;
    docs.push_back(d);
  }
  std::sort(docs.begin(), docs.end());
  docs.erase(std::unique(docs.begin(), docs.end()), docs.end());
  return true;
}

}  // namespace

extern "C" int msa_gather_plan(const msa_bank* bank, const int32_t* doc_sel_host, int32_t B, int32_t k,
                               int64_t* cu_sel_host) {
  MSA_REQUIRE(bank && doc_sel_host && cu_sel_host, "msa_gather_plan: null pointer");
  MSA_REQUIRE(B > 0 && k > 0, "msa_gather_plan: B=%d k=%d", B, k);
  std::vector<int32_t> docs;
  cu_sel_host[0] = 0;
  for (int32_t b = 0; b < B; ++b) {
    MSA_REQUIRE(sample_docs(bank, doc_sel_host + (int64_t)b * k, k, docs),
                "msa_gather_plan: sample %d selects a document outside [0, %lld)", b, (long long)bank->n_docs);
    int64_t n = 0;
    for (int32_t d : docs) n += bank->doc_chunk_off_host[d + 1] - bank->doc_chunk_off_host[d];
    cu_sel_host[b + 1] = cu_sel_host[b] + n;
  }
  return MSA_OK;
}

extern "C" int msa_gather_kv(const msa_bank* bank, int32_t layer, const int32_t* doc_sel_host, int32_t B, int32_t k,
                             void* k_out, void* v_out, int64_t out_capacity_chunks, void* copy_stream) {
  MSA_REQUIRE(bank && doc_sel_host, "msa_gather_kv: null pointer");
  MSA_REQUIRE(B > 0 && k > 0, "msa_gather_kv: B=%d k=%d", B, k);
  MSA_REQUIRE(layer >= 0 && layer < bank->n_layers, "msa_gather_kv: layer %d out of range", layer);
  if (!bank->k_host[layer] || !bank->v_host[layer]) {
    msa_set_error("msa_gather_kv: layer %d has no host K / V set", layer);
    return MSA_ESTATE;
  }
  const size_t row_bytes = (size_t)bank->Hkv * bank->D * elem_bytes(bank->dtype);
  const char* ksrc = static_cast<const char*>(bank->k_host[layer]);
  const char* vsrc = static_cast<const char*>(bank->v_host[layer]);
  char* kdst = static_cast<char*>(k_out);
  char* vdst = static_cast<char*>(v_out);
  hipStream_t st = as_stream(copy_stream);

  // validate everything before the first copy is enqueued
  std::vector<int32_t> docs;
  int64_t total = 0;
  for (int32_t b = 0; b < B; ++b) {
    MSA_REQUIRE(sample_docs(bank, doc_sel_host + (int64_t)b * k, k, docs),
                "msa_gather_kv: sample %d selects a document outside [0, %lld)", b, (long long)bank->n_docs);
    for (int32_t d : docs) total += bank->doc_chunk_off_host[d + 1] - bank->doc_chunk_off_host[d];
  }
  if (total > out_capacity_chunks) {
    msa_set_error("msa_gather_kv: %lld chunks selected, output holds %lld", (long long)total,
                  (long long)out_capacity_chunks);
    return MSA_ESIZE;
  }
  MSA_REQUIRE(total == 0 || (k_out && v_out), "msa_gather_kv: null output");

  int64_t out_row = 0;
  std::unordered_map<int32_t, int64_t> first_row;        // document -> output row of its first copy in this batch
  for (int32_t b = 0; b < B; ++b) {
    sample_docs(bank, doc_sel_host + (int64_t)b * k, k, docs);
    size_t i = 0;
    while (i < docs.size()) {
      const int64_t c0 = bank->doc_chunk_off_host[docs[i]];
      auto seen = first_row.find(docs[i]);
      if (seen != first_row.end()) {                     // fetched for an earlier sample: device-to-device
        const int64_t n = bank->doc_chunk_off_host[docs[i] + 1] - c0;
        const size_t bytes = (size_t)n * row_bytes;
        MSA_HIP(hipMemcpyAsync(kdst + out_row * row_bytes, kdst + seen->second * row_bytes, bytes,
                               hipMemcpyDeviceToDevice, st));
        MSA_HIP(hipMemcpyAsync(vdst + out_row * row_bytes, vdst + seen->second * row_bytes, bytes,
                               hipMemcpyDeviceToDevice, st));
        out_row += n;
        ++i;
        continue;
      }
      size_t j = i;                                      // bank-adjacent documents not seen before: one run
      first_row.emplace(docs[i], out_row);
      while (j + 1 < docs.size() && docs[j + 1] == docs[j] + 1 && first_row.find(docs[j + 1]) == first_row.end()) {
        ++j;
        first_row.emplace(docs[j], out_row + (bank->doc_chunk_off_host[docs[j]] - c0));
      }
      const int64_t c1 = bank->doc_chunk_off_host[docs[j] + 1];
      const size_t bytes = (size_t)(c1 - c0) * row_bytes;
      MSA_HIP(hipMemcpyAsync(kdst + out_row * row_bytes, ksrc + c0 * row_bytes, bytes, hipMemcpyHostToDevice, st));
      MSA_HIP(hipMemcpyAsync(vdst + out_row * row_bytes, vsrc + c0 * row_bytes, bytes, hipMemcpyHostToDevice, st));
      out_row += c1 - c0;
      i = j + 1;
    }
  }
  return MSA_OK;
}

// ------------------------------------------------------------------------------------------
// Device-side gather: no ids on the host, no per-document copies.  A one-workgroup planning
// kernel sorts and de-duplicates each sample's selection (one wavefront per sample, bitonic
// network over the <= 64 picks), prefix-sums the chunk counts into cu_sel and emits one
// (source chunk, rows, destination row, device source row) entry per kept document; a copy kernel
// then pulls the rows straight out of the pinned host bank (the pointers are device-visible) with
// 16-byte loads.  A document that an earlier sample of the batch also picked is not read from the host
// again: its entry names the earlier copy's rows and a second launch copies them on the device.
// ------------------------------------------------------------------------------------------
namespace {

constexpr int kPlanWaves = 4;
using msa_gather::kPlanInts;
using msa_gather::kDedupMaxEntries;
using msa_gather::kCopyRowLanes;

__global__ __launch_bounds__(kPlanWaves * 64) void gather_plan_kernel(const int32_t* __restrict__ doc_sel,
                                                                      const int32_t* __restrict__ doc_chunk_off,
                                                                      int32_t n_docs, int32_t B, int32_t k,
                                                                      int32_t capacity_rows, int32_t dedup,
                                                                      int32_t* __restrict__ cu_sel,
                                                                      int32_t* __restrict__ plan /* [B*k][4] */) {
  extern __shared__ int32_t smem[];
  msa_gather::plan_body(doc_sel, doc_chunk_off, n_docs, B, k, capacity_rows, dedup, cu_sel, plan, smem, (int)threadIdx.x,
                        (int)blockDim.x);
}

// grid.x strides over plan entries, grid.y and the workgroup's groups of 128 lanes over an entry's rows.
// Few workgroups: PCIe reads are slow to return and a compute unit's memory pipeline serves its wavefronts in order, so
// every compute unit that hosts a copy wavefront slows the scoring workgroup beside it.  32 workgroups keep 128 KB in
// flight, enough for the link, and leave the other compute units alone (scan under the copy 5.81 ms against 6.15 ms
// with 2048 workgroups, 5.75 ms without a copy).
constexpr int kCopyGridX = 16, kCopyGridY = 2, kCopyThreads = 128;
template <bool kFromDevice>
__global__ __launch_bounds__(1024) void gather_copy_kernel(const uint4* __restrict__ k_src, const uint4* __restrict__ v_src,
                                                          const int32_t* __restrict__ plan, int32_t n_entries,
                                                          int32_t row_vecs, int64_t capacity_rows, uint4* k_dst,
                                                          uint4* v_dst) {
  const int groups = (int)blockDim.x / kCopyRowLanes;
  msa_gather::copy_body<kFromDevice>(k_src, v_src, plan, n_entries, row_vecs, capacity_rows, k_dst, v_dst, (int)blockIdx.x,
                                     (int)gridDim.x, (int)blockIdx.y * groups + (int)threadIdx.x / kCopyRowLanes,
                                     (int)gridDim.y * groups, (int)threadIdx.x % kCopyRowLanes);
}

}  // namespace

extern "C" size_t msa_gather_device_workspace_bytes(int32_t B, int32_t k) {
  return B > 0 && k > 0 ? align_up((size_t)B * k * kPlanInts * sizeof(int32_t), 256) : 0;
}

extern "C" int msa_gather_kv_device(const msa_bank* bank, int32_t layer, const int32_t* doc_sel, int32_t B, int32_t k,
                                    void* k_out, void* v_out, int64_t out_capacity_chunks, int32_t* cu_sel,
                                    void* workspace, size_t workspace_bytes, void* stream) {
  MSA_REQUIRE(bank && doc_sel && k_out && v_out && cu_sel && workspace, "msa_gather_kv_device: null pointer");
  MSA_REQUIRE(B > 0 && B <= 8192 && k > 0 && k <= 64, "msa_gather_kv_device: B=%d k=%d out of range", B, k);
  MSA_REQUIRE(layer >= 0 && layer < bank->n_layers, "msa_gather_kv_device: layer %d out of range", layer);
  MSA_REQUIRE(out_capacity_chunks > 0, "msa_gather_kv_device: empty output");
  if (!bank->k_host[layer] || !bank->v_host[layer]) {
    msa_set_error("msa_gather_kv_device: layer %d has no host K / V set", layer);
    return MSA_ESTATE;
  }
  if (workspace_bytes < msa_gather_device_workspace_bytes(B, k)) {
    msa_set_error("msa_gather_kv_device: workspace of %zu bytes, need %zu", workspace_bytes,
                  msa_gather_device_workspace_bytes(B, k));
    return MSA_ESIZE;
  }
  hipStream_t st = as_stream(stream);
  int32_t* plan = static_cast<int32_t*>(workspace);
  const int32_t dedup = B > 1 && B * k <= kDedupMaxEntries ? 1 : 0;
  const int32_t cap32 = (int32_t)std::min<int64_t>(out_capacity_chunks, 0x7fffffff);
  const size_t lds = msa_gather::plan_lds_ints(B, k, dedup) * sizeof(int32_t);
  gather_plan_kernel<<<1, kPlanWaves * 64, lds, st>>>(doc_sel, bank->doc_chunk_off_dev, (int32_t)bank->n_docs, B, k,
                                                      cap32, dedup, cu_sel, plan);
  MSA_LAUNCH_CHECK();
  const int32_t row_vecs = (int32_t)((size_t)bank->Hkv * bank->D * elem_bytes(bank->dtype) / 16);
  dim3 grid((unsigned)std::min(B * k, kCopyGridX), kCopyGridY);
  gather_copy_kernel<false><<<grid, kCopyThreads, 0, st>>>(static_cast<const uint4*>(bank->k_host[layer]),
                                                  static_cast<const uint4*>(bank->v_host[layer]), plan, B * k, row_vecs,
                                                  out_capacity_chunks, static_cast<uint4*>(k_out),
                                                  static_cast<uint4*>(v_out));
  MSA_LAUNCH_CHECK();
  if (dedup) {
    gather_copy_kernel<true><<<grid, kCopyThreads, 0, st>>>(nullptr, nullptr, plan, B * k, row_vecs, out_capacity_chunks,
                                                   static_cast<uint4*>(k_out), static_cast<uint4*>(v_out));
    MSA_LAUNCH_CHECK();
  }
  return MSA_OK;
}
