// Gather of the selected documents' pooled K / V from pinned host memory.
// A document's chunks are contiguous rows of the chunk-major bank, so every document — and every
// run of bank-adjacent documents — is one hipMemcpyAsync per tensor on the caller's copy stream.
// A document picked by several samples of the batch crosses the host link once: later samples copy its
// rows from the first sample's segment on the device (the batch-wide unique() of src/msa_service.py:1214).
#include <algorithm>
#include <unordered_map>
#include <vector>

#include "common.h"

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

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
constexpr int kPlanInts = 4;            // ints per plan entry
constexpr int kDedupMaxEntries = 2048;  // batch-wide de-duplication runs while B * k fits this many LDS slots
constexpr int32_t kNoDoc = 0x7fffffff;

__global__ __launch_bounds__(kPlanWaves * 64) void gather_plan_kernel(const int32_t* __restrict__ doc_sel,
                                                                      const int32_t* __restrict__ doc_chunk_off,
                                                                      int32_t n_docs, int32_t B, int32_t k,
                                                                      int32_t capacity_rows, int32_t dedup,
                                                                      int32_t* __restrict__ cu_sel,
                                                                      int32_t* __restrict__ plan /* [B*k][4] */) {
  extern __shared__ int32_t smem[];            // totals [B + 1] | sorted documents [B * k] | destination rows [B * k]
  int32_t* totals = smem;
  int32_t* s_doc = smem + (B + 1);
  int32_t* s_dst = s_doc + (dedup ? B * k : 0);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // pass 1 and 2 share this per-sample routine: sorted unique documents in lanes, chunk counts, in-sample offsets
  auto sample = [&](int b, int32_t& d_out, int32_t& n_out, int32_t& off_out) -> int32_t {
    int32_t d = kNoDoc;
    if (lane < k) {
      const int32_t x = doc_sel[(int64_t)b * k + lane];
      if (x >= 0 && x < n_docs) d = x;
    }
#pragma unroll
    for (int kk = 2; kk <= 64; kk <<= 1)
#pragma unroll
      for (int j = kk >> 1; j > 0; j >>= 1) {            // ascending bitonic sort
        const int32_t o = __shfl_xor(d, j);
        const bool asc = (lane & kk) == 0, lower = (lane & j) == 0;
        d = (lower == asc) ? min(d, o) : max(d, o);
      }
    const int32_t prev = __shfl_up(d, 1);
    const bool keep = d != kNoDoc && (lane == 0 || prev != d);
    int32_t n = keep ? doc_chunk_off[d + 1] - doc_chunk_off[d] : 0;
    int32_t incl = n;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int32_t t = __shfl_up(incl, o);
      if (lane >= o) incl += t;
    }
    d_out = keep ? d : -1; n_out = n; off_out = incl - n;
    return __shfl(incl, 63);
  };
  for (int b = wave; b < B; b += kPlanWaves) {
    int32_t d, n, off;
    const int32_t total = sample(b, d, n, off);
    if (lane == 0) totals[b + 1] = total;
  }
  if (threadIdx.x == 0) totals[0] = 0;
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t run = 0;
    for (int b = 0; b < B; ++b) { run += totals[b + 1]; totals[b + 1] = run; }
  }
  __syncthreads();
  // rows past the output's capacity are never written by the copy kernel: the prefix sums stop there too, so a
  // consumer of cu_sel never addresses a row that was not filled
  for (int i = threadIdx.x; i <= B; i += kPlanWaves * 64) cu_sel[i] = min(totals[i], capacity_rows);
  for (int b = wave; b < B; b += kPlanWaves) {
    int32_t d, n, off;
    sample(b, d, n, off);
    if (lane < k) {
      int32_t* e = plan + ((int64_t)b * k + lane) * kPlanInts;
      e[0] = d >= 0 ? doc_chunk_off[d] : 0;
      e[1] = n;
      e[2] = totals[b] + off;
      e[3] = -1;
      if (dedup) {                               // documents dropped as duplicates inside the sample sort last
        s_doc[b * k + lane] = d >= 0 ? d : kNoDoc;
        s_dst[b * k + lane] = totals[b] + off;
      }
    }
  }
  if (!dedup) return;                            // uniform over the workgroup
  __syncthreads();
  // an entry whose document an earlier sample also holds copies from that sample's rows instead of the host.
  // s_doc rows are ascending except that in-sample duplicates were replaced by kNoDoc in place, so the search
  // below is linear over the k slots (k <= 64).
  for (int i = threadIdx.x; i < B * k; i += kPlanWaves * 64) {
    const int32_t d = s_doc[i];
    if (d == kNoDoc) continue;
    const int b = i / k;
    int32_t from = -1;
    for (int b2 = 0; b2 < b && from < 0; ++b2)
      for (int j = 0; j < k; ++j)
        if (s_doc[b2 * k + j] == d) { from = s_dst[b2 * k + j]; break; }
    if (from >= 0) plan[(int64_t)i * kPlanInts + 3] = from;
  }
}

// grid.x = plan entry, grid.y = row group; 128 lanes move one row of K and of V per step.
// kFromDevice = false: entries without an earlier copy, rows read from the pinned host bank;
// kFromDevice = true: the others, rows read from the earlier copy inside the output itself.
// The kernel stays within 16 vector registers (rows travel through buffer resources, i.e. scalar addresses and one
// vector offset): a scoring workgroup of the routing scan takes 496 of a SIMD's 512, and only a wavefront that fits
// beside it runs under the scan instead of taking a compute unit's turn between two of its workgroups (the copy is
// PCIe-bound: it needs residency, not registers).
// Few workgroups: PCIe reads are slow to return and a compute unit's memory pipeline serves its wavefronts in order, so
// every compute unit that hosts a copy wavefront slows the scoring workgroup beside it.  32 workgroups keep 128 KB in
// flight, enough for the link, and leave the other compute units alone (scan under the copy 5.81 ms against 6.15 ms
// with 2048 workgroups, 5.75 ms without a copy).
constexpr int kCopyGridX = 16, kCopyGridY = 2, kCopyThreads = 128;
constexpr int kCopyRowLanes = 128;      // lanes that share a row (a 2 KB bf16 row is 128 lanes x 16 bytes)
template <bool kFromDevice>
__global__ __launch_bounds__(1024) void gather_copy_kernel(const uint4* __restrict__ k_src, const uint4* __restrict__ v_src,
                                                          const int32_t* __restrict__ plan, int32_t n_entries,
                                                          int32_t row_vecs, int64_t capacity_rows, uint4* k_dst,
                                                          uint4* v_dst) {
  const int row_bytes = row_vecs * 16;
  for (int ent = blockIdx.x; ent < n_entries; ent += gridDim.x) {
  const int32_t* e = plan + (int64_t)ent * kPlanInts;
  const int32_t n = e[1], dst0 = e[2], from = e[3];
  if ((from >= 0) != kFromDevice) continue;
  const int32_t src0 = kFromDevice ? from : e[0];
  for (int r = blockIdx.y * (blockDim.x / kCopyRowLanes) + threadIdx.x / kCopyRowLanes; r < n;
       r += gridDim.y * (blockDim.x / kCopyRowLanes)) {
    if ((int64_t)dst0 + r >= capacity_rows) break;
    if (kFromDevice && (int64_t)src0 + r >= capacity_rows) break;
    const uint4* ks = (kFromDevice ? k_dst : k_src) + ((int64_t)src0 + r) * row_vecs;
    const uint4* vs = (kFromDevice ? v_dst : v_src) + ((int64_t)src0 + r) * row_vecs;
    uint4* kd = k_dst + ((int64_t)dst0 + r) * row_vecs;
    uint4* vd = v_dst + ((int64_t)dst0 + r) * row_vecs;
    const __amdgpu_buffer_rsrc_t rks = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(ks), 0, row_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rvs = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(vs), 0, row_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rkd = __builtin_amdgcn_make_buffer_rsrc(kd, 0, row_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t rvd = __builtin_amdgcn_make_buffer_rsrc(vd, 0, row_bytes, 0x00020000);
    for (int off = (threadIdx.x % kCopyRowLanes) * 16; off < row_bytes; off += kCopyRowLanes * 16) {
      const u32x4_t a = __builtin_amdgcn_raw_buffer_load_b128(rks, off, 0, 0);
      const u32x4_t b = __builtin_amdgcn_raw_buffer_load_b128(rvs, off, 0, 0);
      __builtin_amdgcn_raw_buffer_store_b128(a, rkd, off, 0, 0);
      __builtin_amdgcn_raw_buffer_store_b128(b, rvd, off, 0, 0);
    }
  }
  }
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
  const size_t lds = (size_t)(B + 1 + (dedup ? 2 * B * k : 0)) * sizeof(int32_t);
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
