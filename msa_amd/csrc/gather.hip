// Gather of the selected documents' pooled K / V from pinned host memory (host code only).
// A document's chunks are contiguous rows of the chunk-major bank, so every document — and every
// run of bank-adjacent documents — is one hipMemcpyAsync per tensor on the caller's copy stream.
#include <algorithm>
#include <vector>

#include "common.h"

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
  for (int32_t b = 0; b < B; ++b) {
    sample_docs(bank, doc_sel_host + (int64_t)b * k, k, docs);
    size_t i = 0;
    while (i < docs.size()) {
      size_t j = i;
      while (j + 1 < docs.size() && docs[j + 1] == docs[j] + 1) ++j;   // bank-adjacent documents: one run
      const int64_t c0 = bank->doc_chunk_off_host[docs[i]], c1 = bank->doc_chunk_off_host[docs[j] + 1];
      const size_t bytes = (size_t)(c1 - c0) * row_bytes;
      MSA_HIP(hipMemcpyAsync(kdst + out_row * row_bytes, ksrc + c0 * row_bytes, bytes, hipMemcpyHostToDevice, st));
      MSA_HIP(hipMemcpyAsync(vdst + out_row * row_bytes, vsrc + c0 * row_bytes, bytes, hipMemcpyHostToDevice, st));
      out_row += c1 - c0;
      i = j + 1;
    }
  }
  return MSA_OK;
}
