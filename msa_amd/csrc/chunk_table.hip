// Chunk table of a packed block: two tiny kernels, no host synchronisation.
#include "common.h"

namespace {

constexpr int kScanThreads = 1024;

// One workgroup: exclusive scan of ceil(len_d / P) over all documents.
__global__ __launch_bounds__(kScanThreads) void doc_chunk_scan_kernel(const int32_t* __restrict__ doc_start,
                                                                      int32_t n_docs, int32_t P,
                                                                      int32_t* __restrict__ doc_chunk_off,
                                                                      int64_t* __restrict__ n_chunks_out) {
  __shared__ int32_t part[kScanThreads];
  const int tid = threadIdx.x;
  const int per = (n_docs + kScanThreads - 1) / kScanThreads;
  const int lo = min(tid * per, n_docs), hi = min(lo + per, n_docs);
  int32_t sum = 0;
  for (int d = lo; d < hi; ++d) sum += (doc_start[d + 1] - doc_start[d] + P - 1) / P;
  part[tid] = sum;
  __syncthreads();
  for (int off = 1; off < kScanThreads; off <<= 1) {   // Hillis-Steele inclusive scan
    int32_t add = tid >= off ? part[tid - off] : 0;
    __syncthreads();
    part[tid] += add;
    __syncthreads();
  }
  int32_t run = part[tid] - sum;
  for (int d = lo; d < hi; ++d) {
    doc_chunk_off[d] = run;
    run += (doc_start[d + 1] - doc_start[d] + P - 1) / P;
  }
  if (tid == kScanThreads - 1) {
    doc_chunk_off[n_docs] = part[tid];
    n_chunks_out[0] = part[tid];
  }
}

// One thread per document writes that document's chunk rows.
__global__ void chunk_fill_kernel(const int32_t* __restrict__ doc_start, const int32_t* __restrict__ doc_chunk_off,
                                  int32_t n_docs, int32_t P, int64_t chunk_cap, int32_t* __restrict__ chunk_start,
                                  int32_t* __restrict__ chunk_len, int32_t* __restrict__ chunk_doc) {
  const int d = blockIdx.x * blockDim.x + threadIdx.x;
  if (d >= n_docs) return;
  const int32_t s = doc_start[d], n = doc_start[d + 1] - s;
  const int32_t base = doc_chunk_off[d], nch = (n + P - 1) / P;
  for (int32_t j = 0; j < nch; ++j) {
    const int64_t c = (int64_t)base + j;
    if (c >= chunk_cap) return;
    chunk_start[c] = s + j * P;
    chunk_len[c] = min(P, n - j * P);
    chunk_doc[c] = d;
  }
}

}  // namespace

extern "C" int msa_chunk_table(const int32_t* doc_start, int32_t n_docs, int32_t P, int64_t chunk_cap,
                               int32_t* doc_chunk_off, int32_t* chunk_start, int32_t* chunk_len,
                               int32_t* chunk_doc, int64_t* n_chunks_out, void* stream) {
  MSA_REQUIRE(doc_start && doc_chunk_off && chunk_start && chunk_len && chunk_doc && n_chunks_out,
              "msa_chunk_table: null pointer");
  MSA_REQUIRE(n_docs > 0, "msa_chunk_table: n_docs=%d", n_docs);
  MSA_REQUIRE(P > 0, "msa_chunk_table: P=%d", P);
  MSA_REQUIRE(chunk_cap > 0, "msa_chunk_table: chunk_cap=%lld", (long long)chunk_cap);
  hipStream_t st = as_stream(stream);
  doc_chunk_scan_kernel<<<1, kScanThreads, 0, st>>>(doc_start, n_docs, P, doc_chunk_off, n_chunks_out);
  MSA_LAUNCH_CHECK();
  chunk_fill_kernel<<<(n_docs + 255) / 256, 256, 0, st>>>(doc_start, doc_chunk_off, n_docs, P, chunk_cap,
                                                          chunk_start, chunk_len, chunk_doc);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}
