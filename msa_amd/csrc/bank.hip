// Error plumbing and the memory-bank handle (host code only).
#include <stdarg.h>
#include <stdlib.h>
#include <string.h>

#include "common.h"

static thread_local char g_err[512] = "";

void msa_set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

extern "C" const char* msa_last_error(void) { return g_err; }
extern "C" int msa_abi_version(void) { return 1; }

extern "C" int msa_bank_create(msa_bank** out, int32_t n_layers, int64_t C, int32_t Hkv, int32_t D,
                               int32_t dtype, const int32_t* doc_chunk_off_host,
                               const int64_t* doc_global_id_host, int64_t n_docs) {
  MSA_REQUIRE(out != nullptr, "msa_bank_create: out is null");
  *out = nullptr;
  MSA_REQUIRE(n_layers > 0 && n_layers <= 4096, "msa_bank_create: n_layers=%d out of range", n_layers);
  MSA_REQUIRE(C > 0 && C < (int64_t)1 << 31, "msa_bank_create: C=%lld out of range", (long long)C);
  MSA_REQUIRE(n_docs > 0 && n_docs <= C && n_docs < (int64_t)1 << 31, "msa_bank_create: n_docs=%lld out of range (C=%lld)",
              (long long)n_docs, (long long)C);
  MSA_REQUIRE(D == kHeadDim, "msa_bank_create: head dim %d unsupported (need %d)", D, kHeadDim);
  MSA_REQUIRE(Hkv > 0 && Hkv <= 64, "msa_bank_create: Hkv=%d out of range", Hkv);
  MSA_REQUIRE(dtype == MSA_BF16 || dtype == MSA_F32, "msa_bank_create: bad dtype %d", dtype);
  MSA_REQUIRE(doc_chunk_off_host && doc_global_id_host, "msa_bank_create: null table");
  MSA_REQUIRE(doc_chunk_off_host[0] == 0, "msa_bank_create: doc_chunk_off[0] must be 0");
  for (int64_t d = 0; d < n_docs; ++d)
    MSA_REQUIRE(doc_chunk_off_host[d + 1] > doc_chunk_off_host[d],
                "msa_bank_create: document %lld has no chunks", (long long)d);
  MSA_REQUIRE(doc_chunk_off_host[n_docs] == C, "msa_bank_create: doc_chunk_off[n_docs]=%d != C=%lld",
              doc_chunk_off_host[n_docs], (long long)C);

  msa_bank* b = (msa_bank*)calloc(1, sizeof(msa_bank));
  MSA_REQUIRE(b != nullptr, "msa_bank_create: out of host memory");
  b->n_layers = n_layers; b->C = C; b->Hkv = Hkv; b->D = D; b->dtype = dtype; b->n_docs = n_docs;
  size_t off_bytes = (size_t)(n_docs + 1) * sizeof(int32_t), id_bytes = (size_t)n_docs * sizeof(int64_t);
  b->doc_chunk_off_host = (int32_t*)malloc(off_bytes);
  b->doc_global_id_host = (int64_t*)malloc(id_bytes);
  b->kr_dev = (const void**)calloc(n_layers, sizeof(void*));
  b->k_host = (const void**)calloc(n_layers, sizeof(void*));
  b->v_host = (const void**)calloc(n_layers, sizeof(void*));
  if (!b->doc_chunk_off_host || !b->doc_global_id_host || !b->kr_dev || !b->k_host || !b->v_host) {
    msa_bank_destroy(b);
    msa_set_error("msa_bank_create: out of host memory");
    return MSA_EINVAL;
  }
  memcpy(b->doc_chunk_off_host, doc_chunk_off_host, off_bytes);
  memcpy(b->doc_global_id_host, doc_global_id_host, id_bytes);
  hipError_t e = hipGetDevice(&b->device);
  if (e == hipSuccess) e = hipMalloc((void**)&b->doc_chunk_off_dev, off_bytes);
  if (e == hipSuccess) e = hipMalloc((void**)&b->doc_global_id_dev, id_bytes);
  if (e == hipSuccess) e = hipMemcpy(b->doc_chunk_off_dev, doc_chunk_off_host, off_bytes, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(b->doc_global_id_dev, doc_global_id_host, id_bytes, hipMemcpyHostToDevice);
  if (e == hipSuccess) {
    int32_t* chunk_doc = (int32_t*)malloc((size_t)C * sizeof(int32_t));
    if (chunk_doc == nullptr) {
      msa_bank_destroy(b);
      msa_set_error("msa_bank_create: out of host memory");
      return MSA_EINVAL;
    }
    for (int64_t d = 0; d < n_docs; ++d)
      for (int32_t c = doc_chunk_off_host[d]; c < doc_chunk_off_host[d + 1]; ++c) chunk_doc[c] = (int32_t)d;
    e = hipMalloc((void**)&b->chunk_doc_dev, (size_t)C * sizeof(int32_t));
    if (e == hipSuccess) e = hipMemcpy(b->chunk_doc_dev, chunk_doc, (size_t)C * sizeof(int32_t), hipMemcpyHostToDevice);
    free(chunk_doc);
  }
  if (e != hipSuccess) {
    msa_bank_destroy(b);
    msa_set_error("msa_bank_create: HIP error %s", hipGetErrorString(e));
    return MSA_EHIP;
  }
  *out = b;
  return MSA_OK;
}

extern "C" int msa_bank_set_layer(msa_bank* bank, int32_t layer, const void* kr_dev, const void* k_host,
                                  const void* v_host) {
  MSA_REQUIRE(bank != nullptr, "msa_bank_set_layer: null bank");
  MSA_REQUIRE(layer >= 0 && layer < bank->n_layers, "msa_bank_set_layer: layer %d out of range", layer);
  MSA_REQUIRE(kr_dev != nullptr, "msa_bank_set_layer: kr_dev is null");
  MSA_REQUIRE((k_host == nullptr) == (v_host == nullptr), "msa_bank_set_layer: k_host and v_host go together");
  MSA_REQUIRE(((uintptr_t)kr_dev & 15) == 0, "msa_bank_set_layer: kr_dev must be 16-byte aligned");
  bank->kr_dev[layer] = kr_dev;
  bank->k_host[layer] = k_host;
  bank->v_host[layer] = v_host;
  return MSA_OK;
}

extern "C" int msa_bank_destroy(msa_bank* b) {
  if (!b) return MSA_OK;
  if (b->doc_chunk_off_dev) (void)hipFree(b->doc_chunk_off_dev);
  if (b->doc_global_id_dev) (void)hipFree(b->doc_global_id_dev);
  if (b->chunk_doc_dev) (void)hipFree(b->chunk_doc_dev);
  free(b->doc_chunk_off_host);
  free(b->doc_global_id_host);
  free((void*)b->kr_dev);
  free((void*)b->k_host);
  free((void*)b->v_host);
  free(b);
  return MSA_OK;
}
