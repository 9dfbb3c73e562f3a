// Internal contract between route_score.hip (scores -> chunk keys) and topk.hip (keys -> top-k).
#pragma once
#include "common.h"

constexpr int kTopkMax = 64;          // width of every candidate list (one wavefront)
constexpr int kTopkDocsPerBlock = 2048;   // documents per top-k workgroup: 43 workgroups per query at 87k documents

struct RouteWorkspace {
  int32_t S_pad;        // query tokens padded to a multiple of 32 (one MFMA row block never spans two queries)
  int32_t M_rows;       // B * S_pad
  int32_t topk_blocks;  // candidate lists per query
  int32_t mask_words;   // words of the scored-row bitmask, padded to whole M tiles
  size_t off_qs;        // pre-summed queries [M_rows, Hkv * D]
  size_t off_row_bits;  // scored-row bitmask, one uint32 per 32 rows
  size_t off_key;       // uint32 [B, n_docs] (routing) or [B, C] (chunk scores): order-preserving keys of the unscaled scores
  size_t off_cand;      // uint64 [B, topk_blocks, kTopkMax] sorted candidates
  size_t bytes;
};

static inline int32_t topk_blocks_for(int64_t n_docs) {
  return (int32_t)((n_docs + kTopkDocsPerBlock - 1) / kTopkDocsPerBlock);
}

RouteWorkspace route_workspace_layout(int32_t B, int32_t S, int32_t Hkv, int32_t D, int64_t plane_cols, int64_t n_docs,
                                      int32_t dtype);

// Runs prologue + scoring GEMM on `st`; on success the keys (per document with doc_max, else per chunk) sit at
// layout_out->off_key and score = key_to_f32(key) * (*mul_out); key 0 = nothing scored.
int route_scores_to_keys(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B,
                         int32_t S, int32_t Hq, int32_t mode, float scale, bool doc_max, void* workspace,
                         size_t workspace_bytes, hipStream_t st, RouteWorkspace* layout_out, float* mul_out,
                         const char* who);
