// Internal contract between route_score.hip (scores -> chunk keys) and topk.hip (keys -> top-k).
#pragma once
#include "common.h"

constexpr int kTopkMax = 64;          // width of every candidate list (one wavefront)
constexpr int kTopkDocsPerBlock = 2048;   // documents per top-k workgroup: 43 workgroups per query at 87k documents

// A K / V gather (msa_gather_kv_device's work) that rides along with a routing scan: one workgroup of the scan's launch
// runs it while the others score.  active = 0: none.
struct GatherJob {
  const int32_t* doc_sel;        // [B, k] selected documents (device)
  const int32_t* doc_chunk_off;  // bank table (device)
  int32_t* cu_sel;               // [B + 1] out
  int32_t* plan;                 // [B * k][4] scratch
  const uint4* k_src;            // pinned host K / V of the gathered layer
  const uint4* v_src;
  uint4* k_dst;                  // [capacity_rows, Hkv, D] out
  uint4* v_dst;
  int64_t capacity_rows;
  int32_t n_docs, B, k, dedup, row_vecs, active;
};

struct RouteWorkspace {
  int32_t S_pad;        // query tokens padded to a multiple of 32 (one MFMA row block never spans two queries)
  int32_t M_rows;       // B * S_pad
  int32_t topk_blocks;  // candidate lists per query
  int32_t mask_words;   // words of the scored-row bitmask, padded to whole M tiles
  size_t off_qs;        // pre-summed queries [M_rows, Hkv * D]
  size_t off_row_bits;  // scored-row bitmask, one uint32 per 32 rows
  size_t off_key;       // uint32 [B, n_docs] (routing) or [B, C] (chunk scores): order-preserving keys of the unscaled scores
  size_t off_cand;      // uint64 [B, topk_blocks, kTopkMax] sorted candidates
  size_t off_sched;     // tile pool words of the persistent scan (counter cleared by the prologue kernel)
  size_t off_collapsed; // fp32 [B, Hkv * D] + int32 [B]: a query collapsed to one row (mean / last over its tokens), tokens that counted
  size_t bytes;
};

static inline int32_t topk_blocks_for(int64_t n_docs) {
  return (int32_t)((n_docs + kTopkDocsPerBlock - 1) / kTopkDocsPerBlock);
}

RouteWorkspace route_workspace_layout(int32_t B, int32_t S, int32_t Hkv, int32_t D, int64_t plane_cols, int64_t n_docs,
                                      int32_t dtype);

// query_reduce: MSA_QUERY_*; extra_plane_cols: words per query reserved behind the key plane (the per-document keys
// of the chunk-mean reduction).
// Runs prologue + scoring GEMM on `st`; on success the keys (per document with doc_max, else per chunk) sit at
// layout_out->off_key and score = key_to_f32(key) * (*mul_out); key 0 = nothing scored.
// `job`: an optional gather to run inside the scan's launch; *job_taken tells whether the launch form could carry it
// (only the large-tile form can; the caller runs the gather's own kernels otherwise).
int route_scores_to_keys(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B,
                         int32_t S, int32_t Hq, int32_t mode, float scale, bool doc_max, void* workspace,
                         size_t workspace_bytes, hipStream_t st, RouteWorkspace* layout_out, float* mul_out,
                         const char* who, const GatherJob* job = nullptr, bool* job_taken = nullptr,
                         int32_t query_reduce = MSA_QUERY_MAX, int64_t extra_plane_cols = 0);

// flash_attn.hip: registers and scratch bytes of the loaded wide flash-attention kernel (a diagnostic)
int flash_wide_kernel_resources(int* num_regs, int* scratch_bytes);
