// Shared between attn.hip (split-KV VALU kernel, combine) and flash_attn.hip (MFMA kernels).
#pragma once
#include <algorithm>

#include "common.h"

constexpr int kMinSplitKeys = 256;   // fewest keys worth a workgroup of its own

// Splits of the key range: enough workgroups to fill the chip (about 1024) when there are few
// (query row, KV head) pairs, a single pass over the keys when there are many.  split_keys is a
// multiple of 64.
struct SplitPlan {
  int n_split;
  int split_keys;
};
static inline SplitPlan plan_splits_for(int64_t total_q, int32_t Hkv, int32_t max_kv, int target) {
  const int64_t pairs = std::max<int64_t>(1, total_q * Hkv);
  const int by_fill = (int)std::max<int64_t>(1, (target + pairs - 1) / pairs);
  const int by_size = std::max(1, (max_kv + kMinSplitKeys - 1) / kMinSplitKeys);
  const int n = std::min(by_fill, by_size);
  const int keys = ((max_kv + n - 1) / n + 63) / 64 * 64;
  return {(max_kv + keys - 1) / keys, keys};
}
// MFMA split kernel: about 1024 workgroups.
static inline SplitPlan plan_splits(int64_t total_q, int32_t Hkv, int32_t max_kv) {
  return plan_splits_for(total_q, Hkv, max_kv, 1024);
}
// VALU split kernel (decode): one workgroup per compute unit measured best (fewer, longer key streams); the
// kernel itself divides each sample's own length evenly over n_split.
static inline SplitPlan plan_splits_valu(int64_t total_q, int32_t Hkv, int32_t max_kv) {
  return plan_splits_for(total_q, Hkv, max_kv, 256);
}

// flash_attn.hip: bf16 partial pass over split `blockIdx.z` of the keys; writes un-normalised
// accumulators and (reference max, sum) pairs in the layout attn_combine_kernel reads.
int flash_attn_split_launch(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                            const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, float scale,
                            int32_t causal, SplitPlan plan, float* part_ml, float* part_acc, hipStream_t st);
