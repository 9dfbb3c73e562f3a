// Device-side K / V gather, as functions a kernel calls with its own workgroup: the planning step (sort and
// de-duplicate each sample's selection, prefix-sum the chunk counts, one copy entry per kept document) and the copy
// step (rows out of the pinned host bank, or out of an earlier copy inside the output).  gather.hip wraps them in
// kernels of their own; the routing scan's kernel runs them in one of its workgroups while the others score
// (msa_route_topk_gather).
#pragma once
#include "common.h"

namespace msa_gather {

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kPlanInts = 4;            // ints per plan entry: source chunk, rows, destination row, device source row
constexpr int kDedupMaxEntries = 2048;  // batch-wide de-duplication runs while B * k fits this many LDS slots
constexpr int32_t kNoDoc = 0x7fffffff;
constexpr int kCopyRowLanes = 128;      // lanes that share a row (a 2 KB bf16 row is 128 lanes x 16 bytes)

// LDS ints the planning step needs
__host__ __device__ inline size_t plan_lds_ints(int32_t B, int32_t k, int32_t dedup) {
  return (size_t)(B + 1 + (dedup ? 2 * B * k : 0));
}

// Every thread of the workgroup calls this (it contains workgroup barriers); `smem` holds plan_lds_ints() ints.
// tid / nthreads: the calling workgroup's thread index and size (a multiple of 64).
__device__ __forceinline__ void plan_body(const int32_t* __restrict__ doc_sel, const int32_t* __restrict__ doc_chunk_off,
                                          int32_t n_docs, int32_t B, int32_t k, int32_t capacity_rows, int32_t dedup,
                                          int32_t* __restrict__ cu_sel, int32_t* __restrict__ plan /* [B*k][4] */,
                                          int32_t* smem, int tid, int nthreads) {
  int32_t* totals = smem;                       // totals [B + 1] | sorted documents [B * k] | destination rows [B * k]
  int32_t* s_doc = smem + (B + 1);
  int32_t* s_dst = s_doc + (dedup ? B * k : 0);
  const int lane = tid & 63, wave = tid >> 6, nwaves = nthreads >> 6;
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
  for (int b = wave; b < B; b += nwaves) {
    int32_t d, n, off;
    const int32_t total = sample(b, d, n, off);
    if (lane == 0) totals[b + 1] = total;
  }
  if (tid == 0) totals[0] = 0;
  __syncthreads();
  if (tid == 0) {
    int32_t run = 0;
    for (int b = 0; b < B; ++b) { run += totals[b + 1]; totals[b + 1] = run; }
  }
  __syncthreads();
  // rows past the output's capacity are never written by the copy step: the prefix sums stop there too, so a
  // consumer of cu_sel never addresses a row that was not filled
  for (int i = tid; i <= B; i += nthreads) cu_sel[i] = min(totals[i], capacity_rows);
  for (int b = wave; b < B; b += nwaves) {
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
  for (int i = tid; i < B * k; i += nthreads) {
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

// Copies the rows of plan entries ent0, ent0 + ent_step, ...; of an entry's rows, r0, r0 + r_step, ... (r0 and r_step
// are the same in all 128 lanes that share a row, lane_in_row tells them apart).
// kFromDevice = false: entries without an earlier copy, rows read from the pinned host bank;
// kFromDevice = true: the others, rows read from the earlier copy inside the output itself.
// kRows: rows whose loads are in flight together.  Rows travel through buffer resources (scalar addresses and one
// vector offset), so with kRows = 1 the copy stays within 16 vector registers and a wavefront of it fits beside the
// routing scan's workgroups on a SIMD; a workgroup that has a compute unit to itself takes more rows at a time, since
// a lone workgroup's rate over PCIe is the bytes it keeps in flight over the link's latency.
template <bool kFromDevice, int kRows = 1>
__device__ __forceinline__ void copy_body(const uint4* __restrict__ k_src, const uint4* __restrict__ v_src,
                                          const int32_t* __restrict__ plan, int32_t n_entries, int32_t row_vecs,
                                          int64_t capacity_rows, uint4* k_dst, uint4* v_dst, int ent0, int ent_step,
                                          int r0, int r_step, int lane_in_row) {
  const int row_bytes = row_vecs * 16;
  // Everything that names a row is the same in all lanes of a wavefront (128 lanes share a row).  Said so, the rows'
  // buffer resources are built in scalar registers; left as vector values every load and store sat in a loop that
  // reads the resource back lane by lane.
  const int r0s = __builtin_amdgcn_readfirstlane(r0), r_steps = __builtin_amdgcn_readfirstlane(r_step);
  for (int ent = ent0; ent < n_entries; ent += ent_step) {
    const int32_t* e = plan + (int64_t)ent * kPlanInts;
    const int32_t n = __builtin_amdgcn_readfirstlane(e[1]), dst0 = __builtin_amdgcn_readfirstlane(e[2]);
    const int32_t from = __builtin_amdgcn_readfirstlane(e[3]);
    if ((from >= 0) != kFromDevice) continue;
    const int32_t src0 = kFromDevice ? from : __builtin_amdgcn_readfirstlane(e[0]);
    for (int r = r0s; r < n; r += r_steps * kRows) {
      // a row past the entry's end, or past the capacity on either side, gets an empty extent: its loads return zeros
      // without traffic and its stores are dropped.  The resources are built where they are used (a handful of scalar
      // instructions each) instead of being kept: 4 per row would not fit the scalar registers.
      auto row_of = [&](int j, int64_t& rr, int& ext) {
        const int64_t rj = (int64_t)r + (int64_t)j * r_steps;
        const bool live = rj < n && dst0 + rj < capacity_rows && (!kFromDevice || src0 + rj < capacity_rows);
        rr = live ? rj : 0;
        ext = live ? row_bytes : 0;
      };
      for (int off = lane_in_row * 16; off < row_bytes; off += kCopyRowLanes * 16) {
        u32x4_t a[kRows], b[kRows];
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          int64_t rr; int ext;
          row_of(j, rr, ext);
          const uint4* ks = (kFromDevice ? k_dst : k_src) + (src0 + rr) * row_vecs;
          const uint4* vs = (kFromDevice ? v_dst : v_src) + (src0 + rr) * row_vecs;
          a[j] = __builtin_amdgcn_raw_buffer_load_b128(__builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(ks), 0, ext, 0x00020000), off, 0, 0);
          b[j] = __builtin_amdgcn_raw_buffer_load_b128(__builtin_amdgcn_make_buffer_rsrc(const_cast<uint4*>(vs), 0, ext, 0x00020000), off, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < kRows; ++j) {
          int64_t rr; int ext;
          row_of(j, rr, ext);
          __builtin_amdgcn_raw_buffer_store_b128(a[j], __builtin_amdgcn_make_buffer_rsrc(k_dst + (dst0 + rr) * row_vecs, 0, ext, 0x00020000), off, 0, 0);
          __builtin_amdgcn_raw_buffer_store_b128(b[j], __builtin_amdgcn_make_buffer_rsrc(v_dst + (dst0 + rr) * row_vecs, 0, ext, 0x00020000), off, 0, 0);
        }
      }
    }
  }
}

}  // namespace msa_gather
