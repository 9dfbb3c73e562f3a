// Router scoring: pre-summed query tiles against the HBM-resident pooled K_r bank.
//
// score[b, c] = max over scored tokens t of (scale / Hq) * sum_h q'[b,t,h] . kr[c, h / G]
//             = max_t (scale / Hq) * Qs[b,t,:] . kr[c,:]        with Qs[b,t,g,:] = sum_{h in g} q'[b,t,h,:]
// (the mean over heads is linear, so the G query heads of one KV group are summed first).  That is
// an NT GEMM  [B*S_pad, Hkv*D] x [C, Hkv*D]^T  whose output is never written: each 32-row MFMA
// block is reduced to a column max over its scored rows in registers.  For routing the column maxima
// of a query are folded further, across the chunks of one document, and merged with atomicMax into
// doc_key[B, n_docs] (order-preserving uint32 keys): the max over a document's chunks happens in the
// scoring epilogue and no per-chunk plane exists.  msa_chunk_scores keeps the per-chunk form.
#include <algorithm>
#include <mutex>
#include <type_traits>
#include <vector>

#include "gather_device.h"
#include "route_internal.h"

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// ------------------------------------------------------------------------------------------
// Prologue: normalise (cosine mode), sum the G heads of each KV group, cast, build row masks, clear the key plane.
// One workgroup of Hkv*16 lanes per (b, padded token); lane (g, j) owns 8 contiguous d of group g.
// A row that is not scored (a masked token, or the padding of a query to a multiple of 32 rows) repeats the query's
// first scored row: a repeated row changes no maximum, so the scoring epilogues fold whole 32-row blocks without
// per-row tests.  A query without any scored token keeps rows of zeros and mask words of zero: its row blocks are
// skipped and its keys stay 0.  The workgroup of every 32nd row writes the mask word of its 32 rows (all ones or
// zero), workgroup 0 the zero words that pad the mask to whole M tiles, and all workgroups together clear the
// `clear_words` key words the scoring kernel merges into with atomicMax.
// ------------------------------------------------------------------------------------------
// Words behind the persistent scan's tile pool: the pool's counter, on a cache line of its own, then one word per
// workgroup through which the wavefront that drew a tile tells the workgroup's others.
constexpr int kSchedCounterWords = 32;
constexpr int kSchedMaxWorkgroups = 1024;
constexpr size_t kSchedBytes = (size_t)(kSchedCounterWords + kSchedMaxWorkgroups) * sizeof(uint32_t);

template <typename TIn, typename TOut>
__global__ void presum_queries_kernel(const TIn* __restrict__ q, const uint8_t* __restrict__ qmask, int32_t B,
                                      int32_t S, int32_t S_pad, int32_t Hq, int32_t Hkv, int32_t normalize,
                                      TOut* __restrict__ qs, uint32_t* __restrict__ row_bits, int32_t mask_words,
                                      uint32_t* __restrict__ key_plane, int64_t clear_words, uint32_t* __restrict__ sched) {
  const int row = blockIdx.x;              // b * S_pad + s
  const int b = row / S_pad;
  int s = row % S_pad;
  const int G = Hq / Hkv;
  const int g = threadIdx.x >> 4, j = threadIdx.x & 15;
  bool valid = s < S && (qmask == nullptr || qmask[(int64_t)b * S + s] != 0);
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < clear_words; i += (int64_t)gridDim.x * blockDim.x)
    key_plane[i] = 0u;
  const bool writes_word = (row & 31) == 0;           // rows are padded per query to a multiple of 32
  if (!valid || writes_word) {                        // (uniform over the workgroup)
    // the query's first scored token, found by the workgroup's first wavefront
    __shared__ int first_scored;
    if (threadIdx.x < 64) {
      const int nl = min((int)blockDim.x, 64);
      int found = qmask == nullptr ? 0 : -1;
      for (int base = 0; base < S && found < 0; base += nl) {
        const int t = base + (int)threadIdx.x;
        const bool v = (int)threadIdx.x < nl && t < S && qmask[(int64_t)b * S + t] != 0;
        const uint64_t m = __ballot(v);
        if (m != 0) found = base + __builtin_ctzll(m);
      }
      if (threadIdx.x == 0) {
        first_scored = found;
        if (writes_word) row_bits[row >> 5] = found >= 0 ? 0xffffffffu : 0u;
      }
    }
    __syncthreads();
    if (!valid && first_scored >= 0) {
      s = first_scored;
      valid = true;
    }
  }
  if (blockIdx.x == 0) {
    for (int w = (int)(gridDim.x >> 5) + (int)threadIdx.x; w < mask_words; w += blockDim.x) row_bits[w] = 0u;
    if (threadIdx.x == 0) sched[0] = 0u;        // the scan's pool counter
  }
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  if (valid) {
    const TIn* p0 = q + (((int64_t)b * S + s) * Hq + g * G) * kHeadDim + 8 * j;
    for (int h0 = 0; h0 < G; h0 += 4) {          // four heads' loads in flight before the first is normalised
      float x[4][8];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const TIn* p = p0 + (int64_t)min(h0 + u, G - 1) * kHeadDim;
        if constexpr (sizeof(TIn) == 2) {
          const uint4 w = *reinterpret_cast<const uint4*>(p);
          x[u][0] = bf16lo(w.x); x[u][1] = bf16hi(w.x); x[u][2] = bf16lo(w.y); x[u][3] = bf16hi(w.y);
          x[u][4] = bf16lo(w.z); x[u][5] = bf16hi(w.z); x[u][6] = bf16lo(w.w); x[u][7] = bf16hi(w.w);
        } else {
          const float4 lo = *reinterpret_cast<const float4*>(p);
          const float4 hi = *reinterpret_cast<const float4*>(p + 4);
          x[u][0] = lo.x; x[u][1] = lo.y; x[u][2] = lo.z; x[u][3] = lo.w;
          x[u][4] = hi.x; x[u][5] = hi.y; x[u][6] = hi.z; x[u][7] = hi.w;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        float inv = h0 + u < G ? 1.f : 0.f;      // a clamped repeat of the last head adds nothing
        if (normalize) {
          float ssq = 0.f;
#pragma unroll
          for (int i = 0; i < 8; ++i) ssq += x[u][i] * x[u][i];
          ssq += __shfl_xor(ssq, 1); ssq += __shfl_xor(ssq, 2);     // the 16 lanes of one group
          ssq += __shfl_xor(ssq, 4); ssq += __shfl_xor(ssq, 8);
          inv *= 1.0f / fmaxf(sqrtf(ssq), 1e-12f);
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[i] += x[u][i] * inv;
      }
    }
  }
  TOut* o = qs + ((int64_t)row * Hkv + g) * kHeadDim + 8 * j;
  if constexpr (sizeof(TOut) == 2) {
    uint4 w;
    w.x = pack_bf16x2(acc[0], acc[1]); w.y = pack_bf16x2(acc[2], acc[3]);
    w.z = pack_bf16x2(acc[4], acc[5]); w.w = pack_bf16x2(acc[6], acc[7]);
    *reinterpret_cast<uint4*>(o) = w;
  } else {
    *reinterpret_cast<float4*>(o) = make_float4(acc[0], acc[1], acc[2], acc[3]);
    *reinterpret_cast<float4*>(o + 4) = make_float4(acc[4], acc[5], acc[6], acc[7]);
  }
}

// ------------------------------------------------------------------------------------------
// The other reductions over a query's tokens (src/msa_service.py:751-780): "mean" (sum over the scored tokens / their
// number) and "last" (the token at position count - 1, count = scored tokens).  Both are linear in the query row, or
// pick one, so they collapse the query to ONE pre-summed row before the scan: mean_t (q_t . k) = (mean_t q_t) . k.
// The scan and its max over rows then run unchanged on one row block per query whose 32 rows all hold that row.
//
// collapse_queries_kernel: one workgroup per (query, KV group); its 16 slots of 16 lanes take tokens slot, slot + 16,
// ...; a slot sums, over its tokens that count, the group's (normalised, in cosine mode) heads; the slots meet in LDS in
// a fixed order.  Writes the fp32 row and, from group 0, the number of tokens that counted.
// ------------------------------------------------------------------------------------------
constexpr int kQueryMax = MSA_QUERY_MAX, kQueryMean = MSA_QUERY_MEAN, kQueryLast = MSA_QUERY_LAST;

template <typename TIn>
__global__ __launch_bounds__(256) void collapse_queries_kernel(const TIn* __restrict__ q, const uint8_t* __restrict__ qmask,
                                                               int32_t S, int32_t Hq, int32_t Hkv, int32_t normalize,
                                                               int32_t query_reduce, float* __restrict__ rows,
                                                               int32_t* __restrict__ counts) {
  __shared__ float part[16][kHeadDim];
  __shared__ int n_scored;
  const int b = blockIdx.x, g = blockIdx.y;
  const int G = Hq / Hkv;
  const int slot = threadIdx.x >> 4, j = threadIdx.x & 15;
  // scored tokens of the query (every wavefront counts them: the result is needed by all)
  int count = 0;
  if (qmask == nullptr) {
    count = S;
  } else {
    const int lane = threadIdx.x & 63;
    for (int base = 0; base < S; base += 64) {
      const int t = base + lane;
      count += __builtin_popcountll(__ballot(t < S && qmask[(int64_t)b * S + t] != 0));
    }
  }
  const int last = max(count - 1, 0);
  auto counts_in = [&](int t) {
    const bool scored = qmask == nullptr || qmask[(int64_t)b * S + t] != 0;
    return query_reduce == kQueryLast ? (t == last && scored) : scored;
  };
  float acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) acc[i] = 0.f;
  int used = 0;
  for (int t = slot; t < S; t += 16) {
    if (!counts_in(t)) continue;                       // (uniform over the slot's 16 lanes)
    ++used;
    const TIn* p0 = q + (((int64_t)b * S + t) * Hq + g * G) * kHeadDim + 8 * j;
    for (int h = 0; h < G; ++h) {
      float x[8];
      const TIn* p = p0 + (int64_t)h * kHeadDim;
      if constexpr (sizeof(TIn) == 2) {
        const uint4 w = *reinterpret_cast<const uint4*>(p);
        x[0] = bf16lo(w.x); x[1] = bf16hi(w.x); x[2] = bf16lo(w.y); x[3] = bf16hi(w.y);
        x[4] = bf16lo(w.z); x[5] = bf16hi(w.z); x[6] = bf16lo(w.w); x[7] = bf16hi(w.w);
      } else {
        const float4 lo = *reinterpret_cast<const float4*>(p);
        const float4 hi = *reinterpret_cast<const float4*>(p + 4);
        x[0] = lo.x; x[1] = lo.y; x[2] = lo.z; x[3] = lo.w; x[4] = hi.x; x[5] = hi.y; x[6] = hi.z; x[7] = hi.w;
      }
      float inv = 1.f;
      if (normalize) {
        float ssq = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) ssq += x[i] * x[i];
        inv = 1.0f / fmaxf(sqrtf(row16_sum(ssq)), 1e-12f);
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[i] += x[i] * inv;
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) part[slot][8 * j + i] = acc[i];
  if (threadIdx.x == 0) n_scored = 0;
  __syncthreads();
  if (j == 0 && used) atomicAdd(&n_scored, used);
  __syncthreads();
  if (threadIdx.x < kHeadDim) {
    float sum = 0.f;
    for (int s2 = 0; s2 < 16; ++s2) sum += part[s2][threadIdx.x];
    const int n = n_scored;
    rows[((int64_t)b * Hkv + g) * kHeadDim + threadIdx.x] = n > 0 ? sum / (float)n : 0.f;
    if (g == 0 && threadIdx.x == 0) counts[b] = n;
  }
}

// One row block (32 rows) per query, every row the collapsed row; mask words, padding words, the key plane and the
// tile pool's counter as presum_queries_kernel leaves them.  One workgroup per row.
template <typename TOut>
__global__ void broadcast_rows_kernel(const float* __restrict__ rows, const int32_t* __restrict__ counts, int32_t Hkv,
                                      TOut* __restrict__ qs, uint32_t* __restrict__ row_bits, int32_t mask_words,
                                      uint32_t* __restrict__ key_plane, int64_t clear_words, uint32_t* __restrict__ sched) {
  const int row = blockIdx.x, b = row >> 5;
  const int K = Hkv * kHeadDim;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < clear_words; i += (int64_t)gridDim.x * blockDim.x)
    key_plane[i] = 0u;
  const bool any = counts[b] > 0;
  if ((row & 31) == 0 && threadIdx.x == 0) row_bits[row >> 5] = any ? 0xffffffffu : 0u;
  if (blockIdx.x == 0) {
    for (int w = (int)(gridDim.x >> 5) + (int)threadIdx.x; w < mask_words; w += blockDim.x) row_bits[w] = 0u;
    if (threadIdx.x == 0) sched[0] = 0u;
  }
  for (int c = threadIdx.x; c < K; c += blockDim.x) {
    const float x = any ? rows[(int64_t)b * K + c] : 0.f;
    if constexpr (sizeof(TOut) == 2) qs[(int64_t)row * K + c] = f32_to_bf16(x);
    else qs[(int64_t)row * K + c] = x;
  }
}

// ------------------------------------------------------------------------------------------
// MFMA operand traits.  LDS rows hold 128 bytes of K (64 bf16 or 32 fp32) plus 16 bytes of pad,
// which makes the 16-byte / 4-byte operand reads of a 32-row block bank-conflict free.
// ------------------------------------------------------------------------------------------
constexpr int kRowBytes = 128;
constexpr int kRowStride = kRowBytes + 16;

template <typename T>
struct Mma;
template <>
struct Mma<bf16_t> {
  typedef bf16x8_t Frag;
  static constexpr int kSub = 4;   // 32x32x16 steps per 64-element K tile
  static __device__ __forceinline__ Frag load(const char* row, int sub, int half) {
    return *reinterpret_cast<const Frag*>(row + sub * 32 + half * 16);
  }
  static __device__ __forceinline__ floatx16_t mma(Frag a, Frag b, floatx16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mma<float> {
  typedef float Frag;
  static constexpr int kSub = 16;  // 32x32x2 steps per 32-element K tile
  static __device__ __forceinline__ Frag load(const char* row, int sub, int half) {
    return *reinterpret_cast<const Frag*>(row + sub * 8 + half * 4);
  }
  static __device__ __forceinline__ floatx16_t mma(Frag a, Frag b, floatx16_t c) {
    return __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, 0, 0, 0);
  }
};

// The HBM-bound form for up to 128 query rows (bf16, 128 x 256, streaming over N tiles) stages its operand tiles with
// buffer loads that write LDS directly (no staging registers, no ds_write; un-padded 128-byte rows whose 16-byte units
// are XOR-swizzled by (row >> 1) & 7: a direct load cannot pad, its 64 lanes fill 1 KB of LDS in lane order, so the
// swizzle is applied to the global address each lane fetches), three
// stages of each operand (3 x 16 KB + 3 x 32 KB = 144 KB): both operands are requested two K steps ahead, which keeps
// 96 KB per compute unit in flight (returns are in order, so the query tile has to run as far ahead as the K_r tile for
// the K_r tile's lead to count).
constexpr int kDtlStreamLdsBytes = 3 * (128 + 256) * 128;
template <typename T, int BM, int BN, int kSets, bool kStream>
constexpr bool score_tile_is_direct_stream() {
  return sizeof(T) == 2 && BM == 128 && BN == 256 && kSets == 1 && kStream;
}

// Workgroup tile BM x BN, WAVES_M x WAVES_N wavefronts, each owning TM x TN blocks of 32 x 32.
// kSets: register sets of global loads, i.e. K tiles in flight ahead of the one being multiplied.  One is enough when
// a tile's MFMA work outlasts a load's latency (the MFMA-bound shapes); the HBM-bound shapes (few query rows) need
// more bytes in flight per compute unit than one tile holds.
// kDocMax: keys are folded over the chunks of a document (chunk_doc) and merged into out_key[B, n_docs];
// otherwise one key per (query, chunk) is merged into out_key[B, C].
// kStream: one workgroup per compute-unit slot walks N tiles blockIdx.x, blockIdx.x + gridDim.x, ... (one M tile
// only) with the load / store / multiply pipeline running across tile boundaries: the first K tiles of the next N
// tile are already in flight while the last ones of the current tile are multiplied and its epilogue runs, so the
// HBM stream never drains between tiles.  That is what the HBM-bound shapes need; the fp32 form keeps one
// workgroup per tile.
template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, int kSets, bool kDocMax, bool kStream>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void score_gemm_kernel(
    const T* __restrict__ qs,            // [M_rows, K]  pre-summed queries, M_rows = B * S_pad
    const T* __restrict__ kr,            // [C, K]
    const uint32_t* __restrict__ row_bits,  // [ceil(M_alloc / 32)] scored-row bitmask
    uint32_t* __restrict__ out_key,      // [B, n_docs] or [B, C], zeroed
    const int32_t* __restrict__ chunk_doc,  // [C] document of every chunk (kDocMax)
    int32_t M_rows, int32_t C, int32_t K, int32_t blocks_per_query, int32_t tiles_m, int32_t tiles_n,
    int32_t m_group, int32_t n_docs) {
  constexpr int kThreads = WAVES_M * WAVES_N * 64;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int kVecA = BM * 8 / kThreads, kVecB = BN * 8 / kThreads;   // 16-byte vectors per thread per tile
  static_assert(BM * 8 % kThreads == 0 && BN * 8 % kThreads == 0, "tile/threads mismatch");

  extern __shared__ __align__(16) char lds[];
  constexpr int kBufBytes = (BM + BN) * kRowStride;   // [A tile | B tile] per buffer, two buffers
  constexpr bool kDtlStream = score_tile_is_direct_stream<T, BM, BN, kSets, kStream>();

  // XCD-aware tile order: workgroups are dealt round-robin to the 8 XCDs, so each XCD gets one
  // contiguous range of K_r tiles.  Inside it the M tiles are walked in groups of m_group: a group's
  // query rows stay in that XCD's L2 while its K_r tiles stream past once per group.
  int tile_n, tile_m;
  if constexpr (kStream) {
    tile_n = blockIdx.x;
    tile_m = 0;
  }
  // Position `vb` of the XCD-aware tile order -> (M tile, N tile); false for the padding positions of the order.
  const int n_per_xcd = (tiles_n + 7) / 8, per_group = n_per_xcd * m_group;
  auto decode_tile = [&](int vb, int& tm, int& tn) -> bool {
    const int within = vb / 8;
    const int rem = within % per_group;
    tn = (vb % 8) * n_per_xcd + rem / m_group;
    tm = (within / per_group) * m_group + rem % m_group;
    return tn < tiles_n && tm < tiles_m;
  };
  if constexpr (!kStream) {
    if (!decode_tile(blockIdx.x, tile_m, tile_n)) return;
  }
  if (tile_n >= tiles_n || tile_m >= tiles_m) return;
  int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63;
  // (wave-uniform by construction; said so, the LDS addresses of the direct loads stay in scalar registers instead of
  // being read back from a lane in front of every load: 1.9 % on the large-tile scan)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int half = lane >> 5, l32 = lane & 31;

  const int64_t row_bytes_g = (int64_t)K * sizeof(T);
  const char* ga = reinterpret_cast<const char*>(qs);
  const char* gb = reinterpret_cast<const char*>(kr);

  // Global -> register staging through buffer loads: one resource per operand tile whose extent is
  // the valid part of the tile, so rows past M_rows / C read as zero in hardware (no branches, no
  // clamps).  The range check is defined on the vector offset, so the row displacement of a thread's
  // vectors rides there; the K-tile displacement (which stays inside the row, so it can never carry a
  // load past the extent) is scalar.
  const int rows_a = min(BM, M_rows - m0);
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(ga) + (int64_t)m0 * row_bytes_g, 0, (int)(rows_a * row_bytes_g), 0x00020000);
  const int rows_b = min(BN, C - n0);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(gb) + (int64_t)n0 * row_bytes_g, 0, (int)(rows_b * row_bytes_g), 0x00020000);
  __amdgpu_buffer_rsrc_t rsrc_ld = rsrc_b;      // kStream: the N tile the loads have reached
  const int voff = (tid >> 3) * (int)row_bytes_g + (tid & 7) * 16;
  const int vec_stride = (kThreads / 8) * (int)row_bytes_g;     // rows between a thread's vectors
  static_assert(kSets == 1 || kSets == 2, "one or two K tiles in flight");
  u32x4_t ra[kSets][kVecA], rb[kSets][kVecB];
  // K_r streams through once per M tile group while the query matrix is re-read by every workgroup of an XCD: the
  // non-temporal hint on the K_r loads keeps the queries in the 4 MiB L2 (traffic past L2 9.9 -> 6.9 GB per launch
  // at the 100M-token bank, 1.5 % faster).
  constexpr int kStreamHint = 2;
  constexpr int kPastEnd = 0x40000000;   // vector offset beyond any tile's extent: the load returns zeros, no traffic
  const int k_tiles = (int)(row_bytes_g / kRowBytes);
  auto load_tile = [&](auto set_tag, int kt) {
    constexpr int set = decltype(set_tag)::value;
    const int vo = kt < k_tiles ? voff : kPastEnd;   // a tile past the row is never fetched (keeps the loop branch-free)
#pragma unroll
    for (int i = 0; i < kVecA; ++i)
      ra[set][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, vo + i * vec_stride, kt * kRowBytes, 0);
#pragma unroll
    for (int i = 0; i < kVecB; ++i) {
      if constexpr (kStream)
        rb[set][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_ld, vo + i * vec_stride, kt * kRowBytes, kStreamHint);
      else
        rb[set][i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, vo + i * vec_stride, kt * kRowBytes, kStreamHint);
    }
  };
  // kStream: the loads walk the workgroup's whole sequence of (N tile, K tile) steps; past its last tile they
  // fetch nothing.
  int ld_n0 = n0, ld_kt = 0;
  auto load_next = [&](auto set_tag) {
    load_tile(set_tag, ld_n0 < C ? ld_kt : k_tiles);
    if (++ld_kt == k_tiles) {
      ld_kt = 0;
      ld_n0 = (int)min((int64_t)ld_n0 + (int64_t)gridDim.x * BN, (int64_t)C);
      rsrc_ld = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(gb) + (int64_t)ld_n0 * row_bytes_g, 0,
                                                  (int)(min(BN, C - ld_n0) * row_bytes_g), 0x00020000);
    }
  };
  auto store_tile = [&](auto set_tag, int buf) {
    constexpr int set = decltype(set_tag)::value;
#pragma unroll
    for (int i = 0; i < kVecA; ++i) {
      const int v = tid + i * kThreads, r = v >> 3, c = v & 7;
      *reinterpret_cast<u32x4_t*>(lds + buf * kBufBytes + r * kRowStride + c * 16) = ra[set][i];
    }
#pragma unroll
    for (int i = 0; i < kVecB; ++i) {
      const int v = tid + i * kThreads, r = v >> 3, c = v & 7;
      *reinterpret_cast<u32x4_t*>(lds + buf * kBufBytes + (BM + r) * kRowStride + c * 16) = rb[set][i];
    }
  };
  typedef std::integral_constant<int, 0> Set0;
  typedef std::integral_constant<int, 1 % kSets> Set1;

  floatx16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // Software pipeline over K tiles.  While tile kt is multiplied out of LDS buffer kt&1:
  //   - tile kt+1 (already in registers) is written to the other buffer during sub-step 1, and the
  //     global loads of tile kt+2 are issued right behind it (a whole iteration to land);
  //   - operand fragments are double-buffered in registers, one sub-step ahead of the MFMAs;
  //   - the single barrier per tile sits before the LAST sub-step's MFMAs, after that sub-step's
  //     fragments were read, so the first fragments of tile kt+1 are fetched under those MFMAs.
  // Hazards: buffer (kt+1)&1 held tile kt-1, whose last fragment reads were issued before the
  // barrier of iteration kt-1; the writes of tile kt+1 are complete at the barrier of iteration kt.
  typedef typename Mma<T>::Frag Frag;
  constexpr int kSub = Mma<T>::kSub;
  const int a_row = (wm * WM + l32) * kRowStride, b_row = (BM + wn * WN + l32) * kRowStride;
  Frag fa[2][TM], fb[2][TN];
  auto load_frags = [&](int buf, int sub, int slot) {
    const char* pa = lds + buf * kBufBytes + a_row;
    const char* pb = lds + buf * kBufBytes + b_row;
#pragma unroll
    for (int i = 0; i < TM; ++i) fa[slot][i] = Mma<T>::load(pa + i * 32 * kRowStride, sub, half);
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[slot][j] = Mma<T>::load(pb + j * 32 * kRowStride, sub, half);
  };

  // One K tile out of LDS buffer `step & 1`; kMore says a next step exists (the steady-state loop is
  // compiled without that condition so the wait counters around the barrier stay exact).  Tile t travels in
  // register set t % kSets; `set_tag` names the set that holds the next step's tile, which is stored and then
  // refilled with the tile kSets steps further on.
  auto k_tile = [&](auto more_tag, auto set_tag, int step) {
    constexpr bool kMore = decltype(more_tag)::value;
    const int buf = step & 1;
#pragma unroll
    for (int sub = 0; sub < kSub; ++sub) {
      if (sub + 1 < kSub) {
        load_frags(buf, sub + 1, (sub + 1) & 1);
      } else if (kMore) {
        __syncthreads();
        load_frags(buf ^ 1, 0, 0);
        __builtin_amdgcn_sched_barrier(0);   // keep the last sub-step's MFMAs behind these reads
      }
      if (sub == 1 && kMore) {
        store_tile(set_tag, buf ^ 1);
        if constexpr (kStream) {
          __builtin_amdgcn_sched_barrier(0);   // the refill reuses the registers the stores above read
          load_next(set_tag);
        } else if constexpr (kSets > 1) {
          __builtin_amdgcn_sched_barrier(0);
          load_tile(set_tag, step + 1 + kSets);
        } else if (step + 2 < k_tiles) {
          load_tile(set_tag, step + 2);
        }
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = Mma<T>::mma(fa[sub & 1][i], fb[sub & 1][j], acc[i][j]);
    }
  };

  // ---- direct-to-LDS form (see score_tile_is_direct_stream) ----
  // A wavefront's load instruction covers 8 rows of the operand tile: lane l lands in LDS at byte 16 * l of that 1 KB
  // block, i.e. row l / 8, unit slot l % 8, and fetches the unit that belongs there.
  const int dtl_row = (lane >> 3), dtl_slot = lane & 7;

  // Epilogue of the N tile starting at chunk `tile_n0`.  acc[i][j][e] is row 8*(e/4) + 4*half + e%4, column l32 of
  // its 32x32 block.  Consecutive row blocks of one query are folded into `run` (each half of the wavefront over its
  // own rows); emit() joins the halves and merges the query's column maxima of both blocks into the key plane.
  // Several wavefronts and workgroups hold parts of a query (and of a document), so the merge is an atomicMax into
  // a zeroed plane.  emit() is reached by whole wavefronts (q and any are uniform).
  //
  // With one workgroup per compute unit nothing else runs while an epilogue waits, so it must not wait on memory:
  // the scored-row words of the wavefront's row blocks and the documents of its columns are requested ahead (before
  // the K loop / a tile ahead) and only consumed here, and the lane exchanges of the document fold are row moves.
  const int n_queries = M_rows / (blocks_per_query * 32);
  uint32_t rbits[TM];                                   // scored-row word of each row block (same in every lane)
  // query of the wavefront's first row block and that block's place in the query: later blocks follow by counting
  // (one division per wavefront, under the first tile's load latency, instead of one per block in the epilogue)
  int q_first = 0, r_first = 0;
  auto fetch_rows = [&]() {
#pragma unroll
    for (int i = 0; i < TM; ++i) rbits[i] = row_bits[(m0 + wm * WM + i * 32) >> 5];   // 0 past M_rows (buffer is padded)
    const int blk0 = (m0 + wm * WM) >> 5;
    q_first = blk0 / blocks_per_query;
    r_first = blk0 - q_first * blocks_per_query;
  };
  int cdoc[TN];                                         // document of each column; lanes past the bank never join a run
  auto fetch_docs = [&](int tile_n0) {
    if constexpr (kDocMax) {
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int n = tile_n0 + wn * WN + j * 32 + l32;
        cdoc[j] = n < C ? chunk_doc[n] : -1 - l32;
      }
    }
  };
  // Both column blocks of the wavefront at once: after the halves are joined (one half-wave swap: the upper half of
  // block 0's partial maxima against the lower half of block 1's) the lower 32 lanes hold block 0's 32 column maxima
  // and the upper 32 lanes block 1's, so the segmented scan and the atomics below run once per query for the
  // wavefront's 64 columns instead of once per block with half the lanes idle.
  static_assert(TN == 2, "the epilogue pairs the two column blocks of a wavefront");
  auto emit = [&](int q, int tile_n0, const float (&run_half)[TN], bool any) {
    if (!any || q >= n_queries) return;
    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(run_half[0]), __float_as_uint(run_half[1]), false, false);
    const float run = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
    const int n = tile_n0 + wn * WN + half * 32 + l32;
    const int doc = kDocMax ? (half ? cdoc[1] : cdoc[0]) : 0;
    const bool ok = n < C;
    const uint32_t key = ok ? f32_to_key(run) : 0u;
    if constexpr (kDocMax) {
      // Chunks of a document are adjacent columns: a segmented max-scan over the 32 lanes of each half leaves a
      // document's maximum in the last lane of its run, which alone touches memory (about two atomics per 32
      // chunks instead of 32 stores, and no per-chunk plane to read back).  `dist` is a lane's distance from the
      // first lane of its run, from a ballot of the run heads; the scan itself moves keys only: four shifts inside
      // the rows of 16 lanes, then lane 15 of the lower row joins the runs that cross into the upper one.  Lanes a
      // shift cannot reach read 0, the identity of max over keys.
      const int prev = __builtin_amdgcn_update_dpp(doc, doc, 0x138, 0xF, 0xF, false);      // wave_shr:1
      const uint64_t heads64 = __ballot(l32 == 0 || prev != doc);
      const uint32_t heads = half ? (uint32_t)(heads64 >> 32) : (uint32_t)heads64;
      const uint32_t upto = heads & ((2u << l32) - 1u);                  // heads at or below this lane (never empty)
      const int dist = l32 - (31 - __builtin_clz(upto));
      const bool last = l32 == 31 || ((heads >> (l32 + 1)) & 1u);
      int m = (int)key;
#define MSA_SCAN_STEP(OFF, CTRL)                                                          \
      {                                                                                   \
        const int o = __builtin_amdgcn_update_dpp(0, m, CTRL, 0xF, 0xF, true);            \
        if (dist >= OFF) m = (int)max((uint32_t)m, (uint32_t)o);                          \
      }
      MSA_SCAN_STEP(1, 0x111)   // row_shr:1
      MSA_SCAN_STEP(2, 0x112)
      MSA_SCAN_STEP(4, 0x114)
      MSA_SCAN_STEP(8, 0x118)
#undef MSA_SCAN_STEP
      const int low = __builtin_amdgcn_update_dpp(0, m, 0x142, 0xA, 0xF, false);          // row_bcast:15 into rows 1, 3
      if (dist > (l32 & 15)) m = (int)max((uint32_t)m, (uint32_t)low);
      if (ok && last) atomicMax(&out_key[(int64_t)q * n_docs + doc], (uint32_t)m);
    } else {
      if (ok) atomicMax(&out_key[(int64_t)q * C + n], key);
    }
  };
  auto epilogue = [&](int tile_n0) {
    float run[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) run[j] = -INFINITY;
    bool any = false;
    int run_q = q_first, r = r_first;                      // query of row block i, its block index inside the query
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const uint32_t bits = __builtin_amdgcn_readfirstlane(rbits[i]);
      if (r == blocks_per_query) {                         // row block i opens the next query
        emit(run_q, tile_n0, run, any);
#pragma unroll
        for (int j = 0; j < TN; ++j) run[j] = -INFINITY;
        any = false; ++run_q; r = 0;
      }
      ++r;
      if (bits == 0xffffffffu) {                            // every row scored: no per-row tests
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          float mx = acc[i][j][0];
#pragma unroll
          for (int e = 1; e < 16; ++e) mx = fmaxf(mx, acc[i][j][e]);
          run[j] = fmaxf(run[j], mx);
        }
        any = true;
      } else if (bits != 0) {
        const uint32_t mine = bits >> (4 * half);           // this half's rows: bit 8*(e/4) + e%4
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          float mx = -INFINITY;
#pragma unroll
          for (int e = 0; e < 16; ++e)
            if (mine & (1u << (8 * (e >> 2) + (e & 3)))) mx = fmaxf(mx, acc[i][j][e]);
          run[j] = fmaxf(run[j], mx);
        }
        any = true;
      }
    }
    emit(run_q, tile_n0, run, any);
  };

  if constexpr (kDtlStream) {
    static_assert(kThreads == 512 && kSub == 4 && TM == 2 && TN == 2, "laid out for 8 wavefronts of 64 x 64");
    constexpr int kAStage = BM * 128, kBStage = BN * 128, kStages = 3;
    constexpr int kALoads = BM / 64, kBLoads = BN / 64;      // 1 KB blocks (8 rows) per wavefront and stage
    constexpr int kWaitAllButNewestStep = 0x0F70 + kALoads + kBLoads, kWaitAll = 0x0F70;
    char* const lds_a = lds;
    char* const lds_b = lds + kStages * kAStage;
    auto dtl_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
    auto voff_of = [&](int row) { return row * (int)row_bytes_g + ((dtl_slot ^ ((row >> 1) & 7)) * 16); };
    auto load_a = [&](int stage, int kt) {
#pragma unroll
      for (int i = 0; i < kALoads; ++i) {
        const int blk = wave * kALoads + i;
        MSA_LOAD_TO_LDS(rsrc_a, lds_a + stage * kAStage + blk * 1024, voff_of(blk * 8 + dtl_row), kt * kRowBytes, 0);
      }
    };
    auto load_b = [&](int stage, int kt) {
#pragma unroll
      for (int i = 0; i < kBLoads; ++i) {
        const int blk = wave * kBLoads + i;
        MSA_LOAD_TO_LDS(rsrc_ld, lds_b + stage * kBStage + blk * 1024, voff_of(blk * 8 + dtl_row), kt * kRowBytes,
                        kStreamHint);
      }
    };
    auto frags = [&](int stage, int sub, int slot) {
      const int unit = sub * 2 + half;
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const int row = wm * WM + i * 32 + l32;
        fa[slot][i] = *reinterpret_cast<const Frag*>(lds_a + stage * kAStage + row * 128 + ((unit ^ ((row >> 1) & 7)) * 16));
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const int row = wn * WN + j * 32 + l32;
        fb[slot][j] = *reinterpret_cast<const Frag*>(lds_b + stage * kBStage + row * 128 + ((unit ^ ((row >> 1) & 7)) * 16));
      }
    };
    // The workgroup's N tiles (blockIdx.x, blockIdx.x + gridDim.x, ...) form one sequence of K steps; the loads run two
    // steps ahead of the MFMAs across tile boundaries.
    const int my_tiles = (tiles_n - tile_n + (int)gridDim.x - 1) / (int)gridDim.x;
    int t_ld = 0, kt_ld = 0;                       // tile and K tile the loads have reached
    auto advance_ld = [&]() {
      if (++kt_ld == k_tiles) {
        kt_ld = 0;
        if (++t_ld < my_tiles) {
          const int tn = tile_n + t_ld * (int)gridDim.x;
          rsrc_ld = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(gb) + (int64_t)tn * BN * row_bytes_g, 0,
                                                      (int)(min(BN, C - tn * BN) * row_bytes_g), 0x00020000);
        }
      }
    };
    fetch_rows();                                  // one M tile: the scored-row words serve every N tile
    fetch_docs(n0);
    load_a(0, 0);
    load_b(0, 0);
    advance_ld();
    if (t_ld < my_tiles) {
      load_a(1, kt_ld);
      load_b(1, kt_ld);
      advance_ld();
      __builtin_amdgcn_s_waitcnt(kWaitAllButNewestStep);
    } else {
      __builtin_amdgcn_s_waitcnt(kWaitAll);
    }
    dtl_barrier();
    frags(0, 0, 0);
    int st = 0, t = 0, kt = 0;
    for (;;) {
      const int st1 = st == 2 ? 0 : st + 1, st2 = st1 == 2 ? 0 : st1 + 1;
      const bool more = !(t == my_tiles - 1 && kt == k_tiles - 1);    // a next step exists
      const bool more2 = t_ld < my_tiles;                              // the step behind it exists
      if (more2) {
        load_a(st2, kt_ld);      // stage of the step before this one: its last reads were behind the previous barrier
        load_b(st2, kt_ld);
        advance_ld();
      }
      auto substep = [&](auto sub_tag, auto fresh_tag) {
        constexpr int sub = decltype(sub_tag)::value;
        constexpr bool fresh = decltype(fresh_tag)::value;
        if constexpr (sub + 1 < kSub) {
          frags(st, sub + 1, (sub + 1) & 1);
        } else {
          if (more) {
            if (more2) __builtin_amdgcn_s_waitcnt(kWaitAllButNewestStep);
            else __builtin_amdgcn_s_waitcnt(kWaitAll);
            dtl_barrier();
            frags(st1, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            if constexpr (fresh) acc[i][j] = Mma<T>::mma(fa[sub & 1][i], fb[sub & 1][j], floatx16_t{});
            else acc[i][j] = Mma<T>::mma(fa[sub & 1][i], fb[sub & 1][j], acc[i][j]);
          }
        if constexpr (sub + 1 < kSub) {
#pragma unroll
          for (int g = 0; g < TM + TN; ++g) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
          }
        }
      };
      if (kt == 0) substep(std::integral_constant<int, 0>{}, std::true_type{});
      else substep(std::integral_constant<int, 0>{}, std::false_type{});
      substep(std::integral_constant<int, 1>{}, std::false_type{});
      substep(std::integral_constant<int, 2>{}, std::false_type{});
      substep(std::integral_constant<int, 3>{}, std::false_type{});
      st = st1;
      if (++kt == k_tiles) {
        epilogue(n0);
        if (!more) break;
        kt = 0;
        ++t;
        n0 += (int)gridDim.x * BN;
        fetch_docs(n0);
      }
    }
  } else if constexpr (kStream) {
    // The workgroup's tiles form one sequence of steps (K tiles are even in number, so set tags and LDS buffers
    // alternate the same way in every tile); an epilogue sits where a tile's last step ends, with the next tile's
    // first operand fragments already in registers and its loads in flight.
    const int my_tiles = (tiles_n - tile_n + (int)gridDim.x - 1) / (int)gridDim.x;
    const int steps = my_tiles * k_tiles;
    load_next(Set0{});
    store_tile(Set0{}, 0);
    load_next(Set1{});
    if constexpr (kSets == 2) load_next(Set0{});
    __syncthreads();
    load_frags(0, 0, 0);
    fetch_rows();
    fetch_docs(n0);
    int done_n0 = n0, in_tile = 0;
    for (int step = 0; step + 2 < steps; step += 2) {
      k_tile(std::true_type{}, Set1{}, step);
      k_tile(std::true_type{}, Set0{}, step + 1);
      in_tile += 2;
      if (in_tile == k_tiles) {
        epilogue(done_n0);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
        in_tile = 0;
        done_n0 += (int)gridDim.x * BN;
        fetch_docs(done_n0);
      }
    }
    k_tile(std::true_type{}, Set1{}, steps - 2);
    k_tile(std::false_type{}, Set0{}, steps - 1);
    epilogue(done_n0);
  } else {
    if constexpr (kSets == 2) {
      // tile t travels in register set (t & 1): iteration kt stores tile kt+1 and refills its set with tile kt+3
      load_tile(Set0{}, 0);
      store_tile(Set0{}, 0);
      load_tile(Set1{}, 1);
      load_tile(Set0{}, 2);
      __syncthreads();
      load_frags(0, 0, 0);
      fetch_rows();
      fetch_docs(n0);
      int kt = 0;
      for (; kt + 2 < k_tiles; kt += 2) {
        k_tile(std::true_type{}, Set1{}, kt);
        k_tile(std::true_type{}, Set0{}, kt + 1);
      }
      if (kt + 1 < k_tiles) {
        k_tile(std::true_type{}, Set1{}, kt);
        k_tile(std::false_type{}, Set0{}, kt + 1);
      } else {
        k_tile(std::false_type{}, Set1{}, kt);
      }
    } else {
      load_tile(Set0{}, 0);
      store_tile(Set0{}, 0);
      if (k_tiles > 1) load_tile(Set0{}, 1);
      __syncthreads();
      load_frags(0, 0, 0);
      fetch_rows();
      fetch_docs(n0);
      for (int kt = 0; kt + 1 < k_tiles; ++kt) k_tile(std::true_type{}, Set0{}, kt);
      k_tile(std::false_type{}, Set0{}, k_tiles - 1);
    }
    epilogue(n0);
  }
}

// ------------------------------------------------------------------------------------------
// The MFMA-bound form (bf16, more than 128 query rows): 256 x 256 tile, four wavefronts (one per SIMD) of 128 x 128,
// the sixteen 32 x 32 accumulators of a wavefront in the 256 accumulation registers, and the K step written at the
// instruction level (scan_asm.inc, generated by gen_scan_asm.py, which describes the schedule and the registers the
// asm statements own: v128 - v255 and a0 - a255; the compiler-allocated code of this kernel is held below v128 by the
// register limit on its declaration and uses no accumulation registers, which the build checks).  One wavefront per
// SIMD has nobody to cover a wait, so every wait the step contains is met long before it is reached: operand
// fragments are read a sub-step ahead, the query and K_r tiles are requested two K steps ahead (LDS: two stages of the
// query tile, three of the K_r tile, filled by buffer loads that write LDS directly), and the one barrier per step
// stands behind an MFMA.  Per 128 x 128 wavefront tile a sub-step reads eight operand fragments for sixteen MFMAs,
// against six for eight in a 2 x 4 layout of eight wavefronts.
//
// Persistent: one workgroup per compute unit walks its share of the tile list (scan_walk.h) as one sequence of K
// steps, the loads two steps ahead across tile boundaries.  With a gather job attached the last workgroup of the
// launch copies the K / V rows of an earlier selection instead (gather_device.h).  The last pool_n N tiles are handed
// out one at a time to workgroups that have finished their own share: during the first K steps of the tile in front of
// a pool tile one lane draws a position from the pool's counter (an atomic that returns), publishes it through the
// workgroup's claim word (an exchange that returns, so its arrival says the word is in L2) and every wavefront reads
// it back, one hop per K step, each issued in front of the step's tile loads so that the step's own wait (all but the
// eight newest loads) covers it.  The hops' values live in v217 - v219.
// ------------------------------------------------------------------------------------------
#include "scan_asm.inc"
#include "scan_walk.h"

constexpr int kScan4CompilerVgprs = 128;     // the compiler's share of the vector registers in score_scan4_kernel
constexpr int kScan4LdsBytes = 5 * 256 * 128;

template <bool kDocMax>
__global__ __launch_bounds__(256) __attribute__((amdgpu_num_vgpr(kScan4CompilerVgprs))) void score_scan4_kernel(
    const bf16_t* __restrict__ qs,          // [M_rows, K]  pre-summed queries, M_rows = B * S_pad
    const bf16_t* __restrict__ kr,          // [C, K]
    const uint32_t* __restrict__ row_bits,  // [ceil(M_alloc / 32)] scored-row bitmask
    uint32_t* __restrict__ out_key,         // [B, n_docs] or [B, C], zeroed
    const int32_t* __restrict__ chunk_doc,  // [C] document of every chunk (kDocMax)
    int32_t M_rows, int32_t C, int32_t K, int32_t blocks_per_query, int32_t tiles_m, int32_t tiles_n, int32_t m_group,
    int32_t n_docs, GatherJob job, uint32_t* __restrict__ sched, int32_t pool_n) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int kThreads = 256, BM = 256, BN = 256;
  extern __shared__ __align__(16) char lds[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  if (job.active && (int)blockIdx.x == (int)gridDim.x - 1) {
    // plan (sorted, de-duplicated selection -> copy entries), host rows, then the documents an earlier sample already
    // fetched; the workgroup barriers order the three steps' memory
    msa_gather::plan_body(job.doc_sel, job.doc_chunk_off, job.n_docs, job.B, job.k,
                          (int32_t)min(job.capacity_rows, (int64_t)0x7fffffff), job.dedup, job.cu_sel, job.plan,
                          reinterpret_cast<int32_t*>(lds), tid, kThreads);
    __syncthreads();
    const int groups = kThreads / msa_gather::kCopyRowLanes;
    const int group = tid / msa_gather::kCopyRowLanes, lane_in_row = tid % msa_gather::kCopyRowLanes;
    msa_gather::copy_body<false, 8>(job.k_src, job.v_src, job.plan, job.B * job.k, job.row_vecs, job.capacity_rows,
                                    job.k_dst, job.v_dst, 0, 1, group, groups, lane_in_row);
    __syncthreads();
    if (job.dedup)
      msa_gather::copy_body<true, 8>(nullptr, nullptr, job.plan, job.B * job.k, job.row_vecs, job.capacity_rows, job.k_dst,
                                     job.v_dst, 0, 1, group, groups, lane_in_row);
    return;
  }
  const ScanWalk walk = scan_walk_init((int)blockIdx.x, (int)gridDim.x, job.active ? 1 : 0, tiles_m, tiles_n, m_group, pool_n);
  if (walk.own_count == 0) return;

  const int wm = wave >> 1, wn = wave & 1;
  const int half = lane >> 5, l32 = lane & 31;
  const int row_bytes = K * (int)sizeof(bf16_t);
  const int k_tiles = row_bytes / kRowBytes;
  {
    // per-lane constants of the asm statements: LDS offsets of the operand fragments of sub-steps 0 - 3 (the rows of a
    // wavefront's blocks are 32 apart, which leaves the swizzle term alone) and the global offsets of the lanes' 16
    // bytes in the wavefront's eight 1 KB blocks of a tile (lane l lands at byte 16 * l of its block, i.e. row l / 8,
    // unit slot l % 8, and fetches the unit that belongs there)
    int aa[4], ab[4], vo[8];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int sw = ((s * 2 + half) ^ ((l32 >> 1) & 7)) * 16;
      aa[s] = (wm * 128 + l32) * 128 + sw;
      ab[s] = (wn * 128 + l32) * 128 + sw;
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = (wave * 8 + i) * 8 + (lane >> 3);
      vo[i] = row * row_bytes + (((lane & 7) ^ ((row >> 1) & 7)) * 16);
    }
    asm volatile(MSA_SCAN4_SET_ADDR ::"v"(aa[0]), "v"(aa[1]), "v"(aa[2]), "v"(aa[3]), "v"(ab[0]), "v"(ab[1]), "v"(ab[2]), "v"(ab[3])
                 : MSA_SCAN4_CLOBBERS);
    asm volatile(MSA_SCAN4_SET_VOFF ::"v"(vo[0]), "v"(vo[1]), "v"(vo[2]), "v"(vo[3]), "v"(vo[4]), "v"(vo[5]), "v"(vo[6]), "v"(vo[7])
                 : MSA_SCAN4_CLOBBERS);
    // v222: byte offset of a lane's column in a run of 64 document ids; v223: the pool counter's increment
    asm volatile("v_lshlrev_b32 v222, 2, %0\n\tv_mov_b32 v223, 1" ::"v"(lane) : MSA_SCAN4_CLOBBERS);
    asm volatile(MSA_SCAN4_SET_FOLD ::"v"(l32) : MSA_SCAN4_CLOBBERS);
  }
  const char* ga = reinterpret_cast<const char*>(qs);
  const char* gb = reinterpret_cast<const char*>(kr);
  // One resource per operand tile whose extent is the valid part of the tile: rows past M_rows / C read as zero in
  // hardware (the range check is on the vector offset, where the row displacement rides; the K displacement is
  // scalar and stays inside the row).  A tile that does not exist gets an empty extent: its loads fetch nothing.
  auto make_a = [&](int tm, bool valid) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(ga) + (valid ? (int64_t)tm * BM * row_bytes : 0), 0,
                                             valid ? min(BM, M_rows - tm * BM) * row_bytes : 0, 0x00020000);
  };
  auto make_b = [&](int tn, bool valid) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(gb) + (valid ? (int64_t)tn * BN * row_bytes : 0), 0,
                                             valid ? min(BN, C - tn * BN) * row_bytes : 0, 0x00020000);
  };
  const __amdgpu_buffer_rsrc_t rsrc_docs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<int32_t*>(kDocMax ? chunk_doc : nullptr), 0, kDocMax ? C * 4 : 0, 0x00020000);

  // The workgroup's tiles: `cur` is multiplied, `nxt` is the one behind it (the loads enter it two K steps before the
  // MFMAs do).  Own tiles first, then pool draws.
  int tm_c, tn_c, tm_n = 0, tn_n = 0, own_idx = 0;
  ScanWalkCursor cursor = scan_walk_cursor(walk);
  scan_walk_cursor_tile(walk, cursor, tm_c, tn_c);
  __amdgpu_buffer_rsrc_t ra_c = make_a(tm_c, true), rb_c = make_b(tn_c, true), ra_n, rb_n;
  bool nxt_valid = false, nxt_pending = false;
  auto plan_next = [&]() {
    nxt_valid = own_idx + 1 < walk.own_count;
    nxt_pending = !nxt_valid && pool_n > 0;
    if (nxt_valid) {
      ++own_idx;
      scan_walk_cursor_next(walk, cursor);
      scan_walk_cursor_tile(walk, cursor, tm_n, tn_n);
    }
    ra_n = make_a(tm_n, nxt_valid);
    rb_n = make_b(tn_n, nxt_valid);
  };
  plan_next();
  uint32_t* const pool_counter = sched;
  uint32_t* const my_claim = sched + kSchedCounterWords + blockIdx.x;
  const bool drawer = wave == 0;
  const uint32_t zero_off = 0;

  // ---- epilogue state: see score_gemm_kernel's epilogue, of which this is the 4 x 4 block form ----
  // acc block (i, j), element e: row 8 * (e / 4) + 4 * half + e % 4 of row block i, column l32 of column block j.
  const int n_queries = M_rows / (blocks_per_query * 32);
  typedef const __attribute__((address_space(4))) uint32_t* const_words_t;      // scalar loads
  const const_words_t row_bits_c = (const_words_t)row_bits;
  // floor(2^32 / d) + 1 divides exactly while n * d < 2^32 (row blocks < 2^19, blocks per query <= 2^11)
  const uint32_t bpq_magic = (uint32_t)(0x100000000ull / (uint32_t)blocks_per_query) + 1u;
  uint32_t rbits[4] = {0u, 0u, 0u, 0u};
  int q_first = 0, r_first = 0;
  auto fetch_rows = [&](int m0) {
    const int blk0 = (m0 + wm * 128) >> 5;
#pragma unroll
    for (int i = 0; i < 4; ++i) rbits[i] = row_bits_c[blk0 + i];          // 0 past M_rows (the buffer is padded)
    q_first = blocks_per_query == 1 ? blk0 : (int)__umulhi((uint32_t)blk0, bpq_magic);     // blk0 / blocks_per_query
    r_first = blk0 - q_first * blocks_per_query;
  };
  // the documents of the wavefront's 128 columns, 64 per load, into v220 / v221 (v216: their offsets): requested in
  // front of a K step (whose waits cover them), read when the tile's maxima are folded; columns past the bank read 0
  // and are masked below
  auto fetch_docs = [&](int n0) {
    if constexpr (kDocMax) {
      const int first = (n0 + wn * 128) * 4;      // (in the vector offset, which is what the extent is checked against)
      asm volatile("s_nop 4\n\tv_add_u32 v216, %1, v222\n\tbuffer_load_dword v220, v216, %0, 0 offen\n\t"
                   "buffer_load_dword v221, v216, %0, 0 offen offset:256"
                   ::"s"(rsrc_docs), "s"(first) : MSA_SCAN4_CLOBBERS);
    }
  };
  // One pair of column blocks (64 columns): after the half-wave swap the lower 32 lanes hold block 2p's column maxima
  // and the upper 32 lanes block 2p + 1's; the segmented scan then leaves a document's maximum in the last lane of its
  // run, which alone touches memory.
  auto emit_pair = [&](int q, int n_first, float lo, float hi, int doc_raw) {
    const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(lo), __float_as_uint(hi), false, false);
    const float run = fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
    const int n = n_first + lane;
    const bool ok = n < C;
    const uint32_t key = ok ? f32_to_key(run) : 0u;
    if constexpr (kDocMax) {
      const int doc = ok ? doc_raw : -1 - l32;
      const int prev = __builtin_amdgcn_update_dpp(doc, doc, 0x138, 0xF, 0xF, false);      // wave_shr:1
      const uint64_t heads64 = __ballot(l32 == 0 || prev != doc);
      const uint32_t heads = half ? (uint32_t)(heads64 >> 32) : (uint32_t)heads64;
      const uint32_t upto = heads & ((2u << l32) - 1u);                  // heads at or below this lane (never empty)
      const int dist = l32 - (31 - __builtin_clz(upto));
      const bool last = l32 == 31 || ((heads >> (l32 + 1)) & 1u);
      int m = (int)key;
#define MSA_SCAN_STEP(OFF, CTRL)                                                          \
      {                                                                                   \
        const int o = __builtin_amdgcn_update_dpp(0, m, CTRL, 0xF, 0xF, true);            \
        if (dist >= OFF) m = (int)max((uint32_t)m, (uint32_t)o);                          \
      }
      MSA_SCAN_STEP(1, 0x111)   // row_shr:1
      MSA_SCAN_STEP(2, 0x112)
      MSA_SCAN_STEP(4, 0x114)
      MSA_SCAN_STEP(8, 0x118)
#undef MSA_SCAN_STEP
      const int low = __builtin_amdgcn_update_dpp(0, m, 0x142, 0xA, 0xF, false);          // row_bcast:15 into rows 1, 3
      if (dist > (l32 & 15)) m = (int)max((uint32_t)m, (uint32_t)low);
      if (ok && last) atomicMax(&out_key[(int64_t)q * n_docs + doc], (uint32_t)m);
    } else {
      if (ok) atomicMax(&out_key[(int64_t)q * C + n], key);
    }
  };
  // Folds the finished tile's block maxima (v224 - v239, left by the reduction that rides in the next tile's first K
  // step or by the stand-alone one): row blocks of one query are joined, and at a query's end the two pairs of column
  // blocks are merged into the key plane.  Every row of a scored block counts (the prologue kernel made unscored rows
  // repeat a scored one); a block whose mask word is zero belongs to a query without scored tokens or to the padding
  // past M_rows and is skipped.
  auto fold_tile = [&](int n0) {
    float mx[16];
    asm volatile(MSA_SCAN4_MAX_READ
                 : "=v"(mx[0]), "=v"(mx[1]), "=v"(mx[2]), "=v"(mx[3]), "=v"(mx[4]), "=v"(mx[5]), "=v"(mx[6]), "=v"(mx[7]),
                   "=v"(mx[8]), "=v"(mx[9]), "=v"(mx[10]), "=v"(mx[11]), "=v"(mx[12]), "=v"(mx[13]), "=v"(mx[14]), "=v"(mx[15]));
    int doc0 = 0, doc1 = 0;
    if constexpr (kDocMax) asm volatile("v_mov_b32 %0, v220\n\tv_mov_b32 %1, v221" : "=v"(doc0), "=v"(doc1));
    float run[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    bool any = false;
    int run_q = q_first, r = r_first;
    auto emit = [&]() {
      if (!any || run_q >= n_queries) return;
      emit_pair(run_q, n0 + wn * 128, run[0], run[1], doc0);
      emit_pair(run_q, n0 + wn * 128 + 64, run[2], run[3], doc1);
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      if (r == blocks_per_query) {                         // row block i opens the next query
        emit();
#pragma unroll
        for (int j = 0; j < 4; ++j) run[j] = -INFINITY;
        any = false; ++run_q; r = 0;
      }
      ++r;
      if (rbits[i] != 0) {
        any = true;
#pragma unroll
        for (int j = 0; j < 4; ++j) run[j] = fmaxf(run[j], mx[i * 4 + j]);
      }
    }
    emit();
  };

  // ---- prologue: the first two K tiles of the first tile, the first fragments ----
  const int woff = wave * 8192;
  int sa = 0, sb = 0x10000;
  asm volatile(MSA_SCAN4_LOAD8_NT ::[dst] "s"(0x10000 + woff), [r] "s"(rb_c), [k] "s"(0) : MSA_SCAN4_CLOBBERS);
  asm volatile(MSA_SCAN4_LOAD8 ::[dst] "s"(0 + woff), [r] "s"(ra_c), [k] "s"(0) : MSA_SCAN4_CLOBBERS);
  asm volatile(MSA_SCAN4_LOAD8_NT ::[dst] "s"(0x18000 + woff), [r] "s"(rb_c), [k] "s"(kRowBytes) : MSA_SCAN4_CLOBBERS);
  asm volatile(MSA_SCAN4_LOAD8 ::[dst] "s"(0x8000 + woff), [r] "s"(ra_c), [k] "s"(kRowBytes) : MSA_SCAN4_CLOBBERS);
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  asm volatile(MSA_SCAN4_FRAGS0 ::[sa] "s"(sa), [sb] "s"(sb) : MSA_SCAN4_CLOBBERS);

  // A tile's accumulators are reduced inside the next tile's first K step and folded right behind it, so the fold of
  // tile t uses the row words and the documents fetched for t; those of t + 1 are requested once it is done.
  bool have_prev = false;
  int prev_n0 = 0;
  for (;;) {
    // Step kt requests K tile kt + 2: of this tile while it has one, of the next tile after that.  The steps are laid
    // out so that between two of them the scalar unit has next to nothing to do (a wavefront that is alone on its SIMD
    // pays for every instruction between two MFMAs): the resources a step reads are fixed per loop, and the tile
    // pool's hops ride in front of four peeled steps.
#define MSA_SCAN4_STEP(TEXT, RA, RB, KOFF)                                                                   \
    asm volatile(TEXT : [sa] "+s"(sa), [sb] "+s"(sb)                                                         \
                 : [ra] "s"(RA), [rb] "s"(RB), [k] "s"(KOFF), [woff] "s"(woff) : MSA_SCAN4_CLOBBERS)
    const bool pending = nxt_pending;      // the tile behind this one comes from the pool (k_tiles >= 6 then)
    if (pending && drawer && lane == 0)    // v217 = counter++
      asm volatile("s_nop 4\n\tglobal_atomic_add v217, %0, v223, %1 sc0" ::"v"(zero_off), "s"(pool_counter) : "memory");
    // What the finished tile left is reduced inside this tile's first step.  Usually the wavefront's four row blocks
    // are one query whose rows all count (blocks_per_query a multiple of 4: queries of 128, 256, ... padded tokens) and
    // the tile lies inside the bank: then the step also folds the maxima into the key plane.  Otherwise it leaves one
    // maximum per block and fold_tile() does the rest; a wavefront whose rows are all padding has nothing to fold.
    const bool fold_any = have_prev && (rbits[0] | rbits[1] | rbits[2] | rbits[3]) != 0;
    const bool fold_fast = kDocMax && fold_any && (blocks_per_query & 3) == 0 && rbits[0] != 0 && prev_n0 + BN <= C;
    if (fold_fast) {
      const uint32_t* okey = out_key + (int64_t)q_first * n_docs;
      if (k_tiles > 2)
        asm volatile(MSA_SCAN4_KSTEP_FRESH_FOLD : [sa] "+s"(sa), [sb] "+s"(sb)
                     : [ra] "s"(ra_c), [rb] "s"(rb_c), [k] "s"(2 * kRowBytes), [woff] "s"(woff), [okey] "s"(okey) : MSA_SCAN4_CLOBBERS);
      else
        asm volatile(MSA_SCAN4_KSTEP_FRESH_FOLD : [sa] "+s"(sa), [sb] "+s"(sb)
                     : [ra] "s"(ra_n), [rb] "s"(rb_n), [k] "s"(0), [woff] "s"(woff), [okey] "s"(okey) : MSA_SCAN4_CLOBBERS);
    } else if (fold_any) {
      if (k_tiles > 2) MSA_SCAN4_STEP(MSA_SCAN4_KSTEP_FRESH_REDUCE, ra_c, rb_c, 2 * kRowBytes);
      else MSA_SCAN4_STEP(MSA_SCAN4_KSTEP_FRESH_REDUCE, ra_n, rb_n, 0);
      fold_tile(prev_n0);
    } else {
      if (k_tiles > 2) MSA_SCAN4_STEP(MSA_SCAN4_KSTEP_FRESH, ra_c, rb_c, 2 * kRowBytes);
      else MSA_SCAN4_STEP(MSA_SCAN4_KSTEP_FRESH, ra_n, rb_n, 0);
    }
    const int n0 = tn_c * BN;
    fetch_rows(tm_c * BM);
    fetch_docs(n0);
    int kt = 1;
    if (pending) {
      if (drawer && lane == 0)           // claim word = v217; its old value comes back in v218
        asm volatile("s_nop 4\n\tglobal_atomic_swap v218, %0, v217, %1 sc0" ::"v"(zero_off), "s"(my_claim) : "memory");
      MSA_SCAN4_STEP(MSA_SCAN4_KSTEP, ra_c, rb_c, 3 * kRowBytes);
      // every wavefront reads the word back (past the L1: device scope)
      asm volatile("s_nop 4\n\tglobal_load_dword v219, %0, %1 sc1" ::"v"(zero_off), "s"(my_claim) : "memory");
      MSA_SCAN4_STEP(MSA_SCAN4_KSTEP, ra_c, rb_c, 4 * kRowBytes);
      int p_next;                        // complete since the last step's wait
      asm volatile("v_readfirstlane_b32 %0, v219" : "=s"(p_next));
      nxt_pending = false;
      nxt_valid = p_next < walk.pool_total;
      if (nxt_valid) scan_walk_pool(walk, p_next, tm_n, tn_n);
      ra_n = make_a(tm_n, nxt_valid);
      rb_n = make_b(tn_n, nxt_valid);
      MSA_SCAN4_STEP(MSA_SCAN4_KSTEP, ra_c, rb_c, 5 * kRowBytes);
      kt = 4;
    }
    for (int k_l = (kt + 2) * kRowBytes; k_l < row_bytes; k_l += kRowBytes) MSA_SCAN4_STEP(MSA_SCAN4_KSTEP, ra_c, rb_c, k_l);
    for (int k_l = k_tiles > 2 ? 0 : kRowBytes; k_l < 2 * kRowBytes; k_l += kRowBytes) MSA_SCAN4_STEP(MSA_SCAN4_KSTEP, ra_n, rb_n, k_l);
#undef MSA_SCAN4_STEP
    have_prev = true;
    prev_n0 = n0;
    if (!nxt_valid) break;
    tm_c = tm_n; tn_c = tn_n;
    ra_c = ra_n; rb_c = rb_n;
    plan_next();
  }
  asm volatile(MSA_SCAN4_REDUCE ::: MSA_SCAN4_CLOBBERS);
  fold_tile(prev_n0);
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
#endif
}

// chunk_key -> fp32 scores (times scale / Hq); key 0 (query without a scored token) -> -inf.
__global__ void decode_scores_kernel(const uint32_t* __restrict__ key, int64_t n, float mul,
                                     float* __restrict__ out) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const uint32_t k = key[i];
    out[i] = k == 0 ? -INFINITY : key_to_f32(k) * mul;
  }
}

// Optional timing of the scoring kernel alone: event pairs recorded around its launch.  The lock makes the record
// list safe against concurrent callers; while timing is off a launch only reads one atomic flag.
struct KernelTimer {
  std::mutex mu;
  std::atomic<int> on{0};
  hipEvent_t* start = nullptr;
  hipEvent_t* stop = nullptr;
  int cap = 0;
  int n = 0;
} g_timer;

constexpr size_t kLdsPerCu = 160 * 1024;

// Compute units of the current device (asked once; the library drives one device per process).
int compute_units() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    return cus;
  }();
  return n;
}

template <typename T, int BM, int BN, int WAVES_M, int WAVES_N, int kSets, bool kDocMax, bool kStream>
int launch_gemm(const void* qs, const void* kr, const uint32_t* row_bits, uint32_t* out_key, const int32_t* chunk_doc,
                int32_t M_rows, int32_t C, int32_t K, int32_t blocks_per_query, int32_t n_docs, hipStream_t st) {
  const size_t lds = score_tile_is_direct_stream<T, BM, BN, kSets, kStream>() ? (size_t)kDtlStreamLdsBytes
                                                                               : (size_t)2 * (BM + BN) * kRowStride;
  const int tiles_m = (M_rows + BM - 1) / BM;
  const int tiles_n = (C + BN - 1) / BN;
  // M tiles are walked in groups of 8 per K_r tile: a group's query rows (4 MiB in bf16) are what an XCD's L2
  // holds.  At 8 M tiles that is all of them (groups of 1, 2, 4 lose 2-14 % there); with 16 M tiles groups of 8
  // measured 1.4 % faster than one group, with 256 (a 64k-row prefill batch) 4 %.
  const int m_group = std::min(tiles_m, 8);
  const int m_groups = (tiles_m + m_group - 1) / m_group;
  int grid = 8 * ((tiles_n + 7) / 8) * m_groups * m_group;
  if (kStream) {      // one workgroup per slot the compute units offer (LDS decides how many fit), each walking several tiles
    if (tiles_m != 1) {
      msa_set_error("score_gemm: the streaming form takes one M tile, got %d", tiles_m);
      return MSA_EINVAL;
    }
    grid = std::min(tiles_n, compute_units() * std::max<int>(1, (int)(kLdsPerCu / lds)));
  }
  auto kern = score_gemm_kernel<T, BM, BN, WAVES_M, WAVES_N, kSets, kDocMax, kStream>;
  static std::atomic<int> lds_limit_raised{0};
  MSA_HIP(raise_dynamic_lds_limit(lds_limit_raised, reinterpret_cast<const void*>(kern), (int)lds));
  int slot = -1;
  if (g_timer.on.load(std::memory_order_acquire)) {
    std::lock_guard<std::mutex> lock(g_timer.mu);
    if (g_timer.n < g_timer.cap) slot = g_timer.n++;
  }
  if (slot >= 0) MSA_HIP(hipEventRecord(g_timer.start[slot], st));
  kern<<<grid, WAVES_M * WAVES_N * 64, lds, st>>>(static_cast<const T*>(qs), static_cast<const T*>(kr), row_bits, out_key,
                                                  chunk_doc, M_rows, C, K, blocks_per_query, tiles_m, tiles_n, m_group,
                                                  n_docs);
  MSA_LAUNCH_CHECK();
  if (slot >= 0) MSA_HIP(hipEventRecord(g_timer.stop[slot], st));
  return MSA_OK;
}

// Launch of the MFMA-bound form (score_scan4_kernel): one workgroup per compute unit, persistent.
std::atomic<int> g_tile_pool_enabled{1};

template <bool kDocMax>
int launch_scan4(const void* qs, const void* kr, const uint32_t* row_bits, uint32_t* out_key, const int32_t* chunk_doc,
                 int32_t M_rows, int32_t C, int32_t K, int32_t blocks_per_query, int32_t n_docs, hipStream_t st,
                 const GatherJob* job, bool* job_taken, uint32_t* sched) {
  constexpr int BM = 256, BN = 256;
  const int tiles_m = (M_rows + BM - 1) / BM;
  const int tiles_n = (C + BN - 1) / BN;
  const int k_tiles = K * (int)sizeof(bf16_t) / kRowBytes;
  // the loop requests K tiles two steps ahead: at least two K tiles per tile
  if (K * (int)sizeof(bf16_t) % kRowBytes != 0 || k_tiles < 2) {
    msa_set_error("score_scan4: K=%d is not a multiple of 64 of at least 128", K);
    return MSA_EINVAL;
  }
  // M tiles are walked in groups of 8 per K_r tile: a group's query rows (4 MiB in bf16) are what an XCD's L2 holds.
  // At 8 M tiles that is all of them (groups of 1, 2, 4 lose 2-14 % there); with 16 M tiles groups of 8 measured
  // 1.4 % faster than one group, with 256 (a 64k-row prefill batch) 4 %.
  const int m_group = std::min(tiles_m, 8);
  const int grid = std::min(kSchedMaxWorkgroups, std::max(16, compute_units() / 8 * 8));
  // The XCDs do not run at one speed (their ends lay up to 6 % apart with fixed ranges, in an order that changes from
  // launch to launch): the last eighth of the N tiles is a pool the workgroups draw from one tile at a time once
  // their own share is done.  Worth it when a workgroup has tiles enough for the pool to even the ends out, and
  // possible when a tile is deep enough for a draw to come back in time (three hops, one per K step, in front of the
  // step in which the loads leave the tile).
  int pool_n = 0;
  if (g_tile_pool_enabled.load(std::memory_order_relaxed) && (int64_t)tiles_m * tiles_n >= (int64_t)16 * grid && k_tiles >= 6)
    pool_n = tiles_n / 8;
  GatherJob no_job{};
  const GatherJob* the_job = &no_job;
  if (job != nullptr && job->active) {
    the_job = job;
    if (job_taken) *job_taken = true;
  }
  auto kern = score_scan4_kernel<kDocMax>;
  static std::atomic<int> lds_limit_raised{0}, resources_checked{0};
  if (const int rc = check_asm_kernel_resources(resources_checked, reinterpret_cast<const void*>(kern), "score_scan4_kernel",
                                                nullptr, nullptr))
    return rc;
  MSA_HIP(raise_dynamic_lds_limit(lds_limit_raised, reinterpret_cast<const void*>(kern), kScan4LdsBytes));
  int slot = -1;
  if (g_timer.on.load(std::memory_order_acquire)) {
    std::lock_guard<std::mutex> lock(g_timer.mu);
    if (g_timer.n < g_timer.cap) slot = g_timer.n++;
  }
  if (slot >= 0) MSA_HIP(hipEventRecord(g_timer.start[slot], st));
  kern<<<grid, 256, kScan4LdsBytes, st>>>(static_cast<const bf16_t*>(qs), static_cast<const bf16_t*>(kr), row_bits, out_key,
                                          chunk_doc, M_rows, C, K, blocks_per_query, tiles_m, tiles_n, m_group, n_docs,
                                          *the_job, sched, pool_n);
  MSA_LAUNCH_CHECK();
  if (slot >= 0) MSA_HIP(hipEventRecord(g_timer.stop[slot], st));
  return MSA_OK;
}

// Tile choice by query rows.  Up to 64 rows: narrow M tile, two workgroups per compute unit, two K tiles of global
// loads ahead (3 % faster than one).  Up to 128 rows: 128 x 256 with both operands loaded straight into LDS two K steps
// ahead (1.5 % faster than the register-staged 128 x 384 it replaced, which beat register-staged 128 x 256 by 3 % and
// 128 x 128 by 8 %; more register sets of loads in flight or 16 wavefronts measured 0-6 % slower: the bytes in flight
// are not what limits this shape, the query tile's own traffic and the MFMA work are - with a query tile of zeros the
// same launch streams at the rate of the 64-row form).  More rows are MFMA-bound: the 256 x 256 tile of
// score_scan4_kernel, which is also the form that can carry a gather job.
template <bool kDocMax>
int launch_gemm_for(int32_t dtype, const void* qs, const void* kr, const uint32_t* row_bits, uint32_t* out_key,
                    const int32_t* chunk_doc, int32_t M_rows, int32_t C, int32_t K, int32_t bpq, int32_t n_docs,
                    hipStream_t st, const GatherJob* job, bool* job_taken, uint32_t* sched) {
  if (dtype != MSA_BF16)
    return launch_gemm<float, 128, 128, 2, 2, 1, kDocMax, false>(qs, kr, row_bits, out_key, chunk_doc, M_rows, C, K, bpq, n_docs, st);
  if (M_rows <= 64)
    return launch_gemm<bf16_t, 64, 128, 2, 2, 2, kDocMax, true>(qs, kr, row_bits, out_key, chunk_doc, M_rows, C, K, bpq, n_docs, st);
  if (M_rows <= 128)
    return launch_gemm<bf16_t, 128, 256, 2, 4, 1, kDocMax, true>(qs, kr, row_bits, out_key, chunk_doc, M_rows, C, K, bpq, n_docs, st);
  return launch_scan4<kDocMax>(qs, kr, row_bits, out_key, chunk_doc, M_rows, C, K, bpq, n_docs, st, job, job_taken, sched);
}

}  // namespace

// ------------------------------------------------------------------------------------------
// Workspace layout (shared with topk.hip through route_internal.h)
// ------------------------------------------------------------------------------------------

RouteWorkspace route_workspace_layout(int32_t B, int32_t S, int32_t Hkv, int32_t D, int64_t plane_cols, int64_t n_docs,
                                      int32_t dtype) {
  RouteWorkspace w{};
  w.S_pad = (S + 31) / 32 * 32;
  w.M_rows = B * w.S_pad;
  const int64_t m_alloc = ((int64_t)w.M_rows + 255) / 256 * 256;   // every M tile may read whole mask words
  w.mask_words = (int32_t)(m_alloc / 32);
  size_t off = 0;
  w.off_qs = off;       off = align_up(off + (size_t)w.M_rows * Hkv * D * elem_bytes(dtype), 256);
  w.off_row_bits = off; off = align_up(off + (size_t)w.mask_words * sizeof(uint32_t), 256);
  w.off_key = off;      off = align_up(off + (size_t)B * plane_cols * sizeof(uint32_t), 256);
  w.topk_blocks = topk_blocks_for(n_docs);
  w.off_cand = off;     off = align_up(off + (size_t)B * w.topk_blocks * kTopkMax * sizeof(uint64_t), 256);
  w.off_sched = off;    off = align_up(off + kSchedBytes, 256);
  w.off_collapsed = off; off = align_up(off + (size_t)B * Hkv * D * sizeof(float) + (size_t)B * sizeof(int32_t), 256);
  w.bytes = off;
  return w;
}

// Host-side replay of the large-tile scan's tile order (scan_walk.h): every scoring workgroup walks its own tiles
// with the cursor the kernel uses, then the workgroups draw the pool's tiles in turn from one counter.
extern "C" int msa_diag_scan_walk(int32_t tiles_m, int32_t tiles_n, int32_t grid, int32_t has_copy_workgroup,
                                  int32_t pool_n, int32_t* visits) {
  MSA_REQUIRE(visits != nullptr, "msa_diag_scan_walk: null output");
  MSA_REQUIRE(tiles_m > 0 && tiles_n > 0 && grid >= 16 && grid <= kSchedMaxWorkgroups && pool_n >= 0 && pool_n <= tiles_n,
              "msa_diag_scan_walk: tiles %d x %d, grid %d, pool %d out of range", tiles_m, tiles_n, grid, pool_n);
  const int m_group = std::min(tiles_m, 8);
  for (int64_t i = 0; i < (int64_t)tiles_m * tiles_n; ++i) visits[i] = 0;
  const int scoring = grid - (has_copy_workgroup ? 1 : 0);
  std::vector<int> draws;
  for (int b = 0; b < scoring; ++b) {
    const ScanWalk w = scan_walk_init(b, grid, has_copy_workgroup, tiles_m, tiles_n, m_group, pool_n);
    if (w.own_count == 0) continue;
    ScanWalkCursor c = scan_walk_cursor(w);
    for (int idx = 0; idx < w.own_count; ++idx) {
      int tm, tn, tm2, tn2;
      scan_walk_cursor_tile(w, c, tm, tn);
      scan_walk_own(w, idx, tm2, tn2);
      if (tm != tm2 || tn != tn2 || tm < 0 || tm >= tiles_m || tn < 0 || tn >= tiles_n) {
        msa_set_error("msa_diag_scan_walk: workgroup %d tile %d: cursor (%d, %d), closed form (%d, %d)", b, idx, tm, tn, tm2, tn2);
        return MSA_ESTATE;
      }
      ++visits[(int64_t)tm * tiles_n + tn];
      if (idx + 1 < w.own_count) scan_walk_cursor_next(w, c);
    }
    draws.push_back(b);
  }
  int counter = 0;
  while (pool_n > 0 && !draws.empty()) {
    std::vector<int> still;
    for (int b : draws) {
      const ScanWalk w = scan_walk_init(b, grid, has_copy_workgroup, tiles_m, tiles_n, m_group, pool_n);
      const int p = counter++;
      if (p >= w.pool_total) continue;
      int tm, tn;
      scan_walk_pool(w, p, tm, tn);
      if (tm < 0 || tm >= tiles_m || tn < 0 || tn >= tiles_n) {
        msa_set_error("msa_diag_scan_walk: pool position %d -> (%d, %d)", p, tm, tn);
        return MSA_ESTATE;
      }
      ++visits[(int64_t)tm * tiles_n + tn];
      still.push_back(b);
    }
    draws.swap(still);
  }
  return MSA_OK;
}

// The tile pool of the large-tile scan can be switched off (every tile then belongs to a fixed workgroup).
extern "C" int msa_diag_asm_kernel_resources(int32_t which, int32_t* num_regs, int32_t* scratch_bytes) {
  MSA_REQUIRE(num_regs && scratch_bytes, "msa_diag_asm_kernel_resources: null pointer");
  std::atomic<int> unused{0};
  int regs = 0, scratch = 0, rc;
  if (which == 0)
    rc = check_asm_kernel_resources(unused, reinterpret_cast<const void*>(score_scan4_kernel<true>), "score_scan4_kernel", &regs,
                                    &scratch);
  else if (which == 1)
    rc = flash_wide_kernel_resources(&regs, &scratch);
  else {
    msa_set_error("msa_diag_asm_kernel_resources: which = 0 (routing scan) or 1 (wide flash attention)");
    return MSA_EINVAL;
  }
  *num_regs = regs;
  *scratch_bytes = scratch;
  return rc;
}

extern "C" int msa_route_set_tile_pool(int32_t enabled) {
  g_tile_pool_enabled.store(enabled ? 1 : 0, std::memory_order_relaxed);
  return MSA_OK;
}

extern "C" int msa_profile_enable(int32_t max_records) {
  std::lock_guard<std::mutex> lock(g_timer.mu);
  g_timer.on.store(0, std::memory_order_release);
  for (int i = 0; i < g_timer.cap; ++i) {
    (void)hipEventDestroy(g_timer.start[i]);
    (void)hipEventDestroy(g_timer.stop[i]);
  }
  delete[] g_timer.start;
  delete[] g_timer.stop;
  g_timer.start = g_timer.stop = nullptr;
  g_timer.cap = g_timer.n = 0;
  MSA_REQUIRE(max_records >= 0 && max_records <= 1 << 20, "msa_profile_enable: max_records=%d", max_records);
  if (max_records == 0) return MSA_OK;
  g_timer.start = new hipEvent_t[max_records];
  g_timer.stop = new hipEvent_t[max_records];
  for (int i = 0; i < max_records; ++i) {
    MSA_HIP(hipEventCreate(&g_timer.start[i]));
    MSA_HIP(hipEventCreate(&g_timer.stop[i]));
    g_timer.cap = i + 1;
  }
  g_timer.on.store(1, std::memory_order_release);
  return MSA_OK;
}

extern "C" int msa_profile_collect(float* ms_host, int32_t cap, int32_t* n_out) {
  MSA_REQUIRE(ms_host && n_out, "msa_profile_collect: null pointer");
  std::lock_guard<std::mutex> lock(g_timer.mu);
  const int n = std::min(g_timer.n, cap);
  for (int i = 0; i < n; ++i) {
    MSA_HIP(hipEventSynchronize(g_timer.stop[i]));
    MSA_HIP(hipEventElapsedTime(&ms_host[i], g_timer.start[i], g_timer.stop[i]));
  }
  *n_out = n;
  g_timer.n = 0;
  return MSA_OK;
}

extern "C" size_t msa_route_workspace_bytes(int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D, int64_t C,
                                            int64_t n_docs, int32_t topk) {
  (void)Hq; (void)topk;
  if (B <= 0 || S <= 0 || Hkv <= 0 || D <= 0 || C <= 0 || n_docs <= 0) return 0;
  // sized for fp32 queries so one workspace serves both dtypes, and for the per-chunk plane of msa_chunk_scores
  return route_workspace_layout(B, S, Hkv, D, C + n_docs, n_docs, MSA_F32).bytes;
}

extern "C" size_t msa_route_topk_workspace_bytes(int32_t B, int32_t S, int32_t Hq, int32_t Hkv, int32_t D,
                                                 int64_t n_docs, int32_t topk) {
  (void)Hq; (void)topk;
  if (B <= 0 || S <= 0 || Hkv <= 0 || D <= 0 || n_docs <= 0) return 0;
  return route_workspace_layout(B, S, Hkv, D, n_docs, n_docs, MSA_F32).bytes;
}

int route_scores_to_keys(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B,
                         int32_t S, int32_t Hq, int32_t mode, float scale, bool doc_max, void* workspace,
                         size_t workspace_bytes, hipStream_t st, RouteWorkspace* layout_out, float* mul_out,
                         const char* who, const GatherJob* job, bool* job_taken, int32_t query_reduce,
                         int64_t extra_plane_cols) {
  if (job_taken) *job_taken = false;
  MSA_REQUIRE(query_reduce == kQueryMax || query_reduce == kQueryMean || query_reduce == kQueryLast,
              "%s: bad query reduction %d", who, query_reduce);
  MSA_REQUIRE(bank != nullptr, "%s: null bank", who);
  MSA_REQUIRE(layer >= 0 && layer < bank->n_layers, "%s: layer %d out of range", who, layer);
  if (bank->kr_dev[layer] == nullptr) {
    msa_set_error("%s: layer %d has no K_r set", who, layer);
    return MSA_ESTATE;
  }
  MSA_REQUIRE(q != nullptr && workspace != nullptr, "%s: null pointer", who);
  MSA_REQUIRE(B > 0 && B <= 4096 && S > 0 && S <= 65536, "%s: B=%d S=%d out of range", who, B, S);
  MSA_REQUIRE(Hq > 0 && Hq % bank->Hkv == 0, "%s: Hq=%d not a multiple of Hkv=%d", who, Hq, bank->Hkv);
  MSA_REQUIRE(bank->Hkv <= 16, "%s: Hkv=%d unsupported (max 16)", who, bank->Hkv);
  MSA_REQUIRE(mode == MSA_MODE_COSINE || mode == MSA_MODE_SCALED_DOT, "%s: bad mode %d", who, mode);
  MSA_REQUIRE(((uintptr_t)q & 15) == 0 && ((uintptr_t)workspace & 255) == 0, "%s: q / workspace misaligned", who);
  const float sc = mode == MSA_MODE_COSINE ? 1.0f : scale;
  MSA_REQUIRE(sc > 0.f && sc < INFINITY, "%s: scale must be positive and finite", who);
  MSA_REQUIRE((int64_t)B * ((S + 31) / 32 * 32) < (int64_t)1 << 24, "%s: too many query rows", who);

  const int64_t plane_cols = doc_max ? bank->n_docs : bank->C;
  // a collapsed query (mean / last over its tokens) is one row: one row block per query
  const int32_t S_scan = query_reduce == kQueryMax ? S : 1;
  const RouteWorkspace w = route_workspace_layout(B, S_scan, bank->Hkv, bank->D, plane_cols + extra_plane_cols, bank->n_docs,
                                                  bank->dtype);
  if (w.bytes > workspace_bytes) {
    msa_set_error("%s: workspace of %zu bytes, need %zu", who, workspace_bytes, w.bytes);
    return MSA_ESIZE;
  }
  char* ws = static_cast<char*>(workspace);
  void* qs = ws + w.off_qs;
  uint32_t* row_bits = reinterpret_cast<uint32_t*>(ws + w.off_row_bits);
  uint32_t* key = reinterpret_cast<uint32_t*>(ws + w.off_key);
  uint32_t* sched = reinterpret_cast<uint32_t*>(ws + w.off_sched);

  const int normalize = mode == MSA_MODE_COSINE ? 1 : 0;
  const int pthreads = bank->Hkv * 16;
  const int64_t clear_words = (int64_t)B * plane_cols;
  if (query_reduce != kQueryMax) {
    float* rows = reinterpret_cast<float*>(ws + w.off_collapsed);
    int32_t* counts = reinterpret_cast<int32_t*>(rows + (size_t)B * bank->Hkv * bank->D);
    const dim3 cgrid((unsigned)B, (unsigned)bank->Hkv);
    if (bank->dtype == MSA_BF16) {
      collapse_queries_kernel<bf16_t><<<cgrid, 256, 0, st>>>(static_cast<const bf16_t*>(q), qmask_u8, S, Hq, bank->Hkv,
                                                             normalize, query_reduce, rows, counts);
      MSA_LAUNCH_CHECK();
      broadcast_rows_kernel<bf16_t><<<w.M_rows, 256, 0, st>>>(rows, counts, bank->Hkv, static_cast<bf16_t*>(qs), row_bits,
                                                              w.mask_words, key, clear_words, sched);
    } else {
      collapse_queries_kernel<float><<<cgrid, 256, 0, st>>>(static_cast<const float*>(q), qmask_u8, S, Hq, bank->Hkv,
                                                            normalize, query_reduce, rows, counts);
      MSA_LAUNCH_CHECK();
      broadcast_rows_kernel<float><<<w.M_rows, 256, 0, st>>>(rows, counts, bank->Hkv, static_cast<float*>(qs), row_bits,
                                                             w.mask_words, key, clear_words, sched);
    }
  } else if (bank->dtype == MSA_BF16) {
    presum_queries_kernel<bf16_t, bf16_t><<<w.M_rows, pthreads, 0, st>>>(
        static_cast<const bf16_t*>(q), qmask_u8, B, S, w.S_pad, Hq, bank->Hkv, normalize, static_cast<bf16_t*>(qs),
        row_bits, w.mask_words, key, clear_words, sched);
  } else {
    presum_queries_kernel<float, float><<<w.M_rows, pthreads, 0, st>>>(
        static_cast<const float*>(q), qmask_u8, B, S, w.S_pad, Hq, bank->Hkv, normalize, static_cast<float*>(qs),
        row_bits, w.mask_words, key, clear_words, sched);
  }
  MSA_LAUNCH_CHECK();

  const int32_t K = bank->Hkv * bank->D;
  const int32_t bpq = w.S_pad / 32;
  const int rc = doc_max ? launch_gemm_for<true>(bank->dtype, qs, bank->kr_dev[layer], row_bits, key, bank->chunk_doc_dev,
                                                 w.M_rows, (int32_t)bank->C, K, bpq, (int32_t)bank->n_docs, st, job,
                                                 job_taken, sched)
                         : launch_gemm_for<false>(bank->dtype, qs, bank->kr_dev[layer], row_bits, key, nullptr, w.M_rows,
                                                  (int32_t)bank->C, K, bpq, (int32_t)bank->n_docs, st, job, job_taken, sched);
  if (rc != MSA_OK) return rc;
  *layout_out = w;
  *mul_out = sc / (float)Hq;
  return MSA_OK;
}

extern "C" int msa_chunk_scores(const msa_bank* bank, int32_t layer, const void* q, const uint8_t* qmask_u8, int32_t B,
                                int32_t S, int32_t Hq, int32_t mode, float scale, float* chunk_scores,
                                void* workspace, size_t workspace_bytes, void* stream) {
  MSA_REQUIRE(chunk_scores != nullptr, "msa_chunk_scores: null output");
  RouteWorkspace w;
  float mul;
  hipStream_t st = as_stream(stream);
  int rc = route_scores_to_keys(bank, layer, q, qmask_u8, B, S, Hq, mode, scale, false, workspace, workspace_bytes, st,
                                &w, &mul, "msa_chunk_scores");
  if (rc != MSA_OK) return rc;
  const int64_t n = (int64_t)B * bank->C;
  const uint32_t* key = reinterpret_cast<const uint32_t*>(static_cast<char*>(workspace) + w.off_key);
  decode_scores_kernel<<<(int)std::min<int64_t>((n + 255) / 256, 8192), 256, 0, st>>>(key, n, mul, chunk_scores);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}
