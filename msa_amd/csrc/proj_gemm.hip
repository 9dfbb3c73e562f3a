// Fused projection of a block of tokens: one bf16 NT GEMM  x[T, K] . w[N, K]^T  over the concatenated router / q / k /
// v weights whose epilogue finishes the heads in registers: q and k heads get their per-head RMSNorm and the
// half-split rotary at the token's position, v and router heads are stored as they are.  Replaces the separate
// q_proj / k_proj / v_proj / router_*_proj GEMMs and the norm + rotary pass behind them
// (src/msa/memory_sparse_attention.py:125-133, 178, 263) on the encode (stage 1) and query-prefill (stage 2) paths.
//
// Tile 256 x 256, K tile 64, eight wavefronts as 4 (tokens) x 2 (heads): a wavefront owns 64 tokens x one whole
// 128-wide head; after the main loop it parks the block in LDS and finishes it row-wise (16 lanes per token row), where
// the norm's sum of squares is a 16-lane reduction and a rotary pair (d, d + 64) is the lane 8 places away.  The main
// loop is the one of the
// scoring kernel's large-tile form: operand tiles loaded straight into LDS through buffer resources whose extent is the
// valid part of the tile, two stages of the token tile and three of the weight tile, operand fragments one sub-step
// ahead, one barrier per K tile.
#include <algorithm>
#include <type_traits>

#include "common.h"

namespace {

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kRowBytes = 128;                 // one K tile of a row: 64 bf16
constexpr int BM = 256, BN = 256, WAVES_M = 4, WAVES_N = 2;
constexpr int kThreads = WAVES_M * WAVES_N * 64;
constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;      // 64 tokens x 128 columns (one head) per wavefront
constexpr int TM = WM / 32, TN = WN / 32;
constexpr int kLdsBytes = 5 * 256 * 128;       // two stages of the token tile, three of the weight tile
constexpr int kSub = 4;                        // 32x32x16 steps per K tile
static_assert(WN == kHeadDim, "a wavefront owns whole heads");

struct ProjArgs {
  const bf16_t* x;          // [T, K]
  const bf16_t* w;          // [N, K], heads in the order: front plain heads | q | k | v | back plain heads
  const int64_t* pos;       // [T]
  const bf16_t* q_norm_w;   // [128]
  const bf16_t* k_norm_w;   // [128]
  const float* rope_cos;    // [rope_rows, 64]
  const float* rope_sin;
  bf16_t* q_out;            // [T, Hq, 128]
  bf16_t* k_out;            // [T, Hkv, 128]
  bf16_t* v_out;            // [T, Hkv, 128]
  bf16_t* r_out;            // [T, Hr_front + Hr_back, 128]
  int32_t T, K, N;
  int32_t Hq, Hkv, Hr_front, Hr_back;
  int32_t rope_rows;
  float eps;
  int32_t tiles_m, tiles_n, m_group;
};

__global__ __launch_bounds__(kThreads) void proj_gemm_kernel(ProjArgs a) {
  extern __shared__ __align__(16) char lds[];

  // Each XCD (workgroups are dealt to the 8 XCDs round-robin) takes a contiguous range of token tiles, so the
  // activations are read from HBM once; inside it groups of m_group token tiles share every weight tile while it is hot.
  const int m_per_xcd = (a.tiles_m + 7) / 8;
  const int within = blockIdx.x / 8;
  const int per_group = a.tiles_n * a.m_group;
  const int rem = within % per_group;
  const int tile_m = (blockIdx.x % 8) * m_per_xcd + (within / per_group) * a.m_group + rem % a.m_group;
  const int tile_n = rem / a.m_group;
  if (tile_m >= a.tiles_m || tile_m >= (int)(blockIdx.x % 8 + 1) * m_per_xcd) return;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63;
  // (wave-uniform by construction; said so, the LDS addresses of the direct loads stay in scalar registers instead of
  // being read back from a lane in front of every load: 1.9 % on the large-tile scan)
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int half = lane >> 5, l32 = lane & 31;

  const int row_bytes_g = a.K * 2;
  const int rows_a = min(BM, a.T - m0), rows_b = min(BN, a.N - n0);
  const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(reinterpret_cast<const char*>(a.x)) + (int64_t)m0 * row_bytes_g, 0, rows_a * row_bytes_g, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrc_b = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(reinterpret_cast<const char*>(a.w)) + (int64_t)n0 * row_bytes_g, 0, rows_b * row_bytes_g, 0x00020000);
  const int k_tiles = row_bytes_g / kRowBytes;

  floatx16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // Operand tiles go from global memory straight into LDS (buffer_load ... lds): two stages of the token tile, three of
  // the weight tile, 32 KB each, in un-padded 128-byte rows whose 16-byte units are XOR-swizzled by (row >> 1) & 7 (a
  // direct load cannot pad: its 64 lanes fill 1 KB of LDS in lane order, so the swizzle is applied to the global
  // address each lane fetches; operand reads stay conflict-free).  Token tile kt + 1 and weight tile kt + 2 are
  // requested at the start of step kt; the wait in front of the step's barrier leaves the newest weight tile in
  // flight.  A wavefront's load i covers rows (wave * 4 + i) * 8 .. + 8 of a tile.
  constexpr int kStageBytes = 256 * 128;
  const int dtl_row = lane >> 3, dtl_slot = lane & 7;
  auto dtl_voff = [&](int i) {
    const int row = (wave * 4 + i) * 8 + dtl_row;
    return row * row_bytes_g + ((dtl_slot ^ ((row >> 1) & 7)) * 16);
  };
  auto load_a = [&](int stage, int kt) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      MSA_LOAD_TO_LDS(rsrc_a, lds + stage * kStageBytes + (wave * 4 + i) * 1024, dtl_voff(i), kt * kRowBytes, 0);
  };
  auto load_b = [&](int stage, int kt) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      MSA_LOAD_TO_LDS(rsrc_b, lds + (2 + stage) * kStageBytes + (wave * 4 + i) * 1024, dtl_voff(i), kt * kRowBytes, 0);
  };
  bf16x8_t fa[2][TM], fb[2][TN];
  auto load_frags = [&](int sa, int sb, int sub, int slot) {
    const int unit = sub * 2 + half;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int row = wm * WM + i * 32 + l32;
      fa[slot][i] = *reinterpret_cast<const bf16x8_t*>(lds + sa * kStageBytes + row * 128 + ((unit ^ ((row >> 1) & 7)) * 16));
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int row = wn * WN + j * 32 + l32;
      fb[slot][j] = *reinterpret_cast<const bf16x8_t*>(lds + (2 + sb) * kStageBytes + row * 128 + ((unit ^ ((row >> 1) & 7)) * 16));
    }
  };
  // vmcnt(4) / vmcnt(0) with the other counters left alone: the four newest loads are the weight tile two steps ahead.
  // The barrier is written out: __syncthreads() carries a release fence for which the compiler drains every load that
  // writes LDS, the tile two steps ahead included.
  constexpr int kWaitAllButNewestB = 0x0F74, kWaitAll = 0x0F70;
  auto barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
  load_a(0, 0);
  load_b(0, 0);
  if (k_tiles > 1) {
    load_b(1, 1);
    __builtin_amdgcn_s_waitcnt(kWaitAllButNewestB);
  } else {
    __builtin_amdgcn_s_waitcnt(kWaitAll);
  }
  barrier();
  load_frags(0, 0, 0, 0);
  int sa = 0, sb = 0;
  for (int kt = 0; kt < k_tiles; ++kt) {
    const int sb1 = sb == 2 ? 0 : sb + 1, sb2 = sb1 == 2 ? 0 : sb1 + 1;
    const bool more = kt + 1 < k_tiles, more2 = kt + 2 < k_tiles;
    if (more) load_a(sa ^ 1, kt + 1);       // stage of the step before this one: its last reads were behind the previous barrier
    if (more2) load_b(sb2, kt + 2);
    auto substep = [&](auto sub_tag, auto fresh_tag) {
      constexpr int sub = decltype(sub_tag)::value;
      constexpr bool fresh = decltype(fresh_tag)::value;
      if constexpr (sub + 1 < kSub) {
        load_frags(sa, sb, sub + 1, (sub + 1) & 1);
      } else {
        if (more) {
          if (more2) __builtin_amdgcn_s_waitcnt(kWaitAllButNewestB);
          else __builtin_amdgcn_s_waitcnt(kWaitAll);
          barrier();
          load_frags(sa ^ 1, sb1, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          if constexpr (fresh) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[sub & 1][i], fb[sub & 1][j], floatx16_t{}, 0, 0, 0);
          else acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[sub & 1][i], fb[sub & 1][j], acc[i][j], 0, 0, 0);
        }
      if constexpr (sub + 1 < kSub) {
        // issue order of the sub-step: each of the six operand reads of the next sub-step behind one MFMA of this one
#pragma unroll
        for (int g = 0; g < TM + TN; ++g) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);   // one MFMA
          __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);   // one LDS read
        }
        __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - TM - TN, 0);
      }
    };
    if (kt == 0) substep(std::integral_constant<int, 0>{}, std::true_type{});
    else substep(std::integral_constant<int, 0>{}, std::false_type{});
    substep(std::integral_constant<int, 1>{}, std::false_type{});
    substep(std::integral_constant<int, 2>{}, std::false_type{});
    substep(std::integral_constant<int, 3>{}, std::false_type{});
    sa ^= 1;
    sb = sb1;
  }

  // Epilogue: this wavefront holds head `head` for 64 tokens.  acc[i][j][e] is token row 8*(e/4) + 4*half + e%4 of
  // row block i, column j*32 + l32 of the head.
  const int head = (n0 + wn * WN) / kHeadDim;
  const int h_q0 = a.Hr_front, h_k0 = h_q0 + a.Hq, h_v0 = h_k0 + a.Hkv, h_b0 = h_v0 + a.Hkv, h_end = h_b0 + a.Hr_back;
  __syncthreads();                                         // every wavefront is done reading operand tiles
  if (head >= h_end) return;                               // half of the last N tile may lie past the last head
  bf16_t* dst;
  int dst_heads, dst_h;
  const bf16_t* norm_w = nullptr;
  if (head < h_q0) { dst = a.r_out; dst_heads = a.Hr_front + a.Hr_back; dst_h = head; }
  else if (head < h_k0) { dst = a.q_out; dst_heads = a.Hq; dst_h = head - h_q0; norm_w = a.q_norm_w; }
  else if (head < h_v0) { dst = a.k_out; dst_heads = a.Hkv; dst_h = head - h_k0; norm_w = a.k_norm_w; }
  else if (head < h_b0) { dst = a.v_out; dst_heads = a.Hkv; dst_h = head - h_v0; }
  else { dst = a.r_out; dst_heads = a.Hr_front + a.Hr_back; dst_h = a.Hr_front + head - h_b0; }
  // Each wavefront parks its 64 x 128 block (rounded to bf16, as the projection's output is) in its own slice of LDS
  // and takes it back row-wise: 16 lanes per token row, 8 consecutive dims per lane.  In that layout the norm's sum of
  // squares is a 16-lane DPP reduction, a rotary pair (d, d + 64) is the lane 8 places away, a row's cosines and sines
  // are two 16-byte reads each, and a row leaves as sixteen 16-byte stores (256 contiguous bytes of the dense
  // output).  (Taking the products transposed instead, so that a lane holds half a token's head and nothing is
  // parked, measured 3 % slower: its table reads and 8-byte stores touch 32 cache lines per instruction.)
  constexpr int kOutStride = kHeadDim * 2 + 16;            // bytes per parked row; the pad keeps the two halves apart
  char* park = lds + wave * (WM * kOutStride);
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      const int r = i * 32 + 8 * (e >> 2) + 4 * half + (e & 3);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        *reinterpret_cast<bf16_t*>(park + r * kOutStride + (j * 32 + l32) * 2) = f32_to_bf16(acc[i][j][e]);
    }
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  const int jl = lane & 15, rl = lane >> 4;                // 8 dims [8 jl, 8 jl + 8) of row rl of each group of four
  float w8[8];
  if (norm_w != nullptr) {
    const uint4 ww = *reinterpret_cast<const uint4*>(norm_w + 8 * jl);
    w8[0] = bf16lo(ww.x); w8[1] = bf16hi(ww.x); w8[2] = bf16lo(ww.y); w8[3] = bf16hi(ww.y);
    w8[4] = bf16lo(ww.z); w8[5] = bf16hi(ww.z); w8[6] = bf16lo(ww.w); w8[7] = bf16hi(ww.w);
  }
  const int f = 8 * (jl & 7);                              // frequency index of this lane's first dim
  const float sgn = jl < 8 ? -1.0f : 1.0f;
  // Eight row groups at a time: their positions first, then all their table reads, then the arithmetic, so the two
  // dependent global loads of a row (position, then cosines / sines at it) are each paid once per batch, not per row.
  constexpr int kBatch = 8;
#pragma unroll
  for (int g0 = 0; g0 < WM / 4; g0 += kBatch) {
    int64_t p[kBatch];
    float4 c0[kBatch], c1[kBatch], s0[kBatch], s1[kBatch];
    if (norm_w != nullptr) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int row = m0 + wm * WM + (g0 + u) * 4 + rl;
        p[u] = row < a.T ? a.pos[row] : 0;
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int64_t pc = min((int64_t)max((int64_t)0, p[u]), (int64_t)a.rope_rows - 1);
        const float* ct = a.rope_cos + pc * 64 + f;
        const float* st = a.rope_sin + pc * 64 + f;
        c0[u] = *reinterpret_cast<const float4*>(ct); c1[u] = *reinterpret_cast<const float4*>(ct + 4);
        s0[u] = *reinterpret_cast<const float4*>(st); s1[u] = *reinterpret_cast<const float4*>(st + 4);
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int r = (g0 + u) * 4 + rl;
      const int row = m0 + wm * WM + r;
      const uint4 raw = *reinterpret_cast<const uint4*>(park + r * kOutStride + jl * 16);
      uint4 outw = raw;
      if (norm_w != nullptr) {
        const float x[8] = {bf16lo(raw.x), bf16hi(raw.x), bf16lo(raw.y), bf16hi(raw.y),
                            bf16lo(raw.z), bf16hi(raw.z), bf16lo(raw.w), bf16hi(raw.w)};
        float ssq = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) ssq += x[i] * x[i];
        const float inv = rsqrtf(row16_sum(ssq) * (1.0f / kHeadDim) + a.eps);
        // dims d < 64 (lanes jl < 8) leave as y c - y' s, their partners d + 64 as y c + y' s, y' the value 8 lanes away
        const float cs[8] = {c0[u].x, c0[u].y, c0[u].z, c0[u].w, c1[u].x, c1[u].y, c1[u].z, c1[u].w};
        const float sn[8] = {s0[u].x, s0[u].y, s0[u].z, s0[u].w, s1[u].x, s1[u].y, s1[u].z, s1[u].w};
        float o[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float y = x[i] * (inv * w8[i]);
          o[i] = y * cs[i] + row16_ror8(y) * (sn[i] * sgn);
        }
        outw.x = pack_bf16x2(o[0], o[1]); outw.y = pack_bf16x2(o[2], o[3]);
        outw.z = pack_bf16x2(o[4], o[5]); outw.w = pack_bf16x2(o[6], o[7]);
      }
      if (row < a.T) *reinterpret_cast<uint4*>(dst + ((int64_t)row * dst_heads + dst_h) * kHeadDim + 8 * jl) = outw;
    }
  }
}

}  // namespace

extern "C" int msa_qkv_proj(const void* x, int64_t T, int32_t K, const void* w, int32_t Hq, int32_t Hkv, int32_t Hr_front,
                            int32_t Hr_back, const int64_t* positions, const void* q_norm_w, const void* k_norm_w,
                            float eps, const float* rope_cos, const float* rope_sin, int32_t rope_rows, void* q_out,
                            void* k_out, void* v_out, void* r_out, void* stream) {
  MSA_REQUIRE(x && w && positions && q_norm_w && k_norm_w && rope_cos && rope_sin && q_out && k_out && v_out,
              "msa_qkv_proj: null pointer");
  MSA_REQUIRE(T > 0 && T < ((int64_t)1 << 22), "msa_qkv_proj: T=%lld out of range", (long long)T);
  MSA_REQUIRE(K >= 64 && K % 64 == 0 && K <= 32768, "msa_qkv_proj: K=%d (a multiple of 64 up to 32768)", K);
  MSA_REQUIRE(Hq > 0 && Hkv > 0 && Hr_front >= 0 && Hr_back >= 0, "msa_qkv_proj: bad head counts");
  MSA_REQUIRE((Hr_front + Hr_back == 0) || r_out != nullptr, "msa_qkv_proj: router heads without an output");
  MSA_REQUIRE(rope_rows > 0 && eps > 0.f, "msa_qkv_proj: rope_rows / eps");
  MSA_REQUIRE((((uintptr_t)x | (uintptr_t)w) & 15) == 0, "msa_qkv_proj: x / w must be 16-byte aligned");
  MSA_REQUIRE((((uintptr_t)q_norm_w | (uintptr_t)k_norm_w) & 15) == 0,
              "msa_qkv_proj: q_norm_w / k_norm_w (128 bf16 each) must be 16-byte aligned");
  MSA_REQUIRE((((uintptr_t)rope_cos | (uintptr_t)rope_sin) & 3) == 0 &&
                  (((uintptr_t)q_out | (uintptr_t)k_out | (uintptr_t)v_out | (uintptr_t)r_out) & 15) == 0,
              "msa_qkv_proj: rope tables (fp32 [rope_rows, 64]) 4-byte and outputs 16-byte aligned");
  const int64_t heads = (int64_t)Hq + 2 * Hkv + Hr_front + Hr_back;
  MSA_REQUIRE(heads * kHeadDim < ((int64_t)1 << 20), "msa_qkv_proj: too many heads");
  MSA_REQUIRE((int64_t)BM * K * 2 < ((int64_t)1 << 31), "msa_qkv_proj: K too large");
  ProjArgs a{};
  a.x = static_cast<const bf16_t*>(x); a.w = static_cast<const bf16_t*>(w); a.pos = positions;
  a.q_norm_w = static_cast<const bf16_t*>(q_norm_w); a.k_norm_w = static_cast<const bf16_t*>(k_norm_w);
  a.rope_cos = rope_cos; a.rope_sin = rope_sin;
  a.q_out = static_cast<bf16_t*>(q_out); a.k_out = static_cast<bf16_t*>(k_out); a.v_out = static_cast<bf16_t*>(v_out);
  a.r_out = static_cast<bf16_t*>(r_out);
  a.T = (int32_t)T; a.K = K; a.N = (int32_t)(heads * kHeadDim);
  a.Hq = Hq; a.Hkv = Hkv; a.Hr_front = Hr_front; a.Hr_back = Hr_back; a.rope_rows = rope_rows; a.eps = eps;
  a.tiles_m = (a.T + BM - 1) / BM; a.tiles_n = (a.N + BN - 1) / BN;
  a.m_group = std::min(4, (a.tiles_m + 7) / 8);
  const int m_per_xcd = (a.tiles_m + 7) / 8;
  const int groups = (m_per_xcd + a.m_group - 1) / a.m_group;
  const int64_t grid = (int64_t)8 * groups * a.m_group * a.tiles_n;
  MSA_REQUIRE(grid < ((int64_t)1 << 31), "msa_qkv_proj: grid too large");
  const size_t lds = (size_t)kLdsBytes;
  static std::atomic<int> lds_limit_raised{0};
  MSA_HIP(raise_dynamic_lds_limit(lds_limit_raised, reinterpret_cast<const void*>(proj_gemm_kernel), (int)lds));
  proj_gemm_kernel<<<(unsigned)grid, kThreads, lds, as_stream(stream)>>>(a);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}
