// MFMA flash attention for blocks of query rows (stage-1 document-wise attention, stage-2 query
// prefill): bf16, GQA, ragged samples, bottom-right-aligned causal mask.
//
// A workgroup of 4 wavefronts serves one KV head and a block of 128 / G query tokens of one
// sample (G = query heads per KV head); a wavefront owns 32 (token, head) columns.  K / V tiles of
// 64 keys go through LDS once per workgroup.  Per tile a wavefront computes
//   S^T[64 keys x 32 cols] = K . Q^T          (v_mfma_f32_32x32x16_bf16, contraction over head dim)
// keeps the online softmax per column in registers (a column lives in one lane pair), and
//   O^T[128 dims x 32 cols] += V^T . P^T      (contraction over keys).
// S^T's accumulator layout IS the B-operand layout of the second product (same lane, same
// column), up to the order of keys inside a group of 16, which the V^T operand mirrors, so P never
// leaves registers.  V lies in LDS as it lies in memory ([key][dim] rows) and the V^T operand comes
// out of gfx950's transposing LDS read (ds_read_b64_tr_b16): sixteen lanes hand in the sixteen
// 8-byte pieces of four key rows x 16 dims and lane j of them receives dim j of the four keys, so
// the transpose costs no instruction and the key order is whatever rows the lanes name.
//
// Tiles travel from memory straight into LDS (buffer loads with the LDS bit: no staging registers,
// no LDS store instructions) through a ring of three K tiles and two V tiles (80 KB, so two
// workgroups share a compute unit and one computes while the other starts or ends): iteration t
// reads K(t + 1) and V(t) while K(t + 2) lands and V(t + 1) and K(t + 3) are loaded into the slots
// iteration t - 1 read.  Such a load writes a wavefront's 64 x 16 bytes contiguously, so rows are
// unpadded (256 bytes) and bank conflicts are avoided by which 16-byte piece a lane fetches: piece
// c of K row r sits at position c ^ (r & 15) (the score product reads one piece of 16 consecutive
// rows at a time), piece c of V row r at c ^ ((r & 3) << 2) (a transposing read takes 64 bytes of
// four consecutive rows).
//
// The loop is software-pipelined inside the wavefront: the scores of tile t + 1 are produced in the
// same straight-line block as the exponentials of tile t, and an explicit issue order (scheduling
// groups) puts the LDS reads two products ahead of their use, so one wavefront keeps the matrix pipe,
// the VALU and the LDS busy at once.  One barrier per tile.
#include "attn_internal.h"

namespace {

// 2^x by the bare hardware instruction: the library exp2f wraps it in a range fix-up for results below
// 2^-126 (five more VALU operations per call); softmax arguments are <= 0 and such tails may flush to zero.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }


typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;

constexpr int kKeysPerTile = 64;
constexpr int kRowBytes = 2 * kHeadDim;                    // a key row of one KV head
constexpr int kTileBytes = kKeysPerTile * kRowBytes;       // 16 KB, rows unpadded (see the swizzles above)
constexpr int kRingK = 3, kRingV = 2;                      // tiles of K and of V resident or in flight
constexpr int kVBase = kRingK * kTileBytes;                // the V ring lies behind the K ring
constexpr int kWaves = 4;
constexpr int kLdsBytes = (kRingK + kRingV) * kTileBytes;  // 80 KB: two workgroups per compute unit
// s_waitcnt immediates: vector-memory loads return in order, so "at most n outstanding" names the oldest ones done
constexpr int kWaitVm0 = 0x0F70, kWaitVm4 = 0x0F74, kWaitVm12 = 0x0F7C;

// max / sum of a value over the two half-waves (lane and lane ^ 32), by the half-wave swap instruction
__device__ __forceinline__ float half_wave_max(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_wave_sum(float x) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
// two floats -> packed bf16 pair, round to nearest even (one v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  floatx2_t f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

typedef short shortx4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4_t lds_shortx4_t;

// Transposing LDS read of 16-bit elements: within each group of 16 lanes, lanes 4 r .. 4 r + 3 name the four
// 8-byte pieces of row r (r = 0..3, 16 elements) and lane j receives element j of rows 0..3.
__device__ __forceinline__ shortx4_t lds_read_tr16(const char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_t*)(p));
}

typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) char lds_char_t;

__device__ __forceinline__ uint32_t lds_address(char* p) { return (uint32_t)(uintptr_t)(lds_char_t*)p; }

// 16 bytes per lane from a buffer resource straight into LDS: lane l lands at byte lds_dst + 16 l (lds_dst the same in
// every lane, and handed over in a scalar register).  Written as an asm statement, not through the compiler's builtin,
// so that the compiler does not know of a load in flight that writes LDS: it would drain all of them (vmcnt(0)) in
// front of the first transposing LDS read of every iteration, whose address it cannot tell from the loads' targets.
// The waits are the kernel's own (see the ring).  M0 (the LDS target) is put back as it was, so the statement is
// transparent to whatever the compiler keeps there; the wait states in front of the load cover a resource or an M0
// that the preceding instruction wrote.
// Four loads at once: the wavefront's four consecutive 1 KB blocks of a tile (offsets v0 .. v3).
__device__ __forceinline__ void load4_to_lds(u32x4_t rsrc, uint32_t lds_dst, int v0, int v1, int v2, int v3) {
#if defined(__HIP_DEVICE_COMPILE__)
  uint32_t saved_m0;
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %1\n\t"
      "s_nop 4\n\t"
      "buffer_load_dwordx4 %2, %6, 0 offen lds\n\t"
      "s_add_u32 m0, m0, 0x400\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %3, %6, 0 offen lds\n\t"
      "s_add_u32 m0, m0, 0x400\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %4, %6, 0 offen lds\n\t"
      "s_add_u32 m0, m0, 0x400\n\t"
      "s_nop 0\n\t"
      "buffer_load_dwordx4 %5, %6, 0 offen lds\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(saved_m0) : "s"(lds_dst), "v"(v0), "v"(v1), "v"(v2), "v"(v3), "s"(rsrc) : "scc");
#endif
}

// kSplit: blockIdx.z selects a range of split_keys keys; the un-normalised accumulators and the
// (reference max, sum) pair of every column go to part_acc / part_ml for the combine kernel.
template <int G, bool kSplit>
__global__ __launch_bounds__(kWaves * 64, 2) void flash_attn_kernel(
    const bf16_t* __restrict__ q, const int32_t* __restrict__ cu_q, const bf16_t* __restrict__ k,
    const bf16_t* __restrict__ v, const int64_t* __restrict__ kv_off, const int32_t* __restrict__ kv_len, int32_t B,
    int32_t Hq, int32_t Hkv, float scale_log2e, int32_t causal, bf16_t* __restrict__ out, int32_t n_split,
    int32_t split_keys, float* __restrict__ part_ml, float* __restrict__ part_acc) {
  constexpr int kTokPerWave = 32 / G;
  constexpr int kTokPerBlock = kWaves * kTokPerWave;
  constexpr int kLoads = kTileBytes / (kWaves * 64 * 16);     // load instructions per wavefront, tile and tensor
  extern __shared__ __align__(16) char lds[];                  // [K ring | V ring]

  // which (sample, token block) is this workgroup?  B is small; the scan is uniform.
  // Workgroups go to the eight XCDs round-robin in launch order and each XCD has an L2 of its own (4 MiB).  With the
  // KV head as the fastest index an XCD keeps to one head (eight of them) or a few, and the workgroups resident on
  // it at one time are neighbouring token blocks of one sample: they stream the same 2 MB of K and V, which stay in
  // that L2.  With the head as a grid dimension of its own every XCD held blocks of several samples at once, more
  // K / V than its L2 takes, and most tile loads came from beyond it.
  const int g = blockIdx.x % Hkv;
  int blk = blockIdx.x / Hkv, b = 0;
  bool found = false;
  for (; b < B; ++b) {
    const int sq_b = cu_q ? cu_q[b + 1] - cu_q[b] : 1;
    const int nb = (sq_b + kTokPerBlock - 1) / kTokPerBlock;
    if (blk < nb) {
      // under the causal mask a sample's last token blocks see the most keys: they go first, so that the launch
      // ends on short workgroups instead of waiting for a few long ones
      if (causal) blk = nb - 1 - blk;
      found = true;
      break;
    }
    blk -= nb;
  }
  if (!found) return;
  const int q_first = cu_q ? cu_q[b] : b;
  const int sq = cu_q ? cu_q[b + 1] - q_first : 1;
  const int t0 = blk * kTokPerBlock;
  const int L = kv_len[b];
  const int64_t base = kv_off[b];

  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int col = lane & 31, half = lane >> 5;
  const int tok = t0 + wave * kTokPerWave + col / G;       // token within the sample
  const int head = g * G + col % G;
  const bool col_ok = tok < sq;
  const int limit = col_ok ? (causal ? max(0, L - sq + tok + 1) : L) : 0;   // this column sees keys [0, limit)
  const int last_tok = min(sq, t0 + kTokPerBlock) - 1;
  int kmax = causal ? max(0, min(L, L - sq + last_tok + 1)) : L;             // the block sees keys [0, kmax)
  int first_tile = 0;
  if constexpr (kSplit) {
    first_tile = blockIdx.z * (split_keys / kKeysPerTile);
    kmax = min(kmax, (int)(blockIdx.z + 1) * split_keys);
  }
  const int n_tiles = (kmax + kKeysPerTile - 1) / kKeysPerTile;              // tiles first_tile .. n_tiles - 1
  const int row_elems = Hkv * kHeadDim;

  // Q^T operand fragments stay in registers for the whole pass: lane (col, half), step s holds
  // dims 16 s + 8 half .. + 8 of its column's query row.
  bf16x8_t qf[8];
  {
    const bf16_t* qrow = q + ((int64_t)(q_first + (col_ok ? tok : 0)) * Hq + head) * kHeadDim + 8 * half;
#pragma unroll
    for (int s = 0; s < 8; ++s) {
      uint4 w = col_ok ? *reinterpret_cast<const uint4*>(qrow + 16 * s) : make_uint4(0, 0, 0, 0);
      qf[s] = __builtin_bit_cast(bf16x8_t, w);
    }
  }

  floatx16_t o[4];
#pragma unroll
  for (int d = 0; d < 4; ++d)
#pragma unroll
    for (int e = 0; e < 16; ++e) o[d][e] = 0.f;
  float m = -INFINITY, l = 0.f;
  int wave_min_limit = limit;               // tiles that end below it need no masking in this wavefront
#pragma unroll
  for (int x = 32; x > 0; x >>= 1) wave_min_limit = min(wave_min_limit, __shfl_xor(wave_min_limit, x));

  // Tile loads through buffer resources rebuilt per tile (scalar work only): the extent covers the tile's valid
  // keys and a lane's offset never changes.  Load instruction i of a wavefront fills the 1 KB block of rows
  // 4 (kLoads wave + i) .. + 4: lane l lands at row l / 16, position l % 16 and fetches the piece that belongs there.
  // K rows past the last key may hold anything (their scores are masked by a select); V rows past it are multiplied
  // by probabilities of zero and must be finite, so those lanes fetch the last valid row again.
  const int row_bytes = row_elems * 2;
  int tile_row[kLoads], k_piece[kLoads], v_piece[kLoads], v_full[kLoads];
#pragma unroll
  for (int i = 0; i < kLoads; ++i) {
    tile_row[i] = 4 * (kLoads * wave + i) + (lane >> 4);
    k_piece[i] = ((lane & 15) ^ (tile_row[i] & 15)) * 16;
    v_piece[i] = ((lane & 15) ^ ((tile_row[i] & 3) << 2)) * 16;
    v_full[i] = tile_row[i] * row_bytes + v_piece[i];          // the lane's offset in a tile whose 64 rows all exist
  }
  // Tiles are loaded in order, K and V each from its own running position (address of the next tile to load, keys
  // left from its first row on): a load takes the position's tile and moves it on by one.
  struct TilePos { uintptr_t at; int left; };
  auto first_pos = [&](const bf16_t* src) {
    return TilePos{reinterpret_cast<uintptr_t>(src) + ((base + (int64_t)first_tile * kKeysPerTile) * row_elems + g * kHeadDim) * 2,
                   kmax - first_tile * kKeysPerTile};
  };
  TilePos k_pos = first_pos(k), v_pos = first_pos(v);
  auto tile_rsrc = [&](TilePos& p, int& rows) -> u32x4_t {
    rows = min(kKeysPerTile, p.left);
    const u32x4_t r = {(uint32_t)p.at, (uint32_t)(p.at >> 32) & 0xffffu, (uint32_t)max(0, (rows - 1) * row_bytes + kRowBytes),
                       0x00020000u};                                                        // extent 0 when no row is left
    p.at += (uintptr_t)kKeysPerTile * row_bytes;
    p.left -= kKeysPerTile;
    return r;
  };
  const uint32_t lds_wave = lds_address(lds) + kLoads * wave * 1024;     // this wavefront's first block of a tile
  auto issue_k = [&](int slot) {
    int rows;
    const u32x4_t rsrc = tile_rsrc(k_pos, rows);
    load4_to_lds(rsrc, lds_wave + slot * kTileBytes, tile_row[0] * row_bytes + k_piece[0], tile_row[1] * row_bytes + k_piece[1],
                 tile_row[2] * row_bytes + k_piece[2], tile_row[3] * row_bytes + k_piece[3]);
  };
  auto issue_v = [&](int slot) {
    int rows;
    const u32x4_t rsrc = tile_rsrc(v_pos, rows);
    if (rows == kKeysPerTile) {
      load4_to_lds(rsrc, lds_wave + kVBase + slot * kTileBytes, v_full[0], v_full[1], v_full[2], v_full[3]);
    } else {
      int vo[kLoads];
#pragma unroll
      for (int i = 0; i < kLoads; ++i) vo[i] = min(tile_row[i], rows - 1) * row_bytes + v_piece[i];   // rows <= 0: out of range
      load4_to_lds(rsrc, lds_wave + kVBase + slot * kTileBytes, vo[0], vo[1], vo[2], vo[3]);
    }
  };
  // a barrier that waits for this wavefront's LDS reads but not for its loads in flight
  auto ring_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
  // per-lane read positions inside a tile: K piece 2 ks + half of row col (+ 32 rb), V as the transposing read
  // wants it (rows 4 half + r of a group of 8, 64 bytes at dims 32 d, r = (lane % 16) / 4)
  int k_at[8], v_at[4];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) k_at[ks] = col * kRowBytes + (((2 * ks + half) ^ (col & 15)) * 16);
  {
    const int r = (lane & 15) >> 2;
#pragma unroll
    for (int d = 0; d < 4; ++d)
      v_at[d] = kVBase + (4 * half + r) * kRowBytes + ((d ^ r) * 64) + (lane & 16) * 2 + (lane & 3) * 8;
  }

  // masks the scores of tile t past the column's last visible key and returns their maximum; `between(i)`, i = 0..3,
  // is called at four points spread over the work (the caller's matrix products, so that they issue among these
  // VALU instructions whichever way the branch goes)
  auto tile_max = [&](int t, floatx16_t (&sx)[2], auto between) -> float {
    const int key_base = t * kKeysPerTile + 4 * half;
    float mx_t = -INFINITY;
    if ((t + 1) * kKeysPerTile <= wave_min_limit) {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          if ((e & 7) == 0) { between(2 * rb + (e >> 3)); __builtin_amdgcn_sched_barrier(0); }
          mx_t = fmaxf(mx_t, sx[rb][e]);
        }
    } else {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          if ((e & 7) == 0) { between(2 * rb + (e >> 3)); __builtin_amdgcn_sched_barrier(0); }
          const int key = key_base + 32 * rb + 8 * (e >> 2) + (e & 3);
          const float x = key < limit ? sx[rb][e] : -INFINITY;
          sx[rb][e] = x;
          mx_t = fmaxf(mx_t, x);
        }
    }
    return mx_t;
  };
  float mx_raw = -INFINITY;                  // of the tile the next step consumes
  int ring = 0;                              // (t - first_tile) % kRingK: the slot of K(t)
  auto step = [&](int t, floatx16_t (&sc)[2], floatx16_t (&sn)[2]) {
    const int ring1 = ring == kRingK - 1 ? 0 : ring + 1;
    const int vslot = (t - first_tile) & 1;  // the slot of V(t)
    issue_v(vslot ^ 1);                      // V(t + 1) into V(t - 1)'s slot: last read before the previous barrier
    issue_k(ring);                           // K(t + 3) into K(t)'s slot: likewise
    // (A) the column maximum of this tile's (masked) scores came with the scores: `mx_raw`
    float mx = fmaxf(m, mx_raw * scale_log2e);
    mx = half_wave_max(mx);
    const bool none = mx == -INFINITY;
    // (B) lazy rescaling, as in the plain loop
    const bool grow = !none && mx > m + 6.0f;
    if (__any(grow)) {
      const float mref = none ? m : mx;
      const float alpha = (none || m == -INFINITY) ? (m == -INFINITY ? 0.f : 1.f) : fast_exp2(m - mref);
      l *= alpha;
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int e = 0; e < 16; ++e) o[d][e] *= alpha;
      m = mref;
    }
    const float neg_m = none ? 0.f : -m;
    // (C) / (D) the 16 products of the scores of tile t + 1 (the K slot holds anything past the last tile: never used),
    // the 16 products O^T += V^T . P^T of tile t, and this tile's 32 exponentials in 16 pairs, in an issue order that
    // is written out slot by slot and fenced (the scheduler may not move anything across a slot's end):
    // (slots  0 .. 15: score product s, an exponential pair behind every second one; 16 .. 27: O product, the other
    // pairs; 28 .. 31: O product, the column maximum of the new scores), so that a matrix product has at most VALU
    // work of its own length issued behind it, and each LDS read is issued two products ahead of its use.
    const char* kn = lds + ring1 * kTileBytes;
    const char* vt = lds + vslot * kTileBytes;
    float psum = 0.f;
    uint32_t pw[2][2][4];                   // P as packed bf16 pairs: [key rows 32 rb ..][16 j ..][pair]
    constexpr int kKAhead = 4, kKRing = 3;  // K operand reads issued this many products ahead; ring of score steps
    constexpr int kVAhead = 2, kVRing = 3;  // V^T operands read this many products ahead; ring of operands
    bf16x8_t kf[kKRing][2];
    bf16x8_t va[kVRing];
    auto k_read = [&](int i) {              // i = 2 ks + rb
      kf[(i >> 1) % kKRing][i & 1] = *reinterpret_cast<const bf16x8_t*>(kn + k_at[i >> 1] + (i & 1) * 32 * kRowBytes);
    };
    auto qk = [&](int i) {
      const int ks = i >> 1, rb = i & 1;
      if (ks == 0) {
        floatx16_t z;
#pragma unroll
        for (int e = 0; e < 16; ++e) z[e] = 0.f;
        sn[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[0][rb], qf[0], z, 0, 0, 0);
      } else {
        sn[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks % kKRing][rb], qf[ks], sn[rb], 0, 0, 0);
      }
    };
    auto exp_pair = [&](int gi) {           // elements 2 (gi % 8), + 1 of sc[gi / 8]
      const int prb = gi >> 3, e0 = (gi & 7) * 2;
      const float p0 = fast_exp2(fmaf(sc[prb][e0], scale_log2e, neg_m));
      const float p1 = fast_exp2(fmaf(sc[prb][e0 + 1], scale_log2e, neg_m));
      const uint32_t pk = pack_pair(p0, p1);
      psum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pk), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), psum, false);
      pw[prb][(gi & 7) >> 2][gi & 3] = pk;
    };
    auto v_read = [&](int i) {              // i = (2 rb + j) * 4 + d
      const char* at = vt + v_at[i & 3] + 16 * (i >> 2) * kRowBytes;
      const shortx4_t lo = lds_read_tr16(at), hi = lds_read_tr16(at + 8 * kRowBytes);
      va[i % kVRing] = __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
    };
    auto pv = [&](int i) {
      const int rbj = i >> 2, d = i & 3;
      const u32x4_t pwv = {pw[rbj >> 1][rbj & 1][0], pw[rbj >> 1][rbj & 1][1], pw[rbj >> 1][rbj & 1][2], pw[rbj >> 1][rbj & 1][3]};
      o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[i % kVRing], __builtin_bit_cast(bf16x8_t, pwv), o[d], 0, 0, 0);
    };
    auto fence = [&]() { __builtin_amdgcn_sched_barrier(0); };
    fence();
#pragma unroll
    for (int i = 0; i < kKAhead; ++i) k_read(i);
    fence();
#pragma unroll
    for (int sl = 0; sl < 16; ++sl) {
      if (sl + kKAhead < 16) k_read(sl + kKAhead);
      qk(sl);
      if (sl & 1) exp_pair(sl >> 1);
      if (sl >= 16 - kVAhead) v_read(sl - (16 - kVAhead));
      fence();
    }
    // The O products have little VALU work of their own: with the wavefront's priority raised for their length the
    // SIMD's other wavefront (of the compute unit's other workgroup, usually in a different phase) yields the matrix
    // pipe to them and fills the gaps with its own VALU work instead of the other way round (1.4 %).
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int u = 0; u < 12; ++u) {
      if (u + kVAhead < 16) v_read(u + kVAhead);
      pv(u);
      if (u < 8 && !(u & 1)) exp_pair(8 + (u >> 1));
      if (u >= 8) exp_pair(4 + u);
      fence();
    }
    // the last O products share their issue slots with the maximum of the scores just finished (the next tile's)
    mx_raw = tile_max(t + 1, sn, [&](int i) {
      if (i + 12 + kVAhead < 16) v_read(i + 12 + kVAhead);
      pv(i + 12);
    });
    fence();
    __builtin_amdgcn_s_setprio(0);
    l += half_wave_sum(psum);
    // K(t + 2), issued an iteration ago, and V(t + 1) have landed once only the loads of K(t + 3) are outstanding
    __builtin_amdgcn_s_waitcnt(kWaitVm4);
    ring_barrier();
    ring = ring1;
  };

  static_assert(kLoads == 4, "the wait counts and the load statement assume four loads per wavefront, tile and tensor");
  if (first_tile < n_tiles) {
    issue_k(0);                                // K(first), V(first), K(first + 1), K(first + 2)
    issue_v(0);
    issue_k(1);
    issue_k(2);
    __builtin_amdgcn_s_waitcnt(kWaitVm12);     // K(first) has landed
    ring_barrier();
    floatx16_t s0[2], s1[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int e = 0; e < 16; ++e) s0[rb][e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(lds + k_at[ks] + rb * 32 * kRowBytes);
        s0[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s0[rb], 0, 0, 0);
      }
    // the first step reads V(first) and K(first + 1), and loads K(first + 3) over K(first): every wavefront must
    // have those two and be done with the reads above before any wavefront gets there
    __builtin_amdgcn_s_waitcnt(kWaitVm4);
    ring_barrier();
    mx_raw = tile_max(first_tile, s0, [](int) {});
    for (int t = first_tile; t < n_tiles; t += 2) {
      step(t, s0, s1);
      if (t + 1 < n_tiles) step(t + 1, s1, s0);
    }
    __builtin_amdgcn_s_waitcnt(kWaitVm0);      // nothing may still be writing LDS when the workgroup ends
  }

  if constexpr (kSplit) {
    if (col_ok) {
      const int64_t slot = ((int64_t)(q_first + tok) * Hq + head) * n_split + blockIdx.z;
      if (half == 0) { part_ml[slot * 2] = m; part_ml[slot * 2 + 1] = l; }
      float* prow = part_acc + slot * kHeadDim;
#pragma unroll
      for (int d = 0; d < 4; ++d)
#pragma unroll
        for (int e4 = 0; e4 < 4; ++e4)
          *reinterpret_cast<float4*>(prow + 32 * d + 8 * e4 + 4 * half) =
              make_float4(o[d][4 * e4], o[d][4 * e4 + 1], o[d][4 * e4 + 2], o[d][4 * e4 + 3]);
    }
  } else if (col_ok) {
    const float inv = l > 0.f ? 1.0f / l : 0.f;        // a row that sees no key yields zeros
    bf16_t* orow = out + ((int64_t)(q_first + tok) * Hq + head) * kHeadDim;
#pragma unroll
    for (int d = 0; d < 4; ++d)
#pragma unroll
      for (int e4 = 0; e4 < 4; ++e4) {
        uint2 w;
        w.x = pack_bf16x2(o[d][4 * e4] * inv, o[d][4 * e4 + 1] * inv);
        w.y = pack_bf16x2(o[d][4 * e4 + 2] * inv, o[d][4 * e4 + 3] * inv);
        *reinterpret_cast<uint2*>(orow + 32 * d + 8 * e4 + 4 * half) = w;
      }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// The wide form: one wavefront per SIMD, 64 (token, head) columns per wavefront, 256 per workgroup; the tile step is
// written at the instruction level (flash_asm.inc, generated by gen_flash_asm.py, which describes the schedule, the
// LDS rings and the registers the statements own: v56 - v255, every accumulation register, s84 - s95).  The code the
// compiler allocates stays below v56 (amdgpu_num_vgpr) and only names values for the statements: tile resources,
// the masked-or-not choice per tile, the rescale of O when a reference maximum moved.
#include "flash_asm.inc"

constexpr int kWideLdsBytes = 10 * kTileBytes;  // rings of three K and three V tiles, 16 KB of query rows per wavefront
constexpr int kWideCompilerVgprs = 56;

#define FLASHW_ASM(TEXT) asm volatile(TEXT ::: FLASHW_CLOBBERS)
#define FLASHW_GETO(CB, D, X)                                                                                          \
  asm volatile(FLASHW_GET_O##CB##_##D                                                                                  \
               : "=v"((X)[0]), "=v"((X)[1]), "=v"((X)[2]), "=v"((X)[3]), "=v"((X)[4]), "=v"((X)[5]), "=v"((X)[6]),     \
                 "=v"((X)[7]), "=v"((X)[8]), "=v"((X)[9]), "=v"((X)[10]), "=v"((X)[11]), "=v"((X)[12]), "=v"((X)[13]), \
                 "=v"((X)[14]), "=v"((X)[15]))

// The launch is persistent: one workgroup per compute unit walks the token blocks of its KV head (workgroup w serves
// head w % Hkv, so with eight heads a head keeps to one XCD and its K / V to that XCD's L2, and is the (w / Hkv)-th of
// the n workgroups of the head).  A head's blocks are listed sample by sample, under the causal mask a sample's late
// (long) blocks first, and dealt out in rounds of n that alternate direction: workgroup c takes position c of an even
// round and n - 1 - c of an odd one, so the workgroup that drew the longest block of a round draws the shortest of the
// next (a sample of 2 n causal blocks splits evenly), and the n workgroups stay on the same sample's K / V.
// Blocks are pipelined: once a block's last product is issued its LDS rings are free, so the next block's first tiles
// and its query rows (into 16 KB of LDS per wavefront behind the rings) are requested before the finished block's
// output is scaled and stored, and the block after that is looked up while those loads are awaited.
template <int G>
__global__ __launch_bounds__(256) __attribute__((amdgpu_num_vgpr(kWideCompilerVgprs))) void flash_wide_kernel(
    const bf16_t* __restrict__ q, const int32_t* __restrict__ cu_q, const bf16_t* __restrict__ k,
    const bf16_t* __restrict__ v, const int64_t* __restrict__ kv_off, const int32_t* __restrict__ kv_len, int32_t B,
    int32_t Hq, int32_t Hkv, float scale_log2e, int32_t causal, bf16_t* __restrict__ out, int32_t total_blocks) {
#if defined(__HIP_DEVICE_COMPILE__)
  constexpr int kTokPerWave = 64 / G;
  constexpr int kTokPerBlock = 4 * kTokPerWave;
  extern __shared__ __align__(16) char lds[];

  const int g = blockIdx.x % Hkv, c_wg = blockIdx.x / Hkv, n_wg = gridDim.x / Hkv;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int row_elems = Hkv * kHeadDim;
  const int row_bytes = row_elems * 2;

  // per-lane LDS read positions (slot 0) and global offsets of the wavefront's four 1 KB blocks of a tile: the same
  // row / piece assignment and swizzles as the 32-column form
  {
    const int l32 = lane & 31, half = lane >> 5;
    int k_at[8], v_at[4];
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) k_at[ks] = l32 * kRowBytes + (((2 * ks + half) ^ (l32 & 15)) * 16);
    const int r = (lane & 15) >> 2;
#pragma unroll
    for (int d = 0; d < 4; ++d)
      v_at[d] = 3 * kTileBytes + (4 * half + r) * kRowBytes + ((d ^ r) * 64) + (lane & 16) * 2 + (lane & 3) * 8;
    asm volatile(FLASHW_SET_KAT ::"v"(k_at[0]), "v"(k_at[1]), "v"(k_at[2]), "v"(k_at[3]), "v"(k_at[4]), "v"(k_at[5]),
                 "v"(k_at[6]), "v"(k_at[7])
                 : FLASHW_CLOBBERS);
    asm volatile(FLASHW_SET_VAT ::"v"(v_at[0]), "v"(v_at[1]), "v"(v_at[2]), "v"(v_at[3]) : FLASHW_CLOBBERS);
    int koff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int row = 4 * (4 * wave + i) + (lane >> 4);
      koff[i] = row * row_bytes + ((lane & 15) ^ (row & 15)) * 16;
    }
    asm volatile(FLASHW_SET_KOFF ::"v"(koff[0]), "v"(koff[1]), "v"(koff[2]), "v"(koff[3]) : FLASHW_CLOBBERS);
  }
  const uint32_t ldsw = lds_address(lds) + 4 * wave * 1024;                    // this wavefront's first block of ring slot 0
  const uint32_t ldsq = lds_address(lds) + 6 * kTileBytes + wave * kTileBytes;  // its query rows

  // a block of the walk: everything that names it is wave-uniform
  struct Block {
    int q_first, sq, t0, kmax, n_tiles, L;
    int64_t base;
  };
  // (a workgroup's positions in the list only grow, so the search for a position's sample resumes where the last
  // one ended: `cur_b` is a sample, `before` the number of blocks of the samples in front of it)
  int cur_b = 0, before = 0;
  auto find_block = [&](int& round, Block& blkout) -> bool {
    for (; round * n_wg < total_blocks; ++round) {
      const int pos = round * n_wg + ((round & 1) ? n_wg - 1 - c_wg : c_wg);
      for (; cur_b < B; ++cur_b) {
        const int first = cu_q ? cu_q[cur_b] : cur_b;
        const int sq_b = cu_q ? cu_q[cur_b + 1] - first : 1;
        const int nb = (sq_b + kTokPerBlock - 1) / kTokPerBlock;
        if (pos - before < nb) {
          int blk = pos - before;
          if (causal) blk = nb - 1 - blk;
          blkout.q_first = first;
          blkout.sq = sq_b;
          blkout.t0 = blk * kTokPerBlock;
          blkout.L = kv_len[cur_b];
          blkout.base = kv_off[cur_b];
          const int last_tok = min(sq_b, blkout.t0 + kTokPerBlock) - 1;
          blkout.kmax = causal ? max(0, min(blkout.L, blkout.L - sq_b + last_tok + 1)) : blkout.L;
          blkout.n_tiles = (blkout.kmax + kKeysPerTile - 1) / kKeysPerTile;
          ++round;
          return true;
        }
        before += nb;
      }
    }
    return false;
  };

  // running positions of the K and V tile streams of the block whose tiles are being loaded
  struct TilePos { uintptr_t at; int left; };
  TilePos k_pos{0, 0}, v_pos{0, 0};
  auto tile_rsrc = [&](TilePos& p, int& rows) -> u32x4_t {
    rows = min(kKeysPerTile, p.left);
    const u32x4_t r = {(uint32_t)p.at, (uint32_t)(p.at >> 32) & 0xffffu,
                       (uint32_t)max(0, (rows - 1) * row_bytes + kRowBytes), 0x00020000u};
    p.at += (uintptr_t)kKeysPerTile * row_bytes;
    p.left -= kKeysPerTile;
    return r;
  };
  // the V offsets of a tile of `rows` keys: a last tile of fewer than 64 keys has its missing rows fetched from its
  // last key (they meet probabilities of zero and must be finite), which is the last change a block's offsets see
  auto set_voff = [&](int rows) {
    int lane_v = lane;
    asm volatile("" : "+v"(lane_v));
    const int row0 = 16 * wave + (lane_v >> 4);                          // the lane's row in the first block; + 4 i
    const int piece = ((lane_v & 15) ^ ((row0 & 3) << 2)) * 16;          // (the same for the four blocks)
    int vo[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) vo[i] = min(row0 + 4 * i, rows - 1) * row_bytes + piece;
    asm volatile(FLASHW_SET_VOFF ::"v"(vo[0]), "v"(vo[1]), "v"(vo[2]), "v"(vo[3]) : FLASHW_CLOBBERS);
  };
  auto next_v = [&]() -> u32x4_t {
    int rows;
    const u32x4_t r = tile_rsrc(v_pos, rows);
    if (rows > 0 && rows < kKeysPerTile) set_voff(rows);
    return r;
  };
  auto next_k = [&]() -> u32x4_t {
    int rows;
    return tile_rsrc(k_pos, rows);
  };
  // requests a block's query rows and its first tiles (K(0), K(1), V(0), K(2), V(1): the order the steps' waits count
  // on); every wavefront must be done with the LDS rings
  auto request_block = [&](const Block& nb) {
    {
      // the wavefront's 64 columns are 16 blocks of four rows; a buffer resource over the sample's query rows
      const uintptr_t qa = reinterpret_cast<uintptr_t>(q) + (uintptr_t)nb.q_first * Hq * kRowBytes;
      const u32x4_t rq = {(uint32_t)qa, (uint32_t)(qa >> 32) & 0xffffu, (uint32_t)min((int64_t)nb.sq * Hq * kRowBytes, (int64_t)0xffffff00),
                          0x00020000u};
      int lane_q = lane;
      asm volatile("" : "+v"(lane_q));
#pragma unroll
      for (int j4 = 0; j4 < 4; ++j4) {
        int qo[4];
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
          const int col = 4 * (4 * j4 + jj) + (lane_q >> 4);            // of the wavefront's 64
          const int tok = nb.t0 + wave * kTokPerWave + col / G;
          const int piece = (lane_q & 15) ^ (col & 15);
          // a column past the sample's rows reads from beyond the extent (nothing is fetched; the column is masked)
          qo[jj] = tok < nb.sq ? (tok * Hq + g * G + col % G) * kRowBytes + piece * 16 : -16;
        }
        asm volatile(FLASHW_LOADQ4 ::[dst] "s"(ldsq + j4 * 4096), [r] "s"(rq), [o0] "v"(qo[0]), [o1] "v"(qo[1]),
                     [o2] "v"(qo[2]), [o3] "v"(qo[3])
                     : FLASHW_CLOBBERS);
      }
    }
    const uintptr_t off = (uintptr_t)((nb.base * row_elems + g * kHeadDim) * 2);
    k_pos = TilePos{reinterpret_cast<uintptr_t>(k) + off, nb.kmax};
    v_pos = TilePos{reinterpret_cast<uintptr_t>(v) + off, nb.kmax};
    set_voff(kKeysPerTile);
    if (nb.n_tiles > 0) {
      u32x4_t r = next_k();
      asm volatile(FLASHW_LOAD4_K ::[dst] "s"(ldsw), [r] "s"(r) : FLASHW_CLOBBERS);
      r = next_k();
      asm volatile(FLASHW_LOAD4_K ::[dst] "s"(ldsw + kTileBytes), [r] "s"(r) : FLASHW_CLOBBERS);
      r = next_v();
      asm volatile(FLASHW_LOAD4_V ::[dst] "s"(ldsw + 3 * kTileBytes), [r] "s"(r) : FLASHW_CLOBBERS);
      r = next_k();
      asm volatile(FLASHW_LOAD4_K ::[dst] "s"(ldsw + 2 * kTileBytes), [r] "s"(r) : FLASHW_CLOBBERS);
      r = next_v();
      asm volatile(FLASHW_LOAD4_V ::[dst] "s"(ldsw + 4 * kTileBytes), [r] "s"(r) : FLASHW_CLOBBERS);
    }
  };

  int round = 0;
  Block cur{}, nxt{};
  bool have = find_block(round, cur);
  if (have) request_block(cur);
  while (have) {
    const bool have_next = find_block(round, nxt);      // scalar work under the loads' latency
    const int n_tiles = cur.n_tiles;
    int wave_min_limit;
    {
      int lane_c = lane;
      asm volatile("" : "+v"(lane_c));
      const int half = lane_c >> 5;
      int limit[2];
#pragma unroll
      for (int cb = 0; cb < 2; ++cb) {
        const int col = 32 * cb + (lane_c & 31);
        const int tok = cur.t0 + wave * kTokPerWave + col / G;
        limit[cb] = tok < cur.sq ? (causal ? max(0, cur.L - cur.sq + tok + 1) : cur.L) : 0;
      }
      asm volatile(FLASHW_SET_LIMIT ::"v"(limit[0] - 4 * half), "v"(limit[1] - 4 * half) : FLASHW_CLOBBERS);
      int wm = min(limit[0], limit[1]);
#pragma unroll
      for (int x = 32; x > 0; x >>= 1) wm = min(wm, __shfl_xor(wm, x));
      wave_min_limit = __builtin_amdgcn_readfirstlane(wm);
    }
    // the block's query rows and first tiles have landed (and the last block's output stores are out)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    asm volatile(FLASHW_Q_FROM_LDS ::[qoff] "s"(ldsq) : FLASHW_CLOBBERS);
    FLASHW_ASM(FLASHW_INIT);

    if (n_tiles > 0) {
      asm volatile("s_barrier" ::: "memory");
      FLASHW_ASM(FLASHW_QK_FIRST);
      // The statements repeat with period six (LDS slots and score buffers are immediates), so the loop over the
      // tiles is unrolled by six; tile 0 (nothing to multiply by V yet) stands in front.
      int t = 0, flag;
#define FLASHW_HALF_A(TEXT) asm volatile(TEXT : [flag] "=&s"(flag) : [c] "s"(scale_log2e) : FLASHW_CLOBBERS)
#define FLASHW_STEP(A_TEXT, A_TEXT_M, B_TEXT, B_TEXT_LAST)                                                          \
  {                                                                                                                 \
    if ((t + 1) * kKeysPerTile > wave_min_limit) {                                                                  \
      asm volatile(A_TEXT_M : [flag] "=&s"(flag) : [c] "s"(scale_log2e), [t64] "s"(t * kKeysPerTile) : FLASHW_CLOBBERS); \
    } else {                                                                                                        \
      FLASHW_HALF_A(A_TEXT);                                                                                        \
    }                                                                                                               \
    if (flag) FLASHW_ASM(FLASHW_RESCALE);                                                                           \
    if (++t < n_tiles) {                                                                                            \
      const u32x4_t rk = next_k();                                                                                  \
      const u32x4_t rv = next_v();                                                                                  \
      asm volatile(B_TEXT ::[c] "s"(scale_log2e), [rk] "s"(rk), [rv] "s"(rv), [ldsw] "s"(ldsw) : FLASHW_CLOBBERS);  \
    } else {                                                                                                        \
      asm volatile(B_TEXT_LAST ::[c] "s"(scale_log2e) : FLASHW_CLOBBERS);                                           \
      break;                                                                                                        \
    }                                                                                                               \
  }
      do {
        FLASHW_STEP(FLASHW_A_FIRST, FLASHW_A_FIRST_M, FLASHW_B0, FLASHW_B0_LAST)
        for (;;) {
          FLASHW_STEP(FLASHW_A1, FLASHW_A1_M, FLASHW_B1, FLASHW_B1_LAST)
          FLASHW_STEP(FLASHW_A2, FLASHW_A2_M, FLASHW_B2, FLASHW_B2_LAST)
          FLASHW_STEP(FLASHW_A3, FLASHW_A3_M, FLASHW_B3, FLASHW_B3_LAST)
          FLASHW_STEP(FLASHW_A4, FLASHW_A4_M, FLASHW_B4, FLASHW_B4_LAST)
          FLASHW_STEP(FLASHW_A5, FLASHW_A5_M, FLASHW_B5, FLASHW_B5_LAST)
          FLASHW_STEP(FLASHW_A0, FLASHW_A0_M, FLASHW_B0, FLASHW_B0_LAST)
        }
      } while (false);
#undef FLASHW_STEP
#undef FLASHW_HALF_A
      const int i = t % 6;                      // of the tile behind the last: its half A alone is left (O += V^T . P^T)
      switch (i) {
        case 0: FLASHW_ASM(FLASHW_PV0); break;
        case 1: FLASHW_ASM(FLASHW_PV1); break;
        case 2: FLASHW_ASM(FLASHW_PV2); break;
        case 3: FLASHW_ASM(FLASHW_PV3); break;
        case 4: FLASHW_ASM(FLASHW_PV4); break;
        case 5: FLASHW_ASM(FLASHW_PV5); break;
      }
      // nothing may still be writing LDS (the tiles requested past the block's end), and every wavefront must be
      // done reading the rings, when the next block's tiles are requested (or the workgroup ends)
      asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
    if (have_next) request_block(nxt);

    // ---- the finished block's output
    FLASHW_ASM(FLASHW_DRAIN);
    float m0, m1, lsum[2];
    asm volatile(FLASHW_GET_ML : "=v"(m0), "=v"(m1), "=v"(lsum[0]), "=v"(lsum[1]));
    (void)m0; (void)m1;
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    int64_t orow_e[2];
    bool ok_e[2];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
      const int col = 32 * cb + (lane_e & 31);
      const int tk = cur.t0 + wave * kTokPerWave + col / G;
      ok_e[cb] = tk < cur.sq;
      orow_e[cb] = ((int64_t)(cur.q_first + tk) * Hq + g * G + col % G) * kHeadDim + 8 * (lane_e >> 5);
    }
    // A lane holds dims 8 e4 + 4 half .. + 4 of each group of eight; the two halves of a wavefront trade one group
    // of four per pair of groups (half-wave swap), after which a lane holds eight consecutive dims and stores 16 bytes
#define FLASHW_STORE(CB, D)                                                                              \
  {                                                                                                      \
    float x[16];                                                                                         \
    FLASHW_GETO(CB, D, x);                                                                               \
    uint32_t w[8];                                                                                       \
    _Pragma("unroll") for (int i = 0; i < 8; ++i) w[i] = pack_bf16x2(x[2 * i] * inv[CB], x[2 * i + 1] * inv[CB]); \
    _Pragma("unroll") for (int pr = 0; pr < 2; ++pr) {                                                   \
      const auto r0 = __builtin_amdgcn_permlane32_swap(w[4 * pr], w[4 * pr + 2], false, false);          \
      const auto r1 = __builtin_amdgcn_permlane32_swap(w[4 * pr + 1], w[4 * pr + 3], false, false);      \
      if (ok_e[CB])                                                                                      \
        *reinterpret_cast<uint4*>(out + orow_e[CB] + 32 * D + 16 * pr) = make_uint4(r0[0], r1[0], r0[1], r1[1]); \
    }                                                                                                    \
  }
    float inv[2];
#pragma unroll
    for (int cb = 0; cb < 2; ++cb) {
      const float l = half_wave_sum(lsum[cb]);
      inv[cb] = l > 0.f ? 1.0f / l : 0.f;        // a row that sees no key yields zeros
    }
    FLASHW_STORE(0, 0) FLASHW_STORE(0, 1) FLASHW_STORE(0, 2) FLASHW_STORE(0, 3)
    FLASHW_STORE(1, 0) FLASHW_STORE(1, 1) FLASHW_STORE(1, 2) FLASHW_STORE(1, 3)
#undef FLASHW_STORE
    cur = nxt;
    have = have_next;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#endif
}

template <int G>
int flash_wide_launch_g(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                        const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, float scale,
                        int32_t causal, void* out, hipStream_t st) {
  constexpr int kTokPerBlock = 4 * 64 / G;
  const int64_t blocks = ((int64_t)total_q + kTokPerBlock - 1) / kTokPerBlock + B;   // upper bound over ragged samples
  MSA_REQUIRE(blocks < (int64_t)1 << 30, "flash attention: too many query rows");
  // one workgroup per compute unit, the same number for every KV head
  const int per_head = (int)std::min<int64_t>(blocks, std::max(1, device_compute_units() / Hkv));
  auto kern = flash_wide_kernel<G>;
  static std::atomic<int> lds_limit_raised{0}, resources_checked{0};
  if (const int rc = check_asm_kernel_resources(resources_checked, reinterpret_cast<const void*>(kern), "flash_wide_kernel",
                                                nullptr, nullptr))
    return rc;
  MSA_HIP(raise_dynamic_lds_limit(lds_limit_raised, reinterpret_cast<const void*>(kern), kWideLdsBytes));
  kern<<<dim3((unsigned)(per_head * Hkv)), 256, kWideLdsBytes, st>>>(
      static_cast<const bf16_t*>(q), cu_q, static_cast<const bf16_t*>(k), static_cast<const bf16_t*>(v), kv_off, kv_len,
      B, Hq, Hkv, scale * 1.4426950408889634f, causal, static_cast<bf16_t*>(out), (int32_t)blocks);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

template <typename... Args>
int flash_wide_launch(int G, Args... args) {
  switch (G) {
    case 1: return flash_wide_launch_g<1>(args...);
    case 2: return flash_wide_launch_g<2>(args...);
    case 4: return flash_wide_launch_g<4>(args...);
    case 8: return flash_wide_launch_g<8>(args...);
  }
  msa_set_error("flash attention: GQA group size %d unsupported (1, 2, 4, 8)", G);
  return MSA_EINVAL;
}

std::atomic<int> g_flash_form{0};   // 0: by size, 1: the 32-column form, 2: the wide form

template <int G, bool kSplit>
int flash_launch_g(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                   const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, float scale,
                   int32_t causal, void* out, SplitPlan plan, float* part_ml, float* part_acc, hipStream_t st) {
  constexpr int kTokPerBlock = kWaves * 32 / G;
  const int64_t blocks = ((int64_t)total_q + kTokPerBlock - 1) / kTokPerBlock + B;   // upper bound over ragged samples
  MSA_REQUIRE(blocks * Hkv < (int64_t)1 << 31, "flash attention: too many query rows");
  dim3 grid((unsigned)(blocks * Hkv), 1u, kSplit ? (unsigned)plan.n_split : 1u);
  auto kern = flash_attn_kernel<G, kSplit>;
  static std::atomic<int> lds_limit_raised{0};   // the K and V rings exceed the default dynamic LDS limit
  MSA_HIP(raise_dynamic_lds_limit(lds_limit_raised, reinterpret_cast<const void*>(kern), kLdsBytes));
  kern<<<grid, kWaves * 64, kLdsBytes, st>>>(static_cast<const bf16_t*>(q), cu_q, static_cast<const bf16_t*>(k),
                                             static_cast<const bf16_t*>(v), kv_off, kv_len, B, Hq, Hkv,
                                             scale * 1.4426950408889634f, causal, static_cast<bf16_t*>(out),
                                             kSplit ? plan.n_split : 1, kSplit ? plan.split_keys : 0, part_ml, part_acc);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

template <bool kSplit, typename... Args>
int flash_launch(int G, Args... args) {
  switch (G) {
    case 1: return flash_launch_g<1, kSplit>(args...);
    case 2: return flash_launch_g<2, kSplit>(args...);
    case 4: return flash_launch_g<4, kSplit>(args...);
    case 8: return flash_launch_g<8, kSplit>(args...);
  }
  msa_set_error("flash attention: GQA group size %d unsupported (1, 2, 4, 8)", G);
  return MSA_EINVAL;
}

}  // namespace

namespace {
int flash_attn_entry(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                     const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, int32_t D, float scale,
                     int32_t causal, void* out, int32_t max_sq, void* stream) {
  MSA_REQUIRE(q && k && v && kv_off && kv_len && out, "msa_flash_attn: null pointer");
  MSA_REQUIRE(D == kHeadDim, "msa_flash_attn: head dim %d unsupported (need %d)", D, kHeadDim);
  MSA_REQUIRE(B > 0 && total_q > 0, "msa_flash_attn: bad sizes");
  MSA_REQUIRE(cu_q != nullptr || total_q == B, "msa_flash_attn: cu_q is required when total_q != B");
  MSA_REQUIRE(Hkv > 0 && Hkv <= 65535 && Hq % Hkv == 0, "msa_flash_attn: Hq=%d Hkv=%d unsupported", Hq, Hkv);
  MSA_REQUIRE(scale > 0.f, "msa_flash_attn: scale must be positive");
  MSA_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) == 0,
              "msa_flash_attn: q, k, v and out must be 16-byte aligned");
  const int G = Hq / Hkv;
  MSA_REQUIRE(G == 1 || G == 2 || G == 4 || G == 8, "msa_flash_attn: GQA group size %d unsupported (1, 2, 4, 8)", G);
  // The wide form wants enough columns to fill its 256-column workgroups, and query blocks of about one length: its
  // persistent launch deals the blocks out in a fixed order, which a batch of ragged samples unbalances (a packed
  // block of 30 documents of 256 - 2048 tokens measured 6 % slower than with the 32-column form, whose workgroups
  // the hardware hands out one by one)
  const int form = g_flash_form.load(std::memory_order_relaxed);
  const bool ragged = max_sq > 0 && (int64_t)max_sq * B > (int64_t)total_q + total_q / 4;
  if (form == 2 || (form == 0 && (int64_t)total_q * G >= 4096 && !ragged))
    return flash_wide_launch(G, q, cu_q, k, v, kv_off, kv_len, B, total_q, Hq, Hkv, scale, causal, out, as_stream(stream));
  return flash_launch<false>(G, q, cu_q, k, v, kv_off, kv_len, B, total_q, Hq, Hkv, scale,
                             causal, out, SplitPlan{1, 0}, (float*)nullptr, (float*)nullptr, as_stream(stream));
}
}  // namespace

extern "C" int msa_flash_attn(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                              const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, int32_t D,
                              float scale, int32_t causal, void* out, void* stream) {
  return flash_attn_entry(q, cu_q, k, v, kv_off, kv_len, B, total_q, Hq, Hkv, D, scale, causal, out, 0, stream);
}

extern "C" int msa_flash_attn_hint(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                                   const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, int32_t D,
                                   float scale, int32_t causal, void* out, int32_t max_sq, void* stream) {
  MSA_REQUIRE(max_sq > 0, "msa_flash_attn_hint: max_sq must be the longest query block of the batch");
  return flash_attn_entry(q, cu_q, k, v, kv_off, kv_len, B, total_q, Hq, Hkv, D, scale, causal, out, max_sq, stream);
}

int flash_wide_kernel_resources(int* num_regs, int* scratch_bytes) {
  std::atomic<int> unused{0};
  return check_asm_kernel_resources(unused, reinterpret_cast<const void*>(flash_wide_kernel<4>), "flash_wide_kernel", num_regs,
                                    scratch_bytes);
}

extern "C" int msa_flash_set_form(int32_t form) {
  MSA_REQUIRE(form >= 0 && form <= 2, "msa_flash_set_form: 0 (by size), 1 (32-column form) or 2 (wide form)");
  g_flash_form.store(form, std::memory_order_relaxed);
  return MSA_OK;
}

int flash_attn_split_launch(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                            const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, float scale,
                            int32_t causal, SplitPlan plan, float* part_ml, float* part_acc, hipStream_t st) {
  return flash_launch<true>(Hq / Hkv, q, cu_q, k, v, kv_off, kv_len, B, total_q, Hq,
                            Hkv, scale, causal, (void*)nullptr, plan, part_ml, part_acc, st);
}
