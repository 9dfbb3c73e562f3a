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
// leaves registers.  V goes into LDS as it lies in memory ([key][dim] rows, 16-byte stores) and the
// V^T operand comes out of gfx950's transposing LDS read (ds_read_b64_tr_b16): sixteen lanes hand in
// the sixteen 8-byte pieces of four key rows x 16 dims and lane j of them receives dim j of the four
// keys, so the transpose costs no instruction and the key order is whatever rows the lanes name.
//
// The loop is software-pipelined inside the wavefront: the scores of tile t + 1 are produced in the
// same straight-line block as the exponentials of tile t, and an explicit issue order (scheduling
// groups) puts the LDS reads two products ahead of their use, so one wavefront keeps the matrix pipe,
// the VALU and the LDS busy at once.  K and V are double-buffered out of phase (iteration t reads
// K(t + 1) and V(t) and stores K(t + 2) and V(t + 1)), one barrier per tile.
#include "attn_internal.h"

namespace {

// 2^x by the bare hardware instruction: the library exp2f wraps it in a range fix-up for results below
// 2^-126 (five more VALU operations per call); softmax arguments are <= 0 and such tails may flush to zero.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }


typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;

constexpr int kKeysPerTile = 64;
constexpr int kTileStride = 2 * kHeadDim + 16;   // bytes per key row in LDS: 256 + 16 pad (conflict-free b128 reads)
constexpr int kVStride = 2 * kHeadDim + 64;      // bytes per key row of the V tile: four consecutive keys x 64 bytes
                                                  // (one transposing read of a half-wave) cover all 64 banks once
constexpr int kStageBytes = kKeysPerTile * (kTileStride + kVStride);   // one K tile + one V tile
constexpr int kWaves = 4;
constexpr int kLdsBytes = 2 * kStageBytes;

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
  constexpr int kLoads = kKeysPerTile * 16 / (kWaves * 64);   // 16-byte pieces of a K (or V) tile per thread
  extern __shared__ __align__(16) char lds[];                  // 2 x [K tile | V tile]
  constexpr int kVOffset = kKeysPerTile * kTileStride;

  // which (sample, token block) is this workgroup?  B is small; the scan is uniform.
  int blk = blockIdx.x, b = 0;
  bool found = false;
  for (; b < B; ++b) {
    const int sq_b = cu_q ? cu_q[b + 1] - cu_q[b] : 1;
    const int nb = (sq_b + kTokPerBlock - 1) / kTokPerBlock;
    if (blk < nb) { found = true; break; }
    blk -= nb;
  }
  if (!found) return;
  const int g = blockIdx.y;
  const int q_first = cu_q ? cu_q[b] : b;
  const int sq = cu_q ? cu_q[b + 1] - q_first : 1;
  const int t0 = blk * kTokPerBlock;
  const int L = kv_len[b];
  const int64_t base = kv_off[b];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
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

  uint4 rk[kLoads], rv[kLoads];
  // Tile loads through buffer resources rebuilt per tile (scalar work only): the extent covers the tile's valid
  // keys, so rows past the last key read as zero in hardware and a thread's offset never changes.
  const int row_bytes = row_elems * 2;
  const int voff0 = (tid >> 4) * row_bytes + (tid & 15) * 16;
  auto gload_one = [&](const bf16_t* src, uint4 (&r)[kLoads], int t) {
    const int rows = min(kKeysPerTile, kmax - t * kKeysPerTile);
    const char* at = reinterpret_cast<const char*>(src) + ((base + (int64_t)t * kKeysPerTile) * row_elems + g * kHeadDim) * 2;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<char*>(at), 0, max(0, (rows - 1) * row_bytes + 2 * kHeadDim), 0x00020000);   // 0 when no row is left
#pragma unroll
    for (int i = 0; i < kLoads; ++i)
      r[i] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff0 + i * (kWaves * 4) * row_bytes, 0, 0));
  };
  auto store_k = [&](int slot) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int vv = tid + i * kWaves * 64;
      *reinterpret_cast<uint4*>(lds + slot * kStageBytes + (vv >> 4) * kTileStride + (vv & 15) * 16) = rk[i];
    }
  };
  auto store_v = [&](int slot) {
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
      const int vv = tid + i * kWaves * 64;
      *reinterpret_cast<uint4*>(lds + slot * kStageBytes + kVOffset + (vv >> 4) * kVStride + (vv & 15) * 16) = rv[i];
    }
  };
  const char* k_lane = lds + col * kTileStride + half * 16;
  const char* v_lane = lds + kVOffset + (4 * half + ((lane & 15) >> 2)) * kVStride + (lane & 16) * 2 + (lane & 3) * 8;

  auto step = [&](int t, floatx16_t (&sc)[2], floatx16_t (&sn)[2]) {
    const int slot = (t - first_tile) & 1;
    // (A) mask, column maximum
    const int key_base = t * kKeysPerTile + 4 * half;
    float mx_raw = -INFINITY;
    if ((t + 1) * kKeysPerTile <= wave_min_limit) {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx_raw = fmaxf(mx_raw, sc[rb][e]);
    } else {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = key_base + 32 * rb + 8 * (e >> 2) + (e & 3);
          const float x = key < limit ? sc[rb][e] : -INFINITY;
          sc[rb][e] = x;
          mx_raw = fmaxf(mx_raw, x);
        }
    }
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
    // (C) scores of tile t + 1 next to the exponentials of tile t (the K slot holds zeros past the last tile)
    const char* kn = k_lane + (slot ^ 1) * kStageBytes;
    float psum = 0.f;
    bf16x8_t pf[2][2];
    bf16x8_t kf[3][2];                      // K operands, fetched two steps ahead of their products
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
        kf[ks][rb] = *reinterpret_cast<const bf16x8_t*>(kn + rb * 32 * kTileStride + ks * 32);
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      if (ks + 2 < 8) {
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
          kf[(ks + 2) % 3][rb] = *reinterpret_cast<const bf16x8_t*>(kn + rb * 32 * kTileStride + (ks + 2) * 32);
      }
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        if (ks == 0) {
          floatx16_t z;
#pragma unroll
          for (int e = 0; e < 16; ++e) z[e] = 0.f;
          sn[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[0][rb], qf[0], z, 0, 0, 0);
        } else {
          sn[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[ks % 3][rb], qf[ks], sn[rb], 0, 0, 0);
        }
        // two of this tile's 32 probabilities per product
        const int prb = ks >> 2, e0 = (ks & 3) * 4 + 2 * rb;
        const float p0 = fast_exp2(fmaf(sc[prb][e0], scale_log2e, neg_m));
        const float p1 = fast_exp2(fmaf(sc[prb][e0 + 1], scale_log2e, neg_m));
        const uint32_t pk = pack_pair(p0, p1);
        psum = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, pk), __builtin_bit_cast(bf16x2_t, 0x3f803f80u), psum, false);
        pf[prb][e0 >> 3][e0 & 7] = __builtin_bit_cast(bf16x2_t, pk)[0];
        pf[prb][e0 >> 3][(e0 & 7) + 1] = __builtin_bit_cast(bf16x2_t, pk)[1];
      }
    }
    l += half_wave_sum(psum);
    // (D) O^T += V^T . P^T from this tile's V slot; refill the slots that are free
    const char* vt = v_lane + slot * kStageBytes;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const char* at = vt + (32 * rb + 16 * j) * kVStride + 64 * d;
          const shortx4_t lo = lds_read_tr16(at), hi = lds_read_tr16(at + 8 * kVStride);
          const bf16x8_t a = __builtin_bit_cast(bf16x8_t, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
          o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[rb][j], o[d], 0, 0, 0);
        }
    store_k(slot);           // K(t + 2): this slot's K was last read before the previous barrier
    store_v(slot ^ 1);       // V(t + 1): that slot's V was last read before the previous barrier
    gload_one(k, rk, t + 3);
    gload_one(v, rv, t + 2);
    // Issue order of the straight-line part above: every matrix product is followed by the LDS reads of operands
    // two products ahead and by a share of the exponentials, so neither the reads' latency nor the VALU work
    // leaves the matrix pipe idle; the tile stores and loads ride behind the last products.
    __builtin_amdgcn_sched_group_barrier(0x100, 4, 0);
#pragma unroll
    for (int i = 0; i < 12; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
    }
#pragma unroll
    for (int i = 0; i < 12; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, 1, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
    __syncthreads();
  };

  if (first_tile < n_tiles) {
    gload_one(k, rk, first_tile);
    gload_one(v, rv, first_tile);
    store_k(0);
    store_v(0);
    gload_one(k, rk, first_tile + 1);
    store_k(1);
    gload_one(k, rk, first_tile + 2);
    gload_one(v, rv, first_tile + 1);
    __syncthreads();
    floatx16_t s0[2], s1[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int e = 0; e < 16; ++e) s0[rb][e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(k_lane + rb * 32 * kTileStride + ks * 32);
        s0[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s0[rb], 0, 0, 0);
      }
    // the first step overwrites K slot 0 (with tile first + 2) before its own barrier: every wavefront must have
    // finished the reads of slot 0 above before any wavefront gets there
    __syncthreads();
    for (int t = first_tile; t < n_tiles; t += 2) {
      step(t, s0, s1);
      if (t + 1 < n_tiles) step(t + 1, s1, s0);
    }
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

template <int G, bool kSplit>
int flash_launch_g(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                   const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, float scale,
                   int32_t causal, void* out, SplitPlan plan, float* part_ml, float* part_acc, hipStream_t st) {
  constexpr int kTokPerBlock = kWaves * 32 / G;
  const int64_t blocks = ((int64_t)total_q + kTokPerBlock - 1) / kTokPerBlock + B;   // upper bound over ragged samples
  MSA_REQUIRE(blocks < (int64_t)1 << 31, "flash attention: too many query rows");
  dim3 grid((unsigned)blocks, (unsigned)Hkv, kSplit ? (unsigned)plan.n_split : 1u);
  auto kern = flash_attn_kernel<G, kSplit>;
  static std::atomic<int> lds_limit_raised{0};   // two tiles of K and V exceed the default dynamic LDS limit
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

extern "C" int msa_flash_attn(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                              const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, int32_t D,
                              float scale, int32_t causal, void* out, void* stream) {
  MSA_REQUIRE(q && k && v && kv_off && kv_len && out, "msa_flash_attn: null pointer");
  MSA_REQUIRE(D == kHeadDim, "msa_flash_attn: head dim %d unsupported (need %d)", D, kHeadDim);
  MSA_REQUIRE(B > 0 && total_q > 0, "msa_flash_attn: bad sizes");
  MSA_REQUIRE(cu_q != nullptr || total_q == B, "msa_flash_attn: cu_q is required when total_q != B");
  MSA_REQUIRE(Hkv > 0 && Hkv <= 65535 && Hq % Hkv == 0, "msa_flash_attn: Hq=%d Hkv=%d unsupported", Hq, Hkv);
  MSA_REQUIRE(scale > 0.f, "msa_flash_attn: scale must be positive");
  const int G = Hq / Hkv;
  MSA_REQUIRE(G == 1 || G == 2 || G == 4 || G == 8, "msa_flash_attn: GQA group size %d unsupported (1, 2, 4, 8)", G);
  return flash_launch<false>(G, q, cu_q, k, v, kv_off, kv_len, B, total_q, Hq, Hkv, scale,
                             causal, out, SplitPlan{1, 0}, (float*)nullptr, (float*)nullptr, as_stream(stream));
}

int flash_attn_split_launch(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                            const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, float scale,
                            int32_t causal, SplitPlan plan, float* part_ml, float* part_acc, hipStream_t st) {
  return flash_launch<true>(Hq / Hkv, q, cu_q, k, v, kv_off, kv_len, B, total_q, Hq,
                            Hkv, scale, causal, (void*)nullptr, plan, part_ml, part_acc, st);
}
