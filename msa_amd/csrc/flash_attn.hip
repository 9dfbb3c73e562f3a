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
// leaves registers.  V is transposed on its way into LDS (16-bit stores into [dim][key] rows with
// that key order, XOR-swizzled so the stores of a wavefront spread over all banks) and read back
// as 16-byte operands.
#include "attn_internal.h"

namespace {

// 2^x by the bare hardware instruction: the library exp2f wraps it in a range fix-up for results below
// 2^-126 (five more VALU operations per call); softmax arguments are <= 0 and such tails may flush to zero.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }


typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16_t;

constexpr int kKeysPerTile = 64;
constexpr int kTileStride = 2 * kHeadDim + 16;   // bytes per key row in LDS: 256 + 16 pad (conflict-free b128 reads)
constexpr int kVtStride = 2 * kKeysPerTile + 16;  // bytes per dim row of the transposed V tile
constexpr int kFlashWaves = 4;

// Position of key (0..63) inside a V^T row: bits 2 and 3 swapped (the accumulator layout holds keys
// {0-3, 8-11} in one half-wave and {4-7, 12-15} in the other), then XOR with a per-dim-group value.
__device__ __forceinline__ int vt_pos(int key, int dim) {
  const int p = (key & ~12) | ((key & 4) << 1) | ((key & 8) >> 1);
  return p ^ ((dim >> 4) << 3);
}

// kSplit: blockIdx.z selects a range of split_keys keys; the un-normalised accumulators and the
// (reference max, sum) pair of every column go to part_acc / part_ml for the combine kernel.
template <int G, bool kSplit>
__global__ __launch_bounds__(kFlashWaves * 64, 2) void flash_attn_kernel(
    const bf16_t* __restrict__ q, const int32_t* __restrict__ cu_q, const bf16_t* __restrict__ k,
    const bf16_t* __restrict__ v, const int64_t* __restrict__ kv_off, const int32_t* __restrict__ kv_len, int32_t B,
    int32_t Hq, int32_t Hkv, float scale_log2e, int32_t causal, bf16_t* __restrict__ out, int32_t n_split,
    int32_t split_keys, float* __restrict__ part_ml, float* __restrict__ part_acc) {
  constexpr int kTokPerWave = 32 / G;
  constexpr int kTokPerBlock = kFlashWaves * kTokPerWave;
  __shared__ __align__(16) char lds_k[kKeysPerTile * kTileStride];
  __shared__ __align__(16) char lds_v[kHeadDim * kVtStride];

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

  uint4 rk[4], rv[4];
  auto gload = [&](int t) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int vv = tid + i * kFlashWaves * 64;
      const int key = t * kKeysPerTile + (vv >> 4), dvec = vv & 15;
      if (key < kmax) {
        const int64_t off = (base + key) * row_elems + g * kHeadDim + dvec * 8;
        rk[i] = *reinterpret_cast<const uint4*>(k + off);
        rv[i] = *reinterpret_cast<const uint4*>(v + off);
      } else {
        rk[i] = make_uint4(0, 0, 0, 0);
        rv[i] = make_uint4(0, 0, 0, 0);
      }
    }
  };
  auto lstore = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int vv = tid + i * kFlashWaves * 64;
      const int at = (vv >> 4) * kTileStride + (vv & 15) * 16;
      *reinterpret_cast<uint4*>(lds_k + at) = rk[i];
      const int key = vv >> 4, d0 = (vv & 15) * 8;
      const uint32_t w[4] = {rv[i].x, rv[i].y, rv[i].z, rv[i].w};
#pragma unroll
      for (int e = 0; e < 8; ++e)
        *reinterpret_cast<bf16_t*>(lds_v + (d0 + e) * kVtStride + vt_pos(key, d0 + e) * 2) =
            (bf16_t)(w[e >> 1] >> (16 * (e & 1)));
    }
  };

  if (first_tile < n_tiles) gload(first_tile);
  for (int t = first_tile; t < n_tiles; ++t) {
    __syncthreads();                 // everyone is done reading the previous tile
    lstore();
    __syncthreads();
    if (t + 1 < n_tiles) gload(t + 1);

    // S^T = K . Q^T for the tile's two blocks of 32 keys
    floatx16_t s[2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int e = 0; e < 16; ++e) s[rb][e] = 0.f;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
#pragma unroll
      for (int rb = 0; rb < 2; ++rb) {
        const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(lds_k + (rb * 32 + col) * kTileStride + ks * 32 + half * 16);
        s[rb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s[rb], 0, 0, 0);
      }

    // online softmax of this lane's column; element e of block rb is key 64 t + 32 rb + 8 (e / 4) + 4 half + e % 4
    const int key_base = t * kKeysPerTile + 4 * half;
    // (the maximum is taken over the raw dot products and scaled once: scale > 0; the scale itself is folded
    //  into the exponent's argument with one fma per element further down)
    float mx_raw = -INFINITY;
    if ((t + 1) * kKeysPerTile <= wave_min_limit) {    // interior tile: every key visible to every column
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int e = 0; e < 16; ++e) mx_raw = fmaxf(mx_raw, s[rb][e]);
    } else {
#pragma unroll
      for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int key = key_base + 32 * rb + 8 * (e >> 2) + (e & 3);
          const float x = key < limit ? s[rb][e] : -INFINITY;
          s[rb][e] = x;
          mx_raw = fmaxf(mx_raw, x);
        }
    }
    float mx = fmaxf(m, mx_raw * scale_log2e);
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const bool none = mx == -INFINITY;                 // nothing visible to this column so far
    // Lazy rescaling: keep the old reference maximum while the new one is at most 2^6 above it; the
    // probabilities are then at most 64 (exact in bf16's range) and the accumulators are untouched.
    // The decision is wave-uniform so the 64 accumulator multiplies are skipped as a block.
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
    const float neg_m = none ? 0.f : -m;               // nothing visible yet: every score is -inf, keep the argument -inf
    float psum = 0.f;
    bf16x8_t pf[2][2];
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const float p = fast_exp2(fmaf(s[rb][e], scale_log2e, neg_m));     // -inf (masked) -> 0
        psum += p;
        pf[rb][e >> 3][e & 7] = (__bf16)p;
      }
    psum += __shfl_xor(psum, 32);
    l += psum;

    // O^T += V^T . P^T: the k slots of step (rb, j) are the keys this lane's P values belong to
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const int dim = 32 * d + col;
          const int pos = (32 * rb + 16 * j + 8 * half) ^ ((dim >> 4) << 3);      // 8 keys of this half, in slot order
          const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(lds_v + dim * kVtStride + pos * 2);
          o[d] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf[rb][j], o[d], 0, 0, 0);
        }
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
  const int tok_per_block = kFlashWaves * 32 / G;
  const int64_t blocks = ((int64_t)total_q + tok_per_block - 1) / tok_per_block + B;   // upper bound over ragged samples
  MSA_REQUIRE(blocks < (int64_t)1 << 31, "msa_flash_attn: too many query rows");
  dim3 grid((unsigned)blocks, (unsigned)Hkv);
  const float sl2 = scale * 1.4426950408889634f;
  hipStream_t st = as_stream(stream);
#define MSA_FLASH_CASE(GG)                                                                                        \
  case GG:                                                                                                        \
    flash_attn_kernel<GG, false><<<grid, kFlashWaves * 64, 0, st>>>(                                              \
        static_cast<const bf16_t*>(q), cu_q, static_cast<const bf16_t*>(k), static_cast<const bf16_t*>(v), kv_off, \
        kv_len, B, Hq, Hkv, sl2, causal, static_cast<bf16_t*>(out), 1, 0, nullptr, nullptr);                      \
    break;
  switch (G) {
    MSA_FLASH_CASE(1)
    MSA_FLASH_CASE(2)
    MSA_FLASH_CASE(4)
    MSA_FLASH_CASE(8)
  }
#undef MSA_FLASH_CASE
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

int flash_attn_split_launch(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                            const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, float scale,
                            int32_t causal, SplitPlan plan, float* part_ml, float* part_acc, hipStream_t st) {
  const int G = Hq / Hkv;
  const int tok_per_block = kFlashWaves * 32 / G;
  const int64_t blocks = ((int64_t)total_q + tok_per_block - 1) / tok_per_block + B;   // upper bound over ragged samples
  MSA_REQUIRE(blocks < (int64_t)1 << 31, "msa_sparse_attn: too many query rows");
  dim3 grid((unsigned)blocks, (unsigned)Hkv, (unsigned)plan.n_split);
  const float sl2 = scale * 1.4426950408889634f;
#define MSA_FLASH_SPLIT_CASE(GG)                                                                                  \
  case GG:                                                                                                        \
    flash_attn_kernel<GG, true><<<grid, kFlashWaves * 64, 0, st>>>(                                               \
        static_cast<const bf16_t*>(q), cu_q, static_cast<const bf16_t*>(k), static_cast<const bf16_t*>(v), kv_off, \
        kv_len, B, Hq, Hkv, sl2, causal, nullptr, plan.n_split, plan.split_keys, part_ml, part_acc);              \
    break;
  switch (G) {
    MSA_FLASH_SPLIT_CASE(1)
    MSA_FLASH_SPLIT_CASE(2)
    MSA_FLASH_SPLIT_CASE(4)
    MSA_FLASH_SPLIT_CASE(8)
    default:
      msa_set_error("msa_sparse_attn: GQA group size %d unsupported (1, 2, 4, 8)", G);
      return MSA_EINVAL;
  }
#undef MSA_FLASH_SPLIT_CASE
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}
