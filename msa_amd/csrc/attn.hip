// GQA attention of ragged query rows over per-sample KV ranges (decode and stage-2 prefill).
//
// Split-KV: workgroup (query row, KV head, split) streams its slice of K and V once and serves all
// G query heads of that KV head from the same loads.  A wavefront takes 4 keys per step (16 lanes
// per key, 8 head-dim elements per lane); every (key slot, dim slice) lane keeps an independent
// online-softmax state (m, l, acc[G][8]) that is merged across slots, wavefronts and finally
// splits (second kernel).  K / V rows are [Hkv, 128].
#include "attn_internal.h"

namespace {

// 2^x by the bare hardware instruction: the library exp2f wraps it in a range fix-up for results below
// 2^-126 (five more VALU operations per call); softmax arguments are <= 0 and such tails may flush to zero.
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }


constexpr int kMaxG = 8;

// 16 bytes of K or V with the non-temporal hint: a decode step reads every cache row exactly once, so the rows
// should not displace anything in L2 (the whole decode step runs 3 % faster with the hint).
typedef unsigned int u32x4_stream_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld16_stream(const void* p) {
  const u32x4_stream_t w = __builtin_nontemporal_load(reinterpret_cast<const u32x4_stream_t*>(p));
  return make_uint4(w.x, w.y, w.z, w.w);
}

template <typename T>
__device__ __forceinline__ void ld8(const T* p, float (&x)[8]) {
  if constexpr (sizeof(T) == 2) {
    const uint4 w = ld16_stream(p);
    x[0] = bf16lo(w.x); x[1] = bf16hi(w.x); x[2] = bf16lo(w.y); x[3] = bf16hi(w.y);
    x[4] = bf16lo(w.z); x[5] = bf16hi(w.z); x[6] = bf16lo(w.w); x[7] = bf16hi(w.w);
  } else {
    const uint4 a = ld16_stream(p), b = ld16_stream(p + 4);
    x[0] = __uint_as_float(a.x); x[1] = __uint_as_float(a.y); x[2] = __uint_as_float(a.z); x[3] = __uint_as_float(a.w);
    x[4] = __uint_as_float(b.x); x[5] = __uint_as_float(b.y); x[6] = __uint_as_float(b.z); x[7] = __uint_as_float(b.w);
  }
}

// Finds the sample owning query row `row` in cu_q (B is small: linear scan is fine and uniform).
__device__ __forceinline__ int find_sample(const int32_t* cu_q, int B, int row) {
  int b = 0;
  while (b + 1 < B && cu_q[b + 1] <= row) ++b;
  return b;
}

// sum over the 16 lanes of a DPP row (the lanes sharing one key); every lane gets the total
__device__ __forceinline__ float row16_allsum(float d) {
  d += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, d), 0x128, 0xf, 0xf, false));
  d += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, d), 0x124, 0xf, 0xf, false));
  d += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, d), 0x122, 0xf, 0xf, false));
  d += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, d), 0x121, 0xf, 0xf, false));
  return d;
}

// Streams keys first, first + stride, ... < key1 of one KV head through the running softmax state of this
// lane (key slot = lane / 16, dims 8 j .. 8 j + 8).  Keys go in batches of kBatch steps: all K / V loads of a
// batch are issued before any arithmetic (bytes in flight), scores are reduced over the 16 lanes of a key with
// DPP row rotations, and the running softmax is rescaled once per batch.  `lane_off` is the element offset of
// key 0's slice for this lane.
template <typename T, int G>
__device__ __forceinline__ void attend_keys(const T* __restrict__ k, const T* __restrict__ v, int64_t lane_off,
                                            int row_elems, int first, int key1, int stride, const float (&qv)[G][8],
                                            float (&m)[G], float (&l)[G], float (&acc)[G][8]) {
  constexpr int kBatch = 4;
  for (int kb = first; kb < key1; kb += stride * kBatch) {
    float kx[kBatch][8], vx[kBatch][8];
    bool ok[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int kk = kb + u * stride;
      ok[u] = kk < key1;
      const int64_t off = lane_off + (int64_t)(ok[u] ? kk : kb) * row_elems;   // clamp: always in range
      ld8<T>(k + off, kx[u]);
      ld8<T>(v + off, vx[u]);
    }
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float s[kBatch];
      float mb = m[h];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        float d = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) d += qv[h][i] * kx[u][i];
        d = row16_allsum(d);
        s[u] = ok[u] ? d : -INFINITY;
        mb = fmaxf(mb, s[u]);
      }
      // mb is finite here: the batch's first key is always valid
      const float alpha = fast_exp2(m[h] - mb);
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[h][i] *= alpha;
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const float pu = fast_exp2(s[u] - mb);
        psum += pu;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[h][i] += pu * vx[u][i];
      }
      l[h] = l[h] * alpha + psum;
      m[h] = mb;
    }
  }
}

// bf16 form on packed operands: q.k with v_dot2c_f32_bf16 (two products per instruction, K is never unpacked; q
// stays un-scaled in bf16 and the fp32 dot is scaled afterwards), and p.v over PAIRS of keys: the two keys'
// values of one dim are interleaved with v_perm_b32 and the two probabilities rounded to bf16 (as flash
// attention does before its second product).  qp[h][c] holds dims 8 j + 2 c, 8 j + 2 c + 1 of head h.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ float dot2_bf16(uint32_t a, uint32_t b, float c) {
  union { uint32_t u; bf16x2_t v; } x, y;
  x.u = a; y.u = b;
  return __builtin_amdgcn_fdot2_f32_bf16(x.v, y.v, c, false);
}
__device__ __forceinline__ uint32_t pack_pair_rne(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  union { bf16x2_t b; uint32_t u; } c;
  c.b = __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t);
  return c.u;
}

template <int G>
__device__ __forceinline__ void attend_keys_bf16(const bf16_t* __restrict__ k, const bf16_t* __restrict__ v,
                                                 int64_t lane_off, int row_elems, int first, int key1, int stride,
                                                 const uint32_t (&qp)[G][4], float scale_log2e, float (&m)[G],
                                                 float (&l)[G], float (&acc)[G][8]) {
  constexpr int kBatch = 4;
  for (int kb = first; kb < key1; kb += stride * kBatch) {
    uint4 kx[kBatch], vx[kBatch];
    bool ok[kBatch];
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int kk = kb + u * stride;
      ok[u] = kk < key1;
      const int64_t off = lane_off + (int64_t)(ok[u] ? kk : kb) * row_elems;   // clamp: always in range
      kx[u] = ld16_stream(k + off);
      vx[u] = ld16_stream(v + off);
    }
    // scores of all heads first: they only need K, so the arithmetic starts while V is still arriving
    float s[G][kBatch];
#pragma unroll
    for (int h = 0; h < G; ++h)
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        float d = dot2_bf16(qp[h][0], kx[u].x, 0.f);
        d = dot2_bf16(qp[h][1], kx[u].y, d);
        d = dot2_bf16(qp[h][2], kx[u].z, d);
        d = dot2_bf16(qp[h][3], kx[u].w, d);
        d = row16_allsum(d);
        s[h][u] = ok[u] ? d * scale_log2e : -INFINITY;
      }
    // the two keys of a pair, one dim per 32-bit word: vlo[pr][c] = (v_2pr[2c], v_2pr+1[2c]), vhi the odd dims
    uint32_t vlo[kBatch / 2][4], vhi[kBatch / 2][4];
#pragma unroll
    for (int pr = 0; pr < kBatch / 2; ++pr) {
      const uint32_t a[4] = {vx[2 * pr].x, vx[2 * pr].y, vx[2 * pr].z, vx[2 * pr].w};
      const uint32_t b[4] = {vx[2 * pr + 1].x, vx[2 * pr + 1].y, vx[2 * pr + 1].z, vx[2 * pr + 1].w};
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        vlo[pr][c] = __builtin_amdgcn_perm(b[c], a[c], 0x05040100u);
        vhi[pr][c] = __builtin_amdgcn_perm(b[c], a[c], 0x07060302u);
      }
    }
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float mb = m[h];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) mb = fmaxf(mb, s[h][u]);
      const float alpha = fast_exp2(m[h] - mb);          // mb is finite: the batch's first key is always valid
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[h][i] *= alpha;
#pragma unroll
      for (int pr = 0; pr < kBatch / 2; ++pr) {
        const float p0 = fast_exp2(s[h][2 * pr] - mb), p1 = fast_exp2(s[h][2 * pr + 1] - mb);
        psum += p0 + p1;
        const uint32_t pp = pack_pair_rne(p0, p1);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
          acc[h][2 * c] = dot2_bf16(vlo[pr][c], pp, acc[h][2 * c]);
          acc[h][2 * c + 1] = dot2_bf16(vhi[pr][c], pp, acc[h][2 * c + 1]);
        }
      }
      l[h] = l[h] * alpha + psum;
      m[h] = mb;
    }
  }
}

template <typename T, int G, int kAttnWaves>
__global__ __launch_bounds__(kAttnWaves * 64) void attn_partial_kernel(
    const T* __restrict__ q, const int32_t* __restrict__ cu_q, const T* __restrict__ k, const T* __restrict__ v,
    const int64_t* __restrict__ kv_off, const int32_t* __restrict__ kv_len, int32_t B, int32_t Hq, int32_t Hkv,
    float scale_log2e, int32_t causal, int32_t n_split, int32_t split_keys, float* __restrict__ part_ml,
    float* __restrict__ part_acc) {
  __shared__ float sm_m[kAttnWaves][G], sm_l[kAttnWaves][G];
  __shared__ float sm_acc[kAttnWaves][G][kHeadDim];

  const int row = blockIdx.x, g = blockIdx.y, split = blockIdx.z;
  const int b = cu_q ? find_sample(cu_q, B, row) : row;
  const int q_first = cu_q ? cu_q[b] : row;
  const int sq = cu_q ? cu_q[b + 1] - q_first : 1;
  const int L = kv_len[b];
  const int visible = causal ? max(0, L - sq + (row - q_first) + 1) : L;
  // balanced splits of this sample's own length (the host only knows an upper bound of it)
  const int per_split = split_keys > 0 ? split_keys : (L + n_split - 1) / n_split;
  const int key0 = split * per_split;
  const int key1 = min(visible, key0 + per_split);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slot = lane >> 4, j = lane & 15;
  const int64_t base = kv_off[b];
  const int row_elems = Hkv * kHeadDim;

  float m[G], l[G], acc[G][8];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m[h] = -INFINITY; l[h] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;
  }
  const int64_t lane_off = base * row_elems + g * kHeadDim + 8 * j;     // this lane's slice of key 0
  const T* q_lane = q + ((int64_t)row * Hq + g * G) * kHeadDim + 8 * j;
  // the packed form pays off once several heads share the loads (its dependent dot2 / DPP chains need the
  // other heads' work to hide behind): measured 61 vs 65 us at G = 4, 88 vs 112 at G = 8, but 65 vs 55 at G = 1
  if constexpr (sizeof(T) == 2 && G >= 4) {
    uint32_t qp[G][4];
#pragma unroll
    for (int h = 0; h < G; ++h) {
      const uint4 w = *reinterpret_cast<const uint4*>(q_lane + h * kHeadDim);
      qp[h][0] = w.x; qp[h][1] = w.y; qp[h][2] = w.z; qp[h][3] = w.w;
    }
    attend_keys_bf16<G>(k, v, lane_off, row_elems, key0 + wave * 4 + slot, key1, kAttnWaves * 4, qp, scale_log2e, m, l, acc);
  } else {
    float qv[G][8];
#pragma unroll
    for (int h = 0; h < G; ++h) {
      ld8<T>(q_lane + h * kHeadDim, qv[h]);
#pragma unroll
      for (int i = 0; i < 8; ++i) qv[h][i] *= scale_log2e;      // scores in log2 units: exp2f below
    }
    attend_keys<T, G>(k, v, lane_off, row_elems, key0 + wave * 4 + slot, key1, kAttnWaves * 4, qv, m, l, acc);
  }

  // merge the 4 key slots of the wavefront (lanes differing in bits 4 and 5)
#pragma unroll
  for (int h = 0; h < G; ++h) {
#pragma unroll
    for (int x = 16; x <= 32; x <<= 1) {
      const float mo = __shfl_xor(m[h], x), lo = __shfl_xor(l[h], x);
      const float mn = fmaxf(m[h], mo);
      const float a = mn == -INFINITY ? 0.f : fast_exp2(m[h] - mn), bo = mn == -INFINITY ? 0.f : fast_exp2(mo - mn);
      l[h] = l[h] * a + lo * bo;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[h][i] = acc[h][i] * a + __shfl_xor(acc[h][i], x) * bo;
      m[h] = mn;
    }
  }
  if (slot == 0) {
#pragma unroll
    for (int h = 0; h < G; ++h) {
      if (j == 0) { sm_m[wave][h] = m[h]; sm_l[wave][h] = l[h]; }
#pragma unroll
      for (int i = 0; i < 8; ++i) sm_acc[wave][h][8 * j + i] = acc[h][i];
    }
  }
  __syncthreads();

  // merge the wavefronts; thread (h, d) for h < G
  for (int idx = tid; idx < G * kHeadDim; idx += kAttnWaves * 64) {
    const int h = idx / kHeadDim, d = idx % kHeadDim;
    float mn = -INFINITY;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) mn = fmaxf(mn, sm_m[w][h]);
    float lt = 0.f, at = 0.f;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) {
      const float a = mn == -INFINITY ? 0.f : fast_exp2(sm_m[w][h] - mn);
      lt += sm_l[w][h] * a;
      at += sm_acc[w][h][d] * a;
    }
    const int64_t o = ((int64_t)row * Hq + g * G + h) * n_split + split;
    part_acc[o * kHeadDim + d] = at;
    if (d == 0) { part_ml[o * 2] = mn; part_ml[o * 2 + 1] = lt; }
  }
}

// ------------------------------------------------------------------------------------------------
// Decode step with the q / k RMSNorm, the rotary embedding and the cache append folded into the attention launch
// (bf16, one new token per sample, groups of 4 or 8 query heads).  Row b of `qkv` is the fused projection output
// [Hq q heads | Hkv k heads | Hkv v heads].  Every workgroup (sample, KV head, split) normalises and rotates the q
// heads of its group (16 lanes per head, 8 dims per lane, the same arithmetic as the stand-alone kernel) and shares
// them through LDS; the workgroup of the last split also prepares the new token's k / v row of its KV head, writes it
// to the cache at [b][kv_len[b]] and feeds it to its running softmax as one more key.  kv_len is only read here: the
// combine kernel that follows advances it.  A full cache drops the new row (and the token then does not see itself).
// ------------------------------------------------------------------------------------------------
__device__ __forceinline__ float row16_ror8(float v) {  // value of the lane 8 places away in the 16-lane row
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
}

// RMSNorm over the head's 128 dims (fp32) times the norm weight, then half-split rotary with the table row
// cos_row / sin_row; `src` and `w` point at this lane's 8 elements; returns them packed to bf16.
__device__ __forceinline__ uint4 norm_rope_8(const bf16_t* src, const bf16_t* w, float eps, const float* cos_row,
                                             const float* sin_row, int j) {
  const uint4 xr = *reinterpret_cast<const uint4*>(src), wr = *reinterpret_cast<const uint4*>(w);
  const uint32_t xs[4] = {xr.x, xr.y, xr.z, xr.w}, ws[4] = {wr.x, wr.y, wr.z, wr.w};
  float x[8], wt[8];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    x[2 * c] = bf16lo(xs[c]); x[2 * c + 1] = bf16hi(xs[c]);
    wt[2 * c] = bf16lo(ws[c]); wt[2 * c + 1] = bf16hi(ws[c]);
  }
  float ssq = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) ssq += x[i] * x[i];
  const float inv = rsqrtf(row16_allsum(ssq) * (1.0f / kHeadDim) + eps);
  const int f = 8 * (j & 7);                    // frequency index of this lane's first element
  float out[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float y = x[i] * inv * wt[i];
    const float other = row16_ror8(y);          // the paired dim (d + 64 for j < 8, d - 64 for j >= 8)
    const float c = cos_row[f + i], sn = sin_row[f + i];
    out[i] = j < 8 ? y * c - other * sn : y * c + other * sn;
  }
  uint4 r;
  r.x = pack_bf16x2(out[0], out[1]); r.y = pack_bf16x2(out[2], out[3]);
  r.z = pack_bf16x2(out[4], out[5]); r.w = pack_bf16x2(out[6], out[7]);
  return r;
}

template <int G>
__global__ __launch_bounds__(8 * 64) void attn_decode_fused_kernel(
    const bf16_t* __restrict__ qkv, int64_t row_stride, int32_t Hq, int32_t Hkv, const int64_t* __restrict__ pos,
    const bf16_t* __restrict__ qw, const bf16_t* __restrict__ kw, float eps, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int32_t rope_rows, bf16_t* __restrict__ kcache, bf16_t* __restrict__ vcache,
    int32_t Lcap, const int32_t* __restrict__ kv_len, float scale_log2e, int32_t n_split,
    float* __restrict__ part_ml, float* __restrict__ part_acc) {
  constexpr int kW = 8;
  __shared__ float sm_m[kW][G], sm_l[kW][G];
  __shared__ float sm_acc[kW][G][kHeadDim];
  __shared__ uint4 sm_q[G][16];

  const int b = blockIdx.x, g = blockIdx.y, split = blockIdx.z;
  const int L_old = kv_len[b];
  const bool has_new = L_old < Lcap;
  const int per_split = (L_old + n_split - 1) / n_split;
  const int key0 = split * per_split;
  const int key1 = min(L_old, key0 + per_split);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int slot = lane >> 4, j = lane & 15;
  const int row_elems = Hkv * kHeadDim;
  const int64_t p = min((int64_t)max((int64_t)0, pos[b]), (int64_t)rope_rows - 1);
  const float* cos_row = cos_t + p * 64;
  const float* sin_row = sin_t + p * 64;
  const bf16_t* row = qkv + (int64_t)b * row_stride;

  // q heads of the group: head 4 wave + slot (wavefront 0, and wavefront 1 when G = 8)
  const int hq = wave * 4 + slot;
  if (hq < G) sm_q[hq][j] = norm_rope_8(row + (int64_t)(g * G + hq) * kHeadDim + 8 * j, qw + 8 * j, eps, cos_row, sin_row, j);
  // the new token's key / value of this KV head: the last wavefront's first key slot, in the last split only
  const bool owner = split == n_split - 1 && wave == kW - 1 && slot == 0 && has_new;
  uint4 k_new = make_uint4(0, 0, 0, 0), v_new = k_new;
  if (owner) {
    k_new = norm_rope_8(row + (int64_t)(Hq + g) * kHeadDim + 8 * j, kw + 8 * j, eps, cos_row, sin_row, j);
    v_new = *reinterpret_cast<const uint4*>(row + (int64_t)(Hq + Hkv + g) * kHeadDim + 8 * j);
    const int64_t at = (((int64_t)b * Lcap + L_old) * Hkv + g) * kHeadDim + 8 * j;
    *reinterpret_cast<uint4*>(kcache + at) = k_new;
    *reinterpret_cast<uint4*>(vcache + at) = v_new;
  }
  __syncthreads();

  float m[G], l[G], acc[G][8];
  uint32_t qp[G][4];
#pragma unroll
  for (int h = 0; h < G; ++h) {
    m[h] = -INFINITY; l[h] = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[h][i] = 0.f;
    const uint4 w = sm_q[h][j];
    qp[h][0] = w.x; qp[h][1] = w.y; qp[h][2] = w.z; qp[h][3] = w.w;
  }
  const int64_t lane_off = (int64_t)b * Lcap * row_elems + g * kHeadDim + 8 * j;     // this lane's slice of key 0
  attend_keys_bf16<G>(kcache, vcache, lane_off, row_elems, key0 + wave * 4 + slot, key1, kW * 4, qp, scale_log2e, m, l, acc);
  if (owner) {
    // one more key, straight from registers; the probability is rounded to bf16 as in the paired products above
    const uint32_t vs[4] = {v_new.x, v_new.y, v_new.z, v_new.w};
#pragma unroll
    for (int h = 0; h < G; ++h) {
      float d = dot2_bf16(qp[h][0], k_new.x, 0.f);
      d = dot2_bf16(qp[h][1], k_new.y, d);
      d = dot2_bf16(qp[h][2], k_new.z, d);
      d = dot2_bf16(qp[h][3], k_new.w, d);
      const float sc = row16_allsum(d) * scale_log2e;
      const float mb = fmaxf(m[h], sc);
      const float alpha = fast_exp2(m[h] - mb), pr = fast_exp2(sc - mb);
      const float prb = bf16lo(pack_pair_rne(pr, 0.f));
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        acc[h][2 * c] = acc[h][2 * c] * alpha + prb * bf16lo(vs[c]);
        acc[h][2 * c + 1] = acc[h][2 * c + 1] * alpha + prb * bf16hi(vs[c]);
      }
      l[h] = l[h] * alpha + pr;
      m[h] = mb;
    }
  }

  // merge the 4 key slots of the wavefront (lanes differing in bits 4 and 5)
#pragma unroll
  for (int h = 0; h < G; ++h) {
#pragma unroll
    for (int x = 16; x <= 32; x <<= 1) {
      const float mo = __shfl_xor(m[h], x), lo = __shfl_xor(l[h], x);
      const float mn = fmaxf(m[h], mo);
      const float a = mn == -INFINITY ? 0.f : fast_exp2(m[h] - mn), bo = mn == -INFINITY ? 0.f : fast_exp2(mo - mn);
      l[h] = l[h] * a + lo * bo;
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[h][i] = acc[h][i] * a + __shfl_xor(acc[h][i], x) * bo;
      m[h] = mn;
    }
  }
  if (slot == 0) {
#pragma unroll
    for (int h = 0; h < G; ++h) {
      if (j == 0) { sm_m[wave][h] = m[h]; sm_l[wave][h] = l[h]; }
#pragma unroll
      for (int i = 0; i < 8; ++i) sm_acc[wave][h][8 * j + i] = acc[h][i];
    }
  }
  __syncthreads();
  for (int idx = tid; idx < G * kHeadDim; idx += kW * 64) {
    const int h = idx / kHeadDim, d = idx % kHeadDim;
    float mn = -INFINITY;
#pragma unroll
    for (int w = 0; w < kW; ++w) mn = fmaxf(mn, sm_m[w][h]);
    float lt = 0.f, at = 0.f;
#pragma unroll
    for (int w = 0; w < kW; ++w) {
      const float a = mn == -INFINITY ? 0.f : fast_exp2(sm_m[w][h] - mn);
      lt += sm_l[w][h] * a;
      at += sm_acc[w][h][d] * a;
    }
    const int64_t o = ((int64_t)b * Hq + g * G + h) * n_split + split;
    part_acc[o * kHeadDim + d] = at;
    if (d == 0) { part_ml[o * 2] = mn; part_ml[o * 2 + 1] = lt; }
  }
}

// One workgroup of 128 threads per (query row, head): merge the splits and normalise.
// With `bump_len` (decode step whose attention kernel appended the new token's K / V row itself) the workgroup of
// head 0 of row b also advances bump_len[b], unless the cache was full and the row was dropped.
template <typename T>
__global__ __launch_bounds__(kHeadDim) void attn_combine_kernel(const float* __restrict__ part_ml,
                                                                const float* __restrict__ part_acc, int32_t n_split,
                                                                T* __restrict__ out, int32_t* __restrict__ bump_len = nullptr,
                                                                int32_t Lcap = 0, int32_t Hq = 1) {
  const int64_t rh = blockIdx.x;   // row * Hq + head
  const int d = threadIdx.x;
  if (bump_len != nullptr && d == 0 && rh % Hq == 0) {
    const int64_t b = rh / Hq;
    const int32_t len = bump_len[b];
    if (len < Lcap) bump_len[b] = len + 1;
  }
  float mn = -INFINITY;
  for (int s = 0; s < n_split; ++s) mn = fmaxf(mn, part_ml[(rh * n_split + s) * 2]);
  float lt = 0.f, at = 0.f;
  for (int s = 0; s < n_split; ++s) {
    const float ms = part_ml[(rh * n_split + s) * 2];
    const float a = ms == -INFINITY ? 0.f : fast_exp2(ms - mn);
    lt += part_ml[(rh * n_split + s) * 2 + 1] * a;
    at += part_acc[(rh * n_split + s) * kHeadDim + d] * a;
  }
  const float o = lt > 0.f ? at / lt : 0.f;     // a row that sees no key yields zeros
  if constexpr (sizeof(T) == 2) out[rh * kHeadDim + d] = f32_to_bf16(o);
  else out[rh * kHeadDim + d] = o;
}

template <typename T>
int launch_attn(const void* q, const int32_t* cu_q, const void* k, const void* v, const int64_t* kv_off,
                const int32_t* kv_len, int32_t B, int32_t total_q, int32_t Hq, int32_t Hkv, float scale,
                int32_t causal, SplitPlan plan, void* out, float* part_ml, float* part_acc, hipStream_t st) {
  const int n_split = plan.n_split;
  const int G = Hq / Hkv;
  dim3 grid((unsigned)total_q, (unsigned)Hkv, (unsigned)n_split);
  const float sl2 = scale * 1.4426950408889634f;
  // Wavefronts per workgroup: the VALU work grows with the group size, and one 8-wavefront workgroup per
  // compute unit measured better for G >= 4 than two of 4 (61 vs 64 us on the decode shape).
#define MSA_ATTN_CASE(GG, WW)                                                                                      \
  case GG:                                                                                                         \
    attn_partial_kernel<T, GG, WW><<<grid, WW * 64, 0, st>>>(                                                      \
        static_cast<const T*>(q), cu_q, static_cast<const T*>(k), static_cast<const T*>(v), kv_off, kv_len, B, Hq, \
        Hkv, sl2, causal, n_split, 0, part_ml, part_acc);                                                          \
    break;
  switch (G) {
    MSA_ATTN_CASE(1, 4)
    MSA_ATTN_CASE(2, 4)
    MSA_ATTN_CASE(4, 8)
    MSA_ATTN_CASE(8, 8)
    default:
      msa_set_error("msa_sparse_attn: GQA group size %d unsupported (1, 2, 4, 8)", G);
      return MSA_EINVAL;
  }
#undef MSA_ATTN_CASE
  MSA_LAUNCH_CHECK();
  attn_combine_kernel<T><<<(unsigned)((int64_t)total_q * Hq), kHeadDim, 0, st>>>(part_ml, part_acc, n_split,
                                                                                 static_cast<T*>(out));
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}

}  // namespace

extern "C" size_t msa_attn_workspace_bytes(int32_t total_q, int32_t Hq, int32_t Hkv, int32_t D, int32_t max_kv) {
  if (total_q <= 0 || Hq <= 0 || Hkv <= 0 || D <= 0 || max_kv <= 0) return 0;
  // sized for whichever of the two kernels splits the keys further
  const int splits = std::max(plan_splits(total_q, Hkv, max_kv).n_split, plan_splits_valu(total_q, Hkv, max_kv).n_split);
  const size_t n = (size_t)total_q * Hq * splits;
  return align_up(n * 2 * sizeof(float), 256) + align_up(n * D * sizeof(float), 256);
}

extern "C" int msa_sparse_attn(const void* q, const int32_t* cu_q, const void* k, const void* v,
                               const int64_t* kv_off, const int32_t* kv_len, int32_t B, int32_t total_q,
                               int32_t max_sq, int32_t max_kv, int32_t Hq, int32_t Hkv, int32_t D, int32_t dtype,
                               float scale, int32_t causal, void* out, void* workspace, size_t workspace_bytes,
                               void* stream) {
  MSA_REQUIRE(q && k && v && kv_off && kv_len && out && workspace, "msa_sparse_attn: null pointer");
  MSA_REQUIRE(D == kHeadDim, "msa_sparse_attn: head dim %d unsupported (need %d)", D, kHeadDim);
  MSA_REQUIRE(B > 0 && total_q > 0 && max_sq > 0 && max_kv > 0, "msa_sparse_attn: bad sizes");
  MSA_REQUIRE(cu_q != nullptr || total_q == B, "msa_sparse_attn: cu_q is required when total_q != B");
  MSA_REQUIRE(Hkv > 0 && Hq % Hkv == 0 && Hq / Hkv <= kMaxG, "msa_sparse_attn: Hq=%d Hkv=%d unsupported", Hq, Hkv);
  MSA_REQUIRE(dtype == MSA_BF16 || dtype == MSA_F32, "msa_sparse_attn: bad dtype %d", dtype);
  MSA_REQUIRE(scale > 0.f, "msa_sparse_attn: scale must be positive");
  MSA_REQUIRE((((uintptr_t)q | (uintptr_t)k | (uintptr_t)v | (uintptr_t)out) & 15) == 0,
              "msa_sparse_attn: q, k, v and out must be 16-byte aligned");
  MSA_REQUIRE((int64_t)total_q * Hq < (int64_t)1 << 31 && total_q < 65536 * 32, "msa_sparse_attn: too many rows");
  const bool mfma = dtype == MSA_BF16 && max_sq >= 8;
  const SplitPlan plan = mfma ? plan_splits(total_q, Hkv, max_kv) : plan_splits_valu(total_q, Hkv, max_kv);
  const int n_split = plan.n_split;
  MSA_REQUIRE(n_split <= 65535, "msa_sparse_attn: max_kv=%d too large", max_kv);
  const size_t need = msa_attn_workspace_bytes(total_q, Hq, Hkv, D, max_kv);
  if (need > workspace_bytes) {
    msa_set_error("msa_sparse_attn: workspace of %zu bytes, need %zu", workspace_bytes, need);
    return MSA_ESIZE;
  }
  const size_t n = (size_t)total_q * Hq * n_split;
  float* part_ml = static_cast<float*>(workspace);
  float* part_acc = reinterpret_cast<float*>(static_cast<char*>(workspace) + align_up(n * 2 * sizeof(float), 256));
  hipStream_t st = as_stream(stream);
  if (mfma) {
    // bf16 query blocks: MFMA partial pass (K / V tiles through LDS) + the common combine; single rows
    // (decode) stay on the split-KV kernel below, which keeps more loads in flight per wavefront
    int rc = flash_attn_split_launch(q, cu_q, k, v, kv_off, kv_len, B, total_q, Hq, Hkv, scale, causal, plan, part_ml,
                                     part_acc, st);
    if (rc != MSA_OK) return rc;
    attn_combine_kernel<bf16_t><<<(unsigned)((int64_t)total_q * Hq), kHeadDim, 0, st>>>(part_ml, part_acc, n_split,
                                                                                      static_cast<bf16_t*>(out));
    MSA_LAUNCH_CHECK();
    return MSA_OK;
  }
  if (dtype == MSA_BF16)
    return launch_attn<bf16_t>(q, cu_q, k, v, kv_off, kv_len, B, total_q, Hq, Hkv, scale, causal, plan, out, part_ml,
                               part_acc, st);
  return launch_attn<float>(q, cu_q, k, v, kv_off, kv_len, B, total_q, Hq, Hkv, scale, causal, plan, out, part_ml,
                            part_acc, st);
}

extern "C" int msa_decode_attn_fused(const void* qkv, int64_t row_stride, const int64_t* positions, const void* q_norm_w,
                                     const void* k_norm_w, float eps, const float* rope_cos, const float* rope_sin,
                                     int32_t rope_rows, int32_t B, int32_t Hq, int32_t Hkv, int32_t D, void* kcache,
                                     void* vcache, int32_t Lcap, int32_t* kv_len, float scale, void* out,
                                     void* workspace, size_t workspace_bytes, void* stream) {
  MSA_REQUIRE(qkv && positions && q_norm_w && k_norm_w && rope_cos && rope_sin && kcache && vcache && kv_len && out &&
                  workspace, "msa_decode_attn_fused: null pointer");
  MSA_REQUIRE(D == kHeadDim, "msa_decode_attn_fused: head dim %d unsupported (need %d)", D, kHeadDim);
  MSA_REQUIRE(B > 0 && Hkv > 0 && Hkv <= 65535 && Hq % Hkv == 0 && (Hq / Hkv == 4 || Hq / Hkv == 8),
              "msa_decode_attn_fused: B=%d Hq=%d Hkv=%d (groups of 4 or 8 query heads)", B, Hq, Hkv);
  MSA_REQUIRE(row_stride >= (int64_t)(Hq + 2 * Hkv) * D && row_stride % 8 == 0, "msa_decode_attn_fused: bad row stride");
  MSA_REQUIRE((((uintptr_t)qkv | (uintptr_t)q_norm_w | (uintptr_t)k_norm_w | (uintptr_t)kcache | (uintptr_t)vcache) & 15) == 0,
              "msa_decode_attn_fused: pointers must be 16-byte aligned");
  MSA_REQUIRE(Lcap > 0 && rope_rows > 0 && eps > 0.f && scale > 0.f, "msa_decode_attn_fused: bad scalar argument");
  const SplitPlan plan = plan_splits_valu(B, Hkv, Lcap);
  const int n_split = plan.n_split;
  const size_t need = msa_attn_workspace_bytes(B, Hq, Hkv, D, Lcap);
  if (need > workspace_bytes) {
    msa_set_error("msa_decode_attn_fused: workspace of %zu bytes, need %zu", workspace_bytes, need);
    return MSA_ESIZE;
  }
  const size_t n = (size_t)B * Hq * n_split;
  float* part_ml = static_cast<float*>(workspace);
  float* part_acc = reinterpret_cast<float*>(static_cast<char*>(workspace) + align_up(n * 2 * sizeof(float), 256));
  hipStream_t st = as_stream(stream);
  dim3 grid((unsigned)B, (unsigned)Hkv, (unsigned)n_split);
  const float sl2 = scale * 1.4426950408889634f;
#define MSA_FUSED_CASE(GG)                                                                                           \
  attn_decode_fused_kernel<GG><<<grid, 8 * 64, 0, st>>>(                                                            \
      static_cast<const bf16_t*>(qkv), row_stride, Hq, Hkv, positions, static_cast<const bf16_t*>(q_norm_w),         \
      static_cast<const bf16_t*>(k_norm_w), eps, rope_cos, rope_sin, rope_rows, static_cast<bf16_t*>(kcache),        \
      static_cast<bf16_t*>(vcache), Lcap, kv_len, sl2, n_split, part_ml, part_acc)
  if (Hq / Hkv == 4) MSA_FUSED_CASE(4); else MSA_FUSED_CASE(8);
#undef MSA_FUSED_CASE
  MSA_LAUNCH_CHECK();
  attn_combine_kernel<bf16_t><<<(unsigned)((int64_t)B * Hq), kHeadDim, 0, st>>>(part_ml, part_acc, n_split,
                                                                                static_cast<bf16_t*>(out), kv_len, Lcap, Hq);
  MSA_LAUNCH_CHECK();
  return MSA_OK;
}
