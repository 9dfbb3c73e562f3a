// Shared helpers for the gfx950 kernels: error plumbing, bf16 bit tricks, ordered float keys.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>
#include <stdio.h>

#include "../../include/msa_amd.h"

void msa_set_error(const char* fmt, ...);

#define MSA_REQUIRE(cond, ...)                \
  do {                                        \
    if (!(cond)) {                            \
      msa_set_error(__VA_ARGS__);             \
      return MSA_EINVAL;                      \
    }                                         \
  } while (0)

#define MSA_HIP(call)                                                                  \
  do {                                                                                 \
    hipError_t e__ = (call);                                                           \
    if (e__ != hipSuccess) {                                                           \
      msa_set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e__), __FILE__,  \
                    __LINE__);                                                         \
      return MSA_EHIP;                                                                 \
    }                                                                                  \
  } while (0)

#define MSA_LAUNCH_CHECK() MSA_HIP(hipGetLastError())

// A kernel that needs more dynamic LDS than the default limit gets its limit raised before its first launch, once
// per process whatever the number of host threads (the library drives one device per process).  `done` is the
// per-kernel flag of the call site.
static inline hipError_t raise_dynamic_lds_limit(std::atomic<int>& done, const void* kernel, int bytes) {
  if (done.load(std::memory_order_acquire)) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) done.store(1, std::memory_order_release);   // two threads racing here set the same value twice
  return e;
}

// The kernels whose main loops are asm statements on physical registers keep state in registers across statements:
// that only holds while the compiler spills nothing (a spill's reload is a vector-memory load among hand-counted
// waits, and its address set-up lands in registers the statements own).  The build checks this on the device
// assembly; this is the same check on the code object that was actually loaded, once per kernel, before its first
// launch.
static inline int check_asm_kernel_resources(std::atomic<int>& done, const void* kernel, const char* name, int* num_regs,
                                             int* scratch_bytes) {
  if (done.load(std::memory_order_acquire) && !num_regs) return MSA_OK;
  hipFuncAttributes attr;
  const hipError_t e = hipFuncGetAttributes(&attr, kernel);
  if (e != hipSuccess) {
    msa_set_error("hipFuncGetAttributes(%s) failed: %s", name, hipGetErrorString(e));
    return MSA_EHIP;
  }
  if (num_regs) *num_regs = attr.numRegs;
  if (scratch_bytes) *scratch_bytes = (int)attr.localSizeBytes;
  // (512 registers: the statements name registers up to v255 and a255, and one wavefront per SIMD is what they are
  // scheduled for)
  if (attr.localSizeBytes != 0 || attr.numRegs != 512) {
    msa_set_error("%s was built with %d registers and %d bytes of scratch per lane (512 and 0 expected): its asm "
                  "statements' register contract does not hold", name, attr.numRegs, (int)attr.localSizeBytes);
    return MSA_ESTATE;
  }
  done.store(1, std::memory_order_release);
  return MSA_OK;
}

// Compute units of the current device (asked once; the library drives one device per process).
static inline int device_compute_units() {
  static const int n = [] {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    return cus;
  }();
  return n;
}

typedef uint16_t bf16_t;  // raw bf16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t x) { return __uint_as_float(((uint32_t)x) << 16); }

// round-to-nearest-even, NaN stays NaN: gfx950's packed conversion instruction (v_cvt_pk_bf16_f32)
typedef __bf16 msa_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float msa_f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(msa_f32x2_t{lo, hi}, msa_bf16x2_t));
}
__device__ __forceinline__ bf16_t f32_to_bf16(float f) { return (bf16_t)(pack_bf16x2(f, f) & 0xffffu); }

__device__ __forceinline__ float bf16lo(uint32_t w) { return __uint_as_float(w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }

// Monotone float -> uint32 map (larger float = larger key); key 0 is below every real number.
__device__ __forceinline__ uint32_t f32_to_key(float f) {
  uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_to_f32(uint32_t k) {
  uint32_t u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __uint_as_float(u);
}

__device__ __forceinline__ float row16_sum(float v) {   // all-reduce over the 16 lanes of a DPP row
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x124, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x122, 0xf, 0xf, false));
  v += __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x121, 0xf, 0xf, false));
  return v;
}
__device__ __forceinline__ float row16_ror8(float v) {  // value of the lane 8 places away in the row
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0x128, 0xf, 0xf, false));
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;
// 16 bytes per lane from a buffer resource straight into LDS (lane l lands at byte 16 * l behind `lds_dst`, which must be
// the same in every lane).  The compiler's host pass has no such instruction and only needs the kernel's signature.
#if defined(__HIP_DEVICE_COMPILE__)
#define MSA_LOAD_TO_LDS(rsrc, lds_dst, voffset, soffset, aux) \
  __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_ptr_t)(lds_dst), 16, voffset, soffset, 0, aux)
#else
#define MSA_LOAD_TO_LDS(rsrc, lds_dst, voffset, soffset, aux) ((void)(rsrc), (void)(lds_dst), (void)(voffset), (void)(soffset))
#endif

static inline hipStream_t as_stream(void* s) { return (hipStream_t)s; }
static inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
static inline size_t elem_bytes(int dtype) { return dtype == MSA_F32 ? 4 : 2; }

constexpr int kHeadDim = 128;

// Bank handle (bank.hip).  Tables live on both sides; per-layer tensors are borrowed.
struct msa_bank {
  int32_t n_layers;
  int64_t C;
  int32_t Hkv;
  int32_t D;
  int32_t dtype;
  int64_t n_docs;
  int32_t device;
  int32_t* doc_chunk_off_dev;   // [n_docs+1]
  int32_t* chunk_doc_dev;       // [C] document of every chunk (the scoring epilogue folds chunk maxima per document)
  int64_t* doc_global_id_dev;   // [n_docs]
  int32_t* doc_chunk_off_host;  // [n_docs+1]
  int64_t* doc_global_id_host;  // [n_docs]
  const void** kr_dev;          // [n_layers]
  const void** k_host;
  const void** v_host;
};
