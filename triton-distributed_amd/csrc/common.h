// Shared host/device helpers for libtdist_hip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tdist.h"

#define TDIST_AS1 __attribute__((address_space(1)))
#define TDIST_AS3 __attribute__((address_space(3)))

namespace tdist {

// ---- host side -------------------------------------------------------------------------------
struct DeviceInfo {
  int ok;        // 1 once probed successfully
  int num_cus;   // compute units of the current device
  int num_xcds;  // accelerator complex dies; workgroup i is expected on XCD i % num_xcds (see xcd_round_robin)
  // 1 once tdist_init has SEEN a one-workgroup-per-CU grid land that way on this device (every workgroup read its
  // XCD id from the hardware register and the host compared); 0 = not checked or not so. Only with 1 may a kernel
  // let workgroups that it expects on one XCD exchange data through that XCD's L2 alone.
  int xcd_round_robin;
};

// Records a printf-style message for tdist_last_error_string() and returns `code`.
int fail(int code, const char* fmt, ...) __attribute__((format(printf, 2, 3)));
// hipGetLastError() → TDIST_OK or TDIST_ERR_LAUNCH (message recorded).
int launch_status(const char* what);
const DeviceInfo& device_info();
// The dispatch-order check behind DeviceInfo::xcd_round_robin; run by tdist_init (it allocates and synchronises, so it
// is never run lazily from an entry point).
int probe_xcd_round_robin();
// Test and measurement switches (tdist_debug_set): the value of `key`, -1 = the library decides.
int debug_get(int key);
// Looks up, once per device and with that device current, the device address of the built-in scratch of
// tdist_moe_scatter_index_static (moe.hip). Called by tdist_init and, lazily, by that entry point.
int moe_static_scratch_init();

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// ---- device side -----------------------------------------------------------------------------
typedef __attribute__((__vector_size__(4 * sizeof(int)))) int int4v;
typedef __attribute__((__vector_size__(2 * sizeof(int)))) int int2v;
typedef __attribute__((__vector_size__(8 * sizeof(int)))) int int8v;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float float4v;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float float16v;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8v;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8v;
typedef __attribute__((__vector_size__(4 * sizeof(short)))) short short4v;
typedef __attribute__((__vector_size__(4 * sizeof(_Float16)))) _Float16 f16x4v;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t b) { return __uint_as_float(b << 16); }

// fp32 pair → packed bf16 with v_cvt_pk_bf16_f32: round-to-nearest-even, NaN stays a quiet NaN — the
// rounding of torch's .to(bfloat16).
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((__vector_size__(2 * sizeof(float)))) float float2v;
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2v;
  const float2v f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2v));
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) { return pack_bf16x2(f, 0.f) & 0xffffu; }
__device__ __forceinline__ uint32_t pack_f16x2(float lo, float hi) {
  _Float16 a = (_Float16)lo, b = (_Float16)hi;  // v_cvt_f16_f32: round-to-nearest-even
  return (uint32_t)__builtin_bit_cast(unsigned short, a) | ((uint32_t)__builtin_bit_cast(unsigned short, b) << 16);
}
__device__ __forceinline__ float f16_bits_to_f32(uint32_t b) {
  return (float)__builtin_bit_cast(_Float16, (unsigned short)b);
}

// 16-bit element traits for the two storage dtypes the kernels take.
struct BF16 {
  static constexpr int kDtype = TDIST_BF16;
  __device__ static __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
  __device__ static __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
  __device__ static __forceinline__ float one(uint32_t bits) { return bf16_bits_to_f32(bits); }
  __device__ static __forceinline__ uint32_t pack(float a, float b) { return pack_bf16x2(a, b); }
};
struct F16 {
  static constexpr int kDtype = TDIST_F16;
  __device__ static __forceinline__ float lo(uint32_t w) { return f16_bits_to_f32(w & 0xffffu); }
  __device__ static __forceinline__ float hi(uint32_t w) { return f16_bits_to_f32(w >> 16); }
  __device__ static __forceinline__ float one(uint32_t bits) { return f16_bits_to_f32(bits); }
  __device__ static __forceinline__ uint32_t pack(float a, float b) { return pack_f16x2(a, b); }
};

// OCP e4m3fn byte → fp32 by bit arithmetic (no inf; S.1111.111 is NaN; subnormals m * 2^-9).
__device__ __forceinline__ float e4m3_to_f32(uint32_t b) {
  uint32_t sign = (b & 0x80u) << 24;
  uint32_t em = b & 0x7fu;
  float mag;
  if (em >= 8u) {
    mag = __uint_as_float((em << 20) + (120u << 23));  // exponent bias 7 → 127
    if (em == 0x7fu) mag = __uint_as_float(0x7fc00000u);
  } else {
    mag = (float)em * 0.001953125f;  // 2^-9
  }
  return __uint_as_float(__float_as_uint(mag) | sign);
}

// Four e4m3 bytes of one dword → 4 floats with the gfx950 conversion instruction (OCP format).
__device__ __forceinline__ void e4m3x4_to_f32(uint32_t w, float* out) {
  typedef __attribute__((__vector_size__(2 * sizeof(float)))) float float2v;
  float2v a = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, false);
  float2v b = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, true);
  out[0] = a[0];
  out[1] = a[1];
  out[2] = b[0];
  out[3] = b[1];
}

// Asynchronous 16-byte-per-lane global → LDS copy: lane i of the wave writes lds_base + 16*i.
// lds_base must be wave-uniform. Completion is tracked by vmcnt.
__device__ __forceinline__ void load_lds_16(const void* gptr, void* lds_base) {
  __builtin_amdgcn_global_load_lds((const TDIST_AS1 void*)gptr, (TDIST_AS3 void*)lds_base, 16, 0, 0);
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// Id of the accelerator complex die (XCD) this wave runs on, from the hardware register (bits 3:0 of XCC_ID).
__device__ __forceinline__ int xcc_id() {
  int v;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID, 0, 4)" : "=s"(v));
  return v;
}

__device__ __forceinline__ int lane_id() { return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0)); }

}  // namespace tdist
