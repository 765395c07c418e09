// Shared host/device helpers for libparaattn_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/paraattn_hip.h"

namespace pa {

// ---- error text, one slot per host thread --------------------------------
char* error_slot();  // 512-byte thread-local buffer (defined in pa_api.hip)

#define PA_FAIL(code, ...)                            \
  do {                                                \
    snprintf(pa::error_slot(), 512, __VA_ARGS__);     \
    return (code);                                    \
  } while (0)

#define PA_CHECK_LAUNCH(what)                                                        \
  do {                                                                               \
    hipError_t e_ = hipGetLastError();                                               \
    if (e_ != hipSuccess) PA_FAIL(PA_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e_)); \
  } while (0)

// ---- per-device facts --------------------------------------------------------
constexpr int PA_MAX_DEVICES = 64;

// Index of the current device, or -1 if it cannot be asked or is beyond the cached range.
static inline int current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= PA_MAX_DEVICES) return -1;
  return dev;
}

// Compute units of the current device (0 if it cannot be asked), cached per device.
static inline int device_cus() {
  static int cus[PA_MAX_DEVICES] = {0};
  const int dev = current_device();
  if (dev < 0) return 0;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) return 0;
    cus[dev] = n;  // benign race: every thread writes the same value
  }
  return cus[dev];
}

// ---- vector types ---------------------------------------------------------
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float floatx16;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef __attribute__((__vector_size__(2 * sizeof(float)))) float floatx2;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(2 * sizeof(uint32_t)))) uint32_t u32x2;

// ---- 16-bit element traits --------------------------------------------------
struct BF16 {
  typedef bf16x8 vec8;
  // two fp32 -> packed pair, round to nearest even (v_cvt_pk_bf16_f32)
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    floatx2 v = {a, b};
    bf16x2 r = __builtin_convertvector(v, bf16x2);
    return __builtin_bit_cast(uint32_t, r);
  }
  static __device__ __forceinline__ float lo(uint32_t w) { return __uint_as_float(w << 16); }
  static __device__ __forceinline__ float hi(uint32_t w) { return __uint_as_float(w & 0xffff0000u); }
  // acc + lo(w) + hi(w) in one instruction (v_dot2c_f32_bf16 with a vector of ones)
  static __device__ __forceinline__ float sum2(uint32_t w, float acc) {
    const bf16x2 ones = {(__bf16)1.0f, (__bf16)1.0f};
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), ones, acc, false);
  }
  static __device__ __forceinline__ floatx16 mfma32(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};

struct F16 {
  typedef f16x8 vec8;
  static __device__ __forceinline__ uint32_t pack2(float a, float b) {
    floatx2 v = {a, b};
    f16x2 r = __builtin_convertvector(v, f16x2);
    return __builtin_bit_cast(uint32_t, r);
  }
  static __device__ __forceinline__ float lo(uint32_t w) {
    f16x2 r = __builtin_bit_cast(f16x2, w);
    return (float)r[0];
  }
  static __device__ __forceinline__ float hi(uint32_t w) {
    f16x2 r = __builtin_bit_cast(f16x2, w);
    return (float)r[1];
  }
  static __device__ __forceinline__ float sum2(uint32_t w, float acc) {
    const f16x2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2, w), ones, acc, false);
  }
  static __device__ __forceinline__ floatx16 mfma32(vec8 a, vec8 b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};

}  // namespace pa
