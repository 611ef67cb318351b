// Shared device/host helpers for the gfx950 MoE kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>
#include <utility>

#include "moe_gfx950.h"

typedef __bf16 bf16_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

#define MOE_WAVE 64

__device__ __forceinline__ float bf16_to_f32(uint16_t v) {
  return __builtin_bit_cast(float, (uint32_t)v << 16);
}
// Round-to-nearest-even; gfx950 has a hardware conversion the compiler selects for this cast.
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float bf16lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
__device__ __forceinline__ float bf16hi(uint32_t w) {
  return __builtin_bit_cast(float, w & 0xffff0000u);
}

// Eight consecutive row elements as fp32, loaded from / stored to bf16 or fp32 memory with
// 16-byte accesses.
struct Row8 {
  float v[8];
};
__device__ __forceinline__ Row8 row8_from_bits(u32x4 w) {  // eight bf16 as fp32
  Row8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r.v[2 * i] = bf16lo(w[i]);
    r.v[2 * i + 1] = bf16hi(w[i]);
  }
  return r;
}
__device__ __forceinline__ Row8 load8(const uint16_t* p) {
  return row8_from_bits(*reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ Row8 load8(const float* p) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p);
  const f32x4 b = *reinterpret_cast<const f32x4*>(p + 4);
  Row8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r.v[i] = a[i];
    r.v[4 + i] = b[i];
  }
  return r;
}
__device__ __forceinline__ void store8(uint16_t* p, const Row8& r) {
  u32x4 w;
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(r.v[2 * i], r.v[2 * i + 1]);
  *reinterpret_cast<u32x4*>(p) = w;
}
__device__ __forceinline__ void store8(float* p, const Row8& r) {
  f32x4 a, b;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    a[i] = r.v[i];
    b[i] = r.v[4 + i];
  }
  *reinterpret_cast<f32x4*>(p) = a;
  *reinterpret_cast<f32x4*>(p + 4) = b;
}

#ifndef MOE_STREAMING_STORES
#define MOE_STREAMING_STORES 1
#endif
#ifndef MOE_STREAMING_LOADS
#define MOE_STREAMING_LOADS 1
#endif
// Streaming variants (non-temporal): for rows that are written once and not read again soon,
// or read exactly once.
__device__ __forceinline__ void store_bits_nt(uint16_t* p, u32x4 w) {
#if MOE_STREAMING_STORES
  __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(p));
#else
  *reinterpret_cast<u32x4*>(p) = w;
#endif
}
__device__ __forceinline__ void store8_nt(uint16_t* p, const Row8& r) {
  u32x4 w;
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = pack_bf16x2(r.v[2 * i], r.v[2 * i + 1]);
#if MOE_STREAMING_STORES
  __builtin_nontemporal_store(w, reinterpret_cast<u32x4*>(p));
#else
  *reinterpret_cast<u32x4*>(p) = w;
#endif
}
__device__ __forceinline__ Row8 load8_nt(const uint16_t* p) {
#if MOE_STREAMING_LOADS
  const u32x4 w = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
#else
  const u32x4 w = *reinterpret_cast<const u32x4*>(p);
#endif
  Row8 r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r.v[2 * i] = bf16lo(w[i]);
    r.v[2 * i + 1] = bf16hi(w[i]);
  }
  return r;
}

__device__ __forceinline__ int lane_id() { return threadIdx.x & (MOE_WAVE - 1); }

static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

#define MOE_CHECK_PTR(p) \
  do {                   \
    if ((p) == nullptr) return MOE_ERR_NULL; \
    if (!aligned16(p)) return MOE_ERR_ALIGN; \
  } while (0)

// Facts the host side learns once per GPU and keeps (a compute-unit count, "this kernel's
// attribute is set"): one slot per device id; the caller's current device picks the slot.  Racing
// first calls at worst repeat an idempotent runtime query.
constexpr int MOE_MAX_DEVICES = 64;
static inline int moe_current_device() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= MOE_MAX_DEVICES) dev = 0;
  return dev;
}

static inline int moe_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}
