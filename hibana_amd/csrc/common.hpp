// Shared declarations of the gfx950 kernels: status codes, vector types, small device helpers.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hibana_hip.h"

namespace hb {

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;

constexpr int WAVE = 64;

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// Device pointers the kernels read or write with 16-byte (activations, tile layouts, workspace) or 4-byte accesses.
inline bool aligned(const void* p, size_t bytes) { return (reinterpret_cast<uintptr_t>(p) & (bytes - 1)) == 0; }

inline int launch_status() { return hipGetLastError() == hipSuccess ? HB_OK : HB_ELAUNCH; }

// float32 -> bfloat16 bits, round to nearest even (NaN kept quiet).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  return (uint16_t)((u + 0x7fffu + ((u >> 16) & 1u)) >> 16);
}

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t h) { return __uint_as_float((uint32_t)h << 16); }

__device__ __forceinline__ float round_bf16(float f) { return bf16_bits_to_f32(f32_to_bf16_bits(f)); }

// E4M3 (OCP e4m3fn) byte -> float32 without the conversion instruction (format kernels; also usable for constants).
__device__ __host__ inline float e4m3_to_f32(uint32_t b) {
  uint32_t sign = (b & 0x80u) << 24, e = (b >> 3) & 0xfu, m = b & 7u;
  uint32_t bits;
  if (e == 0) {
    if (m == 0) {
      bits = sign;
    } else {  // subnormal: m * 2^-9
      int lz = (m & 4u) ? 0 : (m & 2u) ? 1 : 2;
      uint32_t mant = (m << (lz + 1)) & 7u;
      bits = sign | ((uint32_t)(127 - 7 - lz) << 23) | (mant << 20);
    }
  } else if (e == 15 && m == 7) {
    bits = sign | 0x7fc00000u;
  } else {
    bits = sign | ((e + 120u) << 23) | (m << 20);
  }
#if defined(__HIP_DEVICE_COMPILE__)
  return __uint_as_float(bits);
#else
  union { uint32_t u; float f; } c;
  c.u = bits;
  return c.f;
#endif
}

}  // namespace hb
