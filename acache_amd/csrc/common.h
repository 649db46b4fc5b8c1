// Shared device/host helpers for the gfx950 affix-KV kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/acache_hip.h"

namespace acache {

// ---------------------------------------------------------------- errors ----
inline char *err_buf() {
  static thread_local char buf[256] = {0};
  return buf;
}

inline int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(err_buf(), 256, fmt, ap);
  va_end(ap);
  return code;
}

inline int launch_status(const char *what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail((int)e, "%s: %s", what, hipGetErrorString(e));
  return 0;
}

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline int dtype_bytes(int dtype) {
  switch (dtype) {
    case ACACHE_BF16: return 2;
    case ACACHE_F16: return 2;
    case ACACHE_F32: return 4;
    default: return 0;
  }
}

// ------------------------------------------------------------ 16-byte IO ----
struct alignas(16) vec16 {
  uint32_t w[4];
};

__device__ __forceinline__ vec16 load16(const void *p) {
  return *reinterpret_cast<const vec16 *>(p);
}
__device__ __forceinline__ void store16(void *p, const vec16 &v) {
  *reinterpret_cast<vec16 *>(p) = v;
}
// Streaming variants: the relocation/scatter payload is touched exactly once,
// so it is kept out of the way of data that is reused (tables, slot maps).
__device__ __forceinline__ vec16 load16_stream(const void *p) {
  vec16 v;
  const uint32_t *s = reinterpret_cast<const uint32_t *>(p);
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  u4 t = __builtin_nontemporal_load(reinterpret_cast<const u4 *>(s));
  v.w[0] = t.x; v.w[1] = t.y; v.w[2] = t.z; v.w[3] = t.w;
  return v;
}
__device__ __forceinline__ void store16_stream(void *p, const vec16 &v) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  u4 t = {v.w[0], v.w[1], v.w[2], v.w[3]};
  __builtin_nontemporal_store(t, reinterpret_cast<u4 *>(p));
}
// Write-through streaming store (nt sc0 sc1): the line goes to memory without being kept in L2 or the
// Infinity Cache.  For the relocation output, 9 GB written once per launch, this measured 2 % faster than
// the plain non-temporal store.
//
// The s_nop behind the store is required: a VALU instruction must not overwrite the data registers of a
// vector store of more than 8 bytes in the two issue slots after it (the store has not read them yet), and
// the compiler's hazard pass does not see a store inside inline assembly; without it the register allocator
// is free to reuse the first data registers for the next address computation right away.
__device__ __forceinline__ void store16_writethrough(void *p, const vec16 &v) {
  typedef uint32_t u4 __attribute__((ext_vector_type(4)));
  const u4 t = {v.w[0], v.w[1], v.w[2], v.w[3]};
  asm volatile("global_store_dwordx4 %0, %1, off nt sc0 sc1\n\ts_nop 1" ::"v"(p), "v"(t) : "memory");
}

// ------------------------------------------------------- element <-> fp32 ----
// bf16 is handled as raw bits so rounding is exactly round-to-nearest-even with
// quiet-NaN canonicalisation (0x7fc0 | sign), the behaviour of torch's bf16 cast.
__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return __uint_as_float(h << 16); }
__device__ __forceinline__ uint32_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
  return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float f16_to_f32(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}
__device__ __forceinline__ uint32_t f32_to_f16(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

template <int DTYPE> struct Elem;
template <> struct Elem<ACACHE_BF16> {
  static constexpr int kBytes = 2;
  static constexpr int kPerVec = 8;
  __device__ static __forceinline__ void unpack(const vec16 &v, float *f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = bf16_to_f32(v.w[i] & 0xffffu);
      f[2 * i + 1] = bf16_to_f32(v.w[i] >> 16);
    }
  }
  __device__ static __forceinline__ vec16 pack(const float *f) {
    vec16 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v.w[i] = f32_to_bf16(f[2 * i]) | (f32_to_bf16(f[2 * i + 1]) << 16);
    return v;
  }
};
template <> struct Elem<ACACHE_F16> {
  static constexpr int kBytes = 2;
  static constexpr int kPerVec = 8;
  __device__ static __forceinline__ void unpack(const vec16 &v, float *f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = f16_to_f32(v.w[i] & 0xffffu);
      f[2 * i + 1] = f16_to_f32(v.w[i] >> 16);
    }
  }
  __device__ static __forceinline__ vec16 pack(const float *f) {
    vec16 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v.w[i] = f32_to_f16(f[2 * i]) | (f32_to_f16(f[2 * i + 1]) << 16);
    return v;
  }
};
template <> struct Elem<ACACHE_F32> {
  static constexpr int kBytes = 4;
  static constexpr int kPerVec = 4;
  __device__ static __forceinline__ void unpack(const vec16 &v, float *f) {
#pragma unroll
    for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(v.w[i]);
  }
  __device__ static __forceinline__ vec16 pack(const float *f) {
    vec16 v;
#pragma unroll
    for (int i = 0; i < 4; ++i) v.w[i] = __float_as_uint(f[i]);
    return v;
  }
};

}  // namespace acache
