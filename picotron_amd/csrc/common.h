// Shared helpers for the gfx950 kernels: vector types, bf16 packing, status plumbing.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <algorithm>
#include <atomic>
#include "../../include/picotron_amd.h"

namespace pico {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;

constexpr int kWave = 64;
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

// Records a failure message for pico_last_error() and returns `code`.
int fail(int code, const char* fmt, ...);
// Maps the result of hipGetLastError() after a launch to a status.
int check_launch(const char* what);

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(static_cast<uint32_t>(b) << 16);
}
// round-to-nearest-even, NaN kept quiet (the hardware conversion on gfx950)
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  __bf16 h = static_cast<__bf16>(f);
  return __builtin_bit_cast(uint16_t, h);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  bf16x2 v;
  v[0] = static_cast<__bf16>(lo);
  v[1] = static_cast<__bf16>(hi);
  return __builtin_bit_cast(uint32_t, v);
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }
__device__ __forceinline__ float fast_log2(float x) { return __builtin_amdgcn_logf(x); }
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

template <typename T> struct io;  // element load/store as float, 16-byte vectors
template <> struct io<__bf16> {
  static constexpr int kVec = 8;  // elements per 16-byte access
  static __device__ __forceinline__ void load(const void* p, float (&out)[8]) {
    u32x4 raw = *reinterpret_cast<const u32x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[2 * i] = __uint_as_float(raw[i] << 16);
      out[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
    }
  }
  // streaming load: for inputs a kernel reads once (they need not stay in the caches)
  static __device__ __forceinline__ void load_stream(const void* p, float (&out)[8]) {
    u32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[2 * i] = __uint_as_float(raw[i] << 16);
      out[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(void* p, const float (&in)[8]) {
    u32x4 raw;
#pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = pack_bf16x2(in[2 * i], in[2 * i + 1]);
    *reinterpret_cast<u32x4*>(p) = raw;
  }
  // streaming (non-temporal) store: for data that nothing on the GPU reads back soon, or that is so large that keeping
  // it in the caches only evicts what is still needed
  static __device__ __forceinline__ void store_stream(void* p, const float (&in)[8]) {
    u32x4 raw;
#pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = pack_bf16x2(in[2 * i], in[2 * i + 1]);
    __builtin_nontemporal_store(raw, reinterpret_cast<u32x4*>(p));
  }
  static __device__ __forceinline__ float round(float v) {
    return bf16_bits_to_float(float_to_bf16_bits(v));
  }
};
template <> struct io<float> {
  static constexpr int kVec = 4;
  static __device__ __forceinline__ void load(const void* p, float (&out)[4]) {
    f32x4 raw = *reinterpret_cast<const f32x4*>(p);
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = raw[i];
  }
  static __device__ __forceinline__ void load_stream(const void* p, float (&out)[4]) {
    f32x4 raw = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = raw[i];
  }
  static __device__ __forceinline__ void store(void* p, const float (&in)[4]) {
    f32x4 raw;
#pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = in[i];
    *reinterpret_cast<f32x4*>(p) = raw;
  }
  static __device__ __forceinline__ void store_stream(void* p, const float (&in)[4]) {
    f32x4 raw;
#pragma unroll
    for (int i = 0; i < 4; ++i) raw[i] = in[i];
    __builtin_nontemporal_store(raw, reinterpret_cast<f32x4*>(p));
  }
  static __device__ __forceinline__ float round(float v) { return v; }
};

template <typename T, bool kStream, int N>
__device__ __forceinline__ void load_as(const void* p, float (&out)[N]) {
  if constexpr (kStream) io<T>::load_stream(p, out);
  else io<T>::load(p, out);
}
// store<kStream>: picks the streaming form at compile time
template <typename T, bool kStream, int N>
__device__ __forceinline__ void store_as(void* p, const float (&in)[N]) {
  if constexpr (kStream) io<T>::store_stream(p, in);
  else io<T>::store(p, in);
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Raises a kernel's dynamic-LDS limit the first time the kernel is launched on a device (the attribute belongs to the
// kernel's code object on that device, so a process that drives several GPUs sets it once on each).  Host threads may
// race here (autograd runs backward on a thread of its own): the per-device bits are atomic and the HIP call is
// idempotent, so two first callers both make it and both proceed only after it has succeeded.
struct LdsOnce {
  std::atomic<uint64_t> devices{0};   // bit d: done on device d (devices 64 and up set the attribute on every launch)
};
inline bool reserve_lds_once(LdsOnce& once, const void* kernel, size_t bytes) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return false;
  const bool tracked = dev >= 0 && dev < 64;
  const uint64_t bit = tracked ? (uint64_t{1} << dev) : 0;
  if (tracked && (once.devices.load(std::memory_order_acquire) & bit)) return true;
  if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)) != hipSuccess)
    return false;
  if (tracked) once.devices.fetch_or(bit, std::memory_order_release);
  return true;
}

}  // namespace pico
