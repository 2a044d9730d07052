// Device-side helpers shared by the gfx950 kernels: bf16 <-> fp32, 16-byte
// vector access, 64-lane wavefront reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/emi.h"

namespace emi {

constexpr int kWave = 64;

struct bf16 {
  uint16_t bits;
};

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return __uint_as_float(((uint32_t)v.bits) << 16); }
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) { return __uint_as_float(((uint32_t)b) << 16); }

// fp32 -> bf16, round to nearest even (v_cvt_pk_bf16_f32 on gfx950).
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  __bf16 b = (__bf16)f;
  return __builtin_bit_cast(uint16_t, b);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
  typedef __attribute__((__vector_size__(2 * sizeof(float)))) float f32x2_t;
  f32x2_t v = {lo, hi};
  bf16x2_t r = __builtin_convertvector(v, bf16x2_t);
  return __builtin_bit_cast(uint32_t, r);
}

template <typename T> __device__ __forceinline__ T from_f32(float f);
template <> __device__ __forceinline__ float from_f32<float>(float f) { return f; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float f) { return bf16{f32_to_bf16_bits(f)}; }

// 16-byte global accesses with the streaming (non-temporal) hint: the HBM-bound kernels touch every element of
// their big operands once, and on this part streamed accesses run 8-12 % faster than plain ones when a wavefront's
// lanes cover consecutive 16-byte pieces (Vec8<bf16>, Chunk<T>).  Vec8<float> keeps plain accesses: its two
// 16-byte halves per lane split every cache line over two instructions, which streams badly.
typedef float emi_f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t emi_u32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ float4 stream_load(const float4* p) {
  const emi_f32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const emi_f32x4_t*>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint4 stream_load(const uint4* p) {
  const emi_u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const emi_u32x4_t*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void stream_store(float4* p, float4 a) {
  const emi_f32x4_t v = {a.x, a.y, a.z, a.w};
  __builtin_nontemporal_store(v, reinterpret_cast<emi_f32x4_t*>(p));
}
__device__ __forceinline__ void stream_store(uint4* p, uint4 a) {
  const emi_u32x4_t v = {a.x, a.y, a.z, a.w};
  __builtin_nontemporal_store(v, reinterpret_cast<emi_u32x4_t*>(p));
}

// SwiGLU of test/llama.py:21-28,229-231 and its adjoint, shared by the elementwise kernels and the GEMM epilogues
// that apply them to a tile: g = a sigmoid(a) b;  da = dg b s (1 + a (1 - s)),  db = dg a s  with s = sigmoid(a).
// The sigmoid costs one hardware exponential and one hardware reciprocal (each good to about one unit in the last
// place; 2^x overflows to inf and underflows to 0 exactly where the sigmoid saturates): an epilogue that applies it
// to a whole tile holds up its CU's matrix cores for as long as its arithmetic lasts, and with the library's expf and
// an IEEE division that was three times longer.
__device__ __forceinline__ float emi_sigmoid(float a) {
  return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(a * -1.44269504088896340736f));
}
__device__ __forceinline__ float emi_swiglu(float a, float b) { return a * emi_sigmoid(a) * b; }
__device__ __forceinline__ void emi_swiglu_adjoint(float a, float b, float dg, float* da, float* db) {
  const float s = emi_sigmoid(a);
  *da = dg * b * s * (1.0f + a * (1.0f - s));
  *db = dg * a * s;
}

// Eight consecutive elements as fp32 (one 16-byte load for bf16, two for fp32).
template <typename T> struct Vec8;
template <> struct Vec8<float> {
  struct Raw { float4 a, b; };
  static __device__ __forceinline__ Raw load_raw(const float* p) {
    return Raw{*reinterpret_cast<const float4*>(p), *reinterpret_cast<const float4*>(p + 4)};
  }
  static __device__ __forceinline__ Raw zero_raw() { return Raw{make_float4(0, 0, 0, 0), make_float4(0, 0, 0, 0)}; }
  static __device__ __forceinline__ void unpack(const Raw& r, float (&v)[8]) {
    v[0] = r.a.x; v[1] = r.a.y; v[2] = r.a.z; v[3] = r.a.w;
    v[4] = r.b.x; v[5] = r.b.y; v[6] = r.b.z; v[7] = r.b.w;
  }
  static __device__ __forceinline__ void load(const float* p, float (&v)[8]) {
    float4 a = *reinterpret_cast<const float4*>(p);
    float4 b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
  static __device__ __forceinline__ void load_cached(const float* p, float (&v)[8]) { load(p, v); }
  static __device__ __forceinline__ void store_cached(float* p, const float (&v)[8]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
  }
};
template <> struct Vec8<bf16> {
  typedef uint4 Raw;
  static __device__ __forceinline__ Raw load_raw(const bf16* p) { return stream_load(reinterpret_cast<const uint4*>(p)); }
  static __device__ __forceinline__ Raw zero_raw() { return make_uint4(0, 0, 0, 0); }
  static __device__ __forceinline__ void unpack(const Raw& a, float (&v)[8]) {
    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void load(const bf16* p, float (&v)[8]) {
    uint4 a = stream_load(reinterpret_cast<const uint4*>(p));
    uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int i = 0; i < 4; i++) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(bf16* p, const float (&v)[8]) {
    uint4 a;
    a.x = pack_bf16x2(v[0], v[1]);
    a.y = pack_bf16x2(v[2], v[3]);
    a.z = pack_bf16x2(v[4], v[5]);
    a.w = pack_bf16x2(v[6], v[7]);
    stream_store(reinterpret_cast<uint4*>(p), a);
  }
  // plain accesses, for kernels that may run in place or whose operand is read again soon
  static __device__ __forceinline__ void load_cached(const bf16* p, float (&v)[8]) { unpack(*reinterpret_cast<const uint4*>(p), v); }
  static __device__ __forceinline__ void store_cached(bf16* p, const float (&v)[8]) {
    uint4 a;
    a.x = pack_bf16x2(v[0], v[1]);
    a.y = pack_bf16x2(v[2], v[3]);
    a.z = pack_bf16x2(v[4], v[5]);
    a.w = pack_bf16x2(v[6], v[7]);
    *reinterpret_cast<uint4*>(p) = a;
  }
};

// Sixteen bytes of T as fp32: 4 floats or 8 bf16.
template <typename T> struct Chunk;
template <> struct Chunk<float> {
  static constexpr int N = 4;
  typedef float4 Raw;
  static __device__ __forceinline__ Raw load_raw(const float* p) { return stream_load(reinterpret_cast<const float4*>(p)); }
  static __device__ __forceinline__ void unpack(const Raw& a, float (&v)[4]) { v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; }
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 a = stream_load(reinterpret_cast<const float4*>(p));
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    stream_store(reinterpret_cast<float4*>(p), make_float4(v[0], v[1], v[2], v[3]));
  }
};
template <> struct Chunk<bf16> {
  static constexpr int N = 8;
  typedef uint4 Raw;
  static __device__ __forceinline__ Raw load_raw(const bf16* p) { return stream_load(reinterpret_cast<const uint4*>(p)); }
  static __device__ __forceinline__ void unpack(const Raw& a, float (&v)[8]) { Vec8<bf16>::unpack(a, v); }
  static __device__ __forceinline__ void load(const bf16* p, float (&v)[8]) { Vec8<bf16>::load(p, v); }
  static __device__ __forceinline__ void store(bf16* p, const float (&v)[8]) { Vec8<bf16>::store(p, v); }
};

// Chunk<T> with plain (cached) accesses, for operands that are read again soon or written in small pieces.
template <typename T> struct ChunkCached;
template <> struct ChunkCached<float> {
  static constexpr int N = 4;
  typedef float4 Raw;
  static __device__ __forceinline__ Raw load_raw(const float* p) { return *reinterpret_cast<const float4*>(p); }
  static __device__ __forceinline__ void unpack(const Raw& a, float (&v)[4]) { v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; }
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) { unpack(load_raw(p), v); }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <> struct ChunkCached<bf16> {
  static constexpr int N = 8;
  typedef uint4 Raw;
  static __device__ __forceinline__ Raw load_raw(const bf16* p) { return *reinterpret_cast<const uint4*>(p); }
  static __device__ __forceinline__ void unpack(const Raw& a, float (&v)[8]) { Vec8<bf16>::unpack(a, v); }
  static __device__ __forceinline__ void load(const bf16* p, float (&v)[8]) { unpack(load_raw(p), v); }
  static __device__ __forceinline__ void store(bf16* p, const float (&v)[8]) {
    uint4 a;
    a.x = pack_bf16x2(v[0], v[1]);
    a.y = pack_bf16x2(v[2], v[3]);
    a.z = pack_bf16x2(v[4], v[5]);
    a.w = pack_bf16x2(v[6], v[7]);
    *reinterpret_cast<uint4*>(p) = a;
  }
};

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

}  // namespace emi

// Host-side error plumbing (defined in status.cc).
extern "C" int emi_fail(int code, const char* fmt, ...);

#define EMI_REQUIRE(cond, ...)                                   \
  do {                                                           \
    if (!(cond)) return emi_fail(EMI_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

#define EMI_CHECK_LAUNCH(name)                                                        \
  do {                                                                                \
    hipError_t e__ = hipGetLastError();                                               \
    if (e__ != hipSuccess) return emi_fail(EMI_INTERNAL, "%s: launch failed: %s", name, hipGetErrorString(e__)); \
  } while (0)
