// Shared device helpers for the LaCT HIP kernels (gfx950 / CDNA4 only).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lact {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

// bf16 is handled as raw uint16_t in memory; conversions go through __bf16 so that the
// compiler emits the hardware round-to-nearest-even convert.
struct bf16 {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_to_f32(uint16_t h) { return __uint_as_float(((uint32_t)h) << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  __bf16 h = (__bf16)f;
  return __builtin_bit_cast(uint16_t, h);
}
// round a float to the nearest bf16-representable float
__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

// Element-type policies: T = uint16_t (bf16 storage) or float.
template <typename T> struct Elem;
template <> struct Elem<uint16_t> {
  static constexpr bool kIsBf16 = true;
  __device__ static __forceinline__ float load(const uint16_t* p) { return bf16_to_f32(*p); }
  __device__ static __forceinline__ void store(uint16_t* p, float v) { *p = f32_to_bf16(v); }
  __device__ static __forceinline__ float rnd(float v) { return round_bf16(v); }
  __device__ static __forceinline__ void store4(uint16_t* p, float a, float b, float c, float d) {
    uint2 u;
    u.x = (uint32_t)f32_to_bf16(a) | ((uint32_t)f32_to_bf16(b) << 16);
    u.y = (uint32_t)f32_to_bf16(c) | ((uint32_t)f32_to_bf16(d) << 16);
    *reinterpret_cast<uint2*>(p) = u;
  }
  __device__ static __forceinline__ void load4(const uint16_t* p, float* o) {
    uint2 u = *reinterpret_cast<const uint2*>(p);
    o[0] = __uint_as_float(u.x << 16);
    o[1] = __uint_as_float(u.x & 0xffff0000u);
    o[2] = __uint_as_float(u.y << 16);
    o[3] = __uint_as_float(u.y & 0xffff0000u);
  }
};
template <> struct Elem<float> {
  static constexpr bool kIsBf16 = false;
  __device__ static __forceinline__ float load(const float* p) { return *p; }
  __device__ static __forceinline__ void store(float* p, float v) { *p = v; }
  __device__ static __forceinline__ float rnd(float v) { return v; }
  __device__ static __forceinline__ void store4(float* p, float a, float b, float c, float d) {
    *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
  }
  __device__ static __forceinline__ void load4(const float* p, float* o) {
    float4 u = *reinterpret_cast<const float4*>(p);
    o[0] = u.x; o[1] = u.y; o[2] = u.z; o[3] = u.w;
  }
};

// one v_exp_f32 and one v_rcp_f32 (1 ulp) instead of the ten-instruction IEEE division: the epilogues that call
// this per element are bound by vector-ALU issue
__device__ __forceinline__ float sigmoidf_(float x) { return __builtin_amdgcn_rcpf(1.0f + __expf(-x)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Sum over the threads of a block (blockDim.x multiple of 64, <= 1024). `red` holds >= 16 floats.
// Every thread receives the total.  Deterministic for a fixed block size.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = (blockDim.x + 63) >> 6;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += red[i];
  return t;
}

// Side job of a kernel that runs right before a fused Newton-Schulz launch: its first block clears the barrier
// lines and the error word (a few KiB), which saves a launch of its own in the dependent chain.
struct ClearWords {
  unsigned* ptr; int n;
};
__device__ __forceinline__ void clear_words(const ClearWords& c, bool first_block) {
  if (c.n > 0 && first_block)
    for (int i = threadIdx.x; i < c.n; i += blockDim.x) c.ptr[i] = 0u;
}

}  // namespace lact
