// Device-side helpers shared by every kernel in this library (gfx950 / CDNA4).
//
// Conventions:
//   * wavefront = 64 lanes; workgroups are a multiple of 64 threads;
//   * the library is compiled with -ffp-contract=off, so `a * b + c` is two
//     roundings exactly like eager torch; fused multiply-adds are written as
//     fmaf()/fma() where they are wanted (the reductions);
//   * cross-lane reductions use wave shuffles, then one LDS hop across the
//     waves of a workgroup, then (for grid-wide sums) a fixed-order pass over
//     per-workgroup partials in a small second kernel, so results do not
//     depend on scheduling.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace unirl {

constexpr int kWave = 64;

// ---------------------------------------------------------------------------
// 16-bit float formats, handled as raw bits (no library types in signatures).
// ---------------------------------------------------------------------------
struct bf16_t {
  uint16_t bits;
};
struct f16_t {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// Round-to-nearest-even fp32 -> bf16, NaN -> quiet NaN (what torch's
// c10::BFloat16 conversion does).
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0u;
  u += 0x7fffu + ((u >> 16) & 1u);
  return u >> 16;
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  union {
    uint16_t u;
    _Float16 f;
  } c;
  c.u = (uint16_t)h;
  return (float)c.f;
}

__device__ __forceinline__ uint32_t f32_to_f16_bits(float f) {
  union {
    uint16_t u;
    _Float16 f;
  } c;
  c.f = (_Float16)f;  // v_cvt_f16_f32, round-to-nearest-even
  return c.u;
}

template <typename T>
struct Elem;

template <>
struct Elem<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float round_trip(float v) { return v; }
};
template <>
struct Elem<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_bits_to_f32(p->bits); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { p->bits = (uint16_t)f32_to_bf16_bits(v); }
  static __device__ __forceinline__ float round_trip(float v) { return bf16_bits_to_f32(f32_to_bf16_bits(v)); }
};
template <>
struct Elem<f16_t> {
  static __device__ __forceinline__ float load(const f16_t* p) { return f16_bits_to_f32(p->bits); }
  static __device__ __forceinline__ void store(f16_t* p, float v) { p->bits = (uint16_t)f32_to_f16_bits(v); }
  static __device__ __forceinline__ float round_trip(float v) { return f16_bits_to_f32(f32_to_f16_bits(v)); }
};

// ---------------------------------------------------------------------------
// Vector loads: N consecutive elements of T -> N floats.  N*sizeof(T) is 8 or
// 16 bytes and `p` is aligned to that, so one lane issues one dwordx2/x4.
// ---------------------------------------------------------------------------
template <typename T, int N>
struct Vec;

template <>
struct Vec<float, 4> {
  static __device__ __forceinline__ void load(const float* p, float (&o)[4]) {
    const float4 v = *reinterpret_cast<const float4*>(p);
    o[0] = v.x;
    o[1] = v.y;
    o[2] = v.z;
    o[3] = v.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&o)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(o[0], o[1], o[2], o[3]);
  }
};
template <>
struct Vec<float, 1> {
  static __device__ __forceinline__ void load(const float* p, float (&o)[1]) { o[0] = *p; }
  static __device__ __forceinline__ void store(float* p, const float (&o)[1]) { *p = o[0]; }
};

template <>
struct Vec<bf16_t, 4> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&o)[4]) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    o[0] = __uint_as_float(v.x << 16);
    o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16);
    o[3] = __uint_as_float(v.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&o)[4]) {
    uint2 v;
    v.x = f32_to_bf16_bits(o[0]) | (f32_to_bf16_bits(o[1]) << 16);
    v.y = f32_to_bf16_bits(o[2]) | (f32_to_bf16_bits(o[3]) << 16);
    *reinterpret_cast<uint2*>(p) = v;
  }
};
template <>
struct Vec<bf16_t, 8> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&o)[8]) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    o[0] = __uint_as_float(v.x << 16);
    o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16);
    o[3] = __uint_as_float(v.y & 0xffff0000u);
    o[4] = __uint_as_float(v.z << 16);
    o[5] = __uint_as_float(v.z & 0xffff0000u);
    o[6] = __uint_as_float(v.w << 16);
    o[7] = __uint_as_float(v.w & 0xffff0000u);
  }
};
template <>
struct Vec<bf16_t, 1> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&o)[1]) { o[0] = Elem<bf16_t>::load(p); }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&o)[1]) { Elem<bf16_t>::store(p, o[0]); }
};

template <>
struct Vec<f16_t, 4> {
  static __device__ __forceinline__ void load(const f16_t* p, float (&o)[4]) {
    const uint2 v = *reinterpret_cast<const uint2*>(p);
    o[0] = f16_bits_to_f32(v.x & 0xffffu);
    o[1] = f16_bits_to_f32(v.x >> 16);
    o[2] = f16_bits_to_f32(v.y & 0xffffu);
    o[3] = f16_bits_to_f32(v.y >> 16);
  }
  static __device__ __forceinline__ void store(f16_t* p, const float (&o)[4]) {
    uint2 v;
    v.x = f32_to_f16_bits(o[0]) | (f32_to_f16_bits(o[1]) << 16);
    v.y = f32_to_f16_bits(o[2]) | (f32_to_f16_bits(o[3]) << 16);
    *reinterpret_cast<uint2*>(p) = v;
  }
};
template <>
struct Vec<f16_t, 8> {
  static __device__ __forceinline__ void load(const f16_t* p, float (&o)[8]) {
    const uint4 v = *reinterpret_cast<const uint4*>(p);
    o[0] = f16_bits_to_f32(v.x & 0xffffu);
    o[1] = f16_bits_to_f32(v.x >> 16);
    o[2] = f16_bits_to_f32(v.y & 0xffffu);
    o[3] = f16_bits_to_f32(v.y >> 16);
    o[4] = f16_bits_to_f32(v.z & 0xffffu);
    o[5] = f16_bits_to_f32(v.z >> 16);
    o[6] = f16_bits_to_f32(v.w & 0xffffu);
    o[7] = f16_bits_to_f32(v.w >> 16);
  }
};
template <>
struct Vec<f16_t, 1> {
  static __device__ __forceinline__ void load(const f16_t* p, float (&o)[1]) { o[0] = Elem<f16_t>::load(p); }
  static __device__ __forceinline__ void store(f16_t* p, const float (&o)[1]) { Elem<f16_t>::store(p, o[0]); }
};

// ---------------------------------------------------------------------------
// Wavefront / workgroup reductions.
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}
__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Sum of `v` over the workgroup, valid in every thread.  `lds` holds at least
// blockDim.x/64 elements of T and may be reused after the call returns.
template <typename T>
__device__ __forceinline__ T block_sum(T v, T* lds) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wid = threadIdx.x / kWave;
  const int nw = blockDim.x / kWave;
  v = wave_sum(v);
  __syncthreads();  // protect lds from a previous use
  if (lane == 0) lds[wid] = v;
  __syncthreads();
  T r = (lane < nw) ? lds[lane] : T(0);
  return wave_sum(r);
}
__device__ __forceinline__ float block_max(float v, float* lds) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wid = threadIdx.x / kWave;
  const int nw = blockDim.x / kWave;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) lds[wid] = v;
  __syncthreads();
  float r = (lane < nw) ? lds[lane] : -INFINITY;
  return wave_max(r);
}
__device__ __forceinline__ float block_min(float v, float* lds) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wid = threadIdx.x / kWave;
  const int nw = blockDim.x / kWave;
  v = wave_min(v);
  __syncthreads();
  if (lane == 0) lds[wid] = v;
  __syncthreads();
  float r = (lane < nw) ? lds[lane] : INFINITY;
  return wave_min(r);
}

// ---------------------------------------------------------------------------
// Grid-wide sums are two launches: the streaming kernel stores one partial per
// workgroup (plain stores), and a finalize kernel of a few wavefronts -- ordered
// after it on the stream -- adds them in index order.  In-kernel alternatives
// were measured and dropped: a device-scope release fence per workgroup writes
// back the XCD's whole L2 (20x slower than the kernel itself), and "last
// arrival finalises" tickets serialise at ~90 ns per same-address atomic,
// which exceeds the ~2 us cost of the second launch beyond ~25 workgroups.
// ---------------------------------------------------------------------------
// Sum of `n` partials at `p`, added in a fixed order by one wavefront; valid in every lane.
__device__ __forceinline__ double wave_ordered_sum(const double* __restrict__ p, int64_t n) {
  const int lane = threadIdx.x & (kWave - 1);
  double q = 0.0;
  for (int64_t j = lane; j < n; j += kWave) q += p[j];
  return wave_sum<double>(q);
}

}  // namespace unirl
