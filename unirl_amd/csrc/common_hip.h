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

// Round-to-nearest-even fp32 -> bf16 on the hardware converter (v_cvt_pk_bf16_f32); NaN stays a
// quiet NaN.  The pair form converts two values with one instruction.
typedef __bf16 hw_bf16x2 __attribute__((ext_vector_type(2)));
typedef float hw_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t f32x2_to_bf16x2_bits(float lo, float hi) {
  const hw_f32x2 v = {lo, hi};
  union {
    hw_bf16x2 h;
    uint32_t u;
  } c;
  c.h = __builtin_convertvector(v, hw_bf16x2);
  return c.u;
}
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
  union {
    __bf16 h;
    uint16_t u;
  } c;
  c.h = (__bf16)f;
  return c.u;
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

// torch.maximum / torch.minimum / torch.clamp propagate NaN; fmaxf / fminf drop it.
__device__ __forceinline__ float nan_max(float a, float b) { return (a != a) ? a : ((b != b) ? b : fmaxf(a, b)); }
__device__ __forceinline__ float nan_min(float a, float b) { return (a != a) ? a : ((b != b) ? b : fminf(a, b)); }
__device__ __forceinline__ float nan_clamp(float v, float lo, float hi) { return (v != v) ? v : fminf(fmaxf(v, lo), hi); }
__device__ __forceinline__ float quiet_nan() { return __uint_as_float(0x7fc00000u); }

// Streaming (non-temporal) 8/16-byte accesses for data that is touched exactly once.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ u32x4 stream_load16(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ u32x2 stream_load8(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
}
__device__ __forceinline__ void stream_store16(void* p, u32x4 v) {
  __builtin_nontemporal_store(v, reinterpret_cast<u32x4*>(p));
}

// ---------------------------------------------------------------------------
// Vector loads: N consecutive elements of T -> N floats.  N*sizeof(T) is 8 or
// 16 bytes and `p` is aligned to that, so one lane issues one dwordx2/x4.  The
// 8- and 16-byte forms are streaming accesses.
// ---------------------------------------------------------------------------
template <typename T, int N>
struct Vec;

template <>
struct Vec<float, 4> {
  static __device__ __forceinline__ void load(const float* p, float (&o)[4]) {
    const u32x4 v = stream_load16(p);
    o[0] = __uint_as_float(v.x);
    o[1] = __uint_as_float(v.y);
    o[2] = __uint_as_float(v.z);
    o[3] = __uint_as_float(v.w);
  }
  static __device__ __forceinline__ void store(float* p, const float (&o)[4]) {
    u32x4 v;
    v.x = __float_as_uint(o[0]);
    v.y = __float_as_uint(o[1]);
    v.z = __float_as_uint(o[2]);
    v.w = __float_as_uint(o[3]);
    stream_store16(p, v);
  }
};
// eight floats: two 16-byte accesses (the pointer needs 16-byte alignment only)
template <>
struct Vec<float, 8> {
  static __device__ __forceinline__ void load(const float* p, float (&o)[8]) {
    const u32x4 a = stream_load16(p), b = stream_load16(p + 4);
    o[0] = __uint_as_float(a.x);
    o[1] = __uint_as_float(a.y);
    o[2] = __uint_as_float(a.z);
    o[3] = __uint_as_float(a.w);
    o[4] = __uint_as_float(b.x);
    o[5] = __uint_as_float(b.y);
    o[6] = __uint_as_float(b.z);
    o[7] = __uint_as_float(b.w);
  }
  static __device__ __forceinline__ void store(float* p, const float (&o)[8]) {
    u32x4 a, b;
    a.x = __float_as_uint(o[0]);
    a.y = __float_as_uint(o[1]);
    a.z = __float_as_uint(o[2]);
    a.w = __float_as_uint(o[3]);
    b.x = __float_as_uint(o[4]);
    b.y = __float_as_uint(o[5]);
    b.z = __float_as_uint(o[6]);
    b.w = __float_as_uint(o[7]);
    stream_store16(p, a);
    stream_store16(p + 4, b);
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
    const u32x2 v = stream_load8(p);
    o[0] = __uint_as_float(v.x << 16);
    o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16);
    o[3] = __uint_as_float(v.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&o)[4]) {
    uint2 v;
    v.x = f32x2_to_bf16x2_bits(o[0], o[1]);
    v.y = f32x2_to_bf16x2_bits(o[2], o[3]);
    *reinterpret_cast<uint2*>(p) = v;
  }
};
template <>
struct Vec<bf16_t, 8> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&o)[8]) {
    const u32x4 v = stream_load16(p);
    o[0] = __uint_as_float(v.x << 16);
    o[1] = __uint_as_float(v.x & 0xffff0000u);
    o[2] = __uint_as_float(v.y << 16);
    o[3] = __uint_as_float(v.y & 0xffff0000u);
    o[4] = __uint_as_float(v.z << 16);
    o[5] = __uint_as_float(v.z & 0xffff0000u);
    o[6] = __uint_as_float(v.w << 16);
    o[7] = __uint_as_float(v.w & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&o)[8]) {
    u32x4 v;
    v.x = f32x2_to_bf16x2_bits(o[0], o[1]);
    v.y = f32x2_to_bf16x2_bits(o[2], o[3]);
    v.z = f32x2_to_bf16x2_bits(o[4], o[5]);
    v.w = f32x2_to_bf16x2_bits(o[6], o[7]);
    stream_store16(p, v);
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
    const u32x2 v = stream_load8(p);
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
    const u32x4 v = stream_load16(p);
    o[0] = f16_bits_to_f32(v.x & 0xffffu);
    o[1] = f16_bits_to_f32(v.x >> 16);
    o[2] = f16_bits_to_f32(v.y & 0xffffu);
    o[3] = f16_bits_to_f32(v.y >> 16);
    o[4] = f16_bits_to_f32(v.z & 0xffffu);
    o[5] = f16_bits_to_f32(v.z >> 16);
    o[6] = f16_bits_to_f32(v.w & 0xffffu);
    o[7] = f16_bits_to_f32(v.w >> 16);
  }
  static __device__ __forceinline__ void store(f16_t* p, const float (&o)[8]) {
    u32x4 v;
    v.x = f32_to_f16_bits(o[0]) | (f32_to_f16_bits(o[1]) << 16);
    v.y = f32_to_f16_bits(o[2]) | (f32_to_f16_bits(o[3]) << 16);
    v.z = f32_to_f16_bits(o[4]) | (f32_to_f16_bits(o[5]) << 16);
    v.w = f32_to_f16_bits(o[6]) | (f32_to_f16_bits(o[7]) << 16);
    stream_store16(p, v);
  }
};
template <>
struct Vec<f16_t, 1> {
  static __device__ __forceinline__ void load(const f16_t* p, float (&o)[1]) { o[0] = Elem<f16_t>::load(p); }
  static __device__ __forceinline__ void store(f16_t* p, const float (&o)[1]) { Elem<f16_t>::store(p, o[0]); }
};

// ---------------------------------------------------------------------------
// Wavefront / workgroup reductions.
//
// Wavefront reductions run on DPP (data-parallel primitives): four row shifts
// leave each 16-lane row's total in its last lane, two row broadcasts carry the
// totals to lane 63, and v_readlane returns it as a wave-uniform scalar.  Full
// rate VALU, no LDS traffic, a fixed association order.  Every lane of the
// wavefront must be active at the call.
// ---------------------------------------------------------------------------
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp_move(int identity, int v) {
  // lanes without a valid source lane (or outside ROW_MASK) receive `identity`
  return __builtin_amdgcn_update_dpp(identity, v, CTRL, ROW_MASK, 0xf, false);
}

#define UNIRL_DPP_REDUCE(v, OP, MOVE)          \
  v = OP(v, MOVE<0x111, 0xf>(v)); /* shr 1  */ \
  v = OP(v, MOVE<0x112, 0xf>(v)); /* shr 2  */ \
  v = OP(v, MOVE<0x114, 0xf>(v)); /* shr 4  */ \
  v = OP(v, MOVE<0x118, 0xf>(v)); /* shr 8  */ \
  v = OP(v, MOVE<0x142, 0xa>(v)); /* bcast15 */ \
  v = OP(v, MOVE<0x143, 0xc>(v)); /* bcast31 */

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_f32_or_zero(float v) {
  return __int_as_float(dpp_move<CTRL, ROW_MASK>(0, __float_as_int(v)));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_f32_or_self(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(__float_as_int(v), __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ unsigned int dpp_u32_or_zero(unsigned int v) {
  return (unsigned int)dpp_move<CTRL, ROW_MASK>(0, (int)v);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_f64_or_zero(double v) {
  const long long b = __double_as_longlong(v);
  const unsigned int lo = (unsigned int)dpp_move<CTRL, ROW_MASK>(0, (int)(unsigned int)b);
  const unsigned int hi = (unsigned int)dpp_move<CTRL, ROW_MASK>(0, (int)(unsigned int)((unsigned long long)b >> 32));
  return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp_f64_or_self(double v) {
  const long long b = __double_as_longlong(v);
  const int l = (int)(unsigned int)b, h = (int)(unsigned int)((unsigned long long)b >> 32);
  const unsigned int lo = (unsigned int)__builtin_amdgcn_update_dpp(l, l, CTRL, ROW_MASK, 0xf, false);
  const unsigned int hi = (unsigned int)__builtin_amdgcn_update_dpp(h, h, CTRL, ROW_MASK, 0xf, false);
  return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

__device__ __forceinline__ float op_add(float a, float b) { return a + b; }
__device__ __forceinline__ double op_add(double a, double b) { return a + b; }
__device__ __forceinline__ unsigned int op_add(unsigned int a, unsigned int b) { return a + b; }
__device__ __forceinline__ float op_max(float a, float b) { return fmaxf(a, b); }
__device__ __forceinline__ double op_max(double a, double b) { return fmax(a, b); }
__device__ __forceinline__ float op_min(float a, float b) { return fminf(a, b); }

__device__ __forceinline__ float last_lane(float v) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), kWave - 1));
}
__device__ __forceinline__ unsigned int last_lane(unsigned int v) {
  return (unsigned int)__builtin_amdgcn_readlane((int)v, kWave - 1);
}
__device__ __forceinline__ double last_lane(double v) {
  const long long b = __double_as_longlong(v);
  const unsigned int lo = (unsigned int)__builtin_amdgcn_readlane((int)(unsigned int)b, kWave - 1);
  const unsigned int hi = (unsigned int)__builtin_amdgcn_readlane((int)(unsigned int)((unsigned long long)b >> 32), kWave - 1);
  return __longlong_as_double((long long)(((unsigned long long)hi << 32) | lo));
}

// Reductions over each 16-lane row of a wavefront (four row shifts); the result is in the
// row's last lane only.
__device__ __forceinline__ double row_sum_last(double v) {
  v += dpp_f64_or_zero<0x111, 0xf>(v);
  v += dpp_f64_or_zero<0x112, 0xf>(v);
  v += dpp_f64_or_zero<0x114, 0xf>(v);
  v += dpp_f64_or_zero<0x118, 0xf>(v);
  return v;
}
__device__ __forceinline__ double row_max_last(double v) {
  v = fmax(v, dpp_f64_or_self<0x111, 0xf>(v));
  v = fmax(v, dpp_f64_or_self<0x112, 0xf>(v));
  v = fmax(v, dpp_f64_or_self<0x114, 0xf>(v));
  v = fmax(v, dpp_f64_or_self<0x118, 0xf>(v));
  return v;
}

__device__ __forceinline__ unsigned int row_sum_last(unsigned int v) {
  v += dpp_u32_or_zero<0x111, 0xf>(v);
  v += dpp_u32_or_zero<0x112, 0xf>(v);
  v += dpp_u32_or_zero<0x114, 0xf>(v);
  v += dpp_u32_or_zero<0x118, 0xf>(v);
  return v;
}
__device__ __forceinline__ float row_max_last(float v) {
  v = fmaxf(v, dpp_f32_or_self<0x111, 0xf>(v));
  v = fmaxf(v, dpp_f32_or_self<0x112, 0xf>(v));
  v = fmaxf(v, dpp_f32_or_self<0x114, 0xf>(v));
  v = fmaxf(v, dpp_f32_or_self<0x118, 0xf>(v));
  return v;
}

// Wave-uniform results.
__device__ __forceinline__ float wave_sum(float v) {
  UNIRL_DPP_REDUCE(v, op_add, dpp_f32_or_zero)
  return last_lane(v);
}
__device__ __forceinline__ double wave_sum(double v) {
  UNIRL_DPP_REDUCE(v, op_add, dpp_f64_or_zero)
  return last_lane(v);
}
__device__ __forceinline__ unsigned int wave_sum(unsigned int v) {
  UNIRL_DPP_REDUCE(v, op_add, dpp_u32_or_zero)
  return last_lane(v);
}
__device__ __forceinline__ float wave_max(float v) {
  UNIRL_DPP_REDUCE(v, op_max, dpp_f32_or_self)
  return last_lane(v);
}
__device__ __forceinline__ double wave_max(double v) {
  UNIRL_DPP_REDUCE(v, op_max, dpp_f64_or_self)
  return last_lane(v);
}
__device__ __forceinline__ float wave_min(float v) {
  UNIRL_DPP_REDUCE(v, op_min, dpp_f32_or_self)
  return last_lane(v);
}

// Reduction over the workgroup, valid in every thread: wavefront totals meet in LDS and are
// combined in wavefront order.  `lds` holds at least blockDim.x/64 elements and may be
// reused after the call returns.  Must be called by every thread of the workgroup.
template <typename T>
__device__ __forceinline__ T block_sum(T v, T* lds) {
  const int wid = threadIdx.x / kWave;
  const int nw = blockDim.x / kWave;
  v = wave_sum(v);
  __syncthreads();  // protect lds from a previous use
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wid] = v;
  __syncthreads();
  T r = lds[0];
  for (int w = 1; w < nw; ++w) r += lds[w];
  return r;
}
__device__ __forceinline__ float block_max(float v, float* lds) {
  const int wid = threadIdx.x / kWave;
  const int nw = blockDim.x / kWave;
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wid] = v;
  __syncthreads();
  float r = lds[0];
  for (int w = 1; w < nw; ++w) r = fmaxf(r, lds[w]);
  return r;
}
__device__ __forceinline__ float block_min(float v, float* lds) {
  const int wid = threadIdx.x / kWave;
  const int nw = blockDim.x / kWave;
  v = wave_min(v);
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) lds[wid] = v;
  __syncthreads();
  float r = lds[0];
  for (int w = 1; w < nw; ++w) r = fminf(r, lds[w]);
  return r;
}

// ---------------------------------------------------------------------------
// Counter-based normal draws: Philox-4x32-10 (Salmon et al., "Parallel random numbers: as easy as
// 1, 2, 3", SC'11) keyed by a 64-bit seed, with the 128-bit counter {element index / 4, offset};
// one block yields the standard normals of four consecutive elements through two Box-Muller
// pairs.  A draw depends only on (seed, offset, element index): not on the launch shape, the
// vector width or which lane computes it.
// ---------------------------------------------------------------------------
struct RngKey {
  uint32_t k0, k1;  // seed
  uint32_t o0, o1;  // offset: counter words 2 and 3
};

__device__ __forceinline__ void philox4x32_10(uint32_t (&c)[4], uint32_t k0, uint32_t k1) {
  constexpr uint32_t kM0 = 0xD2511F53u, kM1 = 0xCD9E8D57u, kW0 = 0x9E3779B9u, kW1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(kM0, c[0]), lo0 = kM0 * c[0];
    const uint32_t hi1 = __umulhi(kM1, c[2]), lo1 = kM1 * c[2];
    c[0] = hi1 ^ c[1] ^ k0;
    c[1] = lo1;
    c[2] = hi0 ^ c[3] ^ k1;
    c[3] = lo0;
    k0 += kW0;
    k1 += kW1;
  }
}

// Two independent standard normals from two 32-bit words: u1 = (a + 1/2) / 2^32 in (0, 1],
// u2 = b / 2^32 in [0, 1]; r = sqrt(-2 ln u1); (r cos 2 pi u2, r sin 2 pi u2).  The hardware
// log2 / sin / cos (arguments in revolutions, so no range reduction) are accurate to about an ulp;
// |z| <= 6.7.
__device__ __forceinline__ void box_muller(uint32_t a, uint32_t b, float& z0, float& z1) {
  const float u1 = fmaf((float)a, 2.3283064365386963e-10f, 1.1641532182693481e-10f);
  const float u2 = (float)b * 2.3283064365386963e-10f;
  const float r = __builtin_amdgcn_sqrtf(-1.3862943611198906f * __builtin_amdgcn_logf(u1));  // -2 ln2 * log2(u1)
  z0 = r * __builtin_amdgcn_cosf(u2);
  z1 = r * __builtin_amdgcn_sinf(u2);
}

// The normals of elements [4 * block, 4 * block + 4).
__device__ __forceinline__ void rng_normal4(const RngKey& K, uint64_t block, uint32_t step, float (&z)[4]) {
  uint32_t c[4] = {(uint32_t)block, (uint32_t)(block >> 32), K.o0 + step, K.o1};
  philox4x32_10(c, K.k0, K.k1);
  box_muller(c[0], c[1], z[0], z[1]);
  box_muller(c[2], c[3], z[2], z[3]);
}

// VEC normals for the elements starting at index e (a multiple of VEC when VEC is 4 or 8).
template <int VEC>
__device__ __forceinline__ void rng_normals(const RngKey& K, uint64_t e, uint32_t step, float (&out)[VEC]) {
  if constexpr (VEC == 1) {
    float z[4];
    rng_normal4(K, e >> 2, step, z);
    const int w = (int)(e & 3);
    out[0] = w == 0 ? z[0] : (w == 1 ? z[1] : (w == 2 ? z[2] : z[3]));
  } else {
    static_assert(VEC % 4 == 0, "whole Philox blocks");
#pragma unroll
    for (int g = 0; g < VEC / 4; ++g) {
      float z[4];
      rng_normal4(K, (e >> 2) + g, step, z);
#pragma unroll
      for (int k = 0; k < 4; ++k) out[4 * g + k] = z[k];
    }
  }
}

// ---------------------------------------------------------------------------
// Timeline marks of measurement builds (-DUNIRL_TRACE); nothing otherwise.  T0 reads the clock
// at kernel entry, MARK reads it again, END has thread 0 of the workgroup store
// {start, mark1, mark2, end} at slot (workgroup index) of the launch's trace slice.
// ---------------------------------------------------------------------------
#ifdef UNIRL_TRACE
#define UNIRL_TRACE_T0() const unsigned long long trace_t0_ = wall_clock64(); unsigned long long trace_m1_ = 0, trace_m2_ = 0
#define UNIRL_TRACE_MARK1() trace_m1_ = wall_clock64()
#define UNIRL_TRACE_MARK2() trace_m2_ = wall_clock64()
#define UNIRL_TRACE_END(tr)                                                                      \
  do {                                                                                           \
    if ((tr) && threadIdx.x == 0) {                                                              \
      unsigned long long* q_ = (tr) + ((size_t)blockIdx.y * gridDim.x + blockIdx.x) * 4;         \
      q_[0] = trace_t0_; q_[1] = trace_m1_; q_[2] = trace_m2_; q_[3] = wall_clock64();           \
    }                                                                                            \
  } while (0)
#else
#define UNIRL_TRACE_T0() ((void)0)
#define UNIRL_TRACE_MARK1() ((void)0)
#define UNIRL_TRACE_MARK2() ((void)0)
#define UNIRL_TRACE_END(tr) ((void)0)
#endif

// ---------------------------------------------------------------------------
// Grid-wide sums are two launches: the streaming kernel stores one partial per
// workgroup (plain stores), and a finalize kernel of a few wavefronts -- ordered
// after it on the stream -- adds them in index order.  In-kernel alternatives
// were measured and dropped: a device-scope release fence per workgroup writes
// back the XCD's whole L2 (20x slower than the kernel itself), and "last
// arrival finalises" tickets serialise at ~90 ns per same-address atomic,
// which exceeds the ~2 us cost of the second launch beyond ~25 workgroups.
// ---------------------------------------------------------------------------
// Fixed-order sums of `n` partials at `p` by one wavefront.  Lane l adds p[first + l],
// p[first + l + 64], ... in that order.  The loads go out in batches of kBatch before the first is
// used -- a plain `for (j) q += p[j]` makes one trip to memory per iteration, each waiting for the
// one before -- and a lane past the end loads the last partial and adds zero instead (a load
// behind a condition would be waited for before the next is issued).
template <int kBatch>
__device__ __forceinline__ double lane_ordered_sum_batched(const double* __restrict__ p, int64_t n, int64_t first) {
  const int lane = threadIdx.x & (kWave - 1);
  double q = 0.0;
  for (int64_t j0 = first + lane; j0 - lane < n; j0 += kWave * kBatch) {
    double y[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int64_t j = j0 + b * kWave;
      y[b] = p[j < n ? j : n - 1];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int b = 0; b < kBatch; ++b) q += (j0 + b * kWave < n) ? y[b] : 0.0;
  }
  return q;
}
// The batch follows the count (wave-uniform): surplus loads of a short row cost more than they hide.
__device__ __forceinline__ double lane_ordered_sum(const double* __restrict__ p, int64_t n, int64_t first) {
  const int64_t rem = n - first;
  if (rem <= kWave) return lane_ordered_sum_batched<1>(p, n, first);
  if (rem <= 2 * kWave) return lane_ordered_sum_batched<2>(p, n, first);
  if (rem <= 4 * kWave) return lane_ordered_sum_batched<4>(p, n, first);
  return lane_ordered_sum_batched<8>(p, n, first);
}
// Two arrays of `n` partials at once (per-lane sums as lane_ordered_sum gives them): both batches of
// loads are in flight before either is used.
__device__ __forceinline__ void lane_ordered_sum2(const double* __restrict__ p1, const double* __restrict__ p2,
                                                  int64_t n, double& q1, double& q2) {
  const int lane = threadIdx.x & (kWave - 1);
  constexpr int kBatch = 8;
  q1 = 0.0;
  q2 = 0.0;
  for (int64_t j0 = lane; j0 - lane < n; j0 += kWave * kBatch) {
    double y1[kBatch], y2[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const int64_t j = j0 + b * kWave;
      const int64_t jc = j < n ? j : n - 1;
      y1[b] = p1[jc];
      y2[b] = p2[jc];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int b = 0; b < kBatch; ++b) {
      const bool ok = j0 + b * kWave < n;
      q1 += ok ? y1[b] : 0.0;
      q2 += ok ? y2[b] : 0.0;
    }
  }
}
// The whole sum, valid in every lane.
__device__ __forceinline__ double wave_ordered_sum(const double* __restrict__ p, int64_t n) {
  return wave_sum(lane_ordered_sum(p, n, 0));
}

}  // namespace unirl
