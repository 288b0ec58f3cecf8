// Device-side helpers shared by the gfx950 kernels: lane exchange, input
// conversion, Philox-4x32-10, reductions.  wave64 only.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace hot {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

struct bf16_t { uint16_t v; };
struct f16_t { _Float16 v; };

template <typename T> struct dtype_of;
template <> struct dtype_of<float> { static constexpr int value = 0; };
template <> struct dtype_of<bf16_t> { static constexpr int value = 1; };
template <> struct dtype_of<f16_t> { static constexpr int value = 2; };

__device__ __forceinline__ float as_f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t as_u(float f) { return __builtin_bit_cast(uint32_t, f); }

// Value held by lane (lane ^ MASK).  1, 2, 3 and 8 are single DPP controls (folded by the compiler
// into the consuming VALU op: quad permutes, and a rotation by 8 inside the row of 16 lanes); 4 is
// two of them (xor 3, then the mirror of each half row, which is xor 7); 16 goes through the LDS
// crossbar without touching memory, 32 uses the wave-wide permute.
template <int MASK>
__device__ __forceinline__ float lane_xor(float v) {
  int i = __builtin_bit_cast(int, v);
  if constexpr (MASK == 1) {
    i = __builtin_amdgcn_update_dpp(0, i, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
  } else if constexpr (MASK == 2) {
    i = __builtin_amdgcn_update_dpp(0, i, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
  } else if constexpr (MASK == 3) {
    i = __builtin_amdgcn_update_dpp(0, i, 0x1B, 0xF, 0xF, true);  // quad_perm [3,2,1,0]
  } else if constexpr (MASK == 4) {
    i = __builtin_amdgcn_update_dpp(0, i, 0x1B, 0xF, 0xF, true);  // quad_perm [3,2,1,0]: xor 3
    i = __builtin_amdgcn_update_dpp(0, i, 0x141, 0xF, 0xF, true); // row_half_mirror: xor 7
  } else if constexpr (MASK == 8) {
    i = __builtin_amdgcn_update_dpp(0, i, 0x128, 0xF, 0xF, true); // row_ror:8
  } else if constexpr (MASK < 32) {
    i = __builtin_amdgcn_ds_swizzle(i, (MASK << 10) | 0x1F);      // bitmask mode: xor MASK
  } else {
    i = __shfl_xor(i, MASK, 64);
  }
  return __builtin_bit_cast(float, i);
}

__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, lane_xor<1>(v));
  v = fmaxf(v, lane_xor<2>(v));
  v = fmaxf(v, lane_xor<4>(v));
  v = fmaxf(v, lane_xor<8>(v));
  v = fmaxf(v, lane_xor<16>(v));
  v = fmaxf(v, lane_xor<32>(v));
  return v;
}

__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
  return v;
}

// ---- 16-byte input vectors -> fp32 ---------------------------------------

template <typename T> struct vec_traits;
template <> struct vec_traits<float> { static constexpr int EPV = 4; };
template <> struct vec_traits<bf16_t> { static constexpr int EPV = 8; };
template <> struct vec_traits<f16_t> { static constexpr int EPV = 8; };

template <typename T>
__device__ __forceinline__ void unpack_vec(const uint4& raw, float* out);

template <>
__device__ __forceinline__ void unpack_vec<float>(const uint4& raw, float* out) {
  out[0] = as_f(raw.x); out[1] = as_f(raw.y); out[2] = as_f(raw.z); out[3] = as_f(raw.w);
}
template <>
__device__ __forceinline__ void unpack_vec<bf16_t>(const uint4& raw, float* out) {
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    out[2 * i] = as_f(w[i] << 16);
    out[2 * i + 1] = as_f(w[i] & 0xFFFF0000u);
  }
}
template <>
__device__ __forceinline__ void unpack_vec<f16_t>(const uint4& raw, float* out) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    h2 p = __builtin_bit_cast(h2, w[i]);
    out[2 * i] = (float)p.x;
    out[2 * i + 1] = (float)p.y;
  }
}

// Scalar element load -> fp32 (used by the column-wise kernels).
template <typename T> __device__ __forceinline__ float load_scalar(const T* p);
template <> __device__ __forceinline__ float load_scalar<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float load_scalar<bf16_t>(const bf16_t* p) { return as_f((uint32_t)p->v << 16); }
template <> __device__ __forceinline__ float load_scalar<f16_t>(const f16_t* p) { return (float)p->v; }

// round-to-nearest-even; gfx950 converts in hardware (v_cvt_pk_bf16_f32)
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }

template <typename T> __device__ __forceinline__ void store_scalar(T* p, float v);
template <> __device__ __forceinline__ void store_scalar<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_scalar<bf16_t>(bf16_t* p, float v) { p->v = f32_to_bf16_rne(v); }
template <> __device__ __forceinline__ void store_scalar<f16_t>(f16_t* p, float v) { p->v = (_Float16)v; }

// ---- Philox-4x32-7 --------------------------------------------------------
// The counter-based generator of stochastic rounding: seven rounds of Philox-4x32 (the fewest that
// Random123 reports as passing BigCrush; its default of ten adds a margin that rounding does not need).

struct philox4 { uint32_t w[4]; };
constexpr int SR_PHILOX_ROUNDS = 7;

__device__ __forceinline__ philox4 philox4x32_sr(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                                 uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < SR_PHILOX_ROUNDS; ++r) {
    // one 32 x 32 -> 64 multiply per product (v_mad_u64_u32) instead of a high and a low multiply
    const uint64_t p0 = (uint64_t)0xD2511F53u * (uint64_t)c0, p1 = (uint64_t)0xCD9E8D57u * (uint64_t)c2;
    const uint32_t hi0 = (uint32_t)(p0 >> 32), lo0 = (uint32_t)p0;
    const uint32_t hi1 = (uint32_t)(p1 >> 32), lo1 = (uint32_t)p1;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n2 = hi0 ^ c3 ^ k1;
    c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  philox4 o; o.w[0] = c0; o.w[1] = c1; o.w[2] = c2; o.w[3] = c3;
  return o;
}

// Uniforms (2^-16 grid) for the eight elements whose linear indices are 8*oct .. 8*oct+7: element
// 2 i + h takes the low (h = 0) or high (h = 1) half of output word i of one Philox call.
__device__ __forceinline__ void sr_uniform8(uint64_t oct, uint64_t seed, uint32_t stream, float* u) {
  const philox4 p = philox4x32_sr((uint32_t)oct, (uint32_t)(oct >> 32), stream, 0u,
                                  (uint32_t)seed, (uint32_t)(seed >> 32));
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    u[2 * i] = (float)(p.w[i] & 0xFFFFu) * 1.52587890625e-05f;      // 2^-16
    u[2 * i + 1] = (float)(p.w[i] >> 16) * 1.52587890625e-05f;
  }
}

// The same numbers one at a time, for callers that walk element indices which are not a compile-time
// sequence: the four output words of the call for octet e / 8 live in named registers (no array, so
// nothing the compiler could turn into an indexed access to scratch memory) and the uniform of
// element e is picked with selects and a shift.
struct philox_words { uint32_t w0, w1, w2, w3; };
__device__ __forceinline__ philox_words sr_octet_words(uint64_t oct, uint64_t seed, uint32_t stream) {
  const philox4 p = philox4x32_sr((uint32_t)oct, (uint32_t)(oct >> 32), stream, 0u,
                                  (uint32_t)seed, (uint32_t)(seed >> 32));
  philox_words o;
  o.w0 = p.w[0]; o.w1 = p.w[1]; o.w2 = p.w[2]; o.w3 = p.w[3];
  return o;
}
// The same draws as 16-bit integers (what the fixed-point rounding below adds): r[2 i + h] = the low
// (h = 0) or high half of output word i of the call for octet `oct`.
__device__ __forceinline__ void sr_bits8(uint64_t oct, uint64_t seed, uint32_t stream, uint32_t* r) {
  const philox4 p = philox4x32_sr((uint32_t)oct, (uint32_t)(oct >> 32), stream, 0u, (uint32_t)seed, (uint32_t)(seed >> 32));
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    r[2 * i] = p.w[i] & 0xFFFFu;
    r[2 * i + 1] = p.w[i] >> 16;
  }
}
__device__ __forceinline__ uint32_t sr_bits_of(const philox_words& p, uint32_t e) {
  const uint32_t i = (e >> 1) & 3u;
  const uint32_t lo = (i & 1u) ? p.w1 : p.w0, hi = (i & 1u) ? p.w3 : p.w2;
  const uint32_t w = (i & 2u) ? hi : lo;
  return (w >> ((e & 1u) * 16u)) & 0xFFFFu;
}

// ---- quantisation of one value --------------------------------------------

// Stochastic rounding of x / d in 16.16 fixed point, rcpk = fl32(1 / d) * 65536, r a 16-bit uniform
// integer: p = fma(|x|, rcpk, 0.5) is |x / d| in units of 2^-16, rounded to the nearest; adding r
// carries into the integer part with probability frac(|x / d|) on a 2^-16 grid.  One fused
// multiply-add, a conversion, an add, a shift, a minimum and the sign: no division, no branch.
__device__ __forceinline__ int q_stoch_fix(float x, float rcpk, uint32_t r, int qmax) {
  const float p = __builtin_fmaf(fabsf(x), rcpk, 0.5f);
  const uint32_t m = min(((uint32_t)p + r) >> 16, (uint32_t)qmax);
  return x < 0.f ? -(int)m : (int)m;
}

// y = x / d already divided.  Nearest: ties to even.
__device__ __forceinline__ int q_nearest(float y) { return (int)rintf(y); }

__device__ __forceinline__ int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// non-negative float max through an integer atomic (bit patterns of
// non-negative floats are ordered like unsigned integers).  The plain read
// first keeps thousands of workgroups from queueing on one address: the value
// only grows, so a stale read can at worst cause a redundant atomic.
__device__ __forceinline__ void atomic_max_nonneg(float* addr, float v) {
  if (v > *reinterpret_cast<volatile float*>(addr)) atomicMax(reinterpret_cast<unsigned int*>(addr), as_u(v));
}

// Per-tensor absmax spread over 16 slots, 32 floats (one 128-byte line) apart: workgroup `wg` folds
// its maximum into slot wg % 16; a reader takes the maximum of the slots (every lane of the calling
// wave gets it).
__device__ __forceinline__ void stat_slot_update(float* slots, unsigned wg, float v) {
  atomic_max_nonneg(slots + (wg & 15u) * 32u, v);
}
__device__ __forceinline__ float stat_slots_max(const float* slots, int lane) {
  return wave_max(lane < 16 ? slots[lane * 32] : 0.f);
}

// rint(x / d) with rcp = 1 / d precomputed: the product x * rcp is within 1.5 * 2^-23 |x/d| of
// the correctly rounded quotient, so it rounds to the same integer unless it lies within 2^-14 of
// a half-integer (|x/d| <= 128); only then is the IEEE division carried out.
__device__ __forceinline__ float rint_div_fast(float x, float d, float rcp) {
  const float p = x * rcp;
  float k = rintf(p);
  if (__builtin_expect(fabsf(p - k) > 0.5f - 6.103515625e-05f, 0)) k = rintf(x / d);
  return k;
}

}  // namespace hot
