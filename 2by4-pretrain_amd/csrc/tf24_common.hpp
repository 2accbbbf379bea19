// Shared device/host helpers for the gfx950 2:4 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <initializer_list>

#include "tf24.h"

namespace tf24 {

// ---------------------------------------------------------------- error reporting (host)
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);
// TF24_ERR_STRIDE unless every listed pointer (NULL is skipped) is aligned to `bytes`: the kernels
// use 128-bit (metadata and byte masks: 64-bit) accesses and do not handle split lines
int check_aligned(const char* fn, int bytes, std::initializer_list<const void*> ptrs);

// ---------------------------------------------------------------- element types
struct f16_t { uint16_t bits; };
struct bf16_t { uint16_t bits; };
struct e4m3_t { uint8_t bits; };
struct e5m2_t { uint8_t bits; };
struct i8_t { uint8_t bits; };      // two's-complement int8

template <typename T> struct dtype_of;
template <> struct dtype_of<float> { static constexpr int value = TF24_F32; };
template <> struct dtype_of<f16_t> { static constexpr int value = TF24_F16; };
template <> struct dtype_of<bf16_t> { static constexpr int value = TF24_BF16; };
template <> struct dtype_of<e4m3_t> { static constexpr int value = TF24_E4M3; };
template <> struct dtype_of<e5m2_t> { static constexpr int value = TF24_E5M2; };
template <> struct dtype_of<i8_t> { static constexpr int value = TF24_I8; };
template <> struct dtype_of<int32_t> { static constexpr int value = TF24_I32; };
__host__ __device__ inline bool is_float8(int dt) { return dt == TF24_E4M3 || dt == TF24_E5M2; }
// value types stored one byte per element: 128 dense columns per panel, int32 metadata words
__host__ __device__ inline bool is_8bit(int dt) { return is_float8(dt) || dt == TF24_I8; }
template <> struct dtype_of<uint8_t> { static constexpr int value = TF24_U8; };

// Panel form of the metadata, [k/32][m][4 bytes]: byte offset of metadata byte `mbyte` (= dense column / 8)
// of row `row` of a matrix with m rows.
__host__ __device__ inline int64_t panel_meta_offset(int64_t mbyte, int64_t row, int64_t m) {
  return ((mbyte >> 2) * m + row) * 4 + (mbyte & 3);
}

// CUTLASS form of the metadata (reorder_meta + ColumnMajorInterleaved<2>, reference csrc .cu:826-851):
// byte offset of metadata byte `mbyte` of row `row`.  WB = bytes per metadata word (2: int16 words of
// 16-bit values, 4: int32 words of 8-bit values).  Word (row, c) moves to row
// row/G*G + (row%8)*I + (row%G)/8 with (G, I) = (32, 4) | (16, 2), is swapped inside 2 x 2 blocks (even
// row, odd column <-> odd row, even column) and lands at word (c'/2)*2m + 2*row' + c'%2.
template <int WB>
__host__ __device__ inline int64_t cutlass_meta_offset(int64_t mbyte, int64_t row, int64_t m) {
  constexpr int G = WB == 2 ? 32 : 16, I = WB == 2 ? 4 : 2;
  const int64_t c = mbyte / WB;
  int64_t dr = row / G * G + (row % 8) * I + (row % G) / 8, dc = c;
  if ((dr & 1) == 0 && (dc & 1) == 1) { dr++; dc--; }
  else if ((dr & 1) == 1 && (dc & 1) == 0) { dr--; dc++; }
  return ((dc >> 1) * m * 2 + dr * 2 + (dc & 1)) * WB + mbyte % WB;
}
// byte offset of metadata byte `mbyte` of row `row` in any of the three storage forms (k = dense columns)
template <int WB>
__host__ __device__ inline int64_t meta_offset(int layout, int64_t mbyte, int64_t row, int64_t m, int64_t k) {
  if (layout == TF24_COMPRESSED_PANEL) return panel_meta_offset(mbyte, row, m);
  if (layout == TF24_COMPRESSED_CUTLASS) return cutlass_meta_offset<WB>(mbyte, row, m);
  return row * (k >> 3) + mbyte;
}

__host__ __device__ inline int dtype_size(int dt) {
  return (dt == TF24_F32 || dt == TF24_I32) ? 4 : (dt == TF24_F16 || dt == TF24_BF16) ? 2 : 1;
}

// ---------------------------------------------------------------- conversions to float (exact)
__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(f16_t v) {
  return (float)__builtin_bit_cast(_Float16, v.bits);
}
__device__ __forceinline__ float to_float(bf16_t v) {
  return __builtin_bit_cast(float, (uint32_t)v.bits << 16);
}
__device__ __forceinline__ float to_float(uint8_t v) { return (float)v; }

// ---------------------------------------------------------------- conversions from float
// round-to-nearest-even everywhere, like a plain tensor cast
template <typename T> __device__ __forceinline__ T from_float(float f);
template <> __device__ __forceinline__ float from_float<float>(float f) { return f; }
template <> __device__ __forceinline__ f16_t from_float<f16_t>(float f) {
  return f16_t{__builtin_bit_cast(uint16_t, (_Float16)f)};
}
// gfx950's V_CVT_PK_BF16_F32: round to nearest even, NaNs quieted with their upper payload bits kept --
// on all 2^32 float32 patterns the same bits as the integer sequence (u + 0x7fff + (u >> 16 & 1)) >> 16 with
// (u >> 16) | 0x40 for NaNs, in one instruction per pair instead of seven per value.
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float f) {
  return bf16_t{__builtin_bit_cast(uint16_t, (__bf16)f)};
}
// OCP e4m3fn (bias 7, no inf, 0x7f = NaN, max 448): values that round past 448 become NaN,
// exactly like the bit pattern arithmetic of a round-to-nearest-even narrowing.
__host__ __device__ inline uint8_t float_to_e4m3(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  uint32_t sign = (u >> 24) & 0x80u;
  u &= 0x7fffffffu;
  uint32_t r;
  if (u >= 0x43f00000u) {            // |f| >= 480, inf, NaN
    r = 0x7fu;
  } else if (u < 0x3c800000u) {      // |f| < 2^-6: subnormal result, multiples of 2^-9
    float a = __builtin_bit_cast(float, u) + 16384.0f;   // ulp(16384) * 2^-23.. aligns 2^-9 to bit 0
    r = __builtin_bit_cast(uint32_t, a) - 0x46800000u;   // 16384.0f == 0x46800000
  } else {
    uint32_t odd = (u >> 20) & 1u;
    u += 0x7ffffu + odd;             // RTNE at bit 20
    r = (u >> 20) - ((127u - 7u) << 3);
  }
  return (uint8_t)(r | sign);
}
// On the device gfx950's V_CVT_PK_FP8_F32 (OCP e4m3fn, round to nearest even, NaN past the range) gives the same
// byte for every float32 pattern that is not a NaN; NaNs take the bit arithmetic's sign | 0x7f (the instruction
// returns 0xff for both signs).  About five instructions instead of twenty.
template <> __device__ __forceinline__ e4m3_t from_float<e4m3_t>(float f) {
  const uint32_t h = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f, f, 0, false) & 0xffu;
  const uint32_t nan = ((__builtin_bit_cast(uint32_t, f) >> 24) & 0x80u) | 0x7fu;
  return e4m3_t{(uint8_t)(f != f ? nan : h)};
}

__host__ __device__ inline float e4m3_to_float(uint8_t b) {
  uint32_t sign = (uint32_t)(b & 0x80u) << 24;
  uint32_t e = (b >> 3) & 0xfu, m = b & 7u;
  float v;
  if (e == 0) v = (float)m * 0.001953125f;                                    // m * 2^-9
  else if (e == 15 && m == 7) v = __builtin_bit_cast(float, 0x7fc00000u);     // NaN
  else v = __builtin_bit_cast(float, ((e + 120u) << 23) | (m << 20));
  return __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, v) | sign);
}
__device__ __forceinline__ float to_float(e4m3_t v) { return e4m3_to_float(v.bits); }

// OCP e5m2 (bias 15, infinities, NaN): the upper byte of an IEEE half.  Round to nearest even from
// float32 on the bit pattern: magnitudes of 2^16 and above become infinity (the rounding carries
// 61440..65535 there as well), subnormals (below 2^-14) are rounded by a float32 addition.
__host__ __device__ inline uint8_t float_to_e5m2(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  const uint32_t sign = (u >> 24) & 0x80u;
  u &= 0x7fffffffu;
  uint32_t r;
  if (u >= (143u << 23)) {
    r = u > 0x7f800000u ? 0x7fu : 0x7cu;
  } else if (u < (113u << 23)) {
    const float v = __builtin_bit_cast(float, u) + __builtin_bit_cast(float, 134u << 23);
    r = __builtin_bit_cast(uint32_t, v) - (134u << 23);
  } else {
    const uint32_t odd = (u >> 21) & 1u;
    u += ((uint32_t)(15 - 127) << 23) + 0xfffffu + odd;
    r = u >> 21;
  }
  return (uint8_t)(r | sign);
}
// V_CVT_PK_BF8_F32: as above (its NaN is 0x7e | sign; the bit arithmetic's, and torch's, 0x7f | sign)
template <> __device__ __forceinline__ e5m2_t from_float<e5m2_t>(float f) {
  const uint32_t h = (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(f, f, 0, false) & 0xffu;
  const uint32_t nan = ((__builtin_bit_cast(uint32_t, f) >> 24) & 0x80u) | 0x7fu;
  return e5m2_t{(uint8_t)(f != f ? nan : h)};
}
// int8: exact for the integers an int8 dense operand holds (the only input the int8 path accepts)
template <> __device__ __forceinline__ i8_t from_float<i8_t>(float f) {
  const float c = f < -128.0f ? -128.0f : (f > 127.0f ? 127.0f : f);
  return i8_t{(uint8_t)(int8_t)(int)c};
}
__device__ __forceinline__ float to_float(i8_t v) { return (float)(int8_t)v.bits; }
__device__ __forceinline__ float to_float(e5m2_t v) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)((uint16_t)v.bits << 8));
}

// ---------------------------------------------------------------- vector loads/stores
template <int BYTES> struct vec_bytes;
template <> struct vec_bytes<2> { using type = uint16_t; };
template <> struct vec_bytes<4> { using type = uint32_t; };
template <> struct vec_bytes<8> { using type = uint2; };
template <> struct vec_bytes<16> { using type = uint4; };
template <> struct vec_bytes<32> { struct alignas(16) type { uint4 a, b; }; };

// load N elements of T (N*sizeof(T) in {2,4,8,16,32} bytes, naturally aligned)
template <typename T, int N>
struct Pack {
  T v[N];
  __device__ __forceinline__ void load(const T* p) {
    using V = typename vec_bytes<sizeof(T) * N>::type;
    *reinterpret_cast<V*>(v) = *reinterpret_cast<const V*>(p);
  }
  __device__ __forceinline__ void store(T* p) const {
    using V = typename vec_bytes<sizeof(T) * N>::type;
    *reinterpret_cast<V*>(p) = *reinterpret_cast<const V*>(v);
  }
  // Streaming variants for data touched once per kernel (non-temporal: the lines are not kept in
  // L2).  On the one-pass conversion kernels they are worth 5-20 %; not for read-modify-write
  // operands, whose loads got slower.
  __device__ __forceinline__ void load_stream(const T* p) {
    constexpr int B = sizeof(T) * N;
    if constexpr (B % 16 == 0) {
      typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int q = 0; q < B / 16; q++) reinterpret_cast<u32x4*>(v)[q] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p) + q);
    } else if constexpr (B == 8) {
      typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
      *reinterpret_cast<u32x2*>(v) = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    } else {
      load(p);
    }
  }
  __device__ __forceinline__ void store_stream(T* p) const {
    constexpr int B = sizeof(T) * N;
    if constexpr (B % 16 == 0) {
      typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
#pragma unroll
      for (int q = 0; q < B / 16; q++) __builtin_nontemporal_store(reinterpret_cast<const u32x4*>(v)[q], reinterpret_cast<u32x4*>(p) + q);
    } else if constexpr (B == 8) {
      typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));
      __builtin_nontemporal_store(*reinterpret_cast<const u32x2*>(v), reinterpret_cast<u32x2*>(p));
    } else {
      store(p);
    }
  }
};

// ---------------------------------------------------------------- 2:4 group math
// The kept elements of one group as four flags, and what the reference's 16-row table
// (_semi_structured_conversions.py:46-82) makes of them: idx0 = 0 if m0, else 1 if m1, else 2;
// idx1 = 1 if m0 & m1 & !m2, else 2 if m2 & (m0 | m1), else 3 -- for any of the 16 flag combinations, not
// only the valid ones with two flags set.  Written on the flags themselves, which the compares leave
// in scalar registers: picking a kept value is two selects on scalar conditions, where the route over
// the packed nibble (bits -> positions -> compares -> three selects per value) costs three times the
// vector instructions.
struct Keep4 {
  bool m0, m1, m2, m3;
  __device__ __forceinline__ bool second_is_1() const { return m0 & m1 & !m2; }
  __device__ __forceinline__ bool second_is_2() const { return m2 & (m0 | m1); }
  template <typename T> __device__ __forceinline__ T first(T v0, T v1, T v2) const { return m0 ? v0 : (m1 ? v1 : v2); }
  template <typename T> __device__ __forceinline__ T second(T v1, T v2, T v3) const { return second_is_1() ? v1 : (second_is_2() ? v2 : v3); }
  // pos0 | pos1 << 2
  __device__ __forceinline__ uint32_t nibble() const {
    const uint32_t lo = m0 ? 0u : (m1 ? 1u : 2u);
    const uint32_t hi = second_is_1() ? 4u : (second_is_2() ? 8u : 12u);
    return lo | hi;
  }
  __device__ __forceinline__ uint32_t bits() const { return (uint32_t)m0 | ((uint32_t)m1 << 1) | ((uint32_t)m2 << 2) | ((uint32_t)m3 << 3); }
};
__device__ __forceinline__ Keep4 keep_from_bits(uint32_t mbits) { return Keep4{(mbits & 1) != 0, (mbits & 2) != 0, (mbits & 4) != 0, (mbits & 8) != 0}; }

// Magnitude mask.  Six strict compares of |x|; ties keep the larger index (all equal -> elements 2 and 3).
__device__ __forceinline__ Keep4 magnitude_keep4(float x0, float x1, float x2, float x3) {
  float a = __builtin_fabsf(x0), b = __builtin_fabsf(x1), c = __builtin_fabsf(x2), d = __builtin_fabsf(x3);
  bool x1_ = a > b, x2_ = a > c, x3_ = a > d, x4_ = b > c, x5_ = b > d, x6_ = c > d;
  Keep4 k;
  k.m0 = (x2_ & x3_) | (x1_ & x2_) | (x1_ & x3_);
  k.m1 = (!x1_ & x5_) | (x4_ & x5_) | (!x1_ & x4_);
  k.m2 = (!x2_ & !x4_) | (!x2_ & x6_) | (!x4_ & x6_);
  k.m3 = (!x3_ & !x5_) | (!x3_ & !x6_) | (!x5_ & !x6_);
  return k;
}
// the same as bits: bit i set = element i kept
__device__ __forceinline__ uint32_t magnitude_mask4(float x0, float x1, float x2, float x3) {
  return magnitude_keep4(x0, x1, x2, x3).bits();
}

// mask bits -> nibble pos0 | pos1<<2 (the 16-row table: masks with other than two bits set
// are mapped as the reference's boolean minimisation maps them)
__device__ __forceinline__ uint32_t encode_nibble(uint32_t mbits) { return keep_from_bits(mbits).nibble(); }

// Magnitude selection of one group of four 16-bit floats (f16 or bf16) held as two dwords
// (x1:x0, x3:x2), in integer arithmetic: for numbers the order of |x| is the order of the low 15
// bits, so key_i = |bits_i| << 2 | i orders the elements by (|x|, index) -- exactly the rule of the
// six compares (a tie keeps the larger index) -- and the two kept elements are the largest and the
// second largest key: four min/max pairs, a max and a max3.  Returns the nibble pos0 | pos1 << 2;
// `top_key` (largest key) lets the caller test for NaN, whose magnitude bits lie above infinity's:
// a group with a NaN follows the float compares instead (NaN compares false either way there).
// About 20 instructions against about 60 for compares, lane-mask logic and the table encoding.
struct Top2 { uint32_t nibble, top_key; };
__device__ __forceinline__ Top2 magnitude_top2_16(uint32_t lo, uint32_t hi) {
  const uint32_t k0 = (lo & 0x7fffu) << 2;
  const uint32_t k1 = (((lo >> 16) & 0x7fffu) << 2) | 1u;
  const uint32_t k2 = ((hi & 0x7fffu) << 2) | 2u;
  const uint32_t k3 = (((hi >> 16) & 0x7fffu) << 2) | 3u;
  const uint32_t hi01 = max(k0, k1), lo01 = min(k0, k1), hi23 = max(k2, k3), lo23 = min(k2, k3);
  const uint32_t top = max(hi01, hi23);
  const uint32_t second = max(min(hi01, hi23), max(lo01, lo23));
  const uint32_t p = top & 3u, q = second & 3u;
  return {min(p, q) | (max(p, q) << 2), top};
}
// the 16-bit element at position pos (0..3) of the group (x1:x0, x3:x2), in the low half of the result
__device__ __forceinline__ uint32_t pick16(uint32_t lo, uint32_t hi, uint32_t pos) {
  const uint64_t both = ((uint64_t)hi << 32) | lo;
  return (uint32_t)(both >> (pos << 4));
}

template <typename T>
__device__ __forceinline__ T select4(uint32_t pos, T v0, T v1, T v2, T v3) {
  T lo = (pos & 1) ? v1 : v0;
  T hi = (pos & 1) ? v3 : v2;
  return (pos & 2) ? hi : lo;
}

// Float32 division for operands inside the normal range.  This is the arithmetic the compiler's
// own division performs between its v_div_scale and v_div_fixup steps: one Newton step on
// v_rcp_f32, then two residual corrections of the quotient.  It returns the correctly rounded
// quotient whenever v_div_scale would leave both operands unscaled and v_div_fixup would pass the
// result through: numerator and denominator finite, non-zero and normal, |numerator| > 2^-104,
// denominator < 2^126, exponent difference below 96 and a normal quotient.  Callers establish those
// bounds and use operator/ outside them.  A reciprocal can be shared between quotients.
__device__ __forceinline__ float refined_rcp(float b) {
  float r = __builtin_amdgcn_rcpf(b);
  return __builtin_fmaf(__builtin_fmaf(-b, r, 1.0f), r, r);
}
__device__ __forceinline__ float div_in_range(float a, float b, float r) {
  float q = a * r;
  q = __builtin_fmaf(__builtin_fmaf(-b, q, a), r, q);
  return __builtin_fmaf(__builtin_fmaf(-b, q, a), r, q);
}

// Counter-based uniforms for MVUE24 when no tensor is supplied: Philox4x32-10 (Salmon et al., the
// generator of Random123 / cuRAND / torch), key = seed, counter = {index, offset}.  One call gives
// the four uniforms of two adjacent groups: `index` = row * (k / 8) + (8-column unit of the row),
// words 0,1 for the even group of the unit and 2,3 for the odd one.
struct Philox4 { uint32_t x, y, z, w; };
__host__ __device__ inline Philox4 philox4x32_10(uint64_t seed, uint64_t index, uint64_t offset) {
  uint32_t c0 = (uint32_t)index, c1 = (uint32_t)(index >> 32), c2 = (uint32_t)offset, c3 = (uint32_t)(offset >> 32);
  uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
#pragma unroll
  for (int round = 0; round < 10; round++) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c0 = n0; c1 = (uint32_t)p1; c2 = n2; c3 = (uint32_t)p0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  return Philox4{c0, c1, c2, c3};
}
// 24 random bits -> [0, 1), exact in float32
__host__ __device__ inline float philox_uniform(uint32_t bits) { return (float)(bits & 0xffffffu) * 5.9604644775390625e-8f; }

// Where MVUE24 takes its uniforms from
enum { RAND_FULL = 0, RAND_PACKED = 1, RAND_SEEDED = 2 };
struct RandSrc {
  const float* ptr;       // RAND_FULL: [m, k] (columns 4g, 4g+1 used); RAND_PACKED: [m, k/2]
  int64_t ld;
  int kind;
  uint64_t seed, offset;  // RAND_SEEDED
  const uint64_t* state;  // RAND_SEEDED: when not null, {seed, offset} are read from here (device memory) by the kernel
  __device__ __forceinline__ uint64_t seed_now() const { return state ? state[0] : seed; }
  __device__ __forceinline__ uint64_t offset_now() const { return state ? state[1] : offset; }
};

// MVUE24 of one group in float32, in the reference's operation order (no contraction): inclusion
// probabilities p_i and the kept-mask bits.  The kept values are x_i / p_i (mvue_rescale); only
// the two kept ones need the division.
//
// in_range: |x_i| + eps >= 2^-23 always, so with sum < 2^40 and every s_i = sum - a_i > 0 (then
// s_i >= 2^-46) the quotients t_i = a_i/sum >= 2^-63 and k_i = t_i/s_i >= 2^-104 meet the bounds of
// div_in_range; p_i >= t_i because k >= k_i for a rounded sum of non-negatives.
struct Mvue4 {
  float p[4];
  Keep4 keep;
  bool in_range;
};

__device__ __forceinline__ Mvue4 mvue4(float x0, float x1, float x2, float x3, float r0, float r1) {
  const float eps = 1.19209e-07f;
  float a0 = __builtin_fabsf(x0) + eps, a1 = __builtin_fabsf(x1) + eps;
  float a2 = __builtin_fabsf(x2) + eps, a3 = __builtin_fabsf(x3) + eps;
  float sum = ((a0 + a1) + a2) + a3;
  float s0 = sum - a0, s1 = sum - a1, s2 = sum - a2, s3 = sum - a3;
  Mvue4 g;
  // every s_i > 0  <=>  their minimum is (none of them is a NaN when sum < 2^40: all a_i are finite then)
  g.in_range = (sum < 0x1p40f) && (__builtin_fminf(__builtin_fminf(s0, s1), __builtin_fminf(s2, s3)) > 0.0f);
  float t0, t1, t2, t3, k0, k1, k2, k3;
  if (g.in_range) {
    const float rs = refined_rcp(sum);
    t0 = div_in_range(a0, sum, rs); t1 = div_in_range(a1, sum, rs);
    t2 = div_in_range(a2, sum, rs); t3 = div_in_range(a3, sum, rs);
    k0 = div_in_range(t0, s0, refined_rcp(s0)); k1 = div_in_range(t1, s1, refined_rcp(s1));
    k2 = div_in_range(t2, s2, refined_rcp(s2)); k3 = div_in_range(t3, s3, refined_rcp(s3));
  } else {
    t0 = a0 / sum; t1 = a1 / sum; t2 = a2 / sum; t3 = a3 / sum;
    k0 = t0 / s0; k1 = t1 / s1; k2 = t2 / s2; k3 = t3 / s3;
  }
  float k = ((k0 + k1) + k2) + k3;
  g.p[0] = t0 + a0 * (k - k0); g.p[1] = t1 + a1 * (k - k1);
  g.p[2] = t2 + a2 * (k - k2); g.p[3] = t3 + a3 * (k - k3);
  bool m0 = r0 <= t0;
  bool m1 = (r0 <= (t0 + t1)) & !m0;
  bool m2 = (r0 <= ((t0 + t1) + t2)) & !m1 & !m0;
  bool m3 = !m2 & !m1 & !m0;
  float d0 = m0 ? 0.0f : a0, d1 = m1 ? 0.0f : a1, d2 = m2 ? 0.0f : a2, d3 = m3 ? 0.0f : a3;
  float dsum = ((d0 + d1) + d2) + d3;
  float t = r1 * dsum;
  bool e0 = t <= d0;
  bool e1 = (t <= (d0 + d1)) & !e0;
  bool e2 = (t <= ((d0 + d1) + d2)) & !e1 & !e0;
  bool e3 = !e2 & !e1 & !e0;
  g.keep.m0 = m0 | e0; g.keep.m1 = m1 | e1; g.keep.m2 = m2 | e2; g.keep.m3 = m3 | e3;
  return g;
}

// x / p for a value of a group whose probabilities came from mvue4.  In range: p in [2^-63, 2],
// |x| <= sum * p (so the exponent difference stays below 96) and |x| >= 2^-100 keeps the quotient
// normal; a zero numerator returns the signed zero the division would.
__device__ __forceinline__ float mvue_rescale(float x, float p, bool in_range) {
  const bool ok = in_range & (p <= 2.0f) & ((x == 0.0f) | (__builtin_fabsf(x) >= 0x1p-100f));
  if (ok) {
    float q = div_in_range(x, p, refined_rcp(p));
    return x == 0.0f ? x : q;
  }
  return x / p;
}

}  // namespace tf24
