// 2:4 sparse x dense matmul on the gfx950 sparse matrix cores (V_SMFMAC), float32 accumulation.
//
//     C[i,j] = act( scale * sum_k A[i,k] * B(k,j) + bias[i] )
//
// A is the compressed operand (values [n_sparse, k/2] + canonical metadata), which is exactly the
// SMFMAC "A" operand: one lane holds a run of consecutive compressed values of one row and the
// matching run of 2-bit positions is a contiguous slice of the row's metadata stream.
//
// Operand layouts of the instructions used (R = 16 or 32 rows, lane l, nkb = 64/R lane blocks,
// K dense depth of the instruction, kper = K/nkb):
//   A: row l%R, block ka = l/R holds the kper/2 compressed values of dense k in [ka*kper, (ka+1)*kper);
//      value e uses index bits [2e+1:2e] (16-bit types: the 16-bit half of the index register
//      selected by ABID; 8-bit types: all 32 bits)
//   B: column l%R, block kb = l/R holds dense k in [kb*kper/2, (kb+1)*kper/2) followed by the same
//      range shifted by K/2
//   D: 16x16: column l%16, rows 4*(l/16)+r;  32x32: column l%32, rows 8*(r/4) + 4*(l/32) + r%4
#pragma once
#include "tf24_common.hpp"
#include <algorithm>
#include <atomic>
#include <type_traits>

namespace tf24 {
namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x16 __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef int int4v __attribute__((ext_vector_type(4)));
typedef int int8v __attribute__((ext_vector_type(8)));
typedef int int16v __attribute__((ext_vector_type(16)));

// ---- element traits: KSTEP = dense depth of one 16x16 instruction; all types move 64 bytes of
// compressed A and 128 bytes of B per row per step.
template <typename T> struct mma16;
template <> struct mma16<f16_t> {
  static constexpr int KSTEP = 64;
  using acc_t = float4v;
  template <int ABID>
  static __device__ __forceinline__ float4v run(int4v a, int8v b, float4v c, int idx) {
    return __builtin_amdgcn_smfmac_f32_16x16x64_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half16, b), c, idx, 0, ABID);
  }
};
template <> struct mma16<bf16_t> {
  static constexpr int KSTEP = 64;
  using acc_t = float4v;
  template <int ABID>
  static __device__ __forceinline__ float4v run(int4v a, int8v b, float4v c, int idx) {
    return __builtin_amdgcn_smfmac_f32_16x16x64_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x16, b), c, idx, 0, ABID);
  }
};
template <> struct mma16<e4m3_t> {
  static constexpr int KSTEP = 128;
  using acc_t = float4v;
  template <int ABID>
  static __device__ __forceinline__ float4v run(int4v a, int8v b, float4v c, int idx) {
    return __builtin_amdgcn_smfmac_f32_16x16x128_fp8_fp8(a, b, c, idx, 0, 0);
  }
};
template <> struct mma16<e5m2_t> {
  static constexpr int KSTEP = 128;
  using acc_t = float4v;
  template <int ABID>
  static __device__ __forceinline__ float4v run(int4v a, int8v b, float4v c, int idx) {
    return __builtin_amdgcn_smfmac_f32_16x16x128_bf8_bf8(a, b, c, idx, 0, 0);
  }
};

template <> struct mma16<i8_t> {
  static constexpr int KSTEP = 128;
  using acc_t = int4v;
  template <int ABID>
  static __device__ __forceinline__ int4v run(int4v a, int8v b, int4v c, int idx) {
    return __builtin_amdgcn_smfmac_i32_16x16x128_i8(a, b, c, idx, 0, 0);
  }
};

// Exact (erf) GELU, 0.5 v (1 + erf(v / sqrt 2)), through the complementary error function of |v| / sqrt 2
// (Abramowitz & Stegun 7.1.26: erfc(z) = t (a1 + t (a2 + t (a3 + t (a4 + t a5)))) exp(-z^2), t = 1 / (1 + p z),
// absolute error <= 1.5e-7):  with q = erfc(|v| / sqrt 2),  gelu(v) = v - v q / 2 for v >= 0 and v q / 2 below,
// so the negative tail is not formed as a difference of nearly equal numbers.  One reciprocal, one exponential
// and nine multiply-adds per element: the library erff costs three times that, which made a GELU output pass
// slower than a plain one plus a separate GELU kernel.  Agrees with the float32 GELU of torch to 3e-7 absolute.
__device__ __forceinline__ float gelu_erf(float v) {
  const float z = __builtin_fabsf(v) * 0.70710678118654752f;
  const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.3275911f, z, 1.0f));
  float poly = __builtin_fmaf(t, 1.061405429f, -1.453152027f);
  poly = __builtin_fmaf(poly, t, 1.421413741f);
  poly = __builtin_fmaf(poly, t, -0.284496736f);
  poly = __builtin_fmaf(poly, t, 0.254829592f);
  const float q = poly * t * __builtin_amdgcn_exp2f(z * z * -1.4426950408889634f);
  // |v| clamped where q has long been 0: an infinite v stays infinite (or becomes -0) instead of inf * 0
  const float h = 0.5f * q * __builtin_amdgcn_fmed3f(v, -65536.0f, 65536.0f);
  return v >= 0.0f ? v - h : (v < 0.0f ? h : v);
}

__device__ __forceinline__ float apply_act(float v, int act) {
  if (act == TF24_ACT_RELU) return v > 0.0f ? v : 0.0f;
  if (act == TF24_ACT_SILU) return v / (1.0f + __expf(-v));
  if (act == TF24_ACT_GELU) return gelu_erf(v);
  return v;
}

// An accumulator element -> the finished output element.  Floating accumulators: scale, bias,
// activation, one rounding.  Integer accumulators (int8 operands): bias and ReLU in int32, exact.
template <typename OutT> __device__ __forceinline__ OutT to_out(float v) { return from_float<OutT>(v); }
template <typename OutT> __device__ __forceinline__ OutT to_out(int v) { return (OutT)v; }
template <typename OutT>
__device__ __forceinline__ float finish_value(float accv, float scale, const OutT* bias, int64_t row, int act) {
  float v = accv * scale;
  if (bias) v += to_float(bias[row]);
  return apply_act(v, act);
}
template <typename OutT>
__device__ __forceinline__ int finish_value(int accv, float, const OutT* bias, int64_t row, int act) {
  int v = accv;
  if (bias) v += (int)bias[row];
  return (act == TF24_ACT_RELU && v < 0) ? 0 : v;
}

// The output pass of the tiled kernel is compiled once per epilogue: plain, bias only, and bias (or none) followed by
// each activation.  Left to run-time tests alone, the per-element selects and the inlined SiLU more than triple the
// time of the pass (21 000 against 6 300 cycles per 256 x 256 tile), which is a tenth of the whole kernel at k = 4096.
// The bias of an element arrives as a value: the pass reads it from LDS, where the wave has put the bias of its rows
// (zeros without one).
enum { EPI_PLAIN = 0, EPI_BIAS = 1, EPI_RELU = 2, EPI_SILU = 3, EPI_GELU = 4 };
template <int MODE>
__device__ __forceinline__ float finish_element(float accv, float scale, float biasv) {
  float v = accv * scale;
  if constexpr (MODE != EPI_PLAIN) v += biasv;
  if constexpr (MODE == EPI_RELU) v = v > 0.0f ? v : 0.0f;
  if constexpr (MODE == EPI_SILU) v = v * __builtin_amdgcn_rcpf(1.0f + __expf(-v));   // (1 ulp reciprocal: the IEEE division is 10 instructions)
  if constexpr (MODE == EPI_GELU) v = gelu_erf(v);
  return v;
}
// integer accumulators: bias and ReLU in int32, exact (the other activations are not defined for them)
template <int MODE>
__device__ __forceinline__ int finish_element(int accv, float, int biasv) {
  int v = accv;
  if constexpr (MODE != EPI_PLAIN) v += biasv;
  if constexpr (MODE == EPI_RELU) v = v < 0 ? 0 : v;
  return v;
}
template <typename OutT> __device__ __forceinline__ float bias_as(float, OutT b) { return to_float(b); }
template <typename OutT> __device__ __forceinline__ int bias_as(int, OutT b) { return (int)b; }
// a bias element as the bits its load leaves in a register, and back
template <typename OutT> __device__ __forceinline__ uint32_t bias_bits(OutT b) {
  if constexpr (sizeof(OutT) == 2) { uint16_t h; __builtin_memcpy(&h, &b, 2); return h; }
  else { uint32_t w; __builtin_memcpy(&w, &b, 4); return w; }
}
template <typename OutT> __device__ __forceinline__ OutT bias_from_bits(uint32_t w) {
  OutT b;
  if constexpr (sizeof(OutT) == 2) { const uint16_t h = (uint16_t)w; __builtin_memcpy(&b, &h, 2); }
  else __builtin_memcpy(&b, &w, 4);
  return b;
}

// ------------------------------------------------------------------------------------------
// General kernel: operands straight from global memory (cached), every supported shape and
// layout.  One wave computes a 32(i) x 32(j) tile with 16x16 instructions; a block is 2x2 waves.
// ------------------------------------------------------------------------------------------
template <typename T, typename OutT, bool B_KCONTIG, bool C_JMAJOR>
__global__ void __launch_bounds__(256)
spmm_general(const uint8_t* __restrict__ a_values, const uint8_t* __restrict__ a_meta, int64_t n_sparse, int64_t k,
             const T* __restrict__ b, int64_t ldb, int64_t n_dense,
             OutT* __restrict__ c, int64_t ldc, const OutT* __restrict__ bias, float scale, int act, int a_layout) {
  constexpr int KSTEP = mma16<T>::KSTEP;
  const bool panel = a_layout == TF24_COMPRESSED_PANEL;
  constexpr int ES = sizeof(T);                       // element size of values and B
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t i0 = (int64_t)blockIdx.y * 64 + (wave >> 1) * 32;
  const int64_t j0 = (int64_t)blockIdx.x * 64 + (wave & 1) * 32;
  if (i0 >= n_sparse || j0 >= n_dense) return;       // whole wave out of range
  const int li = lane & 15, lk = lane >> 4;
  const int64_t a_pitch = (k / 2) * ES;               // bytes per row of compressed values
  typename mma16<T>::acc_t acc[2][2];
#pragma unroll
  for (int ti = 0; ti < 2; ti++)
#pragma unroll
    for (int tj = 0; tj < 2; tj++)
#pragma unroll
      for (int r = 0; r < 4; r++) acc[ti][tj][r] = 0;

  for (int64_t k0 = 0; k0 < k; k0 += KSTEP) {
    int4v af[2];
    int idx[2];
#pragma unroll
    for (int ti = 0; ti < 2; ti++) {
      const int64_t row = i0 + ti * 16 + li;
      // one instruction step is exactly one panel of values (KSTEP dense columns: 64 value bytes); the lane's
      // index word is metadata bytes k0/8 + lk*2.. (16-bit values) or k0/8 + lk*4.. (8-bit) of its row
      const int64_t voff = panel ? ((k0 / KSTEP) * n_sparse + row) * 64 : row * a_pitch + (k0 / 2) * ES;
      const int64_t mbyte = k0 / 8 + lk * (ES == 2 ? 2 : 4);
      const int64_t moff = meta_offset<ES == 2 ? 2 : 4>(a_layout, mbyte, row, n_sparse, k);   // (reordered metadata: the reference's own storage)
      af[ti] = *reinterpret_cast<const int4v*>(a_values + voff + lk * 16);
      if constexpr (ES == 2) idx[ti] = *reinterpret_cast<const uint16_t*>(a_meta + moff);
      else idx[ti] = *reinterpret_cast<const int*>(a_meta + moff);
    }
    int8v bf[2];
#pragma unroll
    for (int tj = 0; tj < 2; tj++) {
      int64_t col = j0 + tj * 16 + li;
      if (col >= n_dense) col = n_dense - 1;          // clamp: the column is never stored
      constexpr int HALF = KSTEP / 8;                 // elements per half run (16 bytes)
      if constexpr (B_KCONTIG) {
        const T* p = b + col * ldb + k0 + lk * HALF;
        int4v lo = *reinterpret_cast<const int4v*>(p);
        int4v hi = *reinterpret_cast<const int4v*>(p + KSTEP / 2);
        bf[tj] = int8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      } else {
        alignas(32) T tmp[2 * HALF];
#pragma unroll
        for (int e = 0; e < HALF; e++) {
          tmp[e] = b[(k0 + lk * HALF + e) * ldb + col];
          tmp[HALF + e] = b[(k0 + KSTEP / 2 + lk * HALF + e) * ldb + col];
        }
        bf[tj] = *reinterpret_cast<int8v*>(tmp);
      }
    }
#pragma unroll
    for (int ti = 0; ti < 2; ti++)
#pragma unroll
      for (int tj = 0; tj < 2; tj++) acc[ti][tj] = mma16<T>::template run<0>(af[ti], bf[tj], acc[ti][tj], idx[ti]);
  }

#pragma unroll
  for (int ti = 0; ti < 2; ti++)
#pragma unroll
    for (int tj = 0; tj < 2; tj++) {
      const int64_t col = j0 + tj * 16 + li;
      if (col >= n_dense) continue;
      const int64_t row = i0 + ti * 16 + lk * 4;
      OutT o[4];
#pragma unroll
      for (int r = 0; r < 4; r++) o[r] = to_out<OutT>(finish_value(acc[ti][tj][r], scale, bias, row + r, act));
      if constexpr (C_JMAJOR) {
        *reinterpret_cast<Pack<OutT, 4>*>(c + col * ldc + row) = *reinterpret_cast<Pack<OutT, 4>*>(o);
      } else {
#pragma unroll
        for (int r = 0; r < 4; r++) c[(row + r) * ldc + col] = o[r];
      }
    }
}


// ------------------------------------------------------------------------------------------
// Tiled kernel: A in the panel layout, B with k contiguous.
//
// A block computes a 256(i) x 256(j) tile with V_SMFMAC_F32_32X32X32_{F16,BF16} / 32X32X64_FP8:
// 8 waves (2 along i x 4 along j), wave tile 128 x 64 = 4 x 2 instructions, 2 waves per SIMD.
// (4 waves with 128 x 128 wave tiles and 256 accumulators read less LDS per instruction but were
// measured slower: with one wave per SIMD nothing covers a wave's own stalls.)
// Operands go global -> LDS directly (GLOBAL_LOAD_LDS_DWORDX4: lane l of a wave writes
// LDS[base + 16*l], a wave fills 1 KB of contiguous LDS) through a ring of three stage buffers of
// 128 bytes of dense k per row (two instruction steps): while stage s is multiplied, the copies of
// stages s+1 and s+2 are in flight.  LDS rows are unpadded; bank conflicts are avoided by
// XOR-swizzling the 16-byte chunk index with row bits (B: chunk ^ ((row>>1)&7) in 128-byte rows,
// A: chunk ^ ((row>>2)&3) in 64-byte rows), applied on the global side of the copy and again in the
// fragment reads.  The three buffers are slices of one LDS array addressed by a rotating
// wave-uniform offset; the copies are written in assembly the compiler does not look into, so the
// only LDS accesses it sees in the main loop are fragment reads.
// Workgroup ids are remapped so that the 8 XCDs (ids are dealt round-robin) each walk a
// contiguous range of tiles in an 8-tile-high grouped raster: the ~32 tiles resident on an XCD
// form an 8 x 4 patch that shares A rows and B columns in that XCD's L2.
// With more tiles than compute units (and no k pieces) one workgroup per compute unit walks its
// tiles in one pipeline (PERSIST): the copies of the next tile's first two stages ride in the last
// two stages of the current one, and the output pass stages through the one buffer that is free.
// At sustained clocks this kernel runs against the board's power limit (the shader clock settles
// well below its 2.4 GHz maximum, the lower the more the operand bits toggle): what buys time is
// fewer bytes moved per instruction, not a tighter schedule.
// ------------------------------------------------------------------------------------------
template <typename T> struct mma32;
template <> struct mma32<f16_t> {
  using acc_t = float16v;
  using acc4_t = float4v;
  static __device__ __forceinline__ float16v run(int4v a, int8v b, float16v c, int idx) {
    return __builtin_amdgcn_smfmac_f32_32x32x32_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half16, b), c, idx, 0, 0);
  }
};
template <> struct mma32<bf16_t> {
  using acc_t = float16v;
  using acc4_t = float4v;
  static __device__ __forceinline__ float16v run(int4v a, int8v b, float16v c, int idx) {
    return __builtin_amdgcn_smfmac_f32_32x32x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x16, b), c, idx, 0, 0);
  }
};
template <> struct mma32<e4m3_t> {
  using acc_t = float16v;
  using acc4_t = float4v;
  static __device__ __forceinline__ float16v run(int4v a, int8v b, float16v c, int idx) {
    return __builtin_amdgcn_smfmac_f32_32x32x64_fp8_fp8(a, b, c, idx, 0, 0);
  }
};
template <> struct mma32<e5m2_t> {
  using acc_t = float16v;
  using acc4_t = float4v;
  static __device__ __forceinline__ float16v run(int4v a, int8v b, float16v c, int idx) {
    return __builtin_amdgcn_smfmac_f32_32x32x64_bf8_bf8(a, b, c, idx, 0, 0);
  }
};

template <> struct mma32<i8_t> {
  using acc_t = int16v;
  using acc4_t = int4v;
  static __device__ __forceinline__ int16v run(int4v a, int8v b, int16v c, int idx) {
    return __builtin_amdgcn_smfmac_i32_32x32x64_i8(a, b, c, idx, 0, 0);
  }
};

template <int WAVES_J_, int TJ_>
struct TileCfgT {
  static constexpr int WAVES_I = 2, WAVES_J = WAVES_J_;
  static constexpr int NW = WAVES_I * WAVES_J;
  static constexpr int THREADS = 64 * NW;
  static constexpr int TI = 4, TJ = TJ_;         // 32x32 instructions per wave
  static constexpr int WI = 32 * TI, WJ = 32 * TJ;
  static constexpr int BI = WI * WAVES_I, BJ = WJ * WAVES_J;
  static_assert(BI == 256 && (BJ == 256 || BJ == 192 || BJ == 128 || BJ == 64), "stage buffers are sized for 256-row tiles of 256, 192, 128 or 64 columns");
  static constexpr int KB = 128;                 // bytes of dense k per row per stage
  static constexpr int STEPS = KB / 64;          // instruction steps per stage
  static constexpr int A_ROW = KB / 2;           // LDS bytes per row per stage: compressed values
  static constexpr int B_ROW = KB;               //                              dense operand
  static constexpr int GH = 8;                   // raster group height in tiles along i
  static constexpr int NB = BJ * B_ROW / 1024 / NW;   // 1 KB copies per wave per stage: B
  static constexpr int NA = BI * A_ROW / 1024 / NW;   //                                 A values
};
using TiledCfg = TileCfgT<4, 2>;
// The same 256 x 256 tile on four waves, one per SIMD, each computing 128 x 128 with 256 accumulator registers
// (the 512-register budget of a wave that has its SIMD to itself).  Every fragment read from LDS then feeds four
// matrix instructions instead of two or four: 100 KB of fragment reads per stage instead of 132 KB.  In cycles the
// two forms are equal (the matrix pipes are busy for 0.72 of them on config 3 either way), but the kernel runs
// against the power limit, and with 29 % fewer LDS cycles the clock settles higher: 0.5 to 2.7 % less time on the
// fp16 products of 8192 x 4096 x 11008 (more on boxes with less power headroom), 2.8 to 4.6 % on the fp8 product of
// 16384 x 8192 x 8192.  With few stages per tile the longer prologue and output pass of a
// 4-wave workgroup cost more than that (12 stages: 8 % slower; 24: equal; 32: 0.6 to 1.3 % faster), so only chained
// tiles of kWave4MinStages or more stages take this form.
using Wave4Cfg = TileCfgT<2, 4>;
// 256 x 192 tiles in the 4-wave form (wave tile 128 x 96): a tile costs 0.89 of a 256 x 256 one, so where the
// narrower tiles need no more rounds of the compute units than the wide ones, every round is that much shorter
// (W[1600, 6400] against 12288 tokens: 336 wide tiles or 448 narrow ones, two rounds either way, 147 against 165 us;
// W[11008, 4096] against 2048 tokens alike).  Long chained tiles only, like the 4-wave form itself.
using Wave4Cfg192 = TileCfgT<2, 3>;
constexpr int kWave4MinStages = 32;
// 256 x 64 tiles, two waves: for dense operands of at most 64 columns (a few dozen tokens), where a
// 256-wide tile would copy and multiply clamped columns.  26 KB per stage, two blocks per CU.
using SlimCfg = TileCfgT<1, 2>;
// 256 x 128 tiles, four waves: dense operands of 65 to 128 columns
using MidCfg = TileCfgT<2, 2>;

typedef __attribute__((address_space(3))) void* lds_ptr_t;

// The copies are issued from inline assembly so that the compiler's wait-count insertion does not
// see them: it would otherwise drain all outstanding copies (vmcnt(0)) before every LDS read, because
// it cannot tell the three stage buffers apart.  Ordering is enforced by hand with s_waitcnt vmcnt(N)
// before the stage barrier.  M0 carries the wave-uniform LDS base of the copy.
__device__ __forceinline__ uint32_t lds_offset(const void* p) {
  return (uint32_t)(uintptr_t)(lds_ptr_t)p;
}
// The source address is a wave-uniform 64-bit base in scalar registers plus a 32-bit offset per lane: with a
// 64-bit address per lane the same copies hold up the matrix instructions issued around them (on an
// instruction mix like the main loop's, 25 % more cycles than the matrix instructions alone against 3 %).
// same with one dword per lane: lane l writes LDS[base + 4*l]
__device__ __forceinline__ void g2l4(const uint8_t* base, uint32_t lane_offset, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1" ::"v"(lane_offset), "s"(base), "s"(lds_base) : "memory", "m0");
}
__device__ __forceinline__ void g2l16(const uint8_t* base, uint32_t lane_offset, uint32_t lds_base) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_offset), "s"(base), "s"(lds_base) : "memory", "m0");
}
// s_waitcnt vmcnt(N) + s_barrier with a compile-time N (a bare s_barrier: __syncthreads() would add
// a fence that drains every outstanding copy)
template <int N>
__device__ __forceinline__ void wait_copies_and_barrier() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" ::"n"(N) : "memory");
}

// workgroup barrier behind this wave's LDS reads only: copies stay in flight
__device__ __forceinline__ void wait_reads_and_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ACTS: the kernel is built twice, for launches without an activation (output pass: plain or bias only) and with one
// (bias or zeros, then ReLU, SiLU or GELU); with all five passes in one kernel the compiler no longer keeps the
// wave-uniform copy addresses in scalar registers.
template <typename T, typename OutT, bool C_JMAJOR, typename C, bool B_KSTRIDED, bool PERSIST, bool ACTS = false>
__global__ void __launch_bounds__(C::THREADS)
spmm_pipe(const uint8_t* __restrict__ a_values, const uint8_t* __restrict__ a_meta, int64_t n_sparse, int64_t k,
          const uint8_t* __restrict__ b, int64_t ldb_bytes, int64_t n_dense,
          OutT* __restrict__ c, int64_t ldc, const OutT* __restrict__ bias, float scale, int act,
          int tiles_i, int tiles_j, int splits, float* __restrict__ partial, int aux) {
  constexpr int ES = sizeof(T);
  constexpr int M_ROW = ES == 2 ? C::KB / 16 : C::KB / 8;   // metadata bytes per row per stage (8 or 16)
  constexpr int M_STEP = M_ROW / C::STEPS;
  // Metadata: in the panel form the words of 32 dense columns of consecutive rows are adjacent, [k/32][m][4 B],
  // so the 256 rows of a tile are one 1 KB run per block of 32 columns and a stage is M_ROW/4 such runs (2 for
  // 16-bit values, 4 for 8-bit ones).  In LDS they lie in the same order, [block][row][4 B], which is the order
  // the index operands are read in: 16-bit values read the halfword of their k half from block = step; 8-bit
  // values the dword of block = 2*step + k half; consecutive lanes read consecutive words either way.
  // A run is one 16-byte-per-lane copy instruction; 8-bit values take those, issued by the last waves of the
  // workgroup (copied a dword per lane, 16 instructions per stage, the same bytes took a fifth of the fp8
  // kernel's copy time).  With 16-bit values and more waves than runs every wave brings a quarter run (or more)
  // with dword copies instead, so that all waves run the same code: a branch in the loop body makes the compiler
  // re-mask the 16-bit index words behind it, and that wait for all of a step's reads costs 5 %.
  constexpr int STAGE_KB = M_ROW / 4;                        // 1 KB metadata runs per stage
  constexpr bool M_DWORD = ES == 2 && C::NW > STAGE_KB;      // quarter runs, every wave
  constexpr int MWAVES = M_DWORD ? C::NW : (STAGE_KB < C::NW ? STAGE_KB : C::NW);   // waves that copy metadata
  constexpr int MW = (M_DWORD ? STAGE_KB * 4 : STAGE_KB) / MWAVES;                  // copies per such wave
  static_assert(MW * MWAVES == (M_DWORD ? STAGE_KB * 4 : STAGE_KB) && C::BI * 4 == 1024, "metadata copies must divide among the waves");
  constexpr bool M_HALF_MAJOR = ES == 1;
  // one stage buffer = [A values | B | A metadata]; three of them rotate
  constexpr int A_STAGE = C::BI * C::A_ROW, B_STAGE = C::BJ * C::B_ROW, M_STAGE = C::BI * M_ROW;
  constexpr int B_AT = A_STAGE, M_AT = A_STAGE + B_STAGE, STAGE_BYTES = A_STAGE + B_STAGE + M_STAGE;
  __shared__ __attribute__((aligned(1024))) uint8_t smem[3 * STAGE_BYTES];

  // ---- XCD-aware work assignment.  A unit of work is (k-split, tile); units are ordered split-major
  // so that the units resident on an XCD belong to the same k range and share operand rows in L2.
  // Workgroup ids are dealt to the 8 XCDs round-robin: XCD x owns the units [x * per_xcd, (x+1) * per_xcd),
  // its workgroup number s = id / 8 takes unit s of that range -- and, PERSIST, every `slots`-th one after
  // it (slots = workgroups per XCD), one tile after the other in the same pipeline.
  const int ntiles = tiles_i * tiles_j;
  const int nunits = ntiles * splits;
  const int per_xcd = (nunits + 7) / 8;
  const int bid = blockIdx.x;
  const int slots = PERSIST ? (int)(gridDim.x >> 3) : per_xcd;
  const int xcd_end = min(((bid & 7) + 1) * per_xcd, nunits);
  int unit = (bid & 7) * per_xcd + (bid >> 3);
  if (unit >= xcd_end) return;
  constexpr int GH = C::GH;
  // aux: chained tiles (PERSIST) -- the start stagger in 10 ns ticks; otherwise the first row of tiles of this launch
  // (a launch may cover the tile rows [aux, aux + tiles_i) of the product; n_sparse stays the row count of the whole operand)
  const int stagger_ticks = PERSIST ? aux : 0;
  const int tile_row0 = PERSIST ? 0 : aux;
  int split = 0;
  int64_t i0 = 0, j0 = 0;
  auto locate = [&](int u, int64_t& ti0, int64_t& tj0) {       // unit -> k piece and tile origin
    split = u / ntiles;
    const int tile = u - split * ntiles;
    const int group = tile / (GH * tiles_j);
    const int gh = min(GH, tiles_i - group * GH);
    const int in_group = tile - group * GH * tiles_j;
    ti0 = (int64_t)(tile_row0 + group * GH + in_group % gh) * C::BI;
    tj0 = (int64_t)(in_group / gh) * C::BJ;
  };
  locate(unit, i0, j0);
  // Chained tiles: every second workgroup of an XCD starts `stagger_ticks` (10 ns each) late.  All compute units
  // otherwise finish their tiles at the same moment and write them out together, at the HBM rate, while no matrix
  // instruction issues (a wave's stores share the counter its copies are waited on, so the next tile stalls until
  // they are acknowledged); with two groups half a burst apart each group's stores drain while the other
  // multiplies.
  if constexpr (PERSIST) {
    if (stagger_ticks > 0 && ((bid >> 3) & 1)) {
      const uint64_t t0 = __builtin_amdgcn_s_memrealtime();
      for (int spin = 0; spin < 1024 && __builtin_amdgcn_s_memrealtime() - t0 < (uint64_t)stagger_ticks; spin++)
        __builtin_amdgcn_s_sleep(4);                 // (also bounded in iterations, whatever the counter does)
    }
  }

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wi = wave / C::WAVES_J, wj = wave % C::WAVES_J;
  const int l32 = lane & 31, lh = lane >> 5;
  const int nstages_total = (int)((k * ES) / C::KB);
  const int st_begin = (int)((int64_t)split * nstages_total / splits);
  const int nstages = (int)((int64_t)(split + 1) * nstages_total / splits) - st_begin;

  // ---- per-lane global sources of the copies (first stage of this unit); LDS destinations are wave-uniform.
  // B: copy q of a wave brings 8 rows x 128 bytes; lane -> (row, swizzled chunk).
  // A: stage st of rows i0..i0+255 is one contiguous run of 256*64 value bytes at (st*n_sparse + i0)*64
  //    (and 256*M_ROW metadata bytes): copy q brings 16 rows x 64 bytes.
  // Every source is (tile base, uniform, advanced by whole stages) + (lane offset inside the tile's first stage).
  uint32_t ob[C::NB], oa[C::NA], om[MW];
  const uint8_t *tile_b, *tile_a, *tile_m;
  // B with k strided (element (k,j) at k*ldb + j, 16-bit types): the stage is kept as [64 k][256 j]
  // in LDS, copy q brings 2 k-rows x 512 bytes; 16-byte chunks are XOR-swizzled with
  // ((k & 3) << 1) | ((k >> 3 & 1) << 3) so that the transposing fragment reads below (four k-rows x
  // 32 bytes per 16 lanes) touch every bank once.  Columns past n_dense re-read the last chunk.
  constexpr int64_t B_STAGE_ADVANCE_ROWS = B_KSTRIDED ? C::KB / ES : 0;
  const int64_t b_stage_stride = B_KSTRIDED ? B_STAGE_ADVANCE_ROWS * ldb_bytes : (int64_t)C::B_ROW;
  auto point_at = [&](int64_t ti0, int64_t tj0) {              // sources of the first stage of the tile at (ti0, tj0)
    // (PERSIST: the lane id is made opaque here and in the output pass, so that the per-lane terms of the
    // addresses are formed again for every tile instead of living in registers through the main loop,
    // where the accumulators and two fragment sets leave none to spare)
    int lane = threadIdx.x & 63;
    if constexpr (PERSIST) asm volatile("" : "+v"(lane));
    const int64_t last_j = n_dense - 1 - tj0, last_i = n_sparse - 1 - ti0;       // >= 0: tile origins lie inside
    if constexpr (B_KSTRIDED) tile_b = b + (int64_t)st_begin * B_STAGE_ADVANCE_ROWS * ldb_bytes;   // columns stay absolute: the clamp may step left of the tile
    else tile_b = b + tj0 * ldb_bytes + (int64_t)st_begin * C::B_ROW;
    tile_a = a_values + (ti0 + (int64_t)st_begin * n_sparse) * 64;
    tile_m = a_meta + (ti0 + (int64_t)st_begin * STAGE_KB * n_sparse) * 4;
#pragma unroll
    for (int q = 0; q < C::NB; q++) {
      if constexpr (B_KSTRIDED) {
        const int krow = (wave * C::NB + q) * 2 + (lane >> 5);
        const int ch = (lane & 31) ^ (((krow & 3) << 1) | (((krow >> 3) & 1) << 3));
        const int64_t col = min(tj0 + ch * 8, n_dense - 8);
        ob[q] = (uint32_t)(krow * ldb_bytes + col * ES);
      } else {
        const int row = (wave * C::NB + q) * 8 + (lane >> 3);
        const int ch = (lane & 7) ^ ((row >> 1) & 7);
        ob[q] = (uint32_t)(min((int64_t)row, last_j) * ldb_bytes + ch * 16);
      }
    }
#pragma unroll
    for (int q = 0; q < C::NA; q++) {
      const int row = (wave * C::NA + q) * 16 + (lane >> 2);
      const int ch = (lane & 3) ^ ((row >> 2) & 3);
      oa[q] = (uint32_t)(min((int64_t)row, last_i) * 64 + ch * 16);
    }
#pragma unroll
    for (int q = 0; q < MW; q++) {
      const int c = (wave - (C::NW - MWAVES)) * MW + q;        // quarter run (a lane brings one row's word) or run (4 rows' words)
      om[q] = M_DWORD ? (uint32_t)(((c >> 2) * n_sparse + min((int64_t)((c & 3) * 64 + lane), last_i)) * 4)
                      : (uint32_t)((c * n_sparse + min((int64_t)lane * 4, last_i - 3)) * 4);
    }
  };
  point_at(i0, j0);
  const int64_t a_stage_stride = n_sparse * 64, m_stage_stride = n_sparse * M_ROW;
  constexpr int NCOPY = C::NB + C::NA + MW;      // copies per wave per stage (MW fewer for the waves without metadata)
  const bool has_meta = MWAVES == C::NW || wave >= C::NW - MWAVES;      // the last waves (measured: 2.7 % better than the first ones at fp8)

  // copy q of this wave for stage st into the stage buffer at LDS byte address `dst`
  const uint32_t smem_at = lds_offset(smem);
  auto issue_one = [&](int q, int st, uint32_t dst) {
    if (q < C::NB) g2l16(tile_b + (int64_t)st * b_stage_stride, ob[q], dst + B_AT + (wave * C::NB + q) * 1024);
    else if (q < C::NB + C::NA) g2l16(tile_a + (int64_t)st * a_stage_stride, oa[q - C::NB], dst + (wave * C::NA + q - C::NB) * 1024);
    else if constexpr (M_DWORD) g2l4(tile_m + (int64_t)st * m_stage_stride, om[q - C::NB - C::NA], dst + M_AT + ((wave - (C::NW - MWAVES)) * MW + q - C::NB - C::NA) * 256);
    else if (has_meta) g2l16(tile_m + (int64_t)st * m_stage_stride, om[q - C::NB - C::NA], dst + M_AT + ((wave - (C::NW - MWAVES)) * MW + q - C::NB - C::NA) * 1024);
  };
  auto issue = [&](int st, uint32_t dst) {
#pragma unroll
    for (int q = 0; q < NCOPY; q++) issue_one(q, st, dst);
  };

  typename mma32<T>::acc_t acc[C::TI][C::TJ];
#pragma unroll
  for (int ti = 0; ti < C::TI; ti++)
#pragma unroll
    for (int tj = 0; tj < C::TJ; tj++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[ti][tj][r] = 0;

  // ---- fragment offsets (swizzled)
  const int a_row = wi * C::WI + l32, b_row = wj * C::WJ + l32;
  const int a_sw = (l32 >> 2) & 3, b_sw = (l32 >> 1) & 7;
  int a_off[C::STEPS], b_off[C::STEPS][2];
#pragma unroll
  for (int step = 0; step < C::STEPS; step++) {
    a_off[step] = a_row * C::A_ROW + (((step * 2 + lh) ^ a_sw) * 16);
#pragma unroll
    for (int h = 0; h < 2; h++) b_off[step][h] = b_row * C::B_ROW + (((step * 4 + h * 2 + lh) ^ b_sw) * 16);
  }
  const int m_off = M_HALF_MAJOR ? lh * (C::BI * 4) + a_row * 4 : a_row * M_STEP + lh * (M_STEP / 2);   // inside a step's block
  constexpr int M_FRAG = M_HALF_MAJOR ? 32 * 4 : 32 * M_STEP;    // from one 32-row fragment to the next
  // k-strided B: transposing reads (DS_READ_B64_TR_B16).  In a group of 16 lanes, lane i receives
  // the halfwords i%4 of the source lanes 4e + i/4 (e = 0..3).  Source lane s therefore addresses
  // k-row k0 + s/4, halfwords 4*(s%4).. of the group's 16 columns, and lane i ends up with
  // k0..k0+3 of column i: four such reads (k0 = 8*kb + {0, 4, 16, 20}) make one dense fragment.
  int bt_off[C::TJ];
  if constexpr (B_KSTRIDED) {
    const int g16 = lane >> 4, s16 = lane & 15;
    const int kb = g16 >> 1, jbase = (g16 & 1) * 16;
    const int swz = ((s16 >> 2) << 1) | (kb << 3);                // (k & 3) << 1 | (k >> 3 & 1) << 3 of the rows read
#pragma unroll
    for (int tj = 0; tj < C::TJ; tj++) {
      const int col = wj * C::WJ + tj * 32 + jbase + (s16 & 3) * 4;  // halfword column in the tile
      bt_off[tj] = (kb * 8 + (s16 >> 2)) * 512 + (((col >> 3) ^ swz) * 16) + ((col >> 2) & 1) * 8;
    }
  }

  // ---- main loop: a software pipeline over instruction steps.  While the matrix instructions of a
  // step run from one register set, the fragments of the next step are read from LDS into the
  // other, a few reads after every row of instructions: read in a block at the start of a step, the
  // eight waves' requests fill the LDS queue, every wave stalls on issue, and the matrix pipes wait.
  // The copies of the stage two ahead are spread over the same gaps (issued in a burst they would
  // queue in the texture-address unit and hold back the fragment reads).
  // One workgroup barrier per stage, B(s), placed before the first fragment read of stage s: every
  // wave arrives having waited for its own copies of stage s and with all its reads of stage s-1
  // complete, so behind B(s) stage s is visible and the buffer of stage s-1 is free for the copies
  // of stage s+2.  The matrix instructions of the last step of stage s-1 are issued behind B(s),
  // from registers, with the first reads of stage s between them.
  int4v af[2][C::TI];
  int idx[2][C::TI];
  int4v bf[2][C::TJ][2];                         // the two 16-byte halves of a dense fragment
  typedef short short4v __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) short4v* lds_short4_ptr;
  short4v bq[2][C::TJ][4];                       // k-strided B: the four 8-byte quarters
  // The reads of a step, in the order the next step's instructions need them: its first row of
  // instructions takes every dense fragment and sparse fragment 0, row r then only needs sparse
  // fragment r.  Read n: dense half-fragment n (fragment n/2, half n%2) for n < 2*TJ, then sparse
  // fragment and index word alternately.
  constexpr int B_READS = (B_KSTRIDED ? 4 : 2) * C::TJ;
  constexpr int N_READS = B_READS + 2 * C::TI;
  constexpr int READS_PER_ROW = (N_READS + C::TI - 1) / C::TI;
  // `src` is the byte offset of the stage buffer in smem (wave-uniform, changes every stage): the
  // per-lane addresses are formed when needed and fragment offsets ride in the instructions' immediates
  auto read_one = [&](int set, int n, uint32_t src, int step) {
    const uint8_t* base = smem + src;
    if (n < B_READS) {
      if constexpr (B_KSTRIDED) {
        const int tj = n >> 2, quarter = n & 3;                  // quarter: k0 = 8*kb + {0, 4, 16, 20}
        const uint8_t* src_q = base + B_AT + bt_off[tj] + step * (32 * 512) + ((quarter & 1) * 4 + (quarter >> 1) * 16) * 512;
        bq[set][tj][quarter] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4_ptr)(lds_ptr_t)src_q);
      } else {
        bf[set][n >> 1][n & 1] = *reinterpret_cast<const int4v*>(base + B_AT + b_off[step][n & 1] + (n >> 1) * 32 * C::B_ROW);
      }
    } else {
      const int f = (n - B_READS) >> 1;
      if (((n - B_READS) & 1) == 0) af[set][f] = *reinterpret_cast<const int4v*>(base + a_off[step] + f * 32 * C::A_ROW);
      else if constexpr (ES == 2) idx[set][f] = *reinterpret_cast<const uint16_t*>(base + M_AT + m_off + f * M_FRAG + step * (C::BI * M_STEP));
      else idx[set][f] = *reinterpret_cast<const int*>(base + M_AT + m_off + f * M_FRAG + step * (C::BI * M_STEP));
    }
  };
  // `half` selects which half of the wave's copies of stage pst is issued between the instructions
  // (into the buffer at LDS address dst); with `reads`, the fragments of step rstep of the buffer at
  // offset src go into the other register set.
  constexpr int PER_SLOT = (NCOPY + 2 * C::TI - 1) / (2 * C::TI);
  // copies of a stage issued during the first of its two steps (the rest during the second)
  constexpr int FIRST_HALF_COPIES = C::NW == 4 ? (NCOPY + 1) / 2 : (C::TI * PER_SLOT < NCOPY ? C::TI * PER_SLOT : NCOPY);
  auto mma_step = [&](int set, int half, bool copies, int pst, uint32_t dst, bool reads, uint32_t src, int rstep) {
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (C::NW == 4) {
      // One wave per SIMD: no other wave fills the matrix pipe while this one issues reads and copies, so they go
      // one by one behind every matrix instruction instead of in a block behind a row of them (in blocks: 5 % slower
      // than the 8-wave form instead of faster).  Ending the reads a few instructions before the step does, so
      // that the stage barrier finds them landed, changes nothing measurable.
      constexpr int SLOTS = C::TI * C::TJ;
      static_assert(!B_KSTRIDED, "the 4-wave form is built for a k-contiguous dense operand (with the transposing reads it spills)");
#pragma unroll
      for (int ti = 0; ti < C::TI; ti++) {
#pragma unroll
        for (int tj = 0; tj < C::TJ; tj++) {
          const int4v lo = bf[set][tj][0], hi = bf[set][tj][1];
          const int8v bfrag = int8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
          acc[ti][tj] = mma32<T>::run(af[set][ti], bfrag, acc[ti][tj], idx[set][ti]);
          __builtin_amdgcn_sched_barrier(0);
          const int n = ti * C::TJ + tj;
          if (reads) {
#pragma unroll
            for (int u = 0; u < (N_READS + SLOTS - 1) / SLOTS; u++)
              if (n * N_READS / SLOTS + u < (n + 1) * N_READS / SLOTS) read_one(set ^ 1, n * N_READS / SLOTS + u, src, rstep);
          }
#pragma unroll
          for (int q = 0; q < NCOPY; q++)
            if ((q * 2 * SLOTS) / NCOPY == half * SLOTS + n && copies) issue_one(q, pst, dst);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      return;
    }
#pragma unroll
    for (int ti = 0; ti < C::TI; ti++) {
#pragma unroll
      for (int tj = 0; tj < C::TJ; tj++) {
        int8v bfrag;
        if constexpr (B_KSTRIDED) {
          typedef int int2v __attribute__((ext_vector_type(2)));
          const int2v q0 = __builtin_bit_cast(int2v, bq[set][tj][0]), q1 = __builtin_bit_cast(int2v, bq[set][tj][1]);
          const int2v q2 = __builtin_bit_cast(int2v, bq[set][tj][2]), q3 = __builtin_bit_cast(int2v, bq[set][tj][3]);
          bfrag = int8v{q0[0], q0[1], q1[0], q1[1], q2[0], q2[1], q3[0], q3[1]};
        } else {
          const int4v lo = bf[set][tj][0], hi = bf[set][tj][1];
          bfrag = int8v{lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
        }
        acc[ti][tj] = mma32<T>::run(af[set][ti], bfrag, acc[ti][tj], idx[set][ti]);
      }
      __builtin_amdgcn_sched_barrier(0);
      if (reads) {
#pragma unroll
        for (int u = 0; u < READS_PER_ROW; u++)
          if (ti * READS_PER_ROW + u < N_READS) read_one(set ^ 1, ti * READS_PER_ROW + u, src, rstep);
      }
#pragma unroll
      for (int u = 0; u < PER_SLOT; u++) {
        const int q = (half * C::TI + ti) * PER_SLOT + u;
        if (q < NCOPY && copies) issue_one(q, pst, dst);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  static_assert(C::STEPS == 2, "the pipeline below is written for two instruction steps per stage");
  static_assert(!PERSIST || C_JMAJOR, "chained tiles rely on the wait inside the j-major output passes");
  auto stage_barrier = [&](bool more) {          // B(st+1): only this wave's copies of stage st+2 may still fly
    if (!more) wait_copies_and_barrier<0>();
    else if (MWAVES == C::NW || has_meta) wait_copies_and_barrier<NCOPY>();
    else wait_copies_and_barrier<NCOPY - MW>();
  };

  issue(0, smem_at);
  if (nstages > 1) issue(1, smem_at + STAGE_BYTES);
  uint32_t cur = 0, nxt = STAGE_BYTES, fre = 2 * STAGE_BYTES;   // buffers of stage st, st+1, st+2 (= st-1)
  // PERSIST (nstages >= 4, no k pieces): the workgroup walks its tiles in one pipeline.  The copies of
  // the next tile's first two stages are issued during the last two stages of the current one, into
  // the two buffers those stages leave free; the output pass then stages through the third (the last
  // stage's) while they fly, and the next tile starts with its operands already in LDS.
  int next_unit = unit;
  int64_t next_i0 = 0, next_j0 = 0;
  bool has_next = false;
  bool chained = false;                          // this tile's first two stages were copied under the previous tile
  for (;;) {
  // A chained tile's first two stages were waited for by every wave before the first store of the previous
  // output pass (below), so its first two barriers only publish them: waiting here on the counter of
  // outstanding memory operations would wait for the acknowledgements of those stores, which it does not
  // tell from copies.  From the third barrier on the usual wait is enough again: stores may complete out of
  // order with loads, but loads complete in order, and after the copies of stage s a wave issues the NCOPY
  // copies of stage s + 1 before it waits -- if one copy of stage s were still in flight, all of those
  // would be too, more than the NCOPY operations the wait allows.
  if (PERSIST && chained) wait_reads_and_barrier();
  else stage_barrier(nstages > 1);
  // stage 0: nothing to multiply yet
  {
    const bool more = 2 < nstages;
#pragma unroll
    for (int n = 0; n < N_READS; n++) read_one(0, n, cur, 0);
    if (more) {
#pragma unroll
      for (int q = 0; q < FIRST_HALF_COPIES; q++) issue_one(q, 2, smem_at + fre);
    }
    mma_step(0, 1, more, 2, smem_at + fre, true, cur, 1);
    if (PERSIST && chained) wait_reads_and_barrier();
    else stage_barrier(more);
  }
  // stage st: behind B(st), register set 1 holds the last step of stage st-1
  int st = 1;
  for (; st + 2 < nstages; st++) {
    const uint32_t t = cur; cur = nxt; nxt = fre; fre = t;
    mma_step(1, 0, true, st + 2, smem_at + fre, true, cur, 0);
    mma_step(0, 1, true, st + 2, smem_at + fre, true, cur, 1);
    stage_barrier(true);
  }
  if constexpr (PERSIST) {
    next_unit = unit + slots;
    has_next = next_unit < xcd_end;
    if (has_next) {                                 // every copy of this tile has been issued: aim at the next one
      locate(next_unit, next_i0, next_j0);
      point_at(next_i0, next_j0);
    }
  }
  for (; st < nstages; st++) {                    // the last two stages: nothing left to copy for this tile
    const uint32_t t = cur; cur = nxt; nxt = fre; fre = t;
    const int pst = st - (nstages - 2);           // stage 0, then 1 of the next tile
    mma_step(1, 0, has_next, pst, smem_at + fre, true, cur, 0);
    mma_step(0, 1, has_next, pst, smem_at + fre, true, cur, 1);
    // behind the last barrier of a tile no wave reads the stage buffers any more; the next tile's
    // copies are not waited for here
    if (st + 1 < nstages) stage_barrier(has_next);
    else if (has_next) wait_reads_and_barrier();
    else stage_barrier(false);
  }
  // ---- bias: every lane fetches the bias of WI/64 of its wave's rows here, one instruction step ahead of the
  // output pass, which hands them round the wave through LDS.  (Fetched per element inside the pass -- 128 two-byte
  // loads per lane, a wait behind every four -- the bias cost 2.8 us per 256 x 256 tile: 59 % on top of a 12-stage
  // tile, 31 % on a 64-stage one.)
  // The loaded bits are first touched behind that step (the empty asm statements): converted right away, the compiler
  // waits for each load -- and with it for every copy in flight -- before the step's matrix instructions.
  using accs_t = std::remove_reference_t<decltype(acc[0][0][0])>;
  uint32_t bias_w[C::WI / 64];
#pragma unroll
  for (int q = 0; q < C::WI / 64; q++) bias_w[q] = 0;
  if (splits == 1 && bias != nullptr) {
#pragma unroll
    for (int q = 0; q < C::WI / 64; q++) {
      const int64_t row = i0 + wi * C::WI + q * 64 + (int)(threadIdx.x & 63);
      bias_w[q] = bias_bits(bias[row < n_sparse ? row : n_sparse - 1]);
    }
  }
  mma_step(1, 0, false, 0, 0, false, 0, 0);       // the last step
  if (splits == 1 && bias != nullptr) {
#pragma unroll
    for (int q = 0; q < C::WI / 64; q++) asm volatile("" : "+v"(bias_w[q]));
  }

  // ---- split-K: park the 32-bit accumulators in the workspace, in register order (every group of
  // four accumulators is one contiguous 16-byte-per-lane slab); spmm_reduce_splits finishes the job.
  if (splits > 1) {
    float* base = partial + (int64_t)unit * (C::BI * C::BJ);
#pragma unroll
    for (int ti = 0; ti < C::TI; ti++)
#pragma unroll
      for (int tj = 0; tj < C::TJ; tj++) {
        if (j0 + wj * C::WJ + tj * 32 >= n_dense) continue;      // columns past the dense operand: never read back
#pragma unroll
        for (int g = 0; g < 4; g++) {
          const int slab = (ti * C::TJ + tj) * 4 + g;
          typename mma32<T>::acc4_t v = {acc[ti][tj][g * 4], acc[ti][tj][g * 4 + 1], acc[ti][tj][g * 4 + 2], acc[ti][tj][g * 4 + 3]};
          *reinterpret_cast<typename mma32<T>::acc4_t*>(base + ((int64_t)slab * C::THREADS + tid) * 4) = v;
        }
      }
    return;
  }

  auto output_pass = [&](auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
    int lane = threadIdx.x & 63;
    if constexpr (PERSIST) asm volatile("" : "+v"(lane));
    const int l32 = lane & 31, lh = lane >> 5;
    // the bias of this wave's WI rows, behind the staging slices of all waves; the wave reads back what its own lanes
    // wrote (LDS accesses of one wave execute in order: no barrier)
    accs_t* bias_lds = reinterpret_cast<accs_t*>(smem + cur + C::NW * 4096 + wave * (C::WI * 4));
    if constexpr (MODE != EPI_PLAIN) {
#pragma unroll
      for (int q = 0; q < C::WI / 64; q++) {
        const accs_t v = bias_as(accs_t(0), bias_from_bits<OutT>(bias_w[q]));
        bias_lds[q * 64 + lane] = i0 + wi * C::WI + q * 64 + lane < n_sparse ? v : accs_t(0);
      }
    }
    // The bias of rows ti*32 + g*8 + lh*4 + 0..3 of the wave's tile, g = 0..3: read for a whole block of the pass
    // ahead of its staging writes.  (Read where it is used, every quad waits behind the LDS writes issued before it,
    // 32 round trips per wave and tile: 1.3 to 2 us.)
    using bias4_t = typename mma32<T>::acc4_t;
    auto bias_quads = [&](int ti, bias4_t (&bq)[4]) {
#pragma unroll
      for (int g = 0; g < 4; g++) {
        bq[g] = bias4_t{0, 0, 0, 0};
        if constexpr (MODE != EPI_PLAIN) bq[g] = *reinterpret_cast<const bias4_t*>(bias_lds + ti * 32 + g * 8 + lh * 4);
      }
    };
    // ---- epilogue.  D layout: column l%32, rows 8*(r/4) + 4*(l/32) + r%4.
    // For 16-bit outputs stored j-major (the Y of X.W^T) a lane owns runs of only 4 consecutive i
    // (8 bytes) in 32 different output rows, so direct stores would touch 32 lines per instruction.
    // Instead every wave stages 32(j) x 64(i) pieces of its sub-tile in a private 4 KB slice of the
    // last stage's buffer (no wave reads it any more: the tile's last barrier is behind us; the other
    // two buffers may already be receiving the next tile) -- 128-byte rows, 16-byte chunks
    // XOR-swizzled with the row -- and streams them out as eight full 128-byte row segments per
    // instruction (streaming stores: the tile is not read again by this kernel and should not
    // displace operand lines in L2).  LDS accesses of one wave execute in order, so the passes need
    // no barrier between them.
    if constexpr (C_JMAJOR && sizeof(OutT) == 2) {
      uint8_t* stage = smem + cur + wave * 4096;
      const int rr = lane >> 3, chr = lane & 7;
  #pragma unroll
      for (int tj = 0; tj < C::TJ; tj++) {
  #pragma unroll
        for (int ip = 0; ip < C::TI / 2; ip++) {                // 64 sparse rows (i) per pass
          bias4_t bq[2][4];
          bias_quads(ip * 2, bq[0]);
          bias_quads(ip * 2 + 1, bq[1]);
  #pragma unroll
          for (int t2 = 0; t2 < 2; t2++) {
            const int ti = ip * 2 + t2;
  #pragma unroll
            for (int g = 0; g < 4; g++) {
              OutT o[4];
  #pragma unroll
              for (int r = 0; r < 4; r++) o[r] = to_out<OutT>(finish_element<MODE>(acc[ti][tj][g * 4 + r], scale, bq[t2][g][r]));
              const int ch = t2 * 4 + g;
              *reinterpret_cast<Pack<OutT, 4>*>(stage + l32 * 128 + ((ch ^ (l32 & 7)) * 16) + lh * 8) = *reinterpret_cast<Pack<OutT, 4>*>(o);
            }
          }
          const int64_t icol = i0 + wi * C::WI + ip * 64 + chr * 8;
          // the next tile's first two stages (issued one and two stages ago) have to be in LDS before this
          // wave's first store joins the outstanding operations
          if (PERSIST && tj == 0 && ip == 0 && has_next) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  #pragma unroll
          for (int it = 0; it < 4; it++) {
            const int jl = it * 8 + rr;
            const int64_t jrow = j0 + wj * C::WJ + tj * 32 + jl;
            const int4v v = *reinterpret_cast<const int4v*>(stage + jl * 128 + ((chr ^ (jl & 7)) * 16));
            if (jrow < n_dense && icol < n_sparse) __builtin_nontemporal_store(v, reinterpret_cast<int4v*>(c + jrow * ldc + icol));
          }
        }
      }
    } else if constexpr (C_JMAJOR && sizeof(OutT) == 4) {
      // j-major 32-bit output (float32 from 8-bit operands, int32 from int8: the reference's output types for
      // them): the same staging with 32(j) x 32(i) pieces -- a lane's four consecutive i are one 16-byte chunk of
      // a 128-byte row -- so that the stores are full 128-byte row segments instead of 32-byte ones.
      uint8_t* stage = smem + cur + wave * 4096;
      const int rr = lane >> 3, chr = lane & 7;
  #pragma unroll
      for (int tj = 0; tj < C::TJ; tj++) {
  #pragma unroll
        for (int ti = 0; ti < C::TI; ti++) {
          bias4_t bq[4];
          bias_quads(ti, bq);
  #pragma unroll
          for (int g = 0; g < 4; g++) {
            typedef OutT out4v __attribute__((ext_vector_type(4)));
            out4v o;
  #pragma unroll
            for (int r = 0; r < 4; r++) o[r] = to_out<OutT>(finish_element<MODE>(acc[ti][tj][g * 4 + r], scale, bq[g][r]));
            const int ch = g * 2 + lh;
            *reinterpret_cast<out4v*>(stage + l32 * 128 + ((ch ^ (l32 & 7)) * 16)) = o;
          }
          const int64_t icol = i0 + wi * C::WI + ti * 32 + chr * 4;
          // (chained tiles: see the 16-bit pass)
          if (PERSIST && tj == 0 && ti == 0 && has_next) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  #pragma unroll
          for (int it = 0; it < 4; it++) {
            const int jl = it * 8 + rr;
            const int64_t jrow = j0 + wj * C::WJ + tj * 32 + jl;
            const int4v v = *reinterpret_cast<const int4v*>(stage + jl * 128 + ((chr ^ (jl & 7)) * 16));
            if (jrow < n_dense && icol < n_sparse) __builtin_nontemporal_store(v, reinterpret_cast<int4v*>(c + jrow * ldc + icol));
          }
        }
      }
    } else if constexpr (!C_JMAJOR && sizeof(OutT) == 2) {
      // i-major 16-bit output (the W.B of `S @ dense`): a lane owns single elements of 64+ different
      // rows.  Stage 32(i) x 64(j) pieces as [i][64 j] (128-byte rows, chunks XOR-swizzled with the
      // row) and stream them out as eight full 128-byte rows per instruction.
      uint8_t* stage = smem + cur + wave * 4096;
      const int rr = lane >> 3, chr = lane & 7;
  #pragma unroll
      for (int half = 0; half < C::TJ / 2; half++) {            // 64 output columns (j) per pass
  #pragma unroll
        for (int ti = 0; ti < C::TI; ti++) {                    // 32 sparse rows (i) per pass
          bias4_t bq[4];
          bias_quads(ti, bq);
  #pragma unroll
          for (int t2 = 0; t2 < 2; t2++) {
            const int tj = half * 2 + t2;
            const int jl = t2 * 32 + l32;
  #pragma unroll
            for (int g = 0; g < 4; g++) {
  #pragma unroll
              for (int r = 0; r < 4; r++) {
                const int il = g * 8 + lh * 4 + r;
                *reinterpret_cast<OutT*>(stage + il * 128 + (((jl >> 3) ^ (il & 7)) * 16) + (jl & 7) * 2) =
                    to_out<OutT>(finish_element<MODE>(acc[ti][tj][g * 4 + r], scale, bq[g][r]));
              }
            }
          }
          const int64_t jcol = j0 + wj * C::WJ + half * 64 + chr * 8;
  #pragma unroll
          for (int it = 0; it < 4; it++) {
            const int il = it * 8 + rr;
            const int64_t irow = i0 + wi * C::WI + ti * 32 + il;
            const int4v v = *reinterpret_cast<const int4v*>(stage + il * 128 + ((chr ^ (il & 7)) * 16));
            if (irow < n_sparse && jcol < n_dense) __builtin_nontemporal_store(v, reinterpret_cast<int4v*>(c + irow * ldc + jcol));
          }
        }
      }
    } else {
  #pragma unroll
      for (int ti = 0; ti < C::TI; ti++) {
        bias4_t bq[4];
        bias_quads(ti, bq);
  #pragma unroll
        for (int tj = 0; tj < C::TJ; tj++) {
          const int64_t col = j0 + wj * C::WJ + tj * 32 + l32;
  #pragma unroll
          for (int g = 0; g < 4; g++) {
            const int64_t row = i0 + wi * C::WI + ti * 32 + g * 8 + lh * 4;
            if (col >= n_dense || row >= n_sparse) continue;
            OutT o[4];
  #pragma unroll
            for (int r = 0; r < 4; r++) o[r] = to_out<OutT>(finish_element<MODE>(acc[ti][tj][g * 4 + r], scale, bq[g][r]));
            if constexpr (C_JMAJOR) {
              *reinterpret_cast<Pack<OutT, 4>*>(c + col * ldc + row) = *reinterpret_cast<Pack<OutT, 4>*>(o);
            } else {
  #pragma unroll
              for (int r = 0; r < 4; r++) c[(row + r) * ldc + col] = o[r];
            }
          }
        }
      }
    }
  };
  constexpr bool INT_ACC = std::is_same<typename mma32<T>::acc4_t, int4v>::value;
  if constexpr (!ACTS) {
    if (!bias) output_pass(std::integral_constant<int, EPI_PLAIN>{});
    else output_pass(std::integral_constant<int, EPI_BIAS>{});
  } else if constexpr (INT_ACC) {
    if (act == TF24_ACT_RELU) output_pass(std::integral_constant<int, EPI_RELU>{});
    else output_pass(std::integral_constant<int, EPI_BIAS>{});
  } else {
    if (act == TF24_ACT_RELU) output_pass(std::integral_constant<int, EPI_RELU>{});
    else if (act == TF24_ACT_SILU) output_pass(std::integral_constant<int, EPI_SILU>{});
    else output_pass(std::integral_constant<int, EPI_GELU>{});
  }
  if (!has_next) break;
  // ---- the next tile: its first two stages are (about to be) in the buffers nxt and fre
  unit = next_unit; i0 = next_i0; j0 = next_j0; chained = true;
  { const uint32_t t = cur; cur = nxt; nxt = fre; fre = t; }
#pragma unroll
  for (int ti = 0; ti < C::TI; ti++)
#pragma unroll
    for (int tj = 0; tj < C::TJ; tj++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[ti][tj][r] = 0;
  }
}

// Second pass of a split-K product: a block handles one eighth of a tile (the accumulator groups
// `slab` of one ti), same lane -> element mapping as spmm_pipe; sums the `splits` partial tiles
// (float32, or int32 for int8 operands) and applies scale / bias / activation / conversion.
template <typename Acc4, typename OutT, bool C_JMAJOR, typename C>
__global__ void __launch_bounds__(C::THREADS)
spmm_reduce_splits(const float* __restrict__ partial, int splits, int tiles_i, int tiles_j, int64_t n_sparse, int64_t n_dense,
                   OutT* __restrict__ c, int64_t ldc, const OutT* __restrict__ bias, float scale, int act) {
  const int ntiles = tiles_i * tiles_j;
  const int tile = blockIdx.x;
  constexpr int GH = C::GH;
  const int group = tile / (GH * tiles_j);
  const int gh = min(GH, tiles_i - group * GH);
  const int in_group = tile - group * GH * tiles_j;
  const int64_t i0 = (int64_t)(group * GH + in_group % gh) * C::BI, j0 = (int64_t)(in_group / gh) * C::BJ;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wi = wave / C::WAVES_J, wj = wave % C::WAVES_J;
  const int l32 = lane & 31, lh = lane >> 5;
  constexpr int NSLAB = C::TI * C::TJ * 4;
  // gridDim.y blocks share the NSLAB accumulator groups of the tile
  for (int slab = blockIdx.y; slab < NSLAB; slab += gridDim.y) {
    const int ti = slab / (C::TJ * 4), tj = (slab / 4) % C::TJ, g = slab % 4;
    if (j0 + wj * C::WJ + tj * 32 >= n_dense) continue;          // the whole 32-column slab lies past the dense operand
    // the pieces are loaded eight at a time (independent loads in flight) and added in piece order
    Acc4 sum = {0, 0, 0, 0};
    const float* first = partial + (int64_t)tile * (C::BI * C::BJ) + ((int64_t)slab * C::THREADS + tid) * 4;
    const int64_t piece = (int64_t)ntiles * (C::BI * C::BJ);
    for (int sp0 = 0; sp0 < splits; sp0 += 8) {
      Acc4 part[8];
#pragma unroll
      for (int u = 0; u < 8; u++)
        part[u] = *reinterpret_cast<const Acc4*>(first + (int64_t)min(sp0 + u, splits - 1) * piece);
#pragma unroll
      for (int u = 0; u < 8; u++)
        if (sp0 + u < splits) sum += part[u];
    }
    const int64_t col = j0 + wj * C::WJ + tj * 32 + l32;
    const int64_t row = i0 + wi * C::WI + ti * 32 + g * 8 + lh * 4;
    if (col >= n_dense || row >= n_sparse) continue;
    OutT o[4];
#pragma unroll
    for (int r = 0; r < 4; r++) o[r] = to_out<OutT>(finish_value(sum[r], scale, bias, row + r, act));
    if constexpr (C_JMAJOR) {
      *reinterpret_cast<Pack<OutT, 4>*>(c + col * ldc + row) = *reinterpret_cast<Pack<OutT, 4>*>(o);
    } else {
#pragma unroll
      for (int r = 0; r < 4; r++) c[(row + r) * ldc + col] = o[r];
    }
  }
}

// k-splits for shapes whose tiles cannot fill the 256 CUs (k-heavy products such as dW): as many as
// fit, each at least 4 stages long, if the caller's workspace holds the float32 partial tiles.
template <typename T, typename C>
int choose_splits(int64_t n_sparse, int64_t k, int64_t n_dense, int64_t workspace_bytes) {
  const int64_t tiles = ((n_sparse + C::BI - 1) / C::BI) * ((n_dense + C::BJ - 1) / C::BJ);
  const int64_t nstages = k * (int64_t)sizeof(T) / C::KB;
  if (tiles >= 160) return 1;
  int64_t splits = 192 / tiles;              // measured: filling all 256 CUs costs more in partial tiles than it gains
  if (splits > nstages / 4) splits = nstages / 4;
  if (splits > 16) splits = 16;
  while (splits > 1 && splits * tiles * C::BI * C::BJ * 4 > workspace_bytes) splits--;
  return splits < 2 ? 1 : (int)splits;
}

// Time estimate of the tiled kernel on one tile configuration, to choose between 256 x 256 and
// 256 x 128 tiles for operands of a few hundred dense columns: rounds of at most 256 blocks (one per
// CU) x stages per block x the stage time measured for that configuration (0.95 us for 256 x 256
// tiles, 0.55 us for 256 x 128), plus, with k pieces, the partial tiles written and read at
// 4.5 TB/s and the second launch.  On W[11008, 4096], W[4096, 11008] and W[8192, 8192] with 256 to
// 1536 dense columns it picks the faster configuration in every case measured (up to 30 % apart).
struct TileCost { int64_t blocks; double us; };
template <typename T, typename C>
TileCost tile_cost(int64_t n_sparse, int64_t k, int64_t n_dense, int64_t workspace_bytes, double stage_us) {
  const int64_t tiles = ((n_sparse + C::BI - 1) / C::BI) * ((n_dense + C::BJ - 1) / C::BJ);
  const int64_t nstages = k * (int64_t)sizeof(T) / C::KB;
  const int64_t splits = workspace_bytes > 0 ? choose_splits<T, C>(n_sparse, k, n_dense, workspace_bytes) : 1;
  const int64_t blocks = tiles * splits, rounds = (blocks + 255) / 256;
  double us = (double)rounds * (double)((nstages + splits - 1) / splits) * stage_us;
  if (splits > 1) us += 2.0 * (double)(splits * tiles * C::BI * C::BJ * 4) / 4.5e6 + 3.0;
  return {blocks, us};
}

// compute units of the current device (looked up once per device; the cache is a table of atomics: two threads
// that meet on an empty entry both look the value up and store the same number)
inline int compute_units() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (!n) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

template <typename T, typename OutT, typename C>
int launch_tiled(const void* av, const void* am, int64_t n_sparse, int64_t k, const void* b, int b_layout, int64_t ldb,
                 int64_t n_dense, void* c, int c_layout, int64_t ldc, const void* bias, float scale, int act,
                 void* workspace, int64_t workspace_bytes, hipStream_t s) {
  int tiles_i = (int)((n_sparse + C::BI - 1) / C::BI);
  const int tiles_j = (int)((n_dense + C::BJ - 1) / C::BJ);
  const int splits = workspace ? choose_splits<T, C>(n_sparse, k, n_dense, workspace_bytes) : 1;
  const int cu_slots = compute_units() / 8;
  // A last round that fills less than half of the compute units: the tile rows that make up the full rounds stay
  // with the chained 256 x 256 tiles, the remaining rows go to a second launch on 256 x 128 tiles, which reach twice
  // as many compute units for half the time each (W[11008, 4096] against 8192 tokens: 1376 tiles = 5 rounds of 256
  // + 96; 40 tile rows chained, 3 rows as 192 half tiles: 351.6 -> 341.6 us).  Long tiles only: what a short
  // tile's round costs is mostly its prologue and output pass, which the second launch pays again.
  int tail_rows = 0;
  if constexpr (std::is_same<C, TiledCfg>::value) {
    const int cus = cu_slots * 8, tiles = tiles_i * tiles_j;
    if (cus > 0 && c_layout == TF24_COL_MAJOR && b_layout == TF24_ROW_MAJOR && splits == 1 && tiles % cus != 0 &&
        k * (int64_t)sizeof(T) / C::KB >= kWave4MinStages) {
      const int rows = tiles / cus * cus / tiles_j;            // tile rows of the full rounds
      const int left = tiles_i - rows;
      const int64_t half_tiles = (int64_t)left * ((n_dense + MidCfg::BJ - 1) / MidCfg::BJ);
      if (rows * tiles_j > cus && left > 0 && half_tiles <= cus) { tiles_i = rows; tail_rows = left; }
    }
  }
  const int per_xcd = (tiles_i * tiles_j * splits + 7) / 8;
  // More tiles than compute units and no k pieces: one workgroup per compute unit walks its tiles in
  // one pipeline (the next tile's operands arrive while the current one is written out).
  const bool persist = C::BJ == 256 && c_layout == TF24_COL_MAJOR && splits == 1 &&
                       k * (int64_t)sizeof(T) / C::KB >= 4 && per_xcd > cu_slots && cu_slots > 0;
  dim3 grid((unsigned)((persist ? cu_slots : per_xcd) * 8));
  const bool jm = c_layout == TF24_COL_MAJOR;
  // Start stagger of chained tiles (see spmm_pipe): half an output burst -- 256 tiles of 128 KB (16-bit) or 256 KB
  // (32-bit) at the HBM write rate are 6 or 12 us -- for short tiles, whose time the bursts are a large part of, and
  // for 32-bit outputs over three or more rounds.  Measured: 576 tiles of 12 stages 48.9 -> 43.4 us (the training
  // step they belong to 0.684 -> 0.679 ms), 2048 tiles of 64 fp8 stages with float32 output 0.521 -> 0.514 ms; with
  // 16-bit outputs the same tiles are unchanged and 1376 tiles of 64 fp16 stages lose 0.2 % (alternating with another
  // product; 1.6 % faster when the same product repeats), so long 16-bit tiles start together.
  const int stagger_rounds = persist ? (per_xcd + cu_slots - 1) / cu_slots : 0;
  const int stagger = !persist ? 0 : k * (int64_t)sizeof(T) / C::KB <= 32 ? (sizeof(OutT) == 2 ? 300 : 600)
                               : (sizeof(OutT) == 4 && stagger_rounds >= 3) ? 600 : 0;
  // long chained tiles of a k-contiguous dense operand take the 4-wave form
  const bool wave4 = persist && std::is_same<C, TiledCfg>::value && b_layout == TF24_ROW_MAJOR &&
                     k * (int64_t)sizeof(T) / C::KB >= kWave4MinStages;
  auto launch_tail = [&]() {                       // the rows behind the full rounds, on 256 x 128 tiles
    if constexpr (std::is_same<C, TiledCfg>::value) {
      if (tail_rows > 0) {
        const int tj = (int)((n_dense + MidCfg::BJ - 1) / MidCfg::BJ);
        const dim3 tgrid((unsigned)((tail_rows * tj + 7) / 8 * 8));
        auto tail = [&](auto acts) {
          hipLaunchKernelGGL((spmm_pipe<T, OutT, true, MidCfg, false, false, decltype(acts)::value>), tgrid, dim3(MidCfg::THREADS), 0, s,
                             (const uint8_t*)av, (const uint8_t*)am, n_sparse, k, (const uint8_t*)b, ldb * (int64_t)sizeof(T), n_dense,
                             (OutT*)c, ldc, (const OutT*)bias, scale, act, tail_rows, tj, 1, (float*)nullptr, tiles_i);
        };
        if (act == TF24_ACT_NONE) tail(std::false_type{}); else tail(std::true_type{});
      }
    }
  };
  if constexpr (std::is_same<C, TiledCfg>::value && sizeof(OutT) == 2) {
    const int tiles_j192 = (int)((n_dense + Wave4Cfg192::BJ - 1) / Wave4Cfg192::BJ);
    const int per_xcd192 = (tiles_i * tiles_j192 + 7) / 8;
    // Also where both widths fit one round and the narrow tiles spread over more compute units (W[768, 3072] against
    // 12288 tokens: 144 wide tiles or 192 narrow ones, 36.1 -> 34.1 us; W[1024, 4096]: 192 or 256 tiles, 56.2 -> 53.9 us).
    const bool one_round192 = C::BJ == 256 && c_layout == TF24_COL_MAJOR && splits == 1 && b_layout == TF24_ROW_MAJOR &&
                              k * (int64_t)sizeof(T) / C::KB >= kWave4MinStages && cu_slots > 0 && per_xcd192 <= cu_slots && per_xcd192 > per_xcd;
    if (one_round192 || (wave4 && per_xcd192 > cu_slots && (per_xcd192 + cu_slots - 1) / cu_slots <= (per_xcd + cu_slots - 1) / cu_slots)) {
      if (one_round192) grid = dim3((unsigned)(cu_slots * 8));    // the chained-tile kernel with one tile per workgroup
      auto narrow = [&](auto acts) {
        hipLaunchKernelGGL((spmm_pipe<T, OutT, true, Wave4Cfg192, false, true, decltype(acts)::value>), grid, dim3(Wave4Cfg192::THREADS), 0, s,
                           (const uint8_t*)av, (const uint8_t*)am, n_sparse, k, (const uint8_t*)b, ldb * (int64_t)sizeof(T), n_dense,
                           (OutT*)c, ldc, (const OutT*)bias, scale, act, tiles_i, tiles_j192, splits, (float*)workspace, stagger);
      };
      if (act == TF24_ACT_NONE) narrow(std::false_type{}); else narrow(std::true_type{});
      launch_tail();
      return check_launch("tf24_spmm");
    }
  }
  auto launch_epi = [&](auto c_jmajor, auto b_kstrided, auto acts) {
    constexpr bool ACTS = decltype(acts)::value;
    if constexpr (C::BJ == 256 && decltype(c_jmajor)::value) {
      if constexpr (std::is_same<C, TiledCfg>::value && !decltype(b_kstrided)::value) {
        if (wave4) {
          hipLaunchKernelGGL((spmm_pipe<T, OutT, true, Wave4Cfg, false, true, ACTS>), grid, dim3(Wave4Cfg::THREADS), 0, s,
                             (const uint8_t*)av, (const uint8_t*)am, n_sparse, k, (const uint8_t*)b, ldb * (int64_t)sizeof(T), n_dense,
                             (OutT*)c, ldc, (const OutT*)bias, scale, act, tiles_i, tiles_j, splits, (float*)workspace, stagger);
          return;
        }
      }
      if (persist) {
        hipLaunchKernelGGL((spmm_pipe<T, OutT, decltype(c_jmajor)::value, C, decltype(b_kstrided)::value, true, ACTS>), grid, dim3(C::THREADS), 0, s,
                           (const uint8_t*)av, (const uint8_t*)am, n_sparse, k, (const uint8_t*)b, ldb * (int64_t)sizeof(T), n_dense,
                           (OutT*)c, ldc, (const OutT*)bias, scale, act, tiles_i, tiles_j, splits, (float*)workspace, stagger);
        return;
      }
    }
    hipLaunchKernelGGL((spmm_pipe<T, OutT, decltype(c_jmajor)::value, C, decltype(b_kstrided)::value, false, ACTS>), grid, dim3(C::THREADS), 0, s,
                       (const uint8_t*)av, (const uint8_t*)am, n_sparse, k, (const uint8_t*)b, ldb * (int64_t)sizeof(T), n_dense,
                       (OutT*)c, ldc, (const OutT*)bias, scale, act, tiles_i, tiles_j, splits, (float*)workspace, 0);
  };
  auto launch = [&](auto c_jmajor, auto b_kstrided) {
    // with k pieces the reduction kernel applies bias and activation, not this one
    if (act == TF24_ACT_NONE || splits > 1) launch_epi(c_jmajor, b_kstrided, std::false_type{});
    else launch_epi(c_jmajor, b_kstrided, std::true_type{});
  };
  bool kstrided = false;
  if constexpr (sizeof(T) == 2 && C::BJ == 256) kstrided = b_layout == TF24_COL_MAJOR;
  if (kstrided) {
    if constexpr (sizeof(T) == 2 && C::BJ == 256) {
      if (jm) launch(std::true_type{}, std::true_type{});
      else launch(std::false_type{}, std::true_type{});
    }
  } else {
    if (jm) launch(std::true_type{}, std::false_type{});
    else launch(std::false_type{}, std::false_type{});
  }
  launch_tail();
  if (splits > 1) {
    dim3 rgrid((unsigned)(tiles_i * tiles_j), C::TI * C::TJ * 4);      // one accumulator group of the tile per block
    if (jm)
      hipLaunchKernelGGL((spmm_reduce_splits<typename mma32<T>::acc4_t, OutT, true, C>), rgrid, dim3(C::THREADS), 0, s, (const float*)workspace, splits, tiles_i, tiles_j,
                         n_sparse, n_dense, (OutT*)c, ldc, (const OutT*)bias, scale, act);
    else
      hipLaunchKernelGGL((spmm_reduce_splits<typename mma32<T>::acc4_t, OutT, false, C>), rgrid, dim3(C::THREADS), 0, s, (const float*)workspace, splits, tiles_i, tiles_j,
                         n_sparse, n_dense, (OutT*)c, ldc, (const OutT*)bias, scale, act);
  }
  return check_launch("tf24_spmm");
}

// ------------------------------------------------------------------------------------------
// Narrow kernels: at most 16 dense columns (decoding a few tokens against a large sparse weight).
// The product is bound by one pass over the compressed operand, so the sparse operand is not
// staged: a wave streams the A fragments of 16 sparse rows straight into registers (in the panel
// layout 1 KB of contiguous memory per panel, 16 bytes per lane, and their index words 128 (256)
// contiguous bytes) and runs one V_SMFMAC_*_16X16 per panel.  Loads are issued a batch of panels at
// a time into one of two register sets, the next batch while the current one is multiplied: left
// to itself the compiler waits for each panel's loads before it issues the next.
// Fewer than 512 row blocks (spmm_narrow): a block owns 16 rows, its up to four waves each take a
// share of the k range, read their dense fragments from global memory (64 contiguous bytes from
// each of the 16 dense rows, twice) and meet in LDS at the end (added in wave order).
// From 512 row blocks on (spmm_narrow_shared): see there.
// ------------------------------------------------------------------------------------------
constexpr int kNarrowMaxDense = 16;
constexpr int kNarrowWaves = 4;
constexpr int kNarrowSharedMin = 160;      // workgroups of four 16-row blocks below which two blocks per workgroup are faster

template <typename T, typename OutT, bool C_JMAJOR>
__global__ void __launch_bounds__(64 * kNarrowWaves)
spmm_narrow(const uint8_t* __restrict__ a_values, const uint8_t* __restrict__ a_meta, int64_t n_sparse, int64_t k,
            const uint8_t* __restrict__ b, int64_t ldb_bytes, int64_t n_dense,
            OutT* __restrict__ c, int64_t ldc, const OutT* __restrict__ bias, float scale, int act) {
  constexpr int KSTEP = mma16<T>::KSTEP;     // dense k per panel = per instruction
  constexpr int M_ROW = KSTEP / 8;           // metadata bytes per row per panel
  constexpr int BATCH = 8;                   // panels per load batch; two batches are in flight
  using acc_t = typename mma16<T>::acc_t;
  __shared__ acc_t s_acc[kNarrowWaves - 1][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, li = lane & 15, lk = lane >> 4;
  const int64_t i0 = (int64_t)blockIdx.x * 16;
  const int64_t npanels = k / KSTEP;
  const int nwaves = blockDim.x >> 6;
  const int64_t p_begin = wave * npanels / nwaves, p_end = (wave + 1) * npanels / nwaves;
  const int64_t col = li < n_dense ? li : n_dense - 1;          // clamp: the column is never stored
  const uint8_t* bp = b + col * ldb_bytes + lk * 16;
  const uint8_t* av = a_values + (i0 + li) * 64 + lk * 16;
  const uint8_t* am = a_meta + panel_meta_offset(lk * (M_ROW / 4), i0 + li, n_sparse);   // (a panel's further words: n_sparse * 4 bytes apart)
  const int64_t a_step = n_sparse * 64, m_step = n_sparse * M_ROW;
  acc_t acc[2];                              // two chains, so that consecutive instructions do not wait on each other
#pragma unroll
  for (int r = 0; r < 4; r++) { acc[0][r] = 0; acc[1][r] = 0; }
  // two register sets: the loads of the next batch are in flight while the current one is multiplied
  int4v af[2][BATCH], lo[2][BATCH], hi[2][BATCH];
  int idx[2][BATCH];
  auto load_batch = [&](int set, int64_t p) {
#pragma unroll
    for (int u = 0; u < BATCH; u++) {
      const int64_t pp = p + u < p_end ? p + u : p_end - 1;     // past the end: re-read the last panel, multiply by zero
      af[set][u] = __builtin_nontemporal_load(reinterpret_cast<const int4v*>(av + pp * a_step));
      if constexpr (sizeof(T) == 2) idx[set][u] = *reinterpret_cast<const uint16_t*>(am + pp * m_step);
      else idx[set][u] = *reinterpret_cast<const int*>(am + pp * m_step);
      lo[set][u] = *reinterpret_cast<const int4v*>(bp + pp * 128);
      hi[set][u] = *reinterpret_cast<const int4v*>(bp + pp * 128 + 64);
    }
  };
  auto multiply_batch = [&](int set, int64_t p) {
#pragma unroll
    for (int u = 0; u < BATCH; u++) {
      const int4v a = p + u < p_end ? af[set][u] : int4v{0, 0, 0, 0};
      const int8v bfrag = {lo[set][u][0], lo[set][u][1], lo[set][u][2], lo[set][u][3], hi[set][u][0], hi[set][u][1], hi[set][u][2], hi[set][u][3]};
      acc[u & 1] = mma16<T>::template run<0>(a, bfrag, acc[u & 1], idx[set][u]);
    }
  };
  if (p_begin < p_end) load_batch(0, p_begin);
  for (int64_t p = p_begin; p < p_end; p += 2 * BATCH) {
    if (p + BATCH < p_end) load_batch(1, p + BATCH);
    __builtin_amdgcn_sched_barrier(0);       // keep the loads ahead of the instructions that wait for the previous batch
    multiply_batch(0, p);
    __builtin_amdgcn_sched_barrier(0);
    if (p + BATCH < p_end) {
      if (p + 2 * BATCH < p_end) load_batch(0, p + 2 * BATCH);
      __builtin_amdgcn_sched_barrier(0);
      multiply_batch(1, p + BATCH);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  acc_t sum = acc[0] + acc[1];
  if (wave > 0) s_acc[wave - 1][lane] = sum;
  __syncthreads();
  if (wave > 0 || li >= n_dense) return;
#pragma unroll
  for (int w = 0; w < nwaves - 1; w++) sum += s_acc[w][lane];
  const int64_t row = i0 + lk * 4;           // D layout: column l%16, rows 4*(l/16) + r
  OutT o[4];
#pragma unroll
  for (int r = 0; r < 4; r++) o[r] = to_out<OutT>(finish_value(sum[r], scale, bias, row + r, act));
  if constexpr (C_JMAJOR) {
    *reinterpret_cast<Pack<OutT, 4>*>(c + (int64_t)li * ldc + row) = *reinterpret_cast<Pack<OutT, 4>*>(o);
  } else {
#pragma unroll
    for (int r = 0; r < 4; r++) c[(row + r) * ldc + li] = o[r];
  }
}

// Narrow kernel for many sparse rows: the NW (2 or 4) waves of a block own adjacent 16-row blocks and
// share the dense operand through LDS, 16 panels (a chunk) at a time in two buffers, so that the
// only loads of the main loop are the sparse operand's: the one-wave form above sends every wave's
// dense fragments through L1 (twice the requests of its share of the sparse operand), and the
// kernel is bound by the number of requests in flight, not by bytes.  LDS holds
// [panel][column][128 bytes] with the 16-byte pieces of a column XOR-swizzled by column / 2, so the
// 16 lanes that read one piece position of 16 columns hit 16 different bank groups.
// NC = dense columns kept in LDS (8 or 16).
template <typename T, typename OutT, bool C_JMAJOR, int NC, int NW>
__global__ void __launch_bounds__(64 * NW)
spmm_narrow_shared(const uint8_t* __restrict__ a_values, const uint8_t* __restrict__ a_meta, int64_t n_sparse, int64_t k,
                   const uint8_t* __restrict__ b, int64_t ldb_bytes, int64_t n_dense,
                   OutT* __restrict__ c, int64_t ldc, const OutT* __restrict__ bias, float scale, int act) {
  constexpr int KSTEP = mma16<T>::KSTEP;
  constexpr int M_ROW = KSTEP / 8;
  constexpr int CH = 16;                              // panels per chunk
  constexpr int THREADS = 64 * NW;
  constexpr int PIECES = NC * CH * 8 / THREADS;       // 16-byte pieces of the dense chunk per thread (4 to 16)
  using acc_t = typename mma16<T>::acc_t;
  __shared__ __attribute__((aligned(16))) uint8_t s_b[2][CH * NC * 128];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, li = lane & 15, lk = lane >> 4;
  const int64_t blocks16 = n_sparse / 16;
  const int64_t rb = (int64_t)blockIdx.x * NW + wave;
  const bool active = rb < blocks16;
  const int64_t i0 = (active ? rb : blocks16 - 1) * 16;
  const int64_t npanels = k / KSTEP;
  const int nchunks = (int)((npanels + CH - 1) / CH);
  const uint8_t* av = a_values + (i0 + li) * 64 + lk * 16;
  const uint8_t* am = a_meta + panel_meta_offset(lk * (M_ROW / 4), i0 + li, n_sparse);   // (a panel's further words: n_sparse * 4 bytes apart)
  const int64_t a_step = n_sparse * 64, m_step = n_sparse * M_ROW;
  // dense chunk: thread's piece q = tid + THREADS j -> column q / (CH * 8), piece q % (CH * 8) of the column's 2 KB
  const uint8_t* bsrc[PIECES];
  int bdst[PIECES], bwithin[PIECES];
#pragma unroll
  for (int j = 0; j < PIECES; j++) {
    const int q = tid + THREADS * j, col = q / (CH * 8), within = q % (CH * 8);
    const int64_t gcol = col < n_dense ? col : n_dense - 1;
    bsrc[j] = b + gcol * ldb_bytes + within * 16;
    bwithin[j] = within;
    bdst[j] = ((within >> 3) * NC + col) * 128 + (((within & 7) ^ ((col >> 1) & 7)) * 16);
  }
  const int64_t row_bytes = npanels * 128;             // bytes of one dense row
  const int colr = li < n_dense ? li : (int)n_dense - 1;
  const int rd_lo = colr * 128 + ((lk ^ ((colr >> 1) & 7)) * 16), rd_hi = colr * 128 + (((lk + 4) ^ ((colr >> 1) & 7)) * 16);
  acc_t acc[2];
#pragma unroll
  for (int r = 0; r < 4; r++) { acc[0][r] = 0; acc[1][r] = 0; }
  int4v af[2][CH], breg[PIECES];
  int idx[2][CH];
  auto load_a = [&](int set, int chunk) {
#pragma unroll
    for (int u = 0; u < CH; u++) {
      const int64_t p = (int64_t)chunk * CH + u;
      const int64_t pp = p < npanels ? p : npanels - 1;          // past the end: re-read the last panel, multiply by zero
      af[set][u] = __builtin_nontemporal_load(reinterpret_cast<const int4v*>(av + pp * a_step));
      if constexpr (sizeof(T) == 2) idx[set][u] = *reinterpret_cast<const uint16_t*>(am + pp * m_step);
      else idx[set][u] = *reinterpret_cast<const int*>(am + pp * m_step);
    }
  };
  auto load_b = [&](int chunk) {
#pragma unroll
    for (int j = 0; j < PIECES; j++) {
      int64_t off = (int64_t)chunk * (CH * 128) + bwithin[j] * 16;
      if (off > row_bytes - 16) off = row_bytes - 16;             // pieces past k are never multiplied
      breg[j] = *reinterpret_cast<const int4v*>(bsrc[j] - bwithin[j] * 16 + off);
    }
  };
  auto multiply = [&](int set, int chunk) {
    const uint8_t* sb = s_b[set];
#pragma unroll
    for (int u = 0; u < CH; u++) {
      const int4v lo = *reinterpret_cast<const int4v*>(sb + u * NC * 128 + rd_lo);
      const int4v hi = *reinterpret_cast<const int4v*>(sb + u * NC * 128 + rd_hi);
      const int4v a = (int64_t)chunk * CH + u < npanels ? af[set][u] : int4v{0, 0, 0, 0};
      const int8v bfrag = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      acc[u & 1] = mma16<T>::template run<0>(a, bfrag, acc[u & 1], idx[set][u]);
    }
  };
  auto store_b = [&](int set) {
#pragma unroll
    for (int j = 0; j < PIECES; j++) *reinterpret_cast<int4v*>(s_b[set] + bdst[j]) = breg[j];
  };
  load_b(0);
  load_a(0, 0);
  __builtin_amdgcn_sched_barrier(0);
  // one barrier per chunk: a buffer is rewritten two iterations after it was read, and every wave
  // passes the barrier in between only after that read
  for (int ch = 0; ch < nchunks; ch += 2) {
    store_b(0);
    if (ch + 1 < nchunks) { load_b(ch + 1); load_a(1, ch + 1); }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    multiply(0, ch);
    __builtin_amdgcn_sched_barrier(0);
    if (ch + 1 < nchunks) {
      store_b(1);
      if (ch + 2 < nchunks) { load_b(ch + 2); load_a(0, ch + 2); }
      __builtin_amdgcn_sched_barrier(0);
      __syncthreads();
      multiply(1, ch + 1);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if (!active || li >= n_dense) return;
  const acc_t sum = acc[0] + acc[1];
  const int64_t row = i0 + lk * 4;           // D layout: column l%16, rows 4*(l/16) + r
  OutT o[4];
#pragma unroll
  for (int r = 0; r < 4; r++) o[r] = to_out<OutT>(finish_value(sum[r], scale, bias, row + r, act));
  if constexpr (C_JMAJOR) {
    *reinterpret_cast<Pack<OutT, 4>*>(c + (int64_t)li * ldc + row) = *reinterpret_cast<Pack<OutT, 4>*>(o);
  } else {
#pragma unroll
    for (int r = 0; r < 4; r++) c[(row + r) * ldc + li] = o[r];
  }
}

template <typename T, typename OutT>
int launch_narrow(const void* av, const void* am, int64_t n_sparse, int64_t k, const void* b, int64_t ldb, int64_t n_dense,
                  void* c, int c_layout, int64_t ldc, const void* bias, float scale, int act, hipStream_t s) {
  dim3 grid((unsigned)(n_sparse / 16));
  const int64_t blocks = n_sparse / 16, npanels = k * (int64_t)sizeof(T) / 128;
  if (blocks >= 512) {          // enough row blocks: several per workgroup, dense operand through LDS
    const bool jm = c_layout == TF24_COL_MAJOR;
    const int nw = blocks / 4 >= kNarrowSharedMin ? 4 : 2;      // four row blocks per workgroup only if that leaves enough workgroups
    dim3 sgrid((unsigned)((blocks + nw - 1) / nw));
    auto go = [&](auto jmajor, auto nc, auto nwc) {
      hipLaunchKernelGGL((spmm_narrow_shared<T, OutT, decltype(jmajor)::value, decltype(nc)::value, decltype(nwc)::value>), sgrid,
                         dim3(64 * decltype(nwc)::value), 0, s,
                         (const uint8_t*)av, (const uint8_t*)am, n_sparse, k, (const uint8_t*)b, ldb * (int64_t)sizeof(T), n_dense,
                         (OutT*)c, ldc, (const OutT*)bias, scale, act);
    };
    auto go_nw = [&](auto jmajor, auto nc) {
      if (nw == 4) go(jmajor, nc, std::integral_constant<int, 4>{}); else go(jmajor, nc, std::integral_constant<int, 2>{});
    };
    if (n_dense <= 8) { if (jm) go_nw(std::true_type{}, std::integral_constant<int, 8>{}); else go_nw(std::false_type{}, std::integral_constant<int, 8>{}); }
    else { if (jm) go_nw(std::true_type{}, std::integral_constant<int, 16>{}); else go_nw(std::false_type{}, std::integral_constant<int, 16>{}); }
    return check_launch("tf24_spmm");
  }
  int nwaves = kNarrowWaves;                 // few row blocks: the waves of a block split k
  while (nwaves > 1 && npanels / nwaves < 4) nwaves /= 2;
  if (c_layout == TF24_COL_MAJOR)
    hipLaunchKernelGGL((spmm_narrow<T, OutT, true>), grid, dim3(64 * nwaves), 0, s, (const uint8_t*)av, (const uint8_t*)am, n_sparse, k,
                       (const uint8_t*)b, ldb * (int64_t)sizeof(T), n_dense, (OutT*)c, ldc, (const OutT*)bias, scale, act);
  else
    hipLaunchKernelGGL((spmm_narrow<T, OutT, false>), grid, dim3(64 * nwaves), 0, s, (const uint8_t*)av, (const uint8_t*)am, n_sparse, k,
                       (const uint8_t*)b, ldb * (int64_t)sizeof(T), n_dense, (OutT*)c, ldc, (const OutT*)bias, scale, act);
  return check_launch("tf24_spmm");
}

template <typename T, typename OutT>
int launch_general(const void* av, const void* am, int a_layout, int64_t n_sparse, int64_t k, const void* b, int b_layout, int64_t ldb,
                   int64_t n_dense, void* c, int c_layout, int64_t ldc, const void* bias, float scale, int act, hipStream_t s) {
  dim3 grid((unsigned)((n_dense + 63) / 64), (unsigned)((n_sparse + 63) / 64));
  const bool kc = b_layout == TF24_ROW_MAJOR, jm = c_layout == TF24_COL_MAJOR;
#define TF24_GO(KC, JM)                                                                                              \
  hipLaunchKernelGGL((spmm_general<T, OutT, KC, JM>), grid, dim3(256), 0, s, (const uint8_t*)av, (const uint8_t*)am, \
                     n_sparse, k, (const T*)b, ldb, n_dense, (OutT*)c, ldc, (const OutT*)bias, scale, act, a_layout)
  if (kc && jm) TF24_GO(true, true);
  else if (kc) TF24_GO(true, false);
  else if (jm) TF24_GO(false, true);
  else TF24_GO(false, false);
#undef TF24_GO
  return check_launch("tf24_spmm");
}

template <typename T>
int dispatch_out(int out_dtype, const void* av, const void* am, int a_layout, int64_t n_sparse, int64_t k, const void* b, int b_layout,
                 int64_t ldb, int64_t n_dense, void* c, int c_layout, int64_t ldc, const void* bias, float scale, int act,
                 void* workspace, int64_t workspace_bytes, hipStream_t s) {
  const bool panel = a_layout == TF24_COMPRESSED_PANEL;
  // the tiled kernel reads a k-strided dense operand through transposing LDS reads (16-bit types only)
  // (also for a narrow dense operand: with its k pieces the tiled kernel beats the general one from 8 columns on)
  const bool tiled = panel && (b_layout == TF24_ROW_MAJOR || sizeof(T) == 2) && n_sparse >= 64;
  // up to 64 dense columns: the tiled kernel on 256 x 64 tiles; up to 128: on 256 x 128 tiles
  const bool slim = tiled && b_layout == TF24_ROW_MAJOR && n_dense <= SlimCfg::BJ;
  // wider operands that still fit one round of 256 x 128 tiles take those when the estimate below says so
  const int64_t ws_bytes = workspace ? workspace_bytes : 0;
  const bool mid = tiled && b_layout == TF24_ROW_MAJOR &&
                   (n_dense <= MidCfg::BJ ||
                    (tile_cost<T, MidCfg>(n_sparse, k, n_dense, ws_bytes, 0.55).blocks <= 256 &&
                     tile_cost<T, MidCfg>(n_sparse, k, n_dense, ws_bytes, 0.55).us < tile_cost<T, TiledCfg>(n_sparse, k, n_dense, ws_bytes, 0.95).us));
  // at most 8 dense columns: one pass over the compressed operand; up to 16 when the sparse operand
  // has enough rows for the four-row-block form of that kernel (13.0 against 15.7 us on 11008 rows,
  // but 19.7 against 18.6 us on 8192), or when the tiled kernel cannot cut k into pieces (no
  // workspace), which it needs to fill the chip
  const bool narrow = panel && b_layout == TF24_ROW_MAJOR &&
                      (n_dense <= 8 || (n_dense <= kNarrowMaxDense && (n_sparse / 64 >= kNarrowSharedMin || !(slim && workspace))));
  if constexpr (std::is_same<T, i8_t>::value) {        // integer product: int32 accumulators, results and bias
    if (narrow) return launch_narrow<T, int32_t>(av, am, n_sparse, k, b, ldb, n_dense, c, c_layout, ldc, bias, scale, act, s);
    if (slim) return launch_tiled<T, int32_t, SlimCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
    if (mid) return launch_tiled<T, int32_t, MidCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
    if (tiled) return launch_tiled<T, int32_t, TiledCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
    return launch_general<T, int32_t>(av, am, a_layout, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, s);
  } else {
  if (narrow) {
    switch (out_dtype) {
      case TF24_F16: return launch_narrow<T, f16_t>(av, am, n_sparse, k, b, ldb, n_dense, c, c_layout, ldc, bias, scale, act, s);
      case TF24_BF16: return launch_narrow<T, bf16_t>(av, am, n_sparse, k, b, ldb, n_dense, c, c_layout, ldc, bias, scale, act, s);
      case TF24_F32: return launch_narrow<T, float>(av, am, n_sparse, k, b, ldb, n_dense, c, c_layout, ldc, bias, scale, act, s);
    }
  }
  if (slim) {
    switch (out_dtype) {
      case TF24_F16: return launch_tiled<T, f16_t, SlimCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
      case TF24_BF16: return launch_tiled<T, bf16_t, SlimCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
      case TF24_F32: return launch_tiled<T, float, SlimCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
    }
  }
  if (mid) {
    switch (out_dtype) {
      case TF24_F16: return launch_tiled<T, f16_t, MidCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
      case TF24_BF16: return launch_tiled<T, bf16_t, MidCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
      case TF24_F32: return launch_tiled<T, float, MidCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
    }
  }
  if (tiled) {
    switch (out_dtype) {
      case TF24_F16: return launch_tiled<T, f16_t, TiledCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
      case TF24_BF16: return launch_tiled<T, bf16_t, TiledCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
      case TF24_F32: return launch_tiled<T, float, TiledCfg>(av, am, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s);
    }
  }
  switch (out_dtype) {
    case TF24_F16: return launch_general<T, f16_t>(av, am, a_layout, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, s);
    case TF24_BF16: return launch_general<T, bf16_t>(av, am, a_layout, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, s);
    case TF24_F32: return launch_general<T, float>(av, am, a_layout, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_spmm: unsupported output dtype %d", out_dtype);
  }
}

}  // namespace

// One translation unit per operand type instantiates the kernels of that type (spmm_<type>.hip) behind
// one of these functions; tf24_spmm (spmm.hip) validates and dispatches on the type.
#define TF24_SPMM_ENTRY_ARGS int out_dtype, const void* av, const void* am, int a_layout, int64_t n_sparse, int64_t k, const void* b, int b_layout, \
                 int64_t ldb, int64_t n_dense, void* c, int c_layout, int64_t ldc, const void* bias, float scale, int act, \
                 void* workspace, int64_t workspace_bytes, hipStream_t s
#define TF24_SPMM_ENTRY_PASS out_dtype, av, am, a_layout, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, act, workspace, workspace_bytes, s
int spmm_f16(TF24_SPMM_ENTRY_ARGS);
int spmm_bf16(TF24_SPMM_ENTRY_ARGS);
int spmm_e4m3(TF24_SPMM_ENTRY_ARGS);
int spmm_e5m2(TF24_SPMM_ENTRY_ARGS);
int spmm_i8(TF24_SPMM_ENTRY_ARGS);
}  // namespace tf24
