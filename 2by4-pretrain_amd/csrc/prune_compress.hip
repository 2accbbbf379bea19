// Dense -> 2:4 prune + compress for gfx950 (HBM-bound streaming kernels).
//
// Row-major input: one lane owns 8 consecutive elements (two groups): 128-bit loads for 16-bit
// inputs, 4 kept values leave as one 64-bit (16-bit values) or 32-bit (fp8) store, and the lane's
// metadata byte is merged across 4 lanes with wave shuffles into one 32-bit store.
// Column-major input (W.T, dY.t() views): one lane owns a 4-column x R-row sub-tile (R groups that
// live entirely in its registers), a 256-lane block covers 8R rows x 128 columns, and the
// compressed tile is transposed through LDS so that values and metadata leave row-major with
// full-line stores.
#include <mutex>
#include <type_traits>

#include "tf24_common.hpp"

namespace tf24 {
namespace {

constexpr int kThreads = 256;
// 8-element units per lane of the row-major kernel.  One input stream (magnitude) is fastest with four
// units per lane (37 against 43 us at 8192 x 8192 with one); with a second stream beside it (mask,
// uniforms) one unit per lane and four times the blocks is (MVUE24 82 against 85 us, mask 67 against 71).
template <int MODE> constexpr int unroll_for() { return MODE == TF24_PRUNE_MAGNITUDE ? 4 : 1; }

// The kept elements of one group; in MVUE mode also the inclusion probabilities the two kept
// values are divided by.
template <typename In, int MODE, typename MaskT>
__device__ __forceinline__ Keep4 prune_group(const float (&x)[4], const MaskT* mk, float r0, float r1, Mvue4& g) {
  if constexpr (MODE == TF24_PRUNE_MAGNITUDE) {
    return magnitude_keep4(x[0], x[1], x[2], x[3]);
  } else if constexpr (MODE == TF24_PRUNE_MASK) {
    return Keep4{to_float(mk[0]) != 0.0f, to_float(mk[1]) != 0.0f, to_float(mk[2]) != 0.0f, to_float(mk[3]) != 0.0f};
  } else {
    g = mvue4(x[0], x[1], x[2], x[3], r0, r1);
    return g.keep;
  }
}

// The two values stored for a group: the kept elements in ascending position (MVUE: rescaled).
template <int MODE>
__device__ __forceinline__ void kept_values(const Keep4& keep, const float (&x)[4], const Mvue4& g, float& first, float& second) {
  first = keep.first(x[0], x[1], x[2]);
  second = keep.second(x[1], x[2], x[3]);
  if constexpr (MODE == TF24_PRUNE_MVUE) {
    first = mvue_rescale(first, keep.first(g.p[0], g.p[1], g.p[2]), g.in_range);
    second = mvue_rescale(second, keep.second(g.p[1], g.p[2], g.p[3]), g.in_range);
  }
}

// Panel output of the row-major kernels: the metadata words of a block ([k/32][m][4 bytes]: one word per
// row and 32 dense columns) are collected in LDS as [block of 32 columns][row] and leave as 16-byte
// pieces of four adjacent rows, whole runs of `rows` words per block of columns.  Stored by the quad
// leaders directly they are 4-byte pieces in 16 places per wave instruction, and partial writes of that
// size cost the memory system whole bursts (magnitude, bf16 -> fp16 at 8192 x 8192: 38.6 us; the same
// kernel with canonical output, whose words are contiguous: 34.4).
// words = rows * kblocks metadata words of the block (at most kThreads); rows % 4 == 0.
__device__ __forceinline__ void store_panel_meta_block(const uint32_t* s_words, int rows, int kblocks, int64_t row0, int64_t mbyte0,
                                                       int64_t upr, int64_t m, uint8_t* __restrict__ meta) {
  const int t4 = threadIdx.x * 4;
  if (t4 < rows * kblocks) {
    const int kb = t4 / rows, r = t4 - kb * rows;
    const int64_t mbyte = mbyte0 + (int64_t)kb * 4;
    if (mbyte < upr) {
      const uint4 w = *reinterpret_cast<const uint4*>(s_words + t4);
      *reinterpret_cast<uint4*>(meta + panel_meta_offset(mbyte, row0 + r, m)) = w;
    }
  }
}

// ------------------------------------------------------------------ row-major
// panel = false: canonical output, values [m, k/2] and metadata [m, k/8 bytes] row-major; units
//   (8 dense elements) are walked along rows.
// panel = true : panel output, [k/KP][m][64 bytes] values (KP = 128 / sizeof(Out) dense elements per
//   panel) and [k/32][m][4 bytes] metadata.  A block covers 64 rows x 128 dense columns
//   (32 x 256 when m is not a multiple of 64): 2^lpr_shift lanes read consecutive columns of one row,
//   the other lanes of the wave take the next rows, so that every store instruction writes, per
//   panel, the contiguous 64-byte pieces of 4 (2) adjacent rows.
template <typename In, typename Out, int MODE, typename MaskT>
__global__ void __launch_bounds__(kThreads)
prune_compress_row(const In* __restrict__ dense, int64_t ld, int64_t m, int64_t k,
                   const MaskT* __restrict__ mask, int64_t mask_ld,
                   RandSrc rs,
                   Out* __restrict__ values, uint8_t* __restrict__ meta, bool contiguous, bool panel, int lpr_shift) {
  constexpr int kUnroll = unroll_for<MODE>();
  constexpr int UPP = (128 / (int)sizeof(Out)) / 8;      // units per panel row (8 or 16)
  __shared__ __attribute__((aligned(16))) uint32_t s_words[kUnroll * kThreads / 4];
  const int64_t upr = k >> 3;                             // 8-element units per row
  const int64_t total = m * upr;
  const int64_t base = (int64_t)blockIdx.x * (kThreads * kUnroll) + threadIdx.x;
#pragma unroll
  for (int it = 0; it < kUnroll; it++) {
    const int64_t u = base + (int64_t)it * kThreads;
    bool live = u < total;
    uint32_t mbyte = 0;
    Pack<Out, 4> out;
    int64_t row = 0, col8 = 0, ounit = 0, ometa = 0;       // unit index among the values, byte offset of its metadata byte
    if (panel) {
      const int rpi = kThreads >> lpr_shift;                 // rows per iteration
      // blocks that run together (consecutive blockIdx.x) read neighbouring column ranges of the same rows
      row = (int64_t)blockIdx.y * (kUnroll * rpi) + it * rpi + (threadIdx.x >> lpr_shift);
      col8 = ((int64_t)blockIdx.x << lpr_shift) + (threadIdx.x & ((1 << lpr_shift) - 1));
      live = col8 < upr;                                   // m is a multiple of 32
    }
    if (live) {
      if (panel) {
        ounit = ((col8 / UPP) * m + row) * UPP + col8 % UPP;
        ometa = panel_meta_offset(col8, row, m);
      } else {
        if (contiguous) {          // every leading dimension equals k: offsets are linear in u
          col8 = u;
        } else {
          row = (int64_t)((uint32_t)u / (uint32_t)upr);
          col8 = u - row * upr;
        }
        ounit = row * upr + col8;
        ometa = ounit;
      }
      Pack<In, 8> in;
      in.load_stream(dense + row * ld + col8 * 8);
      Pack<MaskT, 8> mk;
      float r[4] = {0.f, 0.f, 0.f, 0.f};
      if constexpr (MODE == TF24_PRUNE_MASK) mk.load_stream(mask + row * mask_ld + col8 * 8);
      if constexpr (MODE == TF24_PRUNE_MVUE) {
        if (rs.kind == RAND_SEEDED) {
          const Philox4 c = philox4x32_10(rs.seed_now(), (uint64_t)(row * upr + col8), rs.offset_now());
          r[0] = philox_uniform(c.x); r[1] = philox_uniform(c.y); r[2] = philox_uniform(c.z); r[3] = philox_uniform(c.w);
        } else if (rs.kind == RAND_PACKED) {                   // [m, k/2]: the unit's four uniforms are adjacent
          Pack<float, 4> r4;
          r4.load_stream(rs.ptr + row * rs.ld + col8 * 4);
          r[0] = r4.v[0]; r[1] = r4.v[1]; r[2] = r4.v[2]; r[3] = r4.v[3];
        } else {
          const float* rp = rs.ptr + row * rs.ld + col8 * 8;
          Pack<float, 2> ra, rb;                               // the group's two uniforms: the second load meets the first one's line in L1
          ra.load(rp);
          rb.load(rp + 4);
          r[0] = ra.v[0]; r[1] = ra.v[1]; r[2] = rb.v[0]; r[3] = rb.v[1];
        }
      }
#pragma unroll
      for (int g = 0; g < 2; g++) {
        float x[4];
        Mvue4 pr;
#pragma unroll
        for (int i = 0; i < 4; i++) x[i] = to_float(in.v[4 * g + i]);
        const Keep4 keep = prune_group<In, MODE, MaskT>(x, &mk.v[4 * g], r[2 * g], r[2 * g + 1], pr);
        float v0, v1;
        kept_values<MODE>(keep, x, pr, v0, v1);
        out.v[2 * g] = from_float<Out>(v0);
        out.v[2 * g + 1] = from_float<Out>(v1);
        mbyte |= keep.nibble() << (4 * g);
      }
      out.store_stream(values + ounit * 4);
    }
    // 4 adjacent lanes (32 dense columns of one row) -> one metadata dword
    uint32_t w = mbyte;
    w |= __shfl_down(mbyte, 1) << 8;
    w |= __shfl_down(mbyte, 2) << 16;
    w |= __shfl_down(mbyte, 3) << 24;
    if (panel) {
      const int rpi = kThreads >> lpr_shift;
      if ((threadIdx.x & 3) == 0)
        s_words[((threadIdx.x & ((1 << lpr_shift) - 1)) >> 2) * (kUnroll * rpi) + it * rpi + (threadIdx.x >> lpr_shift)] = w;
    } else if (live && (threadIdx.x & 3) == 0) {
      *reinterpret_cast<uint32_t*>(meta + ometa) = w;
    }
  }
  if (panel) {
    __syncthreads();
    const int rows = kUnroll * (kThreads >> lpr_shift);
    store_panel_meta_block(s_words, rows, 1 << (lpr_shift - 2), (int64_t)blockIdx.y * rows, (int64_t)blockIdx.x << lpr_shift, upr, m, meta);
  }
}

// Magnitude mode on 16-bit floats (the weight conversions of the configs): same work assignment and
// outputs as prune_compress_row, with the selection done on the bit patterns (magnitude_top2_16:
// a third of the instructions of the float compares) and the four dense loads of a lane issued
// before the first is used: with one load in flight per wave the kernel is bound by memory latency,
// a wave alternating between waiting for its load and computing.  A unit that holds a NaN is handed
// to the float compares, whose answer for NaN the integer order does not give.
template <typename In, typename Out>
__global__ void __launch_bounds__(kThreads)
prune_compress_row_mag16(const In* __restrict__ dense, int64_t ld, int64_t m, int64_t k,
                         Out* __restrict__ values, uint8_t* __restrict__ meta, bool contiguous, bool panel, int lpr_shift) {
  constexpr int kUnroll = unroll_for<TF24_PRUNE_MAGNITUDE>();
  constexpr int UPP = (128 / (int)sizeof(Out)) / 8;      // units per panel row (8 or 16)
  constexpr uint32_t kInf = std::is_same<In, f16_t>::value ? 0x7c00u : 0x7f80u;
  __shared__ __attribute__((aligned(16))) uint32_t s_words[kUnroll * kThreads / 4];
  const int64_t upr = k >> 3;
  const int64_t total = m * upr;
  const int64_t base = (int64_t)blockIdx.x * (kThreads * kUnroll) + threadIdx.x;
  bool live[kUnroll];
  int64_t ounit[kUnroll], ometa[kUnroll];
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  u32x4 in[kUnroll];
#pragma unroll
  for (int it = 0; it < kUnroll; it++) {
    const int64_t u = base + (int64_t)it * kThreads;
    int64_t row = 0, col8 = u;
    live[it] = u < total;
    if (panel) {
      const int rpi = kThreads >> lpr_shift;
      row = (int64_t)blockIdx.y * (kUnroll * rpi) + it * rpi + (threadIdx.x >> lpr_shift);
      col8 = ((int64_t)blockIdx.x << lpr_shift) + (threadIdx.x & ((1 << lpr_shift) - 1));
      live[it] = col8 < upr;
      ounit[it] = ((col8 / UPP) * m + row) * UPP + col8 % UPP;
      ometa[it] = panel_meta_offset(col8, row, m);
    } else {
      if (!contiguous) {
        row = (int64_t)((uint32_t)u / (uint32_t)upr);
        col8 = u - row * upr;
      }
      ounit[it] = row * upr + col8;
      ometa[it] = ounit[it];
    }
    in[it] = u32x4{0, 0, 0, 0};
    if (live[it]) in[it] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(dense + row * ld + col8 * 8));
  }
#pragma unroll
  for (int it = 0; it < kUnroll; it++) {
    const uint32_t w0 = in[it][0], w1 = in[it][1], w2 = in[it][2], w3 = in[it][3];
    const Top2 t0 = magnitude_top2_16(w0, w1), t1 = magnitude_top2_16(w2, w3);
    uint32_t n0 = t0.nibble, n1 = t1.nibble;
    if (max(t0.top_key, t1.top_key) > ((kInf << 2) | 3u)) {          // a NaN in the unit
      const In* e = reinterpret_cast<const In*>(&in[it]);
      n0 = encode_nibble(magnitude_mask4(to_float(e[0]), to_float(e[1]), to_float(e[2]), to_float(e[3])));
      n1 = encode_nibble(magnitude_mask4(to_float(e[4]), to_float(e[5]), to_float(e[6]), to_float(e[7])));
    }
    const uint32_t r0 = pick16(w0, w1, n0 & 3u), r1 = pick16(w0, w1, n0 >> 2);
    const uint32_t r2 = pick16(w2, w3, n1 & 3u), r3 = pick16(w2, w3, n1 >> 2);
    Pack<Out, 4> out;
    if constexpr (std::is_same<In, Out>::value) {
      uint32_t* o = reinterpret_cast<uint32_t*>(out.v);
      o[0] = (r0 & 0xffffu) | (r1 << 16);
      o[1] = (r2 & 0xffffu) | (r3 << 16);
    } else {
      out.v[0] = from_float<Out>(to_float(In{(uint16_t)r0}));
      out.v[1] = from_float<Out>(to_float(In{(uint16_t)r1}));
      out.v[2] = from_float<Out>(to_float(In{(uint16_t)r2}));
      out.v[3] = from_float<Out>(to_float(In{(uint16_t)r3}));
    }
    if (live[it]) out.store_stream(values + ounit[it] * 4);
    // 4 adjacent lanes (32 dense columns of one row) -> one metadata dword
    const uint32_t mbyte = live[it] ? n0 | (n1 << 4) : 0u;
    uint32_t w = mbyte;
    w |= __shfl_down(mbyte, 1) << 8;
    w |= __shfl_down(mbyte, 2) << 16;
    w |= __shfl_down(mbyte, 3) << 24;
    if (panel) {
      const int rpi = kThreads >> lpr_shift;
      if ((threadIdx.x & 3) == 0)
        s_words[((threadIdx.x & ((1 << lpr_shift) - 1)) >> 2) * (kUnroll * rpi) + it * rpi + (threadIdx.x >> lpr_shift)] = w;
    } else if (live[it] && (threadIdx.x & 3) == 0) {
      *reinterpret_cast<uint32_t*>(meta + ometa[it]) = w;
    }
  }
  if (panel) {
    __syncthreads();
    const int rows = kUnroll * (kThreads >> lpr_shift);
    store_panel_meta_block(s_words, rows, 1 << (lpr_shift - 2), (int64_t)blockIdx.y * rows, (int64_t)blockIdx.x << lpr_shift, upr, m, meta);
  }
}

// Magnitude mode on 16-bit floats into the PANEL layout: a wave owns 4 adjacent rows x 512 columns.  Each of its
// four load instructions reads 1 KB of one row; a lane holds the same 8-column unit of the 4 rows, so the metadata
// words of its quad for the 4 rows are one 16-byte piece of the [k/32][m] word matrix, stored by the quad leader
// as it is.  (64 rows x 128 columns per block with 256-byte reads per row: 37.0 us at 8192 x 8192 bf16 -> fp16;
// this kernel 35.5; the same without the exchange of the values, 64-byte pieces per store: 41.4.)
template <typename In, typename Out>
__global__ void __launch_bounds__(kThreads)
prune_compress_row_mag16_panel(const In* __restrict__ dense, int64_t ld, int64_t m, int64_t k,
                               Out* __restrict__ values, uint8_t* __restrict__ meta) {
  constexpr int UPP = (128 / (int)sizeof(Out)) / 8;      // units per panel row (8 or 16)
  constexpr uint32_t kInf = std::is_same<In, f16_t>::value ? 0x7c00u : 0x7f80u;
  const int64_t upr = k >> 3;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t row0 = (int64_t)blockIdx.y * 16 + wave * 4;
  const int64_t col8 = (int64_t)blockIdx.x * 64 + lane;
  const bool live = col8 < upr;
  typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
  u32x4 in[4];
#pragma unroll
  for (int it = 0; it < 4; it++) {
    in[it] = u32x4{0, 0, 0, 0};
    if (live) in[it] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(dense + (row0 + it) * ld + col8 * 8));
  }
  // values: a lane's four 8-byte pieces are 64 bytes apart in the panel layout; the wave exchanges them through
  // a private LDS slice (rows padded by 128 bytes: both halves of a 64-lane read fall on all banks) so that a
  // store instruction writes, per panel, the 64-byte pieces of the 4 rows: 256 contiguous bytes (two panels, one of 8-bit values)
  using piece_t = typename vec_bytes<4 * sizeof(Out)>::type;        // a unit's 4 kept values: 8 bytes, or 4 for 8-bit values
  constexpr int XROW = 64 + 128 / (int)sizeof(piece_t);
  __shared__ __attribute__((aligned(16))) piece_t s_x[kThreads / 64][4 * XROW];
  uint32_t words[4];
#pragma unroll
  for (int it = 0; it < 4; it++) {
    const uint32_t w0 = in[it][0], w1 = in[it][1], w2 = in[it][2], w3 = in[it][3];
    const Top2 t0 = magnitude_top2_16(w0, w1), t1 = magnitude_top2_16(w2, w3);
    uint32_t n0 = t0.nibble, n1 = t1.nibble;
    if (max(t0.top_key, t1.top_key) > ((kInf << 2) | 3u)) {          // a NaN in the unit
      const In* e = reinterpret_cast<const In*>(&in[it]);
      n0 = encode_nibble(magnitude_mask4(to_float(e[0]), to_float(e[1]), to_float(e[2]), to_float(e[3])));
      n1 = encode_nibble(magnitude_mask4(to_float(e[4]), to_float(e[5]), to_float(e[6]), to_float(e[7])));
    }
    const uint32_t r0 = pick16(w0, w1, n0 & 3u), r1 = pick16(w0, w1, n0 >> 2);
    const uint32_t r2 = pick16(w2, w3, n1 & 3u), r3 = pick16(w2, w3, n1 >> 2);
    Pack<Out, 4> out;
    if constexpr (std::is_same<In, Out>::value) {
      uint32_t* o = reinterpret_cast<uint32_t*>(out.v);
      o[0] = (r0 & 0xffffu) | (r1 << 16);
      o[1] = (r2 & 0xffffu) | (r3 << 16);
    } else {
      out.v[0] = from_float<Out>(to_float(In{(uint16_t)r0}));
      out.v[1] = from_float<Out>(to_float(In{(uint16_t)r1}));
      out.v[2] = from_float<Out>(to_float(In{(uint16_t)r2}));
      out.v[3] = from_float<Out>(to_float(In{(uint16_t)r3}));
    }
    s_x[wave][it * XROW + lane] = *reinterpret_cast<const piece_t*>(out.v);
    const uint32_t mbyte = live ? n0 | (n1 << 4) : 0u;
    uint32_t w = mbyte;
    w |= __shfl_down(mbyte, 1) << 8;
    w |= __shfl_down(mbyte, 2) << 16;
    w |= __shfl_down(mbyte, 3) << 24;
    words[it] = w;
  }
  // lane l' of store instruction i takes row l'/16, unit 16 i + l'%16 (LDS accesses of one wave execute in order: no barrier)
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int r = lane >> 4, u = 16 * i + (lane & 15);
    Pack<Out, 4> v;
    *reinterpret_cast<piece_t*>(v.v) = s_x[wave][r * XROW + u];
    const int64_t c8 = (int64_t)blockIdx.x * 64 + u;
    if (c8 < upr) v.store_stream(values + (((c8 / UPP) * m + row0 + r) * UPP + c8 % UPP) * 4);
  }
  if (live && (lane & 3) == 0)
    *reinterpret_cast<uint4*>(meta + panel_meta_offset(col8, row0, m)) = make_uint4(words[0], words[1], words[2], words[3]);
}

// ------------------------------------------------------------------ column-major
// element (r,c) at c*ld + r.  R = rows per lane = 16 bytes / sizeof(In).
template <typename In, typename Out, int MODE, typename MaskT>
__global__ void __launch_bounds__(kThreads)
prune_compress_col(const In* __restrict__ dense, int64_t ld, int64_t m, int64_t k,
                   const MaskT* __restrict__ mask, int64_t mask_ld,
                   RandSrc rs,
                   Out* __restrict__ values, uint8_t* __restrict__ meta, bool panel,
                   float* __restrict__ rowsum_partial) {
  constexpr int R = 16 / sizeof(In);
  constexpr int TR = 8 * R;          // tile rows
  constexpr int TC = 128;            // tile columns (32 groups)
  constexpr int VPITCH = (TC / 2) * sizeof(Out) + 4;   // bytes per row of the value tile (+1 bank)
  constexpr int MPITCH = TC / 8 + 4;                   // bytes per row of the metadata tile
  __shared__ __attribute__((aligned(16))) uint8_t s_val[TR * VPITCH];
  __shared__ __attribute__((aligned(16))) uint8_t s_meta[TR * MPITCH];
  // Row sums of the dense input (the bias gradient when the input is dY^T): a lane adds its 4
  // columns, the 32 lanes that share a row meet in LDS, the block leaves one float per row in
  // rowsum_partial[column block][row]; a second kernel adds the column blocks.  Fixed order throughout.
  constexpr int SPITCH = TC / 4 + 1;
  __shared__ float s_sum[TR * SPITCH];

  const int tid = threadIdx.x;
  const int rchunk = tid & 7, grp = tid >> 3;           // 8 row chunks x 32 groups
  // consecutive blockIdx.x walk the contiguous (row) dimension of the column-major input
  const int64_t row0 = (int64_t)blockIdx.x * TR, col0 = (int64_t)blockIdx.y * TC;
  const int64_t r0 = row0 + rchunk * R, c0 = col0 + grp * 4;
  float psum[R];
#pragma unroll
  for (int i = 0; i < R; i++) psum[i] = 0.0f;
  // Seeded uniforms: one generator call serves the two groups of an 8-column unit, which two lanes
  // 8 apart own (grp and grp ^ 1).  Each computes the calls of half of the R rows (the even group's
  // lane the first half) and hands the other lane its two words; every lane of the wave takes part.
  Pack<float, R> su[2];
  if constexpr (MODE == TF24_PRUNE_MVUE) {
    if (rs.kind == RAND_SEEDED) {
      const int par = grp & 1;
#pragma unroll
      for (int j = 0; j < R / 2; j++) {
        const int64_t row = r0 + j + par * (R / 2);
        const Philox4 c = philox4x32_10(rs.seed_now(), (uint64_t)(row * (k >> 3) + (c0 >> 3)), rs.offset_now());
        const float own0 = philox_uniform(par ? c.z : c.x), own1 = philox_uniform(par ? c.w : c.y);
        const float snd0 = philox_uniform(par ? c.x : c.z), snd1 = philox_uniform(par ? c.y : c.w);
        const float rcv0 = __shfl_xor(snd0, 8), rcv1 = __shfl_xor(snd1, 8);
        su[0].v[j] = par ? rcv0 : own0;          su[1].v[j] = par ? rcv1 : own1;            // row j
        su[0].v[j + R / 2] = par ? own0 : rcv0;  su[1].v[j + R / 2] = par ? own1 : rcv1;    // row j + R/2
      }
    }
  }
  if (r0 < m && c0 < k) {
    Pack<In, R> in[4];
    Pack<MaskT, R> mk[4];
    Pack<float, R> rr[2];
#pragma unroll
    for (int c = 0; c < 4; c++) in[c].load_stream(dense + (c0 + c) * ld + r0);
    if constexpr (MODE == TF24_PRUNE_MASK) {
#pragma unroll
      for (int c = 0; c < 4; c++) mk[c].load_stream(mask + (c0 + c) * mask_ld + r0);
    }
    if constexpr (MODE == TF24_PRUNE_MVUE) {
      if (rs.kind == RAND_SEEDED) {
        rr[0] = su[0]; rr[1] = su[1];
      } else {
        const int64_t rc = rs.kind == RAND_PACKED ? c0 >> 1 : c0;   // packed: columns 2g, 2g+1 of a [m, k/2] tensor
        rr[0].load_stream(rs.ptr + (rc + 0) * rs.ld + r0);
        rr[1].load_stream(rs.ptr + (rc + 1) * rs.ld + r0);
      }
    }
#pragma unroll
    for (int i = 0; i < R; i++) {
      float x[4];
      Mvue4 pr;
      MaskT mrow[4];
#pragma unroll
      for (int c = 0; c < 4; c++) { x[c] = to_float(in[c].v[i]); if constexpr (MODE == TF24_PRUNE_MASK) mrow[c] = mk[c].v[i]; }
      float u0 = 0.f, u1 = 0.f;
      if constexpr (MODE == TF24_PRUNE_MVUE) { u0 = rr[0].v[i]; u1 = rr[1].v[i]; }
      if (rowsum_partial) psum[i] = (x[0] + x[1]) + (x[2] + x[3]);
      const Keep4 keep = prune_group<In, MODE, MaskT>(x, mrow, u0, u1, pr);
      const uint32_t nib = keep.nibble();
      float v0, v1;
      kept_values<MODE>(keep, x, pr, v0, v1);
      Pack<Out, 2> o;
      o.v[0] = from_float<Out>(v0);
      o.v[1] = from_float<Out>(v1);
      const int lr = rchunk * R + i;
      o.store(reinterpret_cast<Out*>(s_val + lr * VPITCH) + grp * 2);
      // two groups share a metadata byte: even group low nibble, odd group high nibble
      uint32_t other = __shfl_xor(nib, 8);     // lane with grp^1 (same rchunk)
      if ((grp & 1) == 0) s_meta[lr * MPITCH + (grp >> 1)] = (uint8_t)(nib | (other << 4));
    }
  }
  if (rowsum_partial) {
#pragma unroll
    for (int i = 0; i < R; i++) s_sum[(rchunk * R + i) * SPITCH + grp] = psum[i];
  }
  __syncthreads();
  if (rowsum_partial && tid < TR && row0 + tid < m) {
    float t = 0.0f;
    for (int g = 0; g < TC / 4; g++) t += s_sum[tid * SPITCH + g];
    rowsum_partial[(int64_t)blockIdx.y * m + row0 + tid] = t;
  }
  // values: TR rows x (TC/2)*sizeof(Out) bytes, 16 bytes per lane.  Canonical output: row gr, byte
  // offset (col0/2)*sizeof(Out) + seg*16 of a k/2-element row.  Panel output: the tile covers
  // TC/KP panels (KP = 128/sizeof(Out) dense columns, 64 bytes of values per row); panel p of row gr
  // lives at ((p*m + gr)*64) bytes.
  constexpr int VROW_BYTES = (TC / 2) * sizeof(Out);
  constexpr int LANES_PER_ROW = VROW_BYTES / 16;
  constexpr int ROWS_PER_PASS = kThreads / LANES_PER_ROW;
  constexpr int KP = 128 / (int)sizeof(Out);
  const int64_t vpitch_out = (k >> 1) * sizeof(Out);
#pragma unroll
  for (int pass = 0; pass < (TR + ROWS_PER_PASS - 1) / ROWS_PER_PASS; pass++) {
    const int lr = pass * ROWS_PER_PASS + tid / LANES_PER_ROW;
    const int seg = tid % LANES_PER_ROW;
    const int64_t gr = row0 + lr;
    const int64_t gbyte = (col0 >> 1) * sizeof(Out) + seg * 16;
    if (lr < TR && gr < m && gbyte < vpitch_out) {
      // LDS rows are padded by 4 bytes, so read as four dwords
      const uint32_t* sp = reinterpret_cast<const uint32_t*>(s_val + lr * VPITCH + seg * 16);
      uint4 v = make_uint4(sp[0], sp[1], sp[2], sp[3]);
      int64_t dst = gr * vpitch_out + gbyte;
      if (panel) dst = ((gbyte >> 6) * m + gr) * 64 + (gbyte & 63);
      *reinterpret_cast<uint4*>(reinterpret_cast<uint8_t*>(values) + dst) = v;
    }
  }
  // metadata: TR rows x 16 bytes
  if (tid < TR) {
    const int64_t gr = row0 + tid;
    if (gr < m) {
      const uint32_t* sp = reinterpret_cast<const uint32_t*>(s_meta + tid * MPITCH);
      const int64_t mpitch_out = k >> 3;
      const bool full = col0 + TC <= k;                  // k % 128 == 64 leaves a half tile
      if (!panel) {
        uint8_t* dst = meta + gr * mpitch_out + (col0 >> 3);
        // rows of the metadata matrix are only 8-byte aligned when k % 128 == 64
        *reinterpret_cast<uint2*>(dst) = make_uint2(sp[0], sp[1]);
        if (full) *reinterpret_cast<uint2*>(dst + 8) = make_uint2(sp[2], sp[3]);
      } else {
        const int64_t mbyte0 = col0 >> 3;                // byte offset inside the row's canonical stream
#pragma unroll
        for (int w = 0; w < 4; w++)                      // one word per block of 32 columns; consecutive rows are adjacent
          if (w < 2 || full) *reinterpret_cast<uint32_t*>(meta + panel_meta_offset(mbyte0 + 4 * w, gr, m)) = sp[w];
      }
    }
  }
}

// rowsum[r] = sum over column blocks of partial[b][r], one rounding to T.  A block takes 32 rows;
// its 8 groups of 32 lanes each add every 8th column block (coalesced 128-byte reads), then the 8
// group sums of a row are added in group order.
template <typename T>
__global__ void __launch_bounds__(kThreads)
rowsum_finish(const float* __restrict__ partial, int nblocks, int64_t m, T* __restrict__ out) {
  __shared__ float s_part[8][32];
  const int lr = threadIdx.x & 31, part = threadIdx.x >> 5;
  const int64_t r = (int64_t)blockIdx.x * 32 + lr;
  float t = 0.0f;
  if (r < m)
    for (int b = part; b < nblocks; b += 8) t += partial[(int64_t)b * m + r];
  s_part[part][lr] = t;
  __syncthreads();
  if (part == 0 && r < m) {
    float sum = 0.0f;
#pragma unroll
    for (int q = 0; q < 8; q++) sum += s_part[q][lr];
    out[r] = from_float<T>(sum);
  }
}

// {seed, offset} in device memory: offset += by (vector store from one lane)
__global__ void advance_philox_offset(uint64_t* state, uint64_t by) {
  if (threadIdx.x == 0) state[1] += by;
}

template <typename In, typename Out, int MODE, typename MaskT>
int launch(const void* dense, int layout, int64_t ld, int64_t m, int64_t k, const void* mask, int64_t mask_ld,
           RandSrc rs, void* values, void* meta, bool panel, float* rowsum_partial, hipStream_t stream) {
  if (layout == TF24_ROW_MAJOR) {
    constexpr int kUnroll = unroll_for<MODE>();
    const int64_t per_block = kThreads * kUnroll;
    const bool contiguous = ld == k && (MODE != TF24_PRUNE_MASK || mask_ld == k) && (MODE != TF24_PRUNE_MVUE || rs.kind == RAND_SEEDED || rs.ld == (rs.kind == RAND_PACKED ? k / 2 : k));
    const int64_t total = m * (k >> 3);
    dim3 grid((unsigned)((total + per_block - 1) / per_block));
    // lanes per row (log2): 16 lanes read 256 consecutive bytes of bf16 and the four rows of a wave
    // store 256 contiguous bytes per panel (measured best); 32 lanes when m is not a multiple of 64
    const int lpr_shift = m % (kUnroll * (kThreads >> 4)) == 0 ? 4 : 5;
    if (panel) {
      const int rows_per_block = kUnroll * (kThreads >> lpr_shift), units_per_block = 1 << lpr_shift;
      if (m / rows_per_block > 65535)
        return fail(TF24_ERR_SHAPE, "tf24_prune_compress: %lld rows exceed the %lld the panel-output kernel of this mode covers in one launch; "
                    "write the canonical layout and convert it with tf24_repack", (long long)m, (long long)65535 * rows_per_block);
      grid = dim3((unsigned)(((k >> 3) + units_per_block - 1) / units_per_block), (unsigned)(m / rows_per_block));
    }
    if constexpr (MODE == TF24_PRUNE_MAGNITUDE && (std::is_same<In, f16_t>::value || std::is_same<In, bf16_t>::value)) {
      if (panel && m % 16 == 0 && m / 16 <= 65535) {
        dim3 pgrid((unsigned)(((k >> 3) + 63) / 64), (unsigned)(m / 16));
        hipLaunchKernelGGL((prune_compress_row_mag16_panel<In, Out>), pgrid, dim3(kThreads), 0, stream, (const In*)dense, ld, m, k, (Out*)values, (uint8_t*)meta);
        return check_launch("tf24_prune_compress");
      }
      hipLaunchKernelGGL((prune_compress_row_mag16<In, Out>), grid, dim3(kThreads), 0, stream,
                         (const In*)dense, ld, m, k, (Out*)values, (uint8_t*)meta, contiguous, panel, lpr_shift);
    } else {
      hipLaunchKernelGGL((prune_compress_row<In, Out, MODE, MaskT>), grid, dim3(kThreads), 0, stream,
                         (const In*)dense, ld, m, k, (const MaskT*)mask, mask_ld, rs, (Out*)values, (uint8_t*)meta,
                         contiguous, panel, lpr_shift);
    }
  } else {
    constexpr int R = 16 / sizeof(In);
    dim3 grid((unsigned)((m + 8 * R - 1) / (8 * R)), (unsigned)((k + 127) / 128));
    hipLaunchKernelGGL((prune_compress_col<In, Out, MODE, MaskT>), grid, dim3(kThreads), 0, stream,
                       (const In*)dense, ld, m, k, (const MaskT*)mask, mask_ld, rs, (Out*)values, (uint8_t*)meta, panel,
                       rowsum_partial);
  }
  return check_launch("tf24_prune_compress");
}

template <typename In, typename Out, int MODE>
int dispatch_mask(const void* dense, int layout, int64_t ld, int64_t m, int64_t k, const void* mask, int mask_dtype,
                  int64_t mask_ld, RandSrc rs, void* values, void* meta, bool panel, float* rowsum_partial, hipStream_t s) {
  if constexpr (MODE != TF24_PRUNE_MASK) {
    return launch<In, Out, MODE, uint8_t>(dense, layout, ld, m, k, nullptr, 0, rs, values, meta, panel, rowsum_partial, s);
  } else if constexpr (std::is_same<In, i8_t>::value) {
    // int8 matrices take byte masks only (the column kernel reads 16 rows per lane: 16-byte mask loads)
    if (mask_dtype != TF24_U8) return fail(TF24_ERR_DTYPE, "tf24_prune_compress: int8 input takes a byte mask (dtype %d given)", mask_dtype);
    return launch<In, Out, MODE, uint8_t>(dense, layout, ld, m, k, mask, mask_ld, rs, values, meta, panel, rowsum_partial, s);
  } else {
    switch (mask_dtype) {
      case TF24_U8: return launch<In, Out, MODE, uint8_t>(dense, layout, ld, m, k, mask, mask_ld, rs, values, meta, panel, rowsum_partial, s);
      case TF24_F16: return launch<In, Out, MODE, f16_t>(dense, layout, ld, m, k, mask, mask_ld, rs, values, meta, panel, rowsum_partial, s);
      case TF24_BF16: return launch<In, Out, MODE, bf16_t>(dense, layout, ld, m, k, mask, mask_ld, rs, values, meta, panel, rowsum_partial, s);
      case TF24_F32: return launch<In, Out, MODE, float>(dense, layout, ld, m, k, mask, mask_ld, rs, values, meta, panel, rowsum_partial, s);
    }
    return fail(TF24_ERR_DTYPE, "tf24_prune_compress: unsupported mask dtype %d", mask_dtype);
  }
}

template <typename In, typename Out>
int dispatch_mode(int mode, const void* dense, int layout, int64_t ld, int64_t m, int64_t k, const void* mask,
                  int mask_dtype, int64_t mask_ld, RandSrc rs, void* values, void* meta, bool panel, float* rowsum_partial, hipStream_t s) {
  switch (mode) {
    case TF24_PRUNE_MAGNITUDE:
      return dispatch_mask<In, Out, TF24_PRUNE_MAGNITUDE>(dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s);
    case TF24_PRUNE_MASK:
      return dispatch_mask<In, Out, TF24_PRUNE_MASK>(dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s);
    case TF24_PRUNE_MVUE:
    case TF24_PRUNE_MVUE_PACKED:
    case TF24_PRUNE_MVUE_SEEDED:
    case TF24_PRUNE_MVUE_SEEDED_DEVICE:
      if constexpr (std::is_same<Out, i8_t>::value) break;        // refused by the validator
      else return dispatch_mask<In, Out, TF24_PRUNE_MVUE>(dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s);
  }
  return fail(TF24_ERR_ARG, "tf24_prune_compress: bad mode %d", mode);
}

template <typename In>
int dispatch_out(int out_dtype, int mode, const void* dense, int layout, int64_t ld, int64_t m, int64_t k, const void* mask,
                 int mask_dtype, int64_t mask_ld, RandSrc rs, void* values, void* meta, bool panel, float* rowsum_partial, hipStream_t s) {
  switch (out_dtype) {
    case TF24_F16: return dispatch_mode<In, f16_t>(mode, dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s);
    case TF24_BF16: return dispatch_mode<In, bf16_t>(mode, dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s);
    case TF24_E4M3: return dispatch_mode<In, e4m3_t>(mode, dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s);
    case TF24_E5M2: return dispatch_mode<In, e5m2_t>(mode, dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_prune_compress: unsupported output dtype %d", out_dtype);
}

}  // namespace
}  // namespace tf24

namespace tf24 {
namespace {

int run_prune_compress(const char* fn, const void* dense, int in_dtype, int layout, int64_t ld, int64_t m, int64_t k,
                       int mode, const void* mask, int mask_dtype, int64_t mask_ld, const float* rnd, int64_t rand_ld,
                       void* values, int out_dtype, void* meta, int out_layout, float* rowsum_partial, void* stream) {
  int rc = tf24_prune_compress_validate(in_dtype, layout, ld, m, k, mode, mask != nullptr, mask_dtype, mask_ld,
                                        rnd != nullptr, rand_ld, out_dtype);
  if (rc != TF24_OK) return rc;
  if (!dense || !values || !meta) return fail(TF24_ERR_ARG, "%s: null dense/values/meta pointer", fn);
  if ((rc = check_aligned(fn, 16, {dense, (mode == TF24_PRUNE_MVUE_SEEDED || mode == TF24_PRUNE_MVUE_SEEDED_DEVICE) ? nullptr : rnd, values, mask_dtype == TF24_U8 ? nullptr : mask}))) return rc;
  if ((rc = check_aligned(fn, 8, {meta, mask}))) return rc;
  if (out_layout != TF24_COMPRESSED_CANONICAL && out_layout != TF24_COMPRESSED_PANEL)
    return fail(TF24_ERR_ARG, "%s: bad compressed layout %d", fn, out_layout);
  // panel metadata leaves (and is later copied to LDS by the matmul) in 16-byte pieces
  if (out_layout == TF24_COMPRESSED_PANEL && (rc = check_aligned(fn, 16, {meta}))) return rc;
  const bool panel = out_layout == TF24_COMPRESSED_PANEL;
  RandSrc rs{rnd, rand_ld, mode == TF24_PRUNE_MVUE_PACKED ? RAND_PACKED : RAND_FULL, 0, 0, nullptr};
  if (mode == TF24_PRUNE_MVUE_SEEDED) {          // `rand` points to {seed, offset} in host memory
    const uint64_t* so = reinterpret_cast<const uint64_t*>(rnd);
    rs = RandSrc{nullptr, 0, RAND_SEEDED, so[0], so[1], nullptr};
  } else if (mode == TF24_PRUNE_MVUE_SEEDED_DEVICE) {   // ... in device memory, read by the kernel
    if ((rc = check_aligned(fn, 8, {rnd}))) return rc;
    rs = RandSrc{nullptr, 0, RAND_SEEDED, 0, 0, reinterpret_cast<const uint64_t*>(rnd)};
  }
  hipStream_t s = (hipStream_t)stream;
  rc = fail(TF24_ERR_DTYPE, "%s: unsupported input dtype %d", fn, in_dtype);
  switch (in_dtype) {
    case TF24_F32: rc = dispatch_out<float>(out_dtype, mode, dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s); break;
    case TF24_F16: rc = dispatch_out<f16_t>(out_dtype, mode, dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s); break;
    case TF24_BF16: rc = dispatch_out<bf16_t>(out_dtype, mode, dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s); break;
    case TF24_I8: rc = dispatch_mode<i8_t, i8_t>(mode, dense, layout, ld, m, k, mask, mask_dtype, mask_ld, rs, values, meta, panel, rowsum_partial, s); break;
  }
  if (rc == TF24_OK && mode == TF24_PRUNE_MVUE_SEEDED_DEVICE) {
    // the generator state moves on behind the conversion, in stream order: the next sampling call (or the
    // next replay of a graph holding this one) draws from a fresh offset
    hipLaunchKernelGGL(advance_philox_offset, dim3(1), dim3(64), 0, s, const_cast<uint64_t*>(rs.state), (uint64_t)4);
    rc = check_launch(fn);
  }
  return rc;
}

}  // namespace
}  // namespace tf24

extern "C" int tf24_prune_compress(const void* dense, int in_dtype, int layout, int64_t ld, int64_t m, int64_t k,
                                   int mode, const void* mask, int mask_dtype, int64_t mask_ld,
                                   const float* rnd, int64_t rand_ld,
                                   void* values, int out_dtype, void* meta, int out_layout, void* stream) {
  return tf24::run_prune_compress("tf24_prune_compress", dense, in_dtype, layout, ld, m, k, mode, mask, mask_dtype, mask_ld, rnd, rand_ld,
                                  values, out_dtype, meta, out_layout, nullptr, stream);
}

extern "C" int64_t tf24_prune_compress_rowsum_workspace_bytes(int64_t m, int64_t k) {
  return m > 0 && k > 0 ? ((k + 127) / 128) * m * (int64_t)sizeof(float) : 0;
}

extern "C" int tf24_prune_compress_rowsum(const void* dense, int in_dtype, int layout, int64_t ld, int64_t m, int64_t k,
                                          int mode, const void* mask, int mask_dtype, int64_t mask_ld,
                                          const float* rnd, int64_t rand_ld,
                                          void* values, int out_dtype, void* meta, int out_layout,
                                          void* rowsum, int rowsum_dtype, void* workspace, int64_t workspace_bytes, void* stream) {
  using namespace tf24;
  const char* fn = "tf24_prune_compress_rowsum";
  if (layout != TF24_COL_MAJOR)
    return fail(TF24_ERR_ARG, "%s: row sums are produced for column-major input only (a row of a row-major matrix is contiguous: sum it directly)", fn);
  if (in_dtype == TF24_I8) return fail(TF24_ERR_DTYPE, "%s: int8 input is not supported", fn);
  if (rowsum_dtype != TF24_F32 && rowsum_dtype != TF24_F16 && rowsum_dtype != TF24_BF16)
    return fail(TF24_ERR_DTYPE, "%s: unsupported row-sum dtype %d", fn, rowsum_dtype);
  if (!rowsum || !workspace) return fail(TF24_ERR_ARG, "%s: null rowsum/workspace pointer", fn);
  if (workspace_bytes < tf24_prune_compress_rowsum_workspace_bytes(m, k))
    return fail(TF24_ERR_ARG, "%s: workspace of %lld bytes is too small (%lld needed)", fn, (long long)workspace_bytes,
                (long long)tf24_prune_compress_rowsum_workspace_bytes(m, k));
  int rc = check_aligned(fn, 4, {workspace});
  if (rc) return rc;
  if ((rc = check_aligned(fn, dtype_size(rowsum_dtype), {rowsum}))) return rc;
  rc = run_prune_compress(fn, dense, in_dtype, layout, ld, m, k, mode, mask, mask_dtype, mask_ld, rnd, rand_ld, values, out_dtype, meta,
                          out_layout, (float*)workspace, stream);
  if (rc) return rc;
  const int nblocks = (int)((k + 127) / 128);
  dim3 grid((unsigned)((m + 31) / 32));
  hipStream_t s = (hipStream_t)stream;
  switch (rowsum_dtype) {
    case TF24_F32: hipLaunchKernelGGL((rowsum_finish<float>), grid, dim3(kThreads), 0, s, (const float*)workspace, nblocks, m, (float*)rowsum); break;
    case TF24_F16: hipLaunchKernelGGL((rowsum_finish<f16_t>), grid, dim3(kThreads), 0, s, (const float*)workspace, nblocks, m, (f16_t*)rowsum); break;
    default: hipLaunchKernelGGL((rowsum_finish<bf16_t>), grid, dim3(kThreads), 0, s, (const float*)workspace, nblocks, m, (bf16_t*)rowsum); break;
  }
  return check_launch(fn);
}

// ------------------------------------------------------------------------------------------
// tf24_prune_compress_rowsum without a caller workspace: the partial row sums go to a fixed array in
// the library's own device image.  Each GPU the library runs on holds its own copy of the array (at
// its own address) until the process ends.
// ------------------------------------------------------------------------------------------
namespace tf24 {
namespace {

constexpr int64_t kRowsumScratchFloats = (int64_t)1 << 20;          // 4 MiB: m * ceil(k / 128) <= 2^20
static __device__ __align__(256) float scratch[kRowsumScratchFloats];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
float* g_scratch_ptr[kMaxDevices];                                   // device address of `scratch`, per device

// Device address of `scratch` on the current device (looked up once per device; in host code the
// array's name is only a handle for this lookup, never a device address).
int scratch_address(const char* fn, float** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(TF24_ERR_LAUNCH, "%s: cannot identify the current device (%d)", fn, dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    float* p = nullptr;
    const hipError_t e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fail(TF24_ERR_LAUNCH, "%s: hipGetSymbolAddress failed: %s", fn, hipGetErrorString(e));
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return TF24_OK;
}

}  // namespace
}  // namespace tf24

extern "C" int64_t tf24_prune_compress_rowsum_static_max_bytes(void) {
  return tf24::kRowsumScratchFloats * (int64_t)sizeof(float);
}

extern "C" int tf24_prune_compress_rowsum_static(const void* dense, int in_dtype, int layout, int64_t ld, int64_t m, int64_t k,
                                                 int mode, const void* mask, int mask_dtype, int64_t mask_ld,
                                                 const float* rnd, int64_t rand_ld,
                                                 void* values, int out_dtype, void* meta, int out_layout,
                                                 void* rowsum, int rowsum_dtype, void* stream) {
  using namespace tf24;
  const char* fn = "tf24_prune_compress_rowsum_static";
  const int64_t need = tf24_prune_compress_rowsum_workspace_bytes(m, k);
  if (need > tf24_prune_compress_rowsum_static_max_bytes())
    return fail(TF24_ERR_SHAPE, "%s: a %lld x %lld matrix needs %lld bytes of partial sums, the built-in scratch holds %lld "
                "(m * ceil(k / 128) <= %lld); use tf24_prune_compress_rowsum with a workspace", fn, (long long)m, (long long)k,
                (long long)need, (long long)tf24_prune_compress_rowsum_static_max_bytes(), (long long)kRowsumScratchFloats);
  float* ptr = nullptr;
  if (int rc = scratch_address(fn, &ptr)) return rc;
  // every partial sum the second kernel reads is written by the first one: nothing has to start at zero
  return tf24_prune_compress_rowsum(dense, in_dtype, layout, ld, m, k, mode, mask, mask_dtype, mask_ld, rnd, rand_ld, values, out_dtype,
                                    meta, out_layout, rowsum, rowsum_dtype, ptr, tf24_prune_compress_rowsum_static_max_bytes(), stream);
}

namespace tf24 {
namespace {

// one lane per generator call: the four packed uniforms of an 8-column unit
__global__ void __launch_bounds__(kThreads)
mvue_uniforms_kernel(uint64_t seed, uint64_t offset, int64_t m, int64_t upr, bool col_major, float* __restrict__ out, int64_t ld) {
  const int64_t u = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (u >= m * upr) return;
  const int64_t row = u / upr, unit = u - row * upr;
  const Philox4 c = philox4x32_10(seed, (uint64_t)u, offset);
  const float v[4] = {philox_uniform(c.x), philox_uniform(c.y), philox_uniform(c.z), philox_uniform(c.w)};
  if (col_major) {
#pragma unroll
    for (int i = 0; i < 4; i++) out[(unit * 4 + i) * ld + row] = v[i];
  } else {
#pragma unroll
    for (int i = 0; i < 4; i++) out[row * ld + unit * 4 + i] = v[i];
  }
}

}  // namespace
}  // namespace tf24

extern "C" int tf24_mvue_uniforms(uint64_t seed, uint64_t offset, int64_t m, int64_t k, int layout, float* out, int64_t ld,
                                  void* stream) {
  using namespace tf24;
  const char* fn = "tf24_mvue_uniforms";
  if (m <= 0 || k <= 0 || k % 8) return fail(TF24_ERR_SHAPE, "%s: shape (%lld, %lld): k must be a positive multiple of 8", fn, (long long)m, (long long)k);
  if (layout != TF24_ROW_MAJOR && layout != TF24_COL_MAJOR) return fail(TF24_ERR_ARG, "%s: bad layout %d", fn, layout);
  if (ld < (layout == TF24_ROW_MAJOR ? k / 2 : m)) return fail(TF24_ERR_STRIDE, "%s: leading dimension %lld too small", fn, (long long)ld);
  if (!out) return fail(TF24_ERR_ARG, "%s: null pointer", fn);
  if (int rc = check_aligned(fn, 4, {out})) return rc;
  const int64_t total = m * (k / 8);
  if (total > (int64_t)0x7fffffff * kThreads) return fail(TF24_ERR_SHAPE, "%s: matrix too large", fn);
  dim3 grid((unsigned)((total + kThreads - 1) / kThreads));
  hipLaunchKernelGGL(mvue_uniforms_kernel, grid, dim3(kThreads), 0, (hipStream_t)stream, seed, offset, m, k / 8,
                     layout == TF24_COL_MAJOR, out, ld);
  return check_launch(fn);
}
