// Mask-driven 2:4 compression of W and of W^T from one read of W and of the mask (gfx950).
//
// The training layer keeps two compressed copies of each weight: W [m,k] compressed along k for
// Y = X.W^T and W^T [k,m] compressed along m for dX = dY.W.  Both come from the same master weight
// and the same (transposable) mask, so one kernel reads them once and writes both.
//
// A 256-lane block owns a tile of TR rows x 128 columns (TR = 64 for 16-bit, 128 for 8-bit
// outputs: one panel of W^T).  Pass 1 walks the tile row-wise exactly like the row-major
// compress kernel: a lane owns 8 consecutive elements of a row (two groups along k), stores its 4
// kept values and merges the metadata byte over 4 lanes; it also leaves every converted element,
// tagged with its keep bit, in an LDS copy of the tile.  Pass 2 walks the LDS tile column-wise:
// 4 adjacent lanes own one column (one row of W^T), TR/4 rows each, so the 16-byte value pieces
// and the metadata of 16 consecutive rows of W^T leave as contiguous runs.
#include <type_traits>

#include "tf24_common.hpp"

namespace tf24 {
namespace {

constexpr int kThreads = 256;

template <typename Out> __device__ __forceinline__ uint32_t bits_of(Out v) { return v.bits; }
template <typename Out> __device__ __forceinline__ Out out_from_bits(uint32_t b) {
  Out o;
  o.bits = (decltype(o.bits))b;
  return o;
}

template <typename In, typename Out, typename MaskT>
__global__ void __launch_bounds__(kThreads)
prune_compress_dual(const In* __restrict__ dense, int64_t ld, int64_t m, int64_t k,
                    const MaskT* __restrict__ mask, int64_t mask_ld,
                    Out* __restrict__ values, uint8_t* __restrict__ meta,
                    Out* __restrict__ values_t, uint8_t* __restrict__ meta_t, bool panel) {
  constexpr int OS = sizeof(Out);
  constexpr int TR = 128 / OS;                      // tile rows: the dense columns of one panel of W^T
  constexpr int TC = 128;                           // tile columns
  constexpr int UPP = (128 / OS) / 8;               // 8-element units per panel row
  constexpr int KEEP = 8 * OS;                      // bit position of the keep flag in a tile element
  using E = std::conditional_t<OS == 2, uint32_t, uint16_t>;   // value bits | keep << KEEP
  constexpr int SW = 32 / (int)sizeof(E);           // columns per 32-byte swizzle unit
  constexpr int RL = TR / 4;                        // rows of W per lane in pass 2 (16 or 32)
  constexpr int NG = RL / 4;                        // groups per lane in pass 2 (4 or 8)
  // Row r of the tile is stored with its columns XORed by (r / RL) * SW: the four lanes of a column
  // in pass 2 read rows RL apart, which would otherwise fall into the same banks.
  __shared__ __attribute__((aligned(16))) E tile[TR * TC];

  const int tid = threadIdx.x;
  const int64_t row0 = (int64_t)blockIdx.y * TR, col0 = (int64_t)blockIdx.x * TC;
  const int64_t upr = k >> 3;

  // ---- pass 1: rows of W
  {
    const int lr0 = tid >> 4, c8 = tid & 15;
    const int64_t col8 = (col0 >> 3) + c8;
    const bool live = col8 < upr;                   // k % 128 == 64 leaves half a tile
#pragma unroll
    for (int it = 0; it < TR / 16; it++) {
      const int lr = it * 16 + lr0;
      const int64_t row = row0 + lr;
      uint32_t mbyte = 0;
      int64_t ounit = 0, ometa = 0;
      if (live) {
        Pack<In, 8> in;
        Pack<MaskT, 8> mk;
        in.load_stream(dense + row * ld + col8 * 8);
        mk.load_stream(mask + row * mask_ld + col8 * 8);
        ounit = panel ? ((col8 / UPP) * m + row) * UPP + col8 % UPP : row * upr + col8;
        ometa = panel ? panel_meta_offset(col8, row, m) : ounit;
        Out cv[8];
        bool kept[8];
#pragma unroll
        for (int i = 0; i < 8; i++) {
          cv[i] = from_float<Out>(to_float(in.v[i]));
          kept[i] = to_float(mk.v[i]) != 0.0f;
        }
        Pack<Out, 4> out;
#pragma unroll
        for (int g = 0; g < 2; g++) {
          const Keep4 keep{kept[4 * g], kept[4 * g + 1], kept[4 * g + 2], kept[4 * g + 3]};
          out.v[2 * g] = keep.first(cv[4 * g], cv[4 * g + 1], cv[4 * g + 2]);
          out.v[2 * g + 1] = keep.second(cv[4 * g + 1], cv[4 * g + 2], cv[4 * g + 3]);
          mbyte |= keep.nibble() << (4 * g);
        }
        out.store_stream(values + ounit * 4);
        Pack<E, 8> e;
#pragma unroll
        for (int i = 0; i < 8; i++) e.v[i] = (E)(bits_of(cv[i]) | (kept[i] ? 1u << KEEP : 0u));
        e.store(tile + lr * TC + ((c8 * 8) ^ ((lr / RL) * SW)));
      }
      // 4 adjacent lanes (32 dense columns of one row) -> one metadata dword
      uint32_t w = mbyte;
      w |= __shfl_down(mbyte, 1) << 8;
      w |= __shfl_down(mbyte, 2) << 16;
      w |= __shfl_down(mbyte, 3) << 24;
      if (live && (tid & 3) == 0) *reinterpret_cast<uint32_t*>(meta + ometa) = w;
    }
  }
  __syncthreads();

  // ---- pass 2: columns of W = rows of W^T [k, m]
  const int64_t vrow_bytes = (m >> 1) * OS, mrow_bytes = m >> 3;
#pragma unroll
  for (int pass = 0; pass < 2; pass++) {
    const int c = pass * 64 + (tid >> 2), q = tid & 3;
    const int64_t trow = col0 + c;
    const bool live = trow < k;
    uint32_t mbits = 0;
    if (live) {
      const int cc = c ^ (q * SW);
      Pack<Out, 2 * NG> o;
#pragma unroll
      for (int g = 0; g < NG; g++) {
        uint32_t e[4];
#pragma unroll
        for (int i = 0; i < 4; i++) e[i] = tile[(q * RL + 4 * g + i) * TC + cc];
        const Keep4 keep{((e[0] >> KEEP) & 1u) != 0, ((e[1] >> KEEP) & 1u) != 0, ((e[2] >> KEEP) & 1u) != 0, ((e[3] >> KEEP) & 1u) != 0};
        o.v[2 * g] = out_from_bits<Out>(keep.first(e[0], e[1], e[2]));
        o.v[2 * g + 1] = out_from_bits<Out>(keep.second(e[1], e[2], e[3]));
        mbits |= keep.nibble() << (4 * g);
      }
      // 16 bytes of kept values: byte offset gbyte of the canonical row; panel p = gbyte / 64 of row
      // trow lives at (p * k + trow) * 64
      const int64_t gbyte = ((row0 + q * RL) >> 1) * OS;
      const int64_t dst = panel ? ((gbyte >> 6) * k + trow) * 64 + (gbyte & 63) : trow * vrow_bytes + gbyte;
      o.store_stream(reinterpret_cast<Out*>(reinterpret_cast<uint8_t*>(values_t) + dst));
    }
    // the 4 lanes of a column hold 8 (16) bytes of metadata between them: two (four) words of 32 columns
    const uint32_t b1 = __shfl_down(mbits, 1), b2 = __shfl_down(mbits, 2), b3 = __shfl_down(mbits, 3);
    if (live && q == 0) {
      const int64_t mbyte0 = row0 >> 3;
      if (panel) {
        if constexpr (OS == 2) {
          *reinterpret_cast<uint32_t*>(meta_t + panel_meta_offset(mbyte0, trow, k)) = mbits | (b1 << 16);
          *reinterpret_cast<uint32_t*>(meta_t + panel_meta_offset(mbyte0 + 4, trow, k)) = b2 | (b3 << 16);
        } else {
          *reinterpret_cast<uint32_t*>(meta_t + panel_meta_offset(mbyte0, trow, k)) = mbits;
          *reinterpret_cast<uint32_t*>(meta_t + panel_meta_offset(mbyte0 + 4, trow, k)) = b1;
          *reinterpret_cast<uint32_t*>(meta_t + panel_meta_offset(mbyte0 + 8, trow, k)) = b2;
          *reinterpret_cast<uint32_t*>(meta_t + panel_meta_offset(mbyte0 + 12, trow, k)) = b3;
        }
      } else {
        uint8_t* dst = meta_t + trow * mrow_bytes + mbyte0;
        if constexpr (OS == 2) *reinterpret_cast<uint2*>(dst) = make_uint2(mbits | (b1 << 16), b2 | (b3 << 16));
        else *reinterpret_cast<uint4*>(dst) = make_uint4(mbits, b1, b2, b3);
      }
    }
  }
}

template <typename In, typename Out, typename MaskT>
int launch(const void* dense, int64_t ld, int64_t m, int64_t k, const void* mask, int64_t mask_ld,
           void* values, void* meta, void* values_t, void* meta_t, bool panel, hipStream_t stream) {
  constexpr int TR = 128 / (int)sizeof(Out);
  dim3 grid((unsigned)((k + 127) / 128), (unsigned)(m / TR));
  hipLaunchKernelGGL((prune_compress_dual<In, Out, MaskT>), grid, dim3(kThreads), 0, stream, (const In*)dense, ld, m, k,
                     (const MaskT*)mask, mask_ld, (Out*)values, (uint8_t*)meta, (Out*)values_t, (uint8_t*)meta_t, panel);
  return check_launch("tf24_prune_compress_dual");
}

template <typename In, typename Out>
int dispatch_mask(int mask_dtype, const void* dense, int64_t ld, int64_t m, int64_t k, const void* mask, int64_t mask_ld,
                  void* values, void* meta, void* values_t, void* meta_t, bool panel, hipStream_t s) {
  switch (mask_dtype) {
    case TF24_U8: return launch<In, Out, uint8_t>(dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
    case TF24_F16: return launch<In, Out, f16_t>(dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
    case TF24_BF16: return launch<In, Out, bf16_t>(dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
    case TF24_F32: return launch<In, Out, float>(dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_prune_compress_dual: unsupported mask dtype %d", mask_dtype);
}

template <typename In>
int dispatch_out(int out_dtype, int mask_dtype, const void* dense, int64_t ld, int64_t m, int64_t k, const void* mask,
                 int64_t mask_ld, void* values, void* meta, void* values_t, void* meta_t, bool panel, hipStream_t s) {
  switch (out_dtype) {
    case TF24_F16: return dispatch_mask<In, f16_t>(mask_dtype, dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
    case TF24_BF16: return dispatch_mask<In, bf16_t>(mask_dtype, dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
    case TF24_E4M3: return dispatch_mask<In, e4m3_t>(mask_dtype, dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
    case TF24_E5M2: return dispatch_mask<In, e5m2_t>(mask_dtype, dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_prune_compress_dual: unsupported output dtype %d", out_dtype);
}

}  // namespace
}  // namespace tf24

extern "C" int tf24_prune_compress_dual(const void* dense, int in_dtype, int64_t ld, int64_t m, int64_t k,
                                        const void* mask, int mask_dtype, int64_t mask_ld,
                                        void* values, void* meta, void* values_t, void* meta_t,
                                        int out_dtype, int out_layout, void* stream) {
  using namespace tf24;
  int rc = tf24_prune_compress_dual_validate(in_dtype, ld, m, k, mask_dtype, mask_ld, out_dtype, out_layout);
  if (rc != TF24_OK) return rc;
  if (!dense || !mask || !values || !meta || !values_t || !meta_t)
    return fail(TF24_ERR_ARG, "tf24_prune_compress_dual: null dense/mask/values/meta pointer");
  if ((rc = check_aligned("tf24_prune_compress_dual", 16, {dense, values, values_t, meta_t, mask_dtype == TF24_U8 ? nullptr : mask}))) return rc;
  if ((rc = check_aligned("tf24_prune_compress_dual", 8, {meta, mask}))) return rc;
  const bool panel = out_layout == TF24_COMPRESSED_PANEL;
  hipStream_t s = (hipStream_t)stream;
  switch (in_dtype) {
    case TF24_F32: return dispatch_out<float>(out_dtype, mask_dtype, dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
    case TF24_F16: return dispatch_out<f16_t>(out_dtype, mask_dtype, dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
    case TF24_BF16: return dispatch_out<bf16_t>(out_dtype, mask_dtype, dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
    case TF24_I8: return dispatch_mask<i8_t, i8_t>(mask_dtype, dense, ld, m, k, mask, mask_ld, values, meta, values_t, meta_t, panel, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_prune_compress_dual: unsupported input dtype %d", in_dtype);
}
