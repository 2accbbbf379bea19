// Compressed 2:4 -> dense for gfx950.  Lane owns 8 dense outputs (two groups): loads its 4 kept
// values and one metadata byte, stores 8 elements with one vector store.
#include "tf24_common.hpp"
#include <type_traits>

namespace tf24 {
namespace {

constexpr int kThreads = 256;

// canonical: units in row-major order.  panel: a block covers 8 rows x 32 units (a wave 2 rows),
// blocks numbered along k first, so that a wave reads the two rows' adjacent 64-byte pieces of 4
// (2) panels as whole cache lines and writes 512 contiguous bytes per row.
// cutlass (canonical walk only): the metadata is the reference's reordered form.
template <typename T, bool PANEL>
__global__ void __launch_bounds__(kThreads)
decompress_kernel(const T* __restrict__ values, const uint8_t* __restrict__ meta, int64_t total_units, int64_t m, int64_t k,
                  uint32_t chunks, T* __restrict__ dense, bool cutlass) {
  int64_t u, src, msrc;          // dense unit, its place among the values, byte offset of its metadata byte
  if constexpr (PANEL) {        // values [k/KP][m][KP/8 units], metadata [k/32][m][4 bytes]
    constexpr int UPP = (128 / (int)sizeof(T)) / 8;
    const int64_t upr = k >> 3;
    const uint32_t by = blockIdx.x / chunks, bx = blockIdx.x - by * chunks;        // chunks = 32-unit pieces of a row
    const int64_t col8 = (int64_t)bx * 32 + (threadIdx.x & 31), row = (int64_t)by * 8 + (threadIdx.x >> 5);
    if (col8 >= upr || row >= m) return;
    u = row * upr + col8;
    src = ((col8 / UPP) * m + row) * UPP + col8 % UPP;
    msrc = panel_meta_offset(col8, row, m);
  } else {
    u = (int64_t)blockIdx.x * kThreads + threadIdx.x;   // unit = 8 dense elements, row-major order
    if (u >= total_units) return;
    src = u;
    msrc = u;
    if (cutlass) {
      const int64_t upr = k >> 3, row = u / upr;
      msrc = cutlass_meta_offset<sizeof(T) == 2 ? 2 : 4>(u - row * upr, row, m);
    }
  }
  Pack<T, 4> v;
  v.load_stream(values + src * 4);
  const uint32_t mb = meta[msrc];
  Pack<T, 8> out;
#pragma unroll
  for (int i = 0; i < 8; i++) out.v[i] = T{};
#pragma unroll
  for (int g = 0; g < 2; g++) {
    const uint32_t nib = (mb >> (4 * g)) & 0xf;
    const uint32_t p0 = nib & 3, p1 = nib >> 2;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      if (p0 == (uint32_t)i) out.v[4 * g + i] = v.v[2 * g];
      if (p1 == (uint32_t)i) out.v[4 * g + i] = v.v[2 * g + 1];
    }
  }
  out.store_stream(dense + u * 8);
}

template <typename T>
int launch(const void* values, const void* meta, int layout, int64_t m, int64_t k, void* dense, hipStream_t s) {
  const bool panel = layout == TF24_COMPRESSED_PANEL, cutlass = layout == TF24_COMPRESSED_CUTLASS;
  const int64_t total = m * (k / 8);
  if (panel) {
    const int64_t chunks = (k / 8 + 31) / 32, blocks = chunks * ((m + 7) / 8);
    if (blocks > 0x7fffffffLL) return fail(TF24_ERR_SHAPE, "tf24_decompress: matrix too large");
    hipLaunchKernelGGL((decompress_kernel<T, true>), dim3((unsigned)blocks), dim3(kThreads), 0, s, (const T*)values, (const uint8_t*)meta, total, m, k,
                       (uint32_t)chunks, (T*)dense, false);
  } else {
    dim3 grid((unsigned)((total + kThreads - 1) / kThreads));
    hipLaunchKernelGGL((decompress_kernel<T, false>), grid, dim3(kThreads), 0, s, (const T*)values, (const uint8_t*)meta, total, m, k, 0u, (T*)dense, cutlass);
  }
  return check_launch("tf24_decompress");
}

// Canonical <-> panel storage of a compressed operand.  Per row and panel the 64 value bytes are the
// same in both forms, only their place differs; the metadata moves as 4-byte words (canonical: the row's
// words in a row; panel: [k/32][m]).  A block moves 8 rows x
// 8 panels: a wave the values of 2 rows x 8 panels, 16 bytes per lane (canonical side: 512
// contiguous bytes per row; panel side: the two rows' adjacent pieces, one cache line per panel);
// the first wave also the 64 metadata pieces, lane = (row, panel) (64- or 128-byte runs on both sides).
template <int META_BYTES>
__global__ void __launch_bounds__(kThreads)
repack_kernel(const uint8_t* __restrict__ vin, const uint8_t* __restrict__ min_, int64_t m, int64_t panels, uint32_t chunks,
              bool to_panel, uint8_t* __restrict__ vout, uint8_t* __restrict__ mout) {
  const uint32_t by = blockIdx.x / chunks, bx = blockIdx.x - by * chunks;          // chunks = 8-panel pieces of a row
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  {
    const int part = lane & 3;
    const int64_t p = (int64_t)bx * 8 + ((lane >> 2) & 7), row = (int64_t)by * 8 + wave * 2 + (lane >> 5);
    if (p < panels && row < m) {
      const int64_t canon = row * panels + p, panel = p * m + row;
      const int64_t src = to_panel ? canon : panel, dst = to_panel ? panel : canon;
      *reinterpret_cast<uint4*>(vout + dst * 64 + part * 16) = *reinterpret_cast<const uint4*>(vin + src * 64 + part * 16);
    }
  }
  if (wave == 0 && mout) {
    const int64_t p = (int64_t)bx * 8 + (lane & 7), row = (int64_t)by * 8 + (lane >> 3);
    if (p < panels && row < m) {
#pragma unroll
      for (int w = 0; w < META_BYTES / 4; w++) {
        const int64_t canon = (row * panels + p) * META_BYTES + 4 * w, panel = ((p * (META_BYTES / 4) + w) * m + row) * 4;
        const int64_t src = to_panel ? canon : panel, dst = to_panel ? panel : canon;
        *reinterpret_cast<uint32_t*>(mout + dst) = *reinterpret_cast<const uint32_t*>(min_ + src);
      }
    }
  }
}

// Metadata between any two storage forms, one lane per metadata word (WB bytes), lanes walking the
// words in the order of the reordered form ([word-column pair][row][2]: whole cache lines on that side,
// and on the panel side up to a permutation of 32 adjacent rows).
template <int WB>
__global__ void __launch_bounds__(kThreads)
repack_meta_kernel(const uint8_t* __restrict__ min_, int from_layout, int to_layout, int64_t m, int64_t k, uint8_t* __restrict__ mout) {
  using word_t = typename vec_bytes<WB>::type;
  constexpr int G = WB == 2 ? 32 : 16, I = WB == 2 ? 4 : 2;
  const int64_t ncols = k / (8 * WB);
  const int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (t >= m * ncols) return;
  // t = (dc / 2) * 2m + 2 * dr + dc % 2 -> undo the 2 x 2 swap (its own inverse), then the row permutation
  int64_t dr = (t % (2 * m)) >> 1, dc = (t / (2 * m)) * 2 + (t & 1);
  if ((dr & 1) == 0 && (dc & 1) == 1) { dr++; dc--; }
  else if ((dr & 1) == 1 && (dc & 1) == 0) { dr--; dc++; }
  const int64_t q = dr % G;
  const int64_t row = dr / G * G + (q % I) * 8 + q / I;
  const int64_t src = meta_offset<WB>(from_layout, dc * WB, row, m, k), dst = meta_offset<WB>(to_layout, dc * WB, row, m, k);
  *reinterpret_cast<word_t*>(mout + dst) = *reinterpret_cast<const word_t*>(min_ + src);
}

}  // namespace
}  // namespace tf24

extern "C" int tf24_repack_to(const void* values_in, const void* meta_in, int dtype, int64_t m, int64_t k, int from_layout,
                              int to_layout, void* values_out, void* meta_out, void* stream) {
  using namespace tf24;
  const char* fn = "tf24_repack_to";
  auto known = [](int l) { return l == TF24_COMPRESSED_CANONICAL || l == TF24_COMPRESSED_PANEL || l == TF24_COMPRESSED_CUTLASS; };
  if (!known(from_layout) || !known(to_layout) || from_layout == to_layout)
    return fail(TF24_ERR_ARG, "%s: bad pair of compressed layouts (%d -> %d)", fn, from_layout, to_layout);
  if (from_layout != TF24_COMPRESSED_CUTLASS && to_layout != TF24_COMPRESSED_CUTLASS && values_out && meta_out)
    return tf24_repack(values_in, meta_in, dtype, m, k, from_layout, values_out, meta_out, stream);
  if (dtype != TF24_F16 && dtype != TF24_BF16 && !is_8bit(dtype)) return fail(TF24_ERR_DTYPE, "%s: unsupported dtype %d", fn, dtype);
  const int64_t kp = is_8bit(dtype) ? 128 : 64;
  if (from_layout != TF24_COMPRESSED_CUTLASS && to_layout != TF24_COMPRESSED_CUTLASS && values_out && !meta_out) {
    // canonical <-> panel, values only
    if (m <= 0 || k <= 0 || k % kp) return fail(TF24_ERR_SHAPE, "%s: k=%lld must be a positive multiple of %lld", fn, (long long)k, (long long)kp);
    if (!values_in || values_in == values_out) return fail(TF24_ERR_ARG, "%s: null pointer or in-place conversion", fn);
    if (((uintptr_t)values_in | (uintptr_t)values_out) % 16) return fail(TF24_ERR_STRIDE, "%s: values must be 16-byte aligned", fn);
    const int64_t panels = k / kp, chunks = (panels + 7) / 8, vblocks = chunks * ((m + 7) / 8);
    if (vblocks > 0x7fffffffLL) return fail(TF24_ERR_SHAPE, "%s: matrix too large", fn);
    const bool to_panel = to_layout == TF24_COMPRESSED_PANEL;
    if (kp == 128)
      hipLaunchKernelGGL(repack_kernel<16>, dim3((unsigned)vblocks), dim3(kThreads), 0, (hipStream_t)stream, (const uint8_t*)values_in,
                         (const uint8_t*)nullptr, m, panels, (uint32_t)chunks, to_panel, (uint8_t*)values_out, (uint8_t*)nullptr);
    else
      hipLaunchKernelGGL(repack_kernel<8>, dim3((unsigned)vblocks), dim3(kThreads), 0, (hipStream_t)stream, (const uint8_t*)values_in,
                         (const uint8_t*)nullptr, m, panels, (uint32_t)chunks, to_panel, (uint8_t*)values_out, (uint8_t*)nullptr);
    return check_launch(fn);
  }
  if (m <= 0 || m % 32 || k <= 0 || k % kp)
    return fail(TF24_ERR_SHAPE, "%s: shape (%lld, %lld): m must be a positive multiple of 32 and k of %lld", fn, (long long)m, (long long)k, (long long)kp);
  // from here on the metadata moves through the word-by-word kernel: any pair with the reordered form, or metadata alone
  const bool panel_side = from_layout == TF24_COMPRESSED_PANEL || to_layout == TF24_COMPRESSED_PANEL;
  if (!meta_in || !meta_out || (values_out && !values_in)) return fail(TF24_ERR_ARG, "%s: null pointer", fn);
  if (meta_in == meta_out || (values_out && values_in == values_out)) return fail(TF24_ERR_ARG, "%s: in-place conversion is not supported", fn);
  if ((values_out && ((uintptr_t)values_in | (uintptr_t)values_out) % 16) || ((uintptr_t)meta_in | (uintptr_t)meta_out) % 4)
    return fail(TF24_ERR_STRIDE, "%s: values must be 16-byte and metadata 4-byte aligned", fn);
  const int64_t words = m * (k / (is_8bit(dtype) ? 32 : 16)), blocks = (words + kThreads - 1) / kThreads;
  const int64_t panels = k / kp, chunks = (panels + 7) / 8, vblocks = chunks * ((m + 7) / 8);
  if (blocks > 0x7fffffffLL || vblocks > 0x7fffffffLL) return fail(TF24_ERR_SHAPE, "%s: matrix too large", fn);
  hipStream_t s = (hipStream_t)stream;
  if (is_8bit(dtype))
    hipLaunchKernelGGL(repack_meta_kernel<4>, dim3((unsigned)blocks), dim3(kThreads), 0, s, (const uint8_t*)meta_in, from_layout, to_layout, m, k, (uint8_t*)meta_out);
  else
    hipLaunchKernelGGL(repack_meta_kernel<2>, dim3((unsigned)blocks), dim3(kThreads), 0, s, (const uint8_t*)meta_in, from_layout, to_layout, m, k, (uint8_t*)meta_out);
  if (int rc = check_launch(fn)) return rc;
  if (!values_out) return TF24_OK;
  if (panel_side) {        // the values move as between the canonical and the panel form; the metadata pass of that kernel is switched off
    const bool to_panel = to_layout == TF24_COMPRESSED_PANEL;
    if (kp == 128)
      hipLaunchKernelGGL(repack_kernel<16>, dim3((unsigned)vblocks), dim3(kThreads), 0, s, (const uint8_t*)values_in, (const uint8_t*)nullptr,
                         m, panels, (uint32_t)chunks, to_panel, (uint8_t*)values_out, (uint8_t*)nullptr);
    else
      hipLaunchKernelGGL(repack_kernel<8>, dim3((unsigned)vblocks), dim3(kThreads), 0, s, (const uint8_t*)values_in, (const uint8_t*)nullptr,
                         m, panels, (uint32_t)chunks, to_panel, (uint8_t*)values_out, (uint8_t*)nullptr);
    return check_launch(fn);
  }
  const hipError_t e = hipMemcpyAsync(values_out, values_in, (size_t)(m * (k / 2) * dtype_size(dtype)), hipMemcpyDeviceToDevice, s);
  return e == hipSuccess ? TF24_OK : fail(TF24_ERR_LAUNCH, "%s: %s", fn, hipGetErrorString(e));
}

extern "C" int tf24_repack(const void* values_in, const void* meta_in, int dtype, int64_t m, int64_t k, int from_layout,
                           void* values_out, void* meta_out, void* stream) {
  using namespace tf24;
  const char* fn = "tf24_repack";
  if (dtype != TF24_F16 && dtype != TF24_BF16 && !is_8bit(dtype)) return fail(TF24_ERR_DTYPE, "%s: unsupported dtype %d", fn, dtype);
  const int64_t kp = is_8bit(dtype) ? 128 : 64;
  if (m <= 0 || k <= 0 || k % kp) return fail(TF24_ERR_SHAPE, "%s: k=%lld must be a positive multiple of %lld", fn, (long long)k, (long long)kp);
  if (from_layout != TF24_COMPRESSED_CANONICAL && from_layout != TF24_COMPRESSED_PANEL) return fail(TF24_ERR_ARG, "%s: bad compressed layout %d", fn, from_layout);
  if (!values_in || !meta_in || !values_out || !meta_out) return fail(TF24_ERR_ARG, "%s: null pointer", fn);
  if (values_in == values_out || meta_in == meta_out) return fail(TF24_ERR_ARG, "%s: in-place conversion is not supported", fn);
  if (((uintptr_t)values_in | (uintptr_t)values_out) % 16 || ((uintptr_t)meta_in | (uintptr_t)meta_out) % 4)
    return fail(TF24_ERR_STRIDE, "%s: values must be 16-byte and metadata 4-byte aligned", fn);
  const int64_t panels = k / kp, chunks = (panels + 7) / 8, blocks = chunks * ((m + 7) / 8);
  if (blocks > 0x7fffffffLL) return fail(TF24_ERR_SHAPE, "%s: matrix too large", fn);
  const bool to_panel = from_layout == TF24_COMPRESSED_CANONICAL;
  if (kp == 128)
    hipLaunchKernelGGL(repack_kernel<16>, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream, (const uint8_t*)values_in, (const uint8_t*)meta_in,
                       m, panels, (uint32_t)chunks, to_panel, (uint8_t*)values_out, (uint8_t*)meta_out);
  else
    hipLaunchKernelGGL(repack_kernel<8>, dim3((unsigned)blocks), dim3(kThreads), 0, (hipStream_t)stream, (const uint8_t*)values_in, (const uint8_t*)meta_in,
                       m, panels, (uint32_t)chunks, to_panel, (uint8_t*)values_out, (uint8_t*)meta_out);
  return check_launch(fn);
}

extern "C" int tf24_decompress(const void* values, int dtype, const void* meta, int layout, int64_t m, int64_t k,
                               void* dense_out, void* stream) {
  using namespace tf24;
  const int64_t mult = is_8bit(dtype) ? 32 : 16;
  if (m <= 0 || k <= 0 || k % mult) return fail(TF24_ERR_SHAPE, "tf24_decompress: k=%lld must be a positive multiple of %lld", (long long)k, (long long)mult);
  if (!values || !meta || !dense_out) return fail(TF24_ERR_ARG, "tf24_decompress: null pointer");
  if (int rc = check_aligned("tf24_decompress", 16, {values, dense_out})) return rc;
  if (int rc = check_aligned("tf24_decompress", 8, {meta})) return rc;
  if (layout != TF24_COMPRESSED_CANONICAL && layout != TF24_COMPRESSED_PANEL && layout != TF24_COMPRESSED_CUTLASS)
    return fail(TF24_ERR_ARG, "tf24_decompress: bad compressed layout %d", layout);
  const bool panel = layout == TF24_COMPRESSED_PANEL;
  if (panel && k % (is_8bit(dtype) ? 128 : 64)) return fail(TF24_ERR_SHAPE, "tf24_decompress: panel layout needs whole panels (k=%lld)", (long long)k);
  if (layout == TF24_COMPRESSED_CUTLASS && (m % 32 || k % (is_8bit(dtype) ? 64 : 32)))
    return fail(TF24_ERR_SHAPE, "tf24_decompress: the reordered metadata needs m %% 32 == 0 and an even number of metadata words per row (m=%lld, k=%lld)", (long long)m, (long long)k);
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TF24_F16: return launch<f16_t>(values, meta, layout, m, k, dense_out, s);
    case TF24_BF16: return launch<bf16_t>(values, meta, layout, m, k, dense_out, s);
    case TF24_E4M3: return launch<e4m3_t>(values, meta, layout, m, k, dense_out, s);
    case TF24_E5M2: return launch<e5m2_t>(values, meta, layout, m, k, dense_out, s);
    case TF24_I8: return launch<i8_t>(values, meta, layout, m, k, dense_out, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_decompress: unsupported dtype %d", dtype);
}
