// Compressed 2:4 -> dense for gfx950.  Lane owns 8 dense outputs (two groups): loads its 4 kept
// values and one metadata byte, stores 8 elements with one vector store.
#include "tf24_common.hpp"

namespace tf24 {
namespace {

constexpr int kThreads = 256;

template <typename T>
__global__ void __launch_bounds__(kThreads)
decompress_kernel(const T* __restrict__ values, const uint8_t* __restrict__ meta, int64_t total_units, int64_t m, int64_t k,
                  bool panel, T* __restrict__ dense) {
  const int64_t u = (int64_t)blockIdx.x * kThreads + threadIdx.x;   // unit = 8 dense elements, row-major order
  if (u >= total_units) return;
  int64_t src = u;
  if (panel) {        // [k/KP][m][KP/8 units]
    constexpr int UPP = (128 / (int)sizeof(T)) / 8;
    const int64_t upr = k >> 3, row = u / upr, col8 = u - row * upr;
    src = ((col8 / UPP) * m + row) * UPP + col8 % UPP;
  }
  Pack<T, 4> v;
  v.load_stream(values + src * 4);
  const uint32_t mb = meta[src];
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
int launch(const void* values, const void* meta, bool panel, int64_t m, int64_t k, void* dense, hipStream_t s) {
  const int64_t total = m * (k / 8);
  dim3 grid((unsigned)((total + kThreads - 1) / kThreads));
  hipLaunchKernelGGL((decompress_kernel<T>), grid, dim3(kThreads), 0, s, (const T*)values, (const uint8_t*)meta, total, m, k, panel, (T*)dense);
  return check_launch("tf24_decompress");
}

// Canonical <-> panel storage of a compressed operand.  Per row and panel the 64 value bytes and the
// KP/8 metadata bytes are the same in both forms, only their place differs: a lane moves 16 value
// bytes, the first lanes of a row-panel also its metadata.
__global__ void __launch_bounds__(kThreads)
repack_kernel(const uint8_t* __restrict__ vin, const uint8_t* __restrict__ min_, int64_t m, int64_t panels, int meta_bytes,
              bool to_panel, uint8_t* __restrict__ vout, uint8_t* __restrict__ mout) {
  const int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x;   // 4 lanes per (row, panel), canonical order
  const int64_t chunk = t >> 2;
  const int part = (int)(t & 3);
  if (chunk >= m * panels) return;
  const int64_t row = chunk / panels, p = chunk - row * panels;
  const int64_t canon = row * panels + p, panel = p * m + row;
  const int64_t src = to_panel ? canon : panel, dst = to_panel ? panel : canon;
  *reinterpret_cast<uint4*>(vout + dst * 64 + part * 16) = *reinterpret_cast<const uint4*>(vin + src * 64 + part * 16);
  if (part * 8 < meta_bytes)
    *reinterpret_cast<uint2*>(mout + dst * meta_bytes + part * 8) = *reinterpret_cast<const uint2*>(min_ + src * meta_bytes + part * 8);
}

}  // namespace
}  // namespace tf24

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
  if (((uintptr_t)values_in | (uintptr_t)values_out) % 16 || ((uintptr_t)meta_in | (uintptr_t)meta_out) % 8)
    return fail(TF24_ERR_STRIDE, "%s: values must be 16-byte and metadata 8-byte aligned", fn);
  const int64_t panels = k / kp, threads = m * panels * 4;
  dim3 grid((unsigned)((threads + kThreads - 1) / kThreads));
  hipLaunchKernelGGL(repack_kernel, grid, dim3(kThreads), 0, (hipStream_t)stream, (const uint8_t*)values_in, (const uint8_t*)meta_in, m, panels,
                     (int)(kp / 8), from_layout == TF24_COMPRESSED_CANONICAL, (uint8_t*)values_out, (uint8_t*)meta_out);
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
  if (layout != TF24_COMPRESSED_CANONICAL && layout != TF24_COMPRESSED_PANEL) return fail(TF24_ERR_ARG, "tf24_decompress: bad compressed layout %d", layout);
  const bool panel = layout == TF24_COMPRESSED_PANEL;
  if (panel && k % (is_8bit(dtype) ? 128 : 64)) return fail(TF24_ERR_SHAPE, "tf24_decompress: panel layout needs whole panels (k=%lld)", (long long)k);
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TF24_F16: return launch<f16_t>(values, meta, panel, m, k, dense_out, s);
    case TF24_BF16: return launch<bf16_t>(values, meta, panel, m, k, dense_out, s);
    case TF24_E4M3: return launch<e4m3_t>(values, meta, panel, m, k, dense_out, s);
    case TF24_E5M2: return launch<e5m2_t>(values, meta, panel, m, k, dense_out, s);
    case TF24_I8: return launch<i8_t>(values, meta, panel, m, k, dense_out, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_decompress: unsupported dtype %d", dtype);
}
