// 2-byte / 1-byte element matrix transpose for gfx950: out[c][r] = in[r][c].
// Serves the matmul when the dense operand arrives with k strided (S @ dense with a row-major
// dense, e.g. dW = MVUE(dY^T) @ x): one pass through a 64 x 64 LDS tile, 128-bit loads and stores.
#include "tf24_common.hpp"

namespace tf24 {
namespace {

template <typename T>
__global__ void __launch_bounds__(256)
transpose_kernel(const T* __restrict__ in, int64_t ld_in, int64_t rows, int64_t cols, T* __restrict__ out, int64_t ld_out) {
  constexpr int V = 16 / sizeof(T);            // elements per 16-byte access
  constexpr int TILE = 64;
  __shared__ T tile[TILE][TILE + V];           // padded rows keep the column reads spread over the banks
  const int64_t r0 = (int64_t)blockIdx.y * TILE, c0 = (int64_t)blockIdx.x * TILE;
  const int tid = threadIdx.x;
  constexpr int LPR = TILE / V;                // lanes per tile row
  constexpr int RPP = 256 / LPR;               // rows per pass
#pragma unroll
  for (int p = 0; p < TILE / RPP; p++) {
    const int r = p * RPP + tid / LPR, cv = (tid % LPR) * V;
    if (r0 + r < rows && c0 + cv < cols) {
      Pack<T, V> v;
      v.load(in + (r0 + r) * ld_in + c0 + cv);
#pragma unroll
      for (int e = 0; e < V; e++) tile[r][cv + e] = v.v[e];
    }
  }
  __syncthreads();
#pragma unroll
  for (int p = 0; p < TILE / RPP; p++) {
    const int c = p * RPP + tid / LPR, rv = (tid % LPR) * V;       // output row c, output columns rv..rv+V
    if (c0 + c < cols && r0 + rv < rows) {
      Pack<T, V> v;
#pragma unroll
      for (int e = 0; e < V; e++) v.v[e] = tile[rv + e][c];
      v.store(out + (c0 + c) * ld_out + r0 + rv);
    }
  }
}

template <typename T>
int launch(const void* in, int64_t ld_in, int64_t rows, int64_t cols, void* out, int64_t ld_out, hipStream_t s) {
  dim3 grid((unsigned)((cols + 63) / 64), (unsigned)((rows + 63) / 64));
  hipLaunchKernelGGL((transpose_kernel<T>), grid, dim3(256), 0, s, (const T*)in, ld_in, rows, cols, (T*)out, ld_out);
  return check_launch("tf24_transpose");
}

}  // namespace
}  // namespace tf24

extern "C" int tf24_transpose(const void* in, int dtype, int64_t ld_in, int64_t rows, int64_t cols, void* out, int64_t ld_out,
                              void* stream) {
  using namespace tf24;
  const int es = dtype_size(dtype);
  const int64_t v = 16 / es;
  if (dtype != TF24_F16 && dtype != TF24_BF16 && !is_8bit(dtype) && dtype != TF24_U8)
    return fail(TF24_ERR_DTYPE, "tf24_transpose: unsupported dtype %d", dtype);
  if (rows <= 0 || cols <= 0 || rows % v || cols % v)
    return fail(TF24_ERR_SHAPE, "tf24_transpose: rows and cols must be positive multiples of %lld", (long long)v);
  if (ld_in < cols || ld_in % v || ld_out < rows || ld_out % v)
    return fail(TF24_ERR_STRIDE, "tf24_transpose: leading dimensions must cover the rows and be multiples of %lld", (long long)v);
  if (!in || !out) return fail(TF24_ERR_ARG, "tf24_transpose: null pointer");
  if (int rc = check_aligned("tf24_transpose", 16, {in, out})) return rc;
  hipStream_t s = (hipStream_t)stream;
  if (es == 2) return launch<uint16_t>(in, ld_in, rows, cols, out, ld_out, s);
  return launch<uint8_t>(in, ld_in, rows, cols, out, ld_out, s);
}
