// Dense-shaped 2:4 operators for gfx950: S-STE soft threshold, magnitude pruning, MVUE24.
// Outputs have the input's dtype and layout and are written completely (zeros at dropped
// positions), so no separate memset pass exists: 128-bit loads, 128-bit stores, one pass.
#include "tf24_common.hpp"

namespace tf24 {
namespace {

constexpr int kThreads = 256;
enum { OP_SOFT = 0, OP_SPARSE24 = 1, OP_MVUE = 2 };

// One group: inputs x[4] (float32), outputs y[4] (value to store where kept) and mask bits.
template <int OP>
__device__ __forceinline__ uint32_t group_op(const float (&x)[4], float r0, float r1, float (&y)[4]) {
  if constexpr (OP == OP_MVUE) {
    // only the two kept values are rescaled; with fewer than two mask bits the kept element is
    // still one of the two encoded positions
    const Mvue4 g = mvue4(x[0], x[1], x[2], x[3], r0, r1);
    const uint32_t pa = g.keep.nibble() & 3;
    const float ya = mvue_rescale(g.keep.first(x[0], x[1], x[2]), g.keep.first(g.p[0], g.p[1], g.p[2]), g.in_range);
    const float yb = mvue_rescale(g.keep.second(x[1], x[2], x[3]), g.keep.second(g.p[1], g.p[2], g.p[3]), g.in_range);
#pragma unroll
    for (int i = 0; i < 4; i++) y[i] = (uint32_t)i == pa ? ya : yb;
    return g.keep.bits();
  } else {
    uint32_t mb = magnitude_mask4(x[0], x[1], x[2], x[3]);
    if constexpr (OP == OP_SOFT) {
      float a0 = __builtin_fabsf(x[0]), a1 = __builtin_fabsf(x[1]), a2 = __builtin_fabsf(x[2]), a3 = __builtin_fabsf(x[3]);
      // second smallest magnitude of the four
      float thr = fminf(fmaxf(fminf(a0, a1), fminf(a2, a3)), fminf(fmaxf(a0, a1), fmaxf(a2, a3)));
#pragma unroll
      for (int i = 0; i < 4; i++) y[i] = x[i] > 0.0f ? x[i] - thr : x[i] + thr;
    } else {
#pragma unroll
      for (int i = 0; i < 4; i++) y[i] = x[i];
    }
    return mb;
  }
}

template <typename T> __device__ __forceinline__ T zero_of() { return from_float<T>(0.0f); }
template <typename T> __device__ __forceinline__ T one_of() { return from_float<T>(1.0f); }

// Row-major: lane owns 8 consecutive elements of one row.
template <typename T, int OP>
__global__ void __launch_bounds__(kThreads)
dense_op_row(const T* __restrict__ dense, int64_t ld, int64_t m, int64_t k, const float* __restrict__ rnd, int64_t rand_ld,
             T* __restrict__ sparse, T* __restrict__ mask) {
  // blocks are numbered along the row first: blocks that run together read neighbouring pieces of one row
  const uint32_t chunks = (uint32_t)((k / 8 + kThreads - 1) / kThreads);
  const int64_t row = blockIdx.x / chunks;
  const int64_t col8 = (int64_t)(blockIdx.x - (uint32_t)row * chunks) * kThreads + threadIdx.x;
  if (col8 * 8 >= k) return;
  const int64_t off = row * ld + col8 * 8;
  Pack<T, 8> in, so, mo;
  in.load_stream(dense + off);
  float r[4] = {0.f, 0.f, 0.f, 0.f};
  if constexpr (OP == OP_MVUE) {
    const float* rp = rnd + row * rand_ld + col8 * 8;
    Pack<float, 2> ra, rb;
    ra.load_stream(rp);
    rb.load_stream(rp + 4);
    r[0] = ra.v[0]; r[1] = ra.v[1]; r[2] = rb.v[0]; r[3] = rb.v[1];
  }
#pragma unroll
  for (int g = 0; g < 2; g++) {
    float x[4], y[4];
#pragma unroll
    for (int i = 0; i < 4; i++) x[i] = to_float(in.v[4 * g + i]);
    uint32_t mb = group_op<OP>(x, r[2 * g], r[2 * g + 1], y);
#pragma unroll
    for (int i = 0; i < 4; i++) {
      bool keep = (mb >> i) & 1;
      so.v[4 * g + i] = keep ? from_float<T>(y[i]) : zero_of<T>();
      mo.v[4 * g + i] = keep ? one_of<T>() : zero_of<T>();
    }
  }
  so.store_stream(sparse + off);
  if (mask) mo.store_stream(mask + off);
}

// Column-major: element (r,c) at c*ld + r.  Lane owns a 4-column x R-row sub-tile (R = 16 bytes of T).
template <typename T, int OP>
__global__ void __launch_bounds__(kThreads)
dense_op_col(const T* __restrict__ dense, int64_t ld, int64_t m, int64_t k, const float* __restrict__ rnd, int64_t rand_ld,
             T* __restrict__ sparse, T* __restrict__ mask) {
  constexpr int R = 16 / sizeof(T);
  // blocks are numbered along the contiguous (row) dimension first
  const uint32_t chunks = (uint32_t)((m / R + kThreads - 1) / kThreads);
  const int64_t grp = blockIdx.x / chunks;
  const int64_t r0 = ((int64_t)(blockIdx.x - (uint32_t)grp * chunks) * kThreads + threadIdx.x) * R;
  const int64_t c0 = grp * 4;
  if (r0 >= m) return;
  Pack<T, R> in[4], so[4], mo[4];
  Pack<float, R> rr[2];
#pragma unroll
  for (int c = 0; c < 4; c++) in[c].load_stream(dense + (c0 + c) * ld + r0);
  if constexpr (OP == OP_MVUE) {
    rr[0].load_stream(rnd + (c0 + 0) * rand_ld + r0);
    rr[1].load_stream(rnd + (c0 + 1) * rand_ld + r0);
  }
#pragma unroll
  for (int i = 0; i < R; i++) {
    float x[4], y[4];
#pragma unroll
    for (int c = 0; c < 4; c++) x[c] = to_float(in[c].v[i]);
    float u0 = 0.f, u1 = 0.f;
    if constexpr (OP == OP_MVUE) { u0 = rr[0].v[i]; u1 = rr[1].v[i]; }
    uint32_t mb = group_op<OP>(x, u0, u1, y);
#pragma unroll
    for (int c = 0; c < 4; c++) {
      bool keep = (mb >> c) & 1;
      so[c].v[i] = keep ? from_float<T>(y[c]) : zero_of<T>();
      mo[c].v[i] = keep ? one_of<T>() : zero_of<T>();
    }
  }
#pragma unroll
  for (int c = 0; c < 4; c++) {
    so[c].store_stream(sparse + (c0 + c) * ld + r0);
    if (mask) mo[c].store_stream(mask + (c0 + c) * ld + r0);
  }
}

template <typename T, int OP>
int launch(const void* dense, int layout, int64_t ld, int64_t m, int64_t k, const float* rnd, int64_t rand_ld,
           void* sparse, void* mask, hipStream_t s, const char* fn) {
  if (layout == TF24_ROW_MAJOR) {
    dim3 grid((unsigned)(m * ((k / 8 + kThreads - 1) / kThreads)));
    hipLaunchKernelGGL((dense_op_row<T, OP>), grid, dim3(kThreads), 0, s, (const T*)dense, ld, m, k, rnd, rand_ld, (T*)sparse, (T*)mask);
  } else {
    constexpr int R = 16 / sizeof(T);
    dim3 grid((unsigned)((k / 4) * ((m / R + kThreads - 1) / kThreads)));
    hipLaunchKernelGGL((dense_op_col<T, OP>), grid, dim3(kThreads), 0, s, (const T*)dense, ld, m, k, rnd, rand_ld, (T*)sparse, (T*)mask);
  }
  return check_launch(fn);
}

template <int OP>
int run(const char* fn, const void* dense, int dtype, int layout, int64_t ld, int64_t m, int64_t k, const float* rnd,
        int64_t rand_ld, void* sparse, void* mask, void* stream) {
  if (layout != TF24_ROW_MAJOR && layout != TF24_COL_MAJOR) return fail(TF24_ERR_ARG, "%s: bad layout %d", fn, layout);
  if (m <= 0 || k <= 0 || k % 4) return fail(TF24_ERR_SHAPE, "%s: k=%lld must be a positive multiple of 4", fn, (long long)k);
  if (layout == TF24_ROW_MAJOR && k % 8) return fail(TF24_ERR_SHAPE, "%s: row-major input needs k %% 8 == 0 (k=%lld)", fn, (long long)k);
  if (layout == TF24_COL_MAJOR && m % 8) return fail(TF24_ERR_SHAPE, "%s: column-major input needs m %% 8 == 0 (m=%lld)", fn, (long long)m);
  if (m > 0x7fffffffLL || k > 0x7fffffffLL) return fail(TF24_ERR_SHAPE, "%s: matrix too large", fn);
  const int64_t extent = layout == TF24_ROW_MAJOR ? k : m;
  if (ld < extent || ld % 8) return fail(TF24_ERR_STRIDE, "%s: leading dimension %lld must be >= %lld and a multiple of 8", fn, (long long)ld, (long long)extent);
  if (OP == OP_MVUE && (!rnd || rand_ld < extent || rand_ld % 8)) return fail(TF24_ERR_ARG, "%s: rand tensor missing or bad leading dimension", fn);
  if (!dense || !sparse) return fail(TF24_ERR_ARG, "%s: null pointer", fn);
  if (int rc = check_aligned(fn, 16, {dense, sparse, mask, rnd})) return rc;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TF24_F32: return launch<float, OP>(dense, layout, ld, m, k, rnd, rand_ld, sparse, mask, s, fn);
    case TF24_F16: return launch<f16_t, OP>(dense, layout, ld, m, k, rnd, rand_ld, sparse, mask, s, fn);
    case TF24_BF16: return launch<bf16_t, OP>(dense, layout, ld, m, k, rnd, rand_ld, sparse, mask, s, fn);
  }
  return fail(TF24_ERR_DTYPE, "%s: unsupported dtype %d", fn, dtype);
}

}  // namespace
}  // namespace tf24

extern "C" int tf24_soft_threshold24(const void* dense, int dtype, int layout, int64_t ld, int64_t m, int64_t k,
                                     void* sparse_out, void* mask_out, void* stream) {
  return tf24::run<tf24::OP_SOFT>("tf24_soft_threshold24", dense, dtype, layout, ld, m, k, nullptr, 0, sparse_out, mask_out, stream);
}

extern "C" int tf24_sparse24_dense(const void* dense, int dtype, int layout, int64_t ld, int64_t m, int64_t k,
                                   void* sparse_out, void* mask_out, void* stream) {
  return tf24::run<tf24::OP_SPARSE24>("tf24_sparse24_dense", dense, dtype, layout, ld, m, k, nullptr, 0, sparse_out, mask_out, stream);
}

extern "C" int tf24_mvue24_dense(const void* dense, int dtype, int layout, int64_t ld, int64_t m, int64_t k,
                                 const float* rnd, int64_t rand_ld, void* sparse_out, void* stream) {
  return tf24::run<tf24::OP_MVUE>("tf24_mvue24_dense", dense, dtype, layout, ld, m, k, rnd, rand_ld, sparse_out, nullptr, stream);
}
