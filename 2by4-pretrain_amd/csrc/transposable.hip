// Transposable 4x4 mask search over the 90 row-and-column 2:4 patterns, for gfx950.
//
// One lane owns one 4x4 block, entirely in registers; the whole search is straight-line code
// (compile-time tables), no LDS, no pattern table in memory.  A pattern is a choice of one
// column pair per row, q_r in {(0,1),(0,2),(0,3),(1,2),(1,3),(2,3)}, such that every column is
// covered twice; pattern order (the reference's table, descending lexicographic) is ascending
// lexicographic order of (q0,q1,q2,q3).  The search is two-level:
//   s[r][q]   = B[r][c1(q)] + B[r][c2(q)]                         24 adds
//   bottom    = s[2][q2] + s[3][q3]   for the 36 (q2,q3)          first maximum per class of equal
//                                                                 column-count vector (19 classes)
//   candidate = (s[0][q0] + s[1][q1]) + best_bottom[complement class], first maximum over the 36 tops
// all in float32, strict '>' updates in index order, i.e. the first maximal pattern wins.
#include <type_traits>

#include "tf24_common.hpp"

namespace tf24 {
namespace {

constexpr int kThreads = 256;

constexpr int pair_a(int q) { return q < 3 ? 0 : (q < 5 ? 1 : 2); }
constexpr int pair_b(int q) { return q < 3 ? q + 1 : (q < 5 ? q - 1 : 3); }
constexpr uint32_t row_bits(int q) { return (1u << pair_a(q)) | (1u << pair_b(q)); }

// column-count vector of a pair of rows, 2 bits per column
constexpr uint32_t count_code(int qa, int qb) {
  uint32_t code = 0;
  for (int c = 0; c < 4; c++) code |= (((row_bits(qa) >> c) & 1u) + ((row_bits(qb) >> c) & 1u)) << (2 * c);
  return code;
}
constexpr uint32_t complement_code(uint32_t code) {
  uint32_t out = 0;
  for (int c = 0; c < 4; c++) out |= (2u - ((code >> (2 * c)) & 3u)) << (2 * c);
  return out;
}
// dense class index (0..18) of a count vector: order of first appearance among the 36 combos
constexpr int class_index(uint32_t code) {
  int n = 0;
  for (int b = 0; b < 36; b++) {
    uint32_t cb = count_code(b / 6, b % 6);
    if (cb == code) return n;
    bool seen = false;
    for (int p = 0; p < b; p++) seen = seen || count_code(p / 6, p % 6) == cb;
    if (!seen) n++;
  }
  return -1;
}
constexpr int kClasses = 19;
// is combo b the first member of its class?
constexpr bool first_of_class(int b) {
  for (int p = 0; p < b; p++)
    if (count_code(p / 6, p % 6) == count_code(b / 6, b % 6)) return false;
  return true;
}

template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

// a[r][c] -> 16-bit mask, bit 4r+c
__device__ __forceinline__ uint32_t search_block(const float (&a)[4][4]) {
  float s[4][6];
#pragma unroll
  for (int r = 0; r < 4; r++) {
    s[r][0] = a[r][0] + a[r][1]; s[r][1] = a[r][0] + a[r][2]; s[r][2] = a[r][0] + a[r][3];
    s[r][3] = a[r][1] + a[r][2]; s[r][4] = a[r][1] + a[r][3]; s[r][5] = a[r][2] + a[r][3];
  }
  float bbest[kClasses];
  uint32_t bbits[kClasses];
  static_for<0, 36>([&](auto ic) {
    constexpr int b = decltype(ic)::value;
    constexpr int qa = b / 6, qb = b % 6;
    constexpr int cls = class_index(count_code(qa, qb));
    constexpr uint32_t bits = (row_bits(qa) << 8) | (row_bits(qb) << 12);
    const float v = s[2][qa] + s[3][qb];
    if constexpr (first_of_class(b)) {
      bbest[cls] = v;
      bbits[cls] = bits;
    } else {
      const bool upd = v > bbest[cls];
      bbest[cls] = upd ? v : bbest[cls];
      bbits[cls] = upd ? bits : bbits[cls];
    }
  });
  float best = 0.0f;
  uint32_t mask = 0;
  static_for<0, 36>([&](auto ic) {
    constexpr int t = decltype(ic)::value;
    constexpr int qa = t / 6, qb = t % 6;
    constexpr int cls = class_index(complement_code(count_code(qa, qb)));
    constexpr uint32_t bits = row_bits(qa) | (row_bits(qb) << 4);
    const float cand = (s[0][qa] + s[1][qb]) + bbest[cls];
    if constexpr (t == 0) {
      best = cand;
      mask = bits | bbits[cls];
    } else {
      const bool upd = cand > best;
      best = upd ? cand : best;
      mask = upd ? (bits | bbits[cls]) : mask;
    }
  });
  return mask;
}

// E = elements per row of a block = 4.  TRANS: the matrix is column-major (element (r,c) at c*ld + r),
// so the lane reads the block transposed and writes its results transposed.
template <typename T, bool ABS, bool TRANS>
__global__ void __launch_bounds__(kThreads)
transposable_kernel(const T* __restrict__ dense, int64_t ld, int64_t nmajor4, int64_t nminor8,
                    T* __restrict__ sparse, uint8_t* __restrict__ mask_out) {
  // "major" = the strided dimension in memory, "minor" = the contiguous one.  A lane owns two
  // adjacent 4 x 4 blocks (8 contiguous elements of 4 lines): 16-byte loads and stores for 16-bit
  // types, 8-byte mask stores.
  // blocks are numbered along the contiguous dimension first: blocks that run together read
  // neighbouring pieces of the same four lines
  const uint32_t chunks = (uint32_t)((nminor8 + kThreads - 1) / kThreads);
  const int64_t bmajor = blockIdx.x / chunks;
  const int64_t bminor = (int64_t)(blockIdx.x - (uint32_t)bmajor * chunks) * kThreads + threadIdx.x;
  if (bminor >= nminor8) return;
  const int64_t off = bmajor * 4 * ld + bminor * 8;
  Pack<T, 8> in[4];
#pragma unroll
  for (int p = 0; p < 4; p++) in[p].load_stream(dense + off + p * ld);
  uint32_t mbits[2];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    float a[4][4];
#pragma unroll
    for (int p = 0; p < 4; p++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        float v = to_float(in[p].v[4 * h + e]);
        if (ABS) v = __builtin_fabsf(v);
        if (TRANS) a[e][p] = v; else a[p][e] = v;
      }
    mbits[h] = search_block(a);
  }
#pragma unroll
  for (int p = 0; p < 4; p++) {
    uint32_t bytes[2] = {0, 0};
    Pack<T, 8> out;
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int bit = TRANS ? (4 * e + p) : (4 * p + e);
        const bool keep = (mbits[h] >> bit) & 1;
        bytes[h] |= (uint32_t)keep << (8 * e);
        out.v[4 * h + e] = keep ? in[p].v[4 * h + e] : T{};
      }
    *reinterpret_cast<uint2*>(mask_out + off + p * ld) = make_uint2(bytes[0], bytes[1]);   // streaming here costs 15 %
    if (sparse) out.store_stream(sparse + off + p * ld);
  }
}

template <typename T, bool ABS, bool TRANS>
int launch(const void* dense, int64_t ld, int64_t m, int64_t k, void* sparse, uint8_t* mask, hipStream_t s) {
  const int64_t nmajor4 = (TRANS ? k : m) / 4, nminor8 = (TRANS ? m : k) / 8;     // both extents are multiples of 32
  dim3 grid((unsigned)(nmajor4 * ((nminor8 + kThreads - 1) / kThreads)));
  hipLaunchKernelGGL((transposable_kernel<T, ABS, TRANS>), grid, dim3(kThreads), 0, s, (const T*)dense, ld, nmajor4, nminor8,
                     (T*)sparse, mask);
  return check_launch("tf24_transposable_mask");
}

template <typename T>
int dispatch(const void* dense, int layout, int64_t ld, int64_t m, int64_t k, int use_abs, void* sparse, uint8_t* mask, hipStream_t s) {
  const bool trans = layout == TF24_COL_MAJOR;
  if (use_abs) return trans ? launch<T, true, true>(dense, ld, m, k, sparse, mask, s) : launch<T, true, false>(dense, ld, m, k, sparse, mask, s);
  return trans ? launch<T, false, true>(dense, ld, m, k, sparse, mask, s) : launch<T, false, false>(dense, ld, m, k, sparse, mask, s);
}

}  // namespace
}  // namespace tf24

extern "C" int tf24_transposable_mask_validate(int dtype, int layout, int64_t ld, int64_t m, int64_t k) {
  using namespace tf24;
  const char* fn = "tf24_transposable_mask";
  if (dtype != TF24_F32 && dtype != TF24_F16 && dtype != TF24_BF16) return fail(TF24_ERR_DTYPE, "%s: invalid datatype %d of dense matrix", fn, dtype);
  if (layout != TF24_ROW_MAJOR && layout != TF24_COL_MAJOR) return fail(TF24_ERR_ARG, "%s: bad layout %d", fn, layout);
  if (m <= 0 || m % 32) return fail(TF24_ERR_SHAPE, "%s: number of rows of dense matrix %lld must be divisible by 32", fn, (long long)m);
  if (k <= 0 || k % 64) return fail(TF24_ERR_SHAPE, "%s: number of columns of dense matrix %lld must be divisible by 64", fn, (long long)k);
  const int64_t extent = layout == TF24_ROW_MAJOR ? k : m;
  if (ld < extent || ld % 8) return fail(TF24_ERR_STRIDE, "%s: leading dimension %lld must be >= %lld and a multiple of 8", fn, (long long)ld, (long long)extent);
  if (m > 0x7fffffffLL || k > 0x7fffffffLL) return fail(TF24_ERR_SHAPE, "%s: matrix too large", fn);
  return TF24_OK;
}

extern "C" int tf24_transposable_mask(const void* dense, int dtype, int layout, int64_t ld, int64_t m, int64_t k,
                                      int use_abs, void* sparse_out, uint8_t* mask_out, void* stream) {
  using namespace tf24;
  int rc = tf24_transposable_mask_validate(dtype, layout, ld, m, k);
  if (rc) return rc;
  if (!dense || !mask_out) return fail(TF24_ERR_ARG, "tf24_transposable_mask: null pointer");
  if (int rc2 = check_aligned("tf24_transposable_mask", 16, {dense, sparse_out})) return rc2;
  if (int rc2 = check_aligned("tf24_transposable_mask", 8, {mask_out})) return rc2;
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TF24_F32: return dispatch<float>(dense, layout, ld, m, k, use_abs, sparse_out, mask_out, s);
    case TF24_F16: return dispatch<f16_t>(dense, layout, ld, m, k, use_abs, sparse_out, mask_out, s);
    default: return dispatch<bf16_t>(dense, layout, ld, m, k, use_abs, sparse_out, mask_out, s);
  }
}
