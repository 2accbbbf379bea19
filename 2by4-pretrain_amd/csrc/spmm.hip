// tf24_spmm: argument checks and dispatch on the operand type.  The kernels live in spmm_kernels.hpp and are
// instantiated by one translation unit per operand type (spmm_f16.hip, spmm_bf16.hip, spmm_e4m3.hip,
// spmm_e5m2.hip, spmm_i8.hip), so that they compile side by side.
#include "spmm_kernels.hpp"

extern "C" int tf24_spmm_validate(int dtype, int64_t n_sparse, int64_t k, int b_layout, int64_t ldb, int64_t n_dense,
                                  int out_dtype, int c_layout, int64_t ldc, int activation) {
  using namespace tf24;
  const char* fn = "tf24_spmm";
  if (dtype != TF24_F16 && dtype != TF24_BF16 && !is_8bit(dtype)) return fail(TF24_ERR_DTYPE, "%s: unsupported operand dtype %d", fn, dtype);
  if (dtype == TF24_I8) {
    // integer product (.cu:594-637): int32 results, no or ReLU activation
    if (out_dtype != TF24_I32) return fail(TF24_ERR_DTYPE, "%s: int8 operands give int32 results (output dtype %d)", fn, out_dtype);
    if (activation != TF24_ACT_NONE && activation != TF24_ACT_RELU) return fail(TF24_ERR_ARG, "%s: int8 operands support no activation or ReLU (%d)", fn, activation);
  } else if (out_dtype != TF24_F16 && out_dtype != TF24_BF16 && out_dtype != TF24_F32) {
    return fail(TF24_ERR_DTYPE, "%s: unsupported output dtype %d", fn, out_dtype);
  }
  const bool eight = is_8bit(dtype);
  const int64_t kmult = eight ? 128 : 64, dmult = eight ? 16 : 8;
  if (n_sparse <= 0 || n_sparse % 32) return fail(TF24_ERR_SHAPE, "%s: sparse operand rows %lld must be a positive multiple of 32", fn, (long long)n_sparse);
  if (k <= 0 || k % kmult) return fail(TF24_ERR_SHAPE, "%s: inner dimension %lld must be a positive multiple of %lld", fn, (long long)k, (long long)kmult);
  if (n_dense <= 0 || n_dense % dmult) return fail(TF24_ERR_SHAPE, "%s: dense operand extent %lld must be a positive multiple of %lld", fn, (long long)n_dense, (long long)dmult);
  if (b_layout != TF24_ROW_MAJOR && b_layout != TF24_COL_MAJOR) return fail(TF24_ERR_ARG, "%s: bad b_layout %d", fn, b_layout);
  if (c_layout != TF24_ROW_MAJOR && c_layout != TF24_COL_MAJOR) return fail(TF24_ERR_ARG, "%s: bad c_layout %d", fn, c_layout);
  const int64_t bext = b_layout == TF24_ROW_MAJOR ? k : n_dense;
  if (ldb < bext || ldb % dmult) return fail(TF24_ERR_STRIDE, "%s: ldb %lld must be >= %lld and a multiple of %lld", fn, (long long)ldb, (long long)bext, (long long)dmult);
  // the copies address a tile's rows of B by 32-bit lane offsets from the tile's base: 256 rows must span < 4 GiB
  if (ldb * (eight ? 1 : 2) > ((int64_t)1 << 24)) return fail(TF24_ERR_STRIDE, "%s: ldb %lld exceeds 16 MiB per row", fn, (long long)ldb);
  const int64_t cext = c_layout == TF24_ROW_MAJOR ? n_dense : n_sparse;
  // rows of the output leave as 16-byte stores: 8 elements of a 16-bit type, 4 of a 32-bit one
  const int64_t cmult = (out_dtype == TF24_F16 || out_dtype == TF24_BF16) ? 8 : 4;
  if (ldc < cext || ldc % cmult) return fail(TF24_ERR_STRIDE, "%s: ldc %lld must be >= %lld and a multiple of %lld", fn, (long long)ldc, (long long)cext, (long long)cmult);
  if (activation < TF24_ACT_NONE || activation > TF24_ACT_GELU) return fail(TF24_ERR_ARG, "%s: bad activation %d", fn, activation);
  return TF24_OK;
}

namespace tf24 {
namespace {
template <typename C>
int64_t split_bytes(int dtype, int64_t n_sparse, int64_t k, int64_t n_dense) {
  const int64_t big = (int64_t)1 << 40;
  const int splits = is_8bit(dtype) ? choose_splits<e4m3_t, C>(n_sparse, k, n_dense, big) : choose_splits<f16_t, C>(n_sparse, k, n_dense, big);
  if (splits < 2) return 0;
  const int64_t tiles = ((n_sparse + C::BI - 1) / C::BI) * ((n_dense + C::BJ - 1) / C::BJ);
  return splits * tiles * C::BI * C::BJ * 4;
}
}  // namespace
}  // namespace tf24

// the float32 partial tiles of the k pieces, for whichever tile configuration the shape selects
extern "C" int64_t tf24_spmm_workspace_bytes(int dtype, int64_t n_sparse, int64_t k, int64_t n_dense) {
  using namespace tf24;
  int64_t bytes = split_bytes<TiledCfg>(dtype, n_sparse, k, n_dense);
  bytes = std::max(bytes, split_bytes<MidCfg>(dtype, n_sparse, k, n_dense));
  if (n_dense <= SlimCfg::BJ) bytes = std::max(bytes, split_bytes<SlimCfg>(dtype, n_sparse, k, n_dense));
  return bytes;
}

extern "C" int tf24_spmm(const void* a_values, const void* a_meta, int a_layout, int dtype, int64_t n_sparse, int64_t k,
                         const void* b, int b_layout, int64_t ldb, int64_t n_dense,
                         void* c, int out_dtype, int c_layout, int64_t ldc,
                         const void* bias, float scale, int activation, void* workspace, int64_t workspace_bytes, void* stream) {
  using namespace tf24;
  int rc = tf24_spmm_validate(dtype, n_sparse, k, b_layout, ldb, n_dense, out_dtype, c_layout, ldc, activation);
  if (rc) return rc;
  if (!a_values || !a_meta || !b || !c) return fail(TF24_ERR_ARG, "tf24_spmm: null pointer");
  if ((rc = check_aligned("tf24_spmm", 16, {a_values, b, c, workspace}))) return rc;
  // panel metadata is copied 16 bytes per lane; canonical metadata is read in words of up to 4 bytes, row pitch k/8
  if ((rc = check_aligned("tf24_spmm", a_layout == TF24_COMPRESSED_PANEL ? 16 : a_layout == TF24_COMPRESSED_CUTLASS ? 4 : 8, {a_meta}))) return rc;
  if ((rc = check_aligned("tf24_spmm", dtype_size(out_dtype), {bias}))) return rc;
  if (a_layout != TF24_COMPRESSED_CANONICAL && a_layout != TF24_COMPRESSED_PANEL && a_layout != TF24_COMPRESSED_CUTLASS)
    return fail(TF24_ERR_ARG, "tf24_spmm: bad compressed layout %d", a_layout);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == TF24_I8 && scale != 1.0f) return fail(TF24_ERR_ARG, "tf24_spmm: int8 products are exact, scale must be 1 (%g given)", (double)scale);
  switch (dtype) {
    case TF24_I8: return spmm_i8(out_dtype, a_values, a_meta, a_layout, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, activation, workspace, workspace_bytes, s);
    case TF24_F16: return spmm_f16(out_dtype, a_values, a_meta, a_layout, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, activation, workspace, workspace_bytes, s);
    case TF24_BF16: return spmm_bf16(out_dtype, a_values, a_meta, a_layout, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, activation, workspace, workspace_bytes, s);
    case TF24_E5M2: return spmm_e5m2(out_dtype, a_values, a_meta, a_layout, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, activation, workspace, workspace_bytes, s);
    default: return spmm_e4m3(out_dtype, a_values, a_meta, a_layout, n_sparse, k, b, b_layout, ldb, n_dense, c, c_layout, ldc, bias, scale, activation, workspace, workspace_bytes, s);
  }
}
