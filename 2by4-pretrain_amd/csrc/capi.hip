// Host-only part of the C ABI: version, error reporting, argument validation.
#include <cstdarg>
#include <cstdio>

#include "tf24_common.hpp"

namespace tf24 {

static thread_local char g_error[512] = "";

void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
}

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof g_error, fmt, ap);
  va_end(ap);
  return code;
}

int check_aligned(const char* fn, int bytes, std::initializer_list<const void*> ptrs) {
  for (const void* p : ptrs)
    if (p && (uintptr_t)p % (uintptr_t)bytes) return fail(TF24_ERR_STRIDE, "%s: pointer %p is not %d-byte aligned", fn, p, bytes);
  return TF24_OK;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TF24_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return TF24_OK;
}

static bool is_float_dtype(int dt) { return dt == TF24_F32 || dt == TF24_F16 || dt == TF24_BF16; }
static bool is_mask_dtype(int dt) { return dt == TF24_U8 || is_float_dtype(dt); }
static bool is_layout(int l) { return l == TF24_ROW_MAJOR || l == TF24_COL_MAJOR; }

// leading dimension of an [m,k] matrix: at least the contiguous extent, and a multiple of 8
// elements so that every 128-bit access stays aligned
static int check_ld(const char* fn, const char* name, int layout, int64_t ld, int64_t m, int64_t k) {
  int64_t extent = layout == TF24_ROW_MAJOR ? k : m;
  if (ld < extent) return fail(TF24_ERR_STRIDE, "%s: %s leading dimension %lld < %lld", fn, name, (long long)ld, (long long)extent);
  if (ld % 8) return fail(TF24_ERR_STRIDE, "%s: %s leading dimension %lld must be a multiple of 8", fn, name, (long long)ld);
  return TF24_OK;
}

}  // namespace tf24

using namespace tf24;

extern "C" const char* tf24_version(void) { return "tf24 0.1.0 gfx950"; }

extern "C" const char* tf24_last_error(void) { return g_error; }

extern "C" int tf24_prune_compress_validate(int in_dtype, int layout, int64_t ld, int64_t m, int64_t k, int mode,
                                            int has_mask, int mask_dtype, int64_t mask_ld, int has_rand, int64_t rand_ld,
                                            int out_dtype) {
  const char* fn = "tf24_prune_compress";
  if (!is_float_dtype(in_dtype) && in_dtype != TF24_I8) return fail(TF24_ERR_DTYPE, "%s: unsupported input dtype %d", fn, in_dtype);
  if (out_dtype != TF24_F16 && out_dtype != TF24_BF16 && !is_8bit(out_dtype))
    return fail(TF24_ERR_DTYPE, "%s: unsupported output dtype %d", fn, out_dtype);
  if ((in_dtype == TF24_I8) != (out_dtype == TF24_I8))
    return fail(TF24_ERR_DTYPE, "%s: int8 values come from an int8 dense matrix only (input dtype %d, output dtype %d)", fn, in_dtype, out_dtype);
  if (in_dtype == TF24_I8 && (mode == TF24_PRUNE_MVUE || mode == TF24_PRUNE_MVUE_PACKED || mode == TF24_PRUNE_MVUE_SEEDED || mode == TF24_PRUNE_MVUE_SEEDED_DEVICE))
    return fail(TF24_ERR_ARG, "%s: MVUE24 rescales the kept values and is not defined for int8", fn);
  if (!is_layout(layout)) return fail(TF24_ERR_ARG, "%s: bad layout %d", fn, layout);
  const int64_t min_rows = 32, min_cols = is_8bit(out_dtype) ? 128 : 64;
  if (m < min_rows || m % min_rows || k < min_cols || k % min_cols)
    return fail(TF24_ERR_SHAPE, "%s: shape (%lld, %lld) is not supported: both dimensions must be >= and a multiple of (%lld, %lld)",
                fn, (long long)m, (long long)k, (long long)min_rows, (long long)min_cols);
  if (m * (k / 8) > 0x7fffffffLL) return fail(TF24_ERR_SHAPE, "%s: matrix too large (%lld x %lld)", fn, (long long)m, (long long)k);
  int rc = check_ld(fn, "dense", layout, ld, m, k);
  if (rc) return rc;
  if (in_dtype == TF24_I8) {
    if (has_mask && mask_dtype != TF24_U8) return fail(TF24_ERR_DTYPE, "%s: int8 input takes a byte mask (dtype %d given)", fn, mask_dtype);
    // column-major int8: a lane reads 16 rows of a column with one 16-byte load
    if (layout == TF24_COL_MAJOR && (ld % 16 || (has_mask && mask_ld % 16)))
      return fail(TF24_ERR_STRIDE, "%s: column-major int8 input needs leading dimensions that are multiples of 16", fn);
  }
  switch (mode) {
    case TF24_PRUNE_MAGNITUDE:
      break;
    case TF24_PRUNE_MASK:
      if (!has_mask) return fail(TF24_ERR_ARG, "%s: mode MASK needs a mask", fn);
      if (!is_mask_dtype(mask_dtype)) return fail(TF24_ERR_DTYPE, "%s: unsupported mask dtype %d", fn, mask_dtype);
      if ((rc = check_ld(fn, "mask", layout, mask_ld, m, k))) return rc;
      break;
    case TF24_PRUNE_MVUE:
      if (!has_rand) return fail(TF24_ERR_ARG, "%s: mode MVUE needs a rand tensor", fn);
      if ((rc = check_ld(fn, "rand", layout, rand_ld, m, k))) return rc;
      break;
    case TF24_PRUNE_MVUE_PACKED:
      if (!has_rand) return fail(TF24_ERR_ARG, "%s: mode MVUE_PACKED needs a rand tensor", fn);
      if ((rc = check_ld(fn, "rand", layout, rand_ld, m, k / 2))) return rc;
      break;
    case TF24_PRUNE_MVUE_SEEDED:
    case TF24_PRUNE_MVUE_SEEDED_DEVICE:
      if (!has_rand) return fail(TF24_ERR_ARG, "%s: mode MVUE_SEEDED needs `rand` to point to {seed, offset}", fn);
      break;
    default:
      return fail(TF24_ERR_ARG, "%s: bad mode %d", fn, mode);
  }
  if (has_mask && has_rand) return fail(TF24_ERR_ARG, "%s: using MVUE24 with mask is not supported", fn);
  return TF24_OK;
}

extern "C" int tf24_prune_compress_dual_validate(int in_dtype, int64_t ld, int64_t m, int64_t k, int mask_dtype,
                                                 int64_t mask_ld, int out_dtype, int out_layout) {
  const char* fn = "tf24_prune_compress_dual";
  if (!is_float_dtype(in_dtype) && in_dtype != TF24_I8) return fail(TF24_ERR_DTYPE, "%s: unsupported input dtype %d", fn, in_dtype);
  if (out_dtype != TF24_F16 && out_dtype != TF24_BF16 && !is_8bit(out_dtype))
    return fail(TF24_ERR_DTYPE, "%s: unsupported output dtype %d", fn, out_dtype);
  if ((in_dtype == TF24_I8) != (out_dtype == TF24_I8))
    return fail(TF24_ERR_DTYPE, "%s: int8 values come from an int8 dense matrix only (input dtype %d, output dtype %d)", fn, in_dtype, out_dtype);
  if (!is_mask_dtype(mask_dtype)) return fail(TF24_ERR_DTYPE, "%s: unsupported mask dtype %d", fn, mask_dtype);
  if (out_layout != TF24_COMPRESSED_CANONICAL && out_layout != TF24_COMPRESSED_PANEL)
    return fail(TF24_ERR_ARG, "%s: bad compressed layout %d", fn, out_layout);
  const int64_t unit = is_8bit(out_dtype) ? 128 : 64;
  if (m < unit || m % unit || k < unit || k % unit)
    return fail(TF24_ERR_SHAPE, "%s: shape (%lld, %lld) is not supported: both dimensions must be >= and a multiple of %lld",
                fn, (long long)m, (long long)k, (long long)unit);
  int rc = check_ld(fn, "dense", TF24_ROW_MAJOR, ld, m, k);
  if (rc) return rc;
  return check_ld(fn, "mask", TF24_ROW_MAJOR, mask_ld, m, k);
}
