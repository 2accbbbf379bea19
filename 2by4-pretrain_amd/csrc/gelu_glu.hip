// GELU-GLU for gfx950: out = gelu_tanh(gate) * x with [x | gate] the two halves of the input's
// last dimension, and its backward pass; float32 arithmetic, one rounding to the storage type.
//
// Both memory orders of the reference's two code paths are one indexing scheme: element (i, j) of
// the x half at i*ld + j and its gate at the same place + gate_off.  Row-major input [rows, cols]:
// i = row, j = column < cols/2, gate_off = cols/2.  Column-major input (the reference's "fall back
// to 2D" path, memory [cols][ld]): i = column < cols/2, j = row, gate_off = (cols/2)*ld.
// A lane owns 8 consecutive j (16-byte accesses for 16-bit types) when the extents allow it.
#include "tf24_common.hpp"

namespace tf24 {
namespace {

constexpr int kThreads = 256;
constexpr float kBeta = 0.7978845608028654f;     // sqrt(2/pi)
constexpr float kKappa = 0.044715f;

// 0.5 * (1 + tanh(u)) is the logistic function of 2u: one exponential and one reciprocal per
// element (written with tanh, exp and a division, as the reference does, the forward kernel is
// bound by the vector ALUs at 0.59 of the HBM peak instead of by memory).  exp of a large
// argument gives +inf and the reciprocal 0, so no range split is needed.
struct GluTerms {
  float gelu;      // gelu_tanh(gate) = gate * sig
  float dgelu;     // d gelu_tanh / d gate = sig + gate * sig * (1 - sig) * 2 * du/dgate
};
template <bool GRAD>
__device__ __forceinline__ GluTerms glu_terms(float gate) {
  const float g2 = gate * gate;
  const float u = kBeta * (gate + kKappa * g2 * gate);
  const float sig = __builtin_amdgcn_rcpf(1.0f + __expf(-2.0f * u));
  GluTerms r;
  r.gelu = gate * sig;
  r.dgelu = 0.0f;
  if constexpr (GRAD) r.dgelu = sig + gate * (sig * (1.0f - sig)) * ((2.0f * kBeta) * (1.0f + (3.0f * kKappa) * g2));
  return r;
}

// V = elements per lane (8 or 1); blocks are numbered along j first
template <typename T, int V>
__global__ void __launch_bounds__(kThreads)
gelu_glu_fwd(const T* __restrict__ in, int64_t ld_in, int64_t gate_off, int64_t ni, int64_t nj,
             T* __restrict__ out, int64_t ld_out) {
  const uint32_t chunks = (uint32_t)((nj / V + kThreads - 1) / kThreads);
  const int64_t i = blockIdx.x / chunks;
  const int64_t j = ((int64_t)(blockIdx.x - (uint32_t)i * chunks) * kThreads + threadIdx.x) * V;
  if (j >= nj) return;
  Pack<T, V> x, g, o;
  x.load_stream(in + i * ld_in + j);
  g.load_stream(in + i * ld_in + j + gate_off);
#pragma unroll
  for (int e = 0; e < V; e++) o.v[e] = from_float<T>(glu_terms<false>(to_float(g.v[e])).gelu * to_float(x.v[e]));
  o.store_stream(out + i * ld_out + j);
}

template <typename T, int V>
__global__ void __launch_bounds__(kThreads)
gelu_glu_bwd(const T* __restrict__ grad_out, int64_t ld_go, const T* __restrict__ in, int64_t ld_in, int64_t gate_off,
             int64_t ni, int64_t nj, T* __restrict__ grad_in, int64_t ld_gi, int64_t gate_off_gi) {
  const uint32_t chunks = (uint32_t)((nj / V + kThreads - 1) / kThreads);
  const int64_t i = blockIdx.x / chunks;
  const int64_t j = ((int64_t)(blockIdx.x - (uint32_t)i * chunks) * kThreads + threadIdx.x) * V;
  if (j >= nj) return;
  Pack<T, V> go, x, g, gx, gg;
  go.load_stream(grad_out + i * ld_go + j);
  x.load_stream(in + i * ld_in + j);
  g.load_stream(in + i * ld_in + j + gate_off);
#pragma unroll
  for (int e = 0; e < V; e++) {
    const GluTerms t = glu_terms<true>(to_float(g.v[e]));
    const float dy = to_float(go.v[e]);
    gx.v[e] = from_float<T>(dy * t.gelu);
    gg.v[e] = from_float<T>(dy * to_float(x.v[e]) * t.dgelu);
  }
  gx.store_stream(grad_in + i * ld_gi + j);
  gg.store_stream(grad_in + i * ld_gi + j + gate_off_gi);
}

struct View {
  int64_t ni, nj, gate_off;
};
// layout of the [rows, cols] input -> the (i, j) scheme above
View view_of(int layout, int64_t rows, int64_t cols, int64_t ld) {
  if (layout == TF24_ROW_MAJOR) return {rows, cols / 2, cols / 2};
  return {cols / 2, rows, (cols / 2) * ld};
}
bool vectorizable(int64_t nj, std::initializer_list<int64_t> offsets, std::initializer_list<const void*> ptrs) {
  if (nj % 8) return false;
  for (int64_t o : offsets) if (o % 8) return false;
  for (const void* p : ptrs) if ((uintptr_t)p % 16) return false;
  return true;
}

template <typename T>
int forward(const void* in, int layout, int64_t ld_in, int64_t rows, int64_t cols, void* out, int64_t ld_out, hipStream_t s) {
  const View v = view_of(layout, rows, cols, ld_in);
  if (vectorizable(v.nj, {ld_in, ld_out, v.gate_off}, {in, out})) {
    dim3 grid((unsigned)(v.ni * ((v.nj / 8 + kThreads - 1) / kThreads)));
    hipLaunchKernelGGL((gelu_glu_fwd<T, 8>), grid, dim3(kThreads), 0, s, (const T*)in, ld_in, v.gate_off, v.ni, v.nj, (T*)out, ld_out);
  } else {
    dim3 grid((unsigned)(v.ni * ((v.nj + kThreads - 1) / kThreads)));
    hipLaunchKernelGGL((gelu_glu_fwd<T, 1>), grid, dim3(kThreads), 0, s, (const T*)in, ld_in, v.gate_off, v.ni, v.nj, (T*)out, ld_out);
  }
  return check_launch("tf24_gelu_glu_forward");
}

template <typename T>
int backward(const void* go, int64_t ld_go, const void* in, int layout, int64_t ld_in, int64_t rows, int64_t cols,
             void* gi, int64_t ld_gi, hipStream_t s) {
  const View v = view_of(layout, rows, cols, ld_in);
  const int64_t gate_off_gi = view_of(layout, rows, cols, ld_gi).gate_off;
  if (vectorizable(v.nj, {ld_go, ld_in, ld_gi, v.gate_off, gate_off_gi}, {go, in, gi})) {
    dim3 grid((unsigned)(v.ni * ((v.nj / 8 + kThreads - 1) / kThreads)));
    hipLaunchKernelGGL((gelu_glu_bwd<T, 8>), grid, dim3(kThreads), 0, s, (const T*)go, ld_go, (const T*)in, ld_in, v.gate_off, v.ni, v.nj,
                       (T*)gi, ld_gi, gate_off_gi);
  } else {
    dim3 grid((unsigned)(v.ni * ((v.nj + kThreads - 1) / kThreads)));
    hipLaunchKernelGGL((gelu_glu_bwd<T, 1>), grid, dim3(kThreads), 0, s, (const T*)go, ld_go, (const T*)in, ld_in, v.gate_off, v.ni, v.nj,
                       (T*)gi, ld_gi, gate_off_gi);
  }
  return check_launch("tf24_gelu_glu_backward");
}

int check_args(const char* fn, int dtype, int layout, int64_t rows, int64_t cols, std::initializer_list<int64_t> lds_full,
               std::initializer_list<int64_t> lds_half) {
  if (dtype != TF24_F32 && dtype != TF24_F16 && dtype != TF24_BF16) return fail(TF24_ERR_DTYPE, "%s: unsupported dtype %d", fn, dtype);
  if (layout != TF24_ROW_MAJOR && layout != TF24_COL_MAJOR) return fail(TF24_ERR_ARG, "%s: bad layout %d", fn, layout);
  if (rows < 1 || cols < 2 || cols % 2) return fail(TF24_ERR_SHAPE, "%s: shape (%lld, %lld) is not supported: the last dimension must be even", fn, (long long)rows, (long long)cols);
  const int64_t ni = layout == TF24_ROW_MAJOR ? rows : cols / 2, nj = layout == TF24_ROW_MAJOR ? cols / 2 : rows;
  if (ni * ((nj + kThreads - 1) / kThreads) > 0x7fffffffLL) return fail(TF24_ERR_SHAPE, "%s: tensor too large", fn);
  // leading dimensions: the contiguous extent is cols (row-major) or rows (column-major) for the
  // full-width tensors, cols/2 or rows for the half-width ones
  for (int64_t ld : lds_full)
    if (ld < (layout == TF24_ROW_MAJOR ? cols : rows)) return fail(TF24_ERR_STRIDE, "%s: leading dimension %lld too small", fn, (long long)ld);
  for (int64_t ld : lds_half)
    if (ld < (layout == TF24_ROW_MAJOR ? cols / 2 : rows)) return fail(TF24_ERR_STRIDE, "%s: leading dimension %lld too small", fn, (long long)ld);
  return TF24_OK;
}

}  // namespace
}  // namespace tf24

extern "C" int tf24_gelu_glu_forward(const void* in, int dtype, int layout, int64_t ld_in, int64_t rows, int64_t cols,
                                     void* out, int64_t ld_out, void* stream) {
  using namespace tf24;
  int rc = check_args("tf24_gelu_glu_forward", dtype, layout, rows, cols, {ld_in}, {ld_out});
  if (rc != TF24_OK) return rc;
  if (!in || !out) return fail(TF24_ERR_ARG, "tf24_gelu_glu_forward: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TF24_F32: return forward<float>(in, layout, ld_in, rows, cols, out, ld_out, s);
    case TF24_F16: return forward<f16_t>(in, layout, ld_in, rows, cols, out, ld_out, s);
    default: return forward<bf16_t>(in, layout, ld_in, rows, cols, out, ld_out, s);
  }
}

extern "C" int tf24_gelu_glu_backward(const void* grad_out, int64_t ld_grad_out, const void* in, int dtype, int layout,
                                      int64_t ld_in, int64_t rows, int64_t cols, void* grad_in, int64_t ld_grad_in,
                                      void* stream) {
  using namespace tf24;
  int rc = check_args("tf24_gelu_glu_backward", dtype, layout, rows, cols, {ld_in, ld_grad_in}, {ld_grad_out});
  if (rc != TF24_OK) return rc;
  if (!grad_out || !in || !grad_in) return fail(TF24_ERR_ARG, "tf24_gelu_glu_backward: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (dtype) {
    case TF24_F32: return backward<float>(grad_out, ld_grad_out, in, layout, ld_in, rows, cols, grad_in, ld_grad_in, s);
    case TF24_F16: return backward<f16_t>(grad_out, ld_grad_out, in, layout, ld_in, rows, cols, grad_in, ld_grad_in, s);
    default: return backward<bf16_t>(grad_out, ld_grad_out, in, layout, ld_in, rows, cols, grad_in, ld_grad_in, s);
  }
}
