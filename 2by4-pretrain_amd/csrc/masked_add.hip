// Masked decay for gfx950: grad[i] += alpha * p[i] where mask[i] == 0, in place, one pass.
// Lane owns 8 consecutive elements (vector loads of every operand); float32 arithmetic as a
// rounded product followed by a rounded sum (no fused multiply-add).
#include "tf24_common.hpp"

namespace tf24 {
namespace {

constexpr int kThreads = 256;

template <typename G, typename P, typename M>
__global__ void __launch_bounds__(kThreads)
masked_add_vec(G* __restrict__ grad, const P* __restrict__ p, const M* __restrict__ mask, int64_t n8, float alpha) {
  const int64_t u = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (u >= n8) return;
  Pack<G, 8> g;
  Pack<P, 8> pv;
  Pack<M, 8> mk;
  g.load(grad + u * 8);
  pv.load_stream(p + u * 8);        // read once; the gradient is read and written: ordinary accesses
  mk.load_stream(mask + u * 8);
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const float prod = to_float(pv.v[i]) * alpha;
    const float sum = to_float(g.v[i]) + prod;
    if (to_float(mk.v[i]) == 0.0f) g.v[i] = from_float<G>(sum);
  }
  g.store(grad + u * 8);
}

template <typename G, typename P, typename M>
__global__ void __launch_bounds__(kThreads)
masked_add_scalar(G* __restrict__ grad, const P* __restrict__ p, const M* __restrict__ mask, int64_t begin, int64_t n, float alpha) {
  const int64_t i = begin + (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n) return;
  if (to_float(mask[i]) == 0.0f) {
    const float prod = to_float(p[i]) * alpha;
    grad[i] = from_float<G>(to_float(grad[i]) + prod);
  }
}

template <typename G, typename P, typename M>
int launch(void* grad, const void* p, const void* mask, int64_t n, float alpha, hipStream_t s) {
  const bool aligned = ((uintptr_t)grad % 16 == 0) && ((uintptr_t)p % 16 == 0) && ((uintptr_t)mask % 8 == 0);
  const int64_t n8 = aligned ? n / 8 : 0;
  if (n8 > 0) {
    dim3 grid((unsigned)((n8 + kThreads - 1) / kThreads));
    hipLaunchKernelGGL((masked_add_vec<G, P, M>), grid, dim3(kThreads), 0, s, (G*)grad, (const P*)p, (const M*)mask, n8, alpha);
  }
  const int64_t begin = n8 * 8;
  if (begin < n) {
    dim3 grid((unsigned)((n - begin + kThreads - 1) / kThreads));
    hipLaunchKernelGGL((masked_add_scalar<G, P, M>), grid, dim3(kThreads), 0, s, (G*)grad, (const P*)p, (const M*)mask, begin, n, alpha);
  }
  return check_launch("tf24_masked_add");
}

template <typename G, typename P>
int dispatch_mask(int mask_dtype, void* grad, const void* p, const void* mask, int64_t n, float alpha, hipStream_t s) {
  switch (mask_dtype) {
    case TF24_U8: return launch<G, P, uint8_t>(grad, p, mask, n, alpha, s);
    case TF24_F32: return launch<G, P, float>(grad, p, mask, n, alpha, s);
    case TF24_F16: return launch<G, P, f16_t>(grad, p, mask, n, alpha, s);
    case TF24_BF16: return launch<G, P, bf16_t>(grad, p, mask, n, alpha, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_masked_add: unsupported mask dtype %d", mask_dtype);
}

template <typename G>
int dispatch_p(int p_dtype, int mask_dtype, void* grad, const void* p, const void* mask, int64_t n, float alpha, hipStream_t s) {
  switch (p_dtype) {
    case TF24_F32: return dispatch_mask<G, float>(mask_dtype, grad, p, mask, n, alpha, s);
    case TF24_F16: return dispatch_mask<G, f16_t>(mask_dtype, grad, p, mask, n, alpha, s);
    case TF24_BF16: return dispatch_mask<G, bf16_t>(mask_dtype, grad, p, mask, n, alpha, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_masked_add: unsupported parameter dtype %d", p_dtype);
}

}  // namespace
}  // namespace tf24

extern "C" int tf24_masked_add(void* grad, int grad_dtype, const void* p, int p_dtype, const void* mask, int mask_dtype,
                               int64_t n, float alpha, void* stream) {
  using namespace tf24;
  if (n < 0) return fail(TF24_ERR_SHAPE, "tf24_masked_add: negative element count");
  if (n == 0) return TF24_OK;
  if (!grad || !p || !mask) return fail(TF24_ERR_ARG, "tf24_masked_add: null pointer");
  hipStream_t s = (hipStream_t)stream;
  switch (grad_dtype) {
    case TF24_F32: return dispatch_p<float>(p_dtype, mask_dtype, grad, p, mask, n, alpha, s);
    case TF24_F16: return dispatch_p<f16_t>(p_dtype, mask_dtype, grad, p, mask, n, alpha, s);
    case TF24_BF16: return dispatch_p<bf16_t>(p_dtype, mask_dtype, grad, p, mask, n, alpha, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_masked_add: unsupported gradient dtype %d", grad_dtype);
}
