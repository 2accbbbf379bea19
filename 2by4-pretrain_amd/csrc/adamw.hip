// AdamW step with the masked decay folded in, for gfx950: one pass over parameter, gradient, both
// moments and the mask instead of a masked_add_ pass over (grad, p, mask) followed by the optimizer's
// passes.  Per element, float32, every product and sum rounded separately (no fused multiply-add),
// in the order of the reference's optimizer (sparse/adamw.py:70-113) preceded by its decay
// (sparse/decay.py:27-37, applied in README.md:205-213 before optimizer.step()):
//     g  = grad (+ alpha * p where mask == 0)
//     p  = p * (1 - lr * weight_decay)
//     m  = m * beta1 + (1 - beta1) * g
//     v  = v * beta2 + ((1 - beta2) * g) * g
//     p  = p + (-(lr / bc1)) * (m / (sqrt(v) / sqrt(bc2) + eps))
// The gradient is only read.  Lane owns 4 consecutive elements (16-byte accesses of the float32
// operands).
#include "tf24_common.hpp"

namespace tf24 {
namespace {

constexpr int kThreads = 256;

struct AdamArgs {
  float decay_mul;        // 1 - lr * weight_decay
  float beta1, one_m_beta1, beta2, one_m_beta2;
  float sqrt_bc2;         // sqrt(v) is divided by it
  float eps, neg_step_size, alpha;
};

// The hyper-parameters as the caller gave them.  The per-step scalars are formed in double like the Python of the
// reference and rounded once to float32 where a tensor meets them -- on the host when the step count is a host
// number, by the first lane of every block when it lives in device memory (a recorded graph replays with the
// count of the replay, not of the recording).
struct AdamHyper {
  double lr, beta1, beta2, eps, weight_decay, alpha;
};

__host__ __device__ inline AdamArgs adam_args(const AdamHyper& h, int64_t step) {
  const double bc1 = 1.0 - pow(h.beta1, (double)step), bc2 = 1.0 - pow(h.beta2, (double)step);
  AdamArgs a;
  a.decay_mul = (float)(1.0 - h.lr * h.weight_decay);
  a.beta1 = (float)h.beta1; a.one_m_beta1 = (float)(1.0 - h.beta1);
  a.beta2 = (float)h.beta2; a.one_m_beta2 = (float)(1.0 - h.beta2);
  a.sqrt_bc2 = (float)sqrt(bc2);
  a.eps = (float)h.eps;
  a.neg_step_size = (float)(-(h.lr / bc1));
  a.alpha = (float)h.alpha;
  return a;
}

// step_dev == nullptr: `a` holds the step's scalars; otherwise they are formed here from *step_dev
__device__ __forceinline__ AdamArgs block_args(const AdamArgs& a, const AdamHyper& h, const int64_t* step_dev) {
  if (!step_dev) return a;
  __shared__ AdamArgs shared;
  if (threadIdx.x == 0) shared = adam_args(h, *step_dev);
  __syncthreads();
  return shared;
}

__device__ __forceinline__ void adam_element(float& p, float g, float& m, float& v, bool decay, const AdamArgs& a) {
  if (decay) g = g + p * a.alpha;
  p = p * a.decay_mul;
  m = m * a.beta1 + a.one_m_beta1 * g;
  v = v * a.beta2 + (a.one_m_beta2 * g) * g;
  const float denom = __builtin_sqrtf(v) / a.sqrt_bc2 + a.eps;
  p = p + a.neg_step_size * (m / denom);
}

template <typename G, typename M, bool HAS_MASK>
__global__ void __launch_bounds__(kThreads)
adamw_vec(float* __restrict__ p, const G* __restrict__ grad, float* __restrict__ m, float* __restrict__ v,
          const M* __restrict__ mask, int64_t n4, AdamArgs a_host, AdamHyper h, const int64_t* __restrict__ step_dev) {
  const AdamArgs a = block_args(a_host, h, step_dev);
  const int64_t u = (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (u >= n4) return;
  Pack<float, 4> pv, mv, vv;
  Pack<G, 4> gv;
  Pack<M, 4> mk;
  pv.load(p + u * 4); mv.load(m + u * 4); vv.load(v + u * 4); gv.load_stream(grad + u * 4);
  if constexpr (HAS_MASK) mk.load_stream(mask + u * 4);
#pragma unroll
  for (int i = 0; i < 4; i++) {
    bool decay = false;
    if constexpr (HAS_MASK) decay = to_float(mk.v[i]) == 0.0f;
    adam_element(pv.v[i], to_float(gv.v[i]), mv.v[i], vv.v[i], decay, a);
  }
  pv.store(p + u * 4); mv.store(m + u * 4); vv.store(v + u * 4);
}

template <typename G, typename M, bool HAS_MASK>
__global__ void __launch_bounds__(kThreads)
adamw_scalar(float* __restrict__ p, const G* __restrict__ grad, float* __restrict__ m, float* __restrict__ v,
             const M* __restrict__ mask, int64_t begin, int64_t n, AdamArgs a_host, AdamHyper h, const int64_t* __restrict__ step_dev) {
  const AdamArgs a = block_args(a_host, h, step_dev);
  const int64_t i = begin + (int64_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n) return;
  bool decay = false;
  if constexpr (HAS_MASK) decay = to_float(mask[i]) == 0.0f;
  float pi = p[i], mi = m[i], vi = v[i];
  adam_element(pi, to_float(grad[i]), mi, vi, decay, a);
  p[i] = pi; m[i] = mi; v[i] = vi;
}

template <typename G, typename M, bool HAS_MASK>
int launch(float* p, const void* grad, float* m, float* v, const void* mask, int64_t n, const AdamArgs& a, const AdamHyper& h,
           const int64_t* step_dev, hipStream_t s) {
  const bool aligned = ((uintptr_t)p % 16 == 0) && ((uintptr_t)m % 16 == 0) && ((uintptr_t)v % 16 == 0) &&
                       ((uintptr_t)grad % (4 * sizeof(G)) == 0) && (!HAS_MASK || (uintptr_t)mask % (4 * sizeof(M)) == 0);
  const int64_t n4 = aligned ? n / 4 : 0;
  if (n4 > 0) {
    dim3 grid((unsigned)((n4 + kThreads - 1) / kThreads));
    hipLaunchKernelGGL((adamw_vec<G, M, HAS_MASK>), grid, dim3(kThreads), 0, s, p, (const G*)grad, m, v, (const M*)mask, n4, a, h, step_dev);
  }
  const int64_t begin = n4 * 4;
  if (begin < n) {
    dim3 grid((unsigned)((n - begin + kThreads - 1) / kThreads));
    hipLaunchKernelGGL((adamw_scalar<G, M, HAS_MASK>), grid, dim3(kThreads), 0, s, p, (const G*)grad, m, v, (const M*)mask, begin, n, a, h, step_dev);
  }
  return check_launch("tf24_adamw_masked_decay");
}

template <typename G>
int dispatch_mask(const void* mask, int mask_dtype, float* p, const void* grad, float* m, float* v, int64_t n, const AdamArgs& a,
                  const AdamHyper& h, const int64_t* step_dev, hipStream_t s) {
  if (!mask) return launch<G, uint8_t, false>(p, grad, m, v, nullptr, n, a, h, step_dev, s);
  switch (mask_dtype) {
    case TF24_U8: return launch<G, uint8_t, true>(p, grad, m, v, mask, n, a, h, step_dev, s);
    case TF24_F32: return launch<G, float, true>(p, grad, m, v, mask, n, a, h, step_dev, s);
    case TF24_F16: return launch<G, f16_t, true>(p, grad, m, v, mask, n, a, h, step_dev, s);
    case TF24_BF16: return launch<G, bf16_t, true>(p, grad, m, v, mask, n, a, h, step_dev, s);
  }
  return fail(TF24_ERR_DTYPE, "tf24_adamw_masked_decay: unsupported mask dtype %d", mask_dtype);
}

}  // namespace
}  // namespace tf24

// step_host >= 1 with step_dev == nullptr, or step_dev (device memory) and step_host ignored
static int adamw_masked_decay(const char* fn, float* p, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                              const void* mask, int mask_dtype, int64_t n, double lr, double beta1, double beta2, double eps,
                              double weight_decay, double decay_alpha, int64_t step_host, const int64_t* step_dev, void* stream) {
  using namespace tf24;
  if (n < 0) return fail(TF24_ERR_SHAPE, "%s: negative element count", fn);
  if (n == 0) return TF24_OK;
  if (!p || !grad || !exp_avg || !exp_avg_sq) return fail(TF24_ERR_ARG, "%s: null pointer", fn);
  if (!step_dev && step_host < 1) return fail(TF24_ERR_ARG, "%s: step %lld must be >= 1", fn, (long long)step_host);
  if (step_dev && (uintptr_t)step_dev % 8 != 0) return fail(TF24_ERR_STRIDE, "%s: the step count must be 8-byte aligned", fn);
  if (!(lr >= 0.0) || !(eps >= 0.0) || !(beta1 >= 0.0 && beta1 < 1.0) || !(beta2 >= 0.0 && beta2 < 1.0))
    return fail(TF24_ERR_ARG, "%s: invalid hyper-parameter (lr %g, eps %g, betas %g %g)", fn, lr, eps, beta1, beta2);
  const AdamHyper h{lr, beta1, beta2, eps, weight_decay, decay_alpha};
  const AdamArgs a = adam_args(h, step_dev ? 1 : step_host);
  hipStream_t s = (hipStream_t)stream;
  switch (grad_dtype) {
    case TF24_F32: return dispatch_mask<float>(mask, mask_dtype, p, grad, exp_avg, exp_avg_sq, n, a, h, step_dev, s);
    case TF24_F16: return dispatch_mask<f16_t>(mask, mask_dtype, p, grad, exp_avg, exp_avg_sq, n, a, h, step_dev, s);
    case TF24_BF16: return dispatch_mask<bf16_t>(mask, mask_dtype, p, grad, exp_avg, exp_avg_sq, n, a, h, step_dev, s);
  }
  return fail(TF24_ERR_DTYPE, "%s: unsupported gradient dtype %d", fn, grad_dtype);
}

extern "C" int tf24_adamw_masked_decay(float* p, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                                       const void* mask, int mask_dtype, int64_t n, double lr, double beta1, double beta2,
                                       double eps, double weight_decay, double decay_alpha, int64_t step, void* stream) {
  return adamw_masked_decay("tf24_adamw_masked_decay", p, grad, grad_dtype, exp_avg, exp_avg_sq, mask, mask_dtype, n, lr, beta1, beta2,
                            eps, weight_decay, decay_alpha, step, nullptr, stream);
}

extern "C" int tf24_adamw_masked_decay_device_step(float* p, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                                                   const void* mask, int mask_dtype, int64_t n, double lr, double beta1,
                                                   double beta2, double eps, double weight_decay, double decay_alpha,
                                                   const int64_t* step, void* stream) {
  if (!step) return tf24::fail(TF24_ERR_ARG, "tf24_adamw_masked_decay_device_step: null step pointer");
  return adamw_masked_decay("tf24_adamw_masked_decay_device_step", p, grad, grad_dtype, exp_avg, exp_avg_sq, mask, mask_dtype, n, lr,
                            beta1, beta2, eps, weight_decay, decay_alpha, 0, step, stream);
}
