// The update of the STEP optimizer (AdamW with a frozen-variance second phase) for gfx950, one pass
// per tensor.  Per element, float32, every product and sum rounded separately, in the order of
// sparse/adamw_step.py:84-148:
//     p  = p * (1 - lr * weight_decay)
//     m  = m * beta1 + (1 - beta1) * g
//     v' = v * beta2 + ((1 - beta2) * g) * g
//     phase 1:            denom = sqrt(v') / sqrt(bc2) + eps          (amsgrad: of max(vmax, v'))
//     phase 2 (precond):  denom = sqrt(precond) + eps^(3/4)           (the variance frozen at the switch)
//     p  = p + (-(lr / bc1)) * (m / denom)
// In phase 1 the optimizer also needs Z = a mean over all tracked elements of |v' - v| (option 1) or of
// log|v' - v| (option 2, a geometric mean after exp): every block of 1024 elements leaves the sum of
// its terms in z_partial[block] (lanes, waves and blocks are added in a fixed order), so the old
// variance is never copied.
#include "tf24_common.hpp"

namespace tf24 {
namespace {

constexpr int kThreads = 256;
constexpr int kPerBlock = kThreads * 4;

struct StepArgs {
  float decay_mul, beta1, one_m_beta1, beta2, one_m_beta2, sqrt_bc2, eps, eps34, neg_step_size;
  int z_option;      // 0: no statistic, 1: |dv|, 2: log|dv|
};

// returns this element's term of the statistic
__device__ __forceinline__ float step_element(float& p, float g, float& m, float& v, float* vmax, const float* precond,
                                              const StepArgs& a) {
  p = p * a.decay_mul;
  m = m * a.beta1 + a.one_m_beta1 * g;
  const float v_old = v;
  v = v * a.beta2 + (a.one_m_beta2 * g) * g;
  float denom;
  if (precond) {
    denom = __builtin_sqrtf(*precond) + a.eps34;
  } else {
    float second = v;
    if (vmax) { *vmax = *vmax > v ? *vmax : v; second = *vmax; }
    denom = __builtin_sqrtf(second) / a.sqrt_bc2 + a.eps;
  }
  p = p + a.neg_step_size * (m / denom);
  if (a.z_option == 0) return 0.0f;
  const float dv = __builtin_fabsf(v - v_old);
  return a.z_option == 1 ? dv : logf(dv);
}

// VEC: 16-byte accesses (all pointers 16-byte aligned, gradient 4-element aligned); otherwise the
// same lane -> element mapping with scalar accesses, so that block b always covers elements
// [1024 b, 1024 b + 1024) and the partial sums do not depend on the variant.
template <typename G, bool VEC>
__global__ void __launch_bounds__(kThreads)
adamw_step_kernel(float* __restrict__ p, const G* __restrict__ grad, float* __restrict__ m, float* __restrict__ v,
                  float* __restrict__ vmax, const float* __restrict__ precond, int64_t n, StepArgs a,
                  float* __restrict__ z_partial) {
  const int64_t e0 = ((int64_t)blockIdx.x * kThreads + threadIdx.x) * 4;
  float z = 0.0f;
  if (e0 < n) {
    if (VEC && e0 + 4 <= n) {
      Pack<float, 4> pv, mv, vv, xv, cv;
      Pack<G, 4> gv;
      pv.load(p + e0); mv.load(m + e0); vv.load(v + e0); gv.load_stream(grad + e0);
      if (vmax) xv.load(vmax + e0);
      if (precond) cv.load(precond + e0);
#pragma unroll
      for (int i = 0; i < 4; i++)
        z += step_element(pv.v[i], to_float(gv.v[i]), mv.v[i], vv.v[i], vmax ? &xv.v[i] : nullptr, precond ? &cv.v[i] : nullptr, a);
      pv.store(p + e0); mv.store(m + e0); vv.store(v + e0);
      if (vmax) xv.store(vmax + e0);
    } else {
      for (int i = 0; i < 4 && e0 + i < n; i++) {
        const int64_t e = e0 + i;
        float pe = p[e], me = m[e], ve = v[e], xe = vmax ? vmax[e] : 0.0f, ce = precond ? precond[e] : 0.0f;
        z += step_element(pe, to_float(grad[e]), me, ve, vmax ? &xe : nullptr, precond ? &ce : nullptr, a);
        p[e] = pe; m[e] = me; v[e] = ve;
        if (vmax) vmax[e] = xe;
      }
    }
  }
  if (!z_partial) return;
  // lanes -> wave (butterfly order is fixed), waves -> block in wave order
  __shared__ float s_wave[kThreads / 64];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) z += __shfl_down(z, off);
  if ((threadIdx.x & 63) == 0) s_wave[threadIdx.x >> 6] = z;
  __syncthreads();
  if (threadIdx.x == 0) z_partial[blockIdx.x] = ((s_wave[0] + s_wave[1]) + s_wave[2]) + s_wave[3];
}

template <typename G>
int launch(float* p, const void* grad, float* m, float* v, float* vmax, const float* precond, int64_t n, const StepArgs& a,
           float* z_partial, hipStream_t s) {
  const uintptr_t all = (uintptr_t)p | (uintptr_t)m | (uintptr_t)v | (uintptr_t)vmax | (uintptr_t)precond;
  const bool vec = all % 16 == 0 && (uintptr_t)grad % (4 * sizeof(G)) == 0;
  dim3 grid((unsigned)((n + kPerBlock - 1) / kPerBlock));
  if (vec) hipLaunchKernelGGL((adamw_step_kernel<G, true>), grid, dim3(kThreads), 0, s, p, (const G*)grad, m, v, vmax, precond, n, a, z_partial);
  else hipLaunchKernelGGL((adamw_step_kernel<G, false>), grid, dim3(kThreads), 0, s, p, (const G*)grad, m, v, vmax, precond, n, a, z_partial);
  return check_launch("tf24_adamw_step");
}

}  // namespace
}  // namespace tf24

extern "C" int64_t tf24_adamw_step_partials(int64_t n) { return n > 0 ? (n + tf24::kPerBlock - 1) / tf24::kPerBlock : 0; }

extern "C" int tf24_adamw_step(float* p, const void* grad, int grad_dtype, float* exp_avg, float* exp_avg_sq,
                               float* max_exp_avg_sq, const float* precond_variance, int64_t n,
                               double lr, double beta1, double beta2, double eps, double weight_decay, int64_t step,
                               float* z_partial, int z_option, void* stream) {
  using namespace tf24;
  const char* fn = "tf24_adamw_step";
  if (n < 0) return fail(TF24_ERR_SHAPE, "%s: negative element count", fn);
  if (n == 0) return TF24_OK;
  if (n > (int64_t)0x7fffffff * kPerBlock) return fail(TF24_ERR_SHAPE, "%s: tensor too large", fn);
  if (!p || !grad || !exp_avg || !exp_avg_sq) return fail(TF24_ERR_ARG, "%s: null pointer", fn);
  if (step < 1) return fail(TF24_ERR_ARG, "%s: step %lld must be >= 1", fn, (long long)step);
  if (!(lr >= 0.0) || !(eps >= 0.0) || !(beta1 >= 0.0 && beta1 < 1.0) || !(beta2 >= 0.0 && beta2 < 1.0))
    return fail(TF24_ERR_ARG, "%s: invalid hyper-parameter (lr %g, eps %g, betas %g %g)", fn, lr, eps, beta1, beta2);
  if (z_option < 0 || z_option > 2) return fail(TF24_ERR_ARG, "%s: bad statistic option %d", fn, z_option);
  if ((z_option != 0) != (z_partial != nullptr)) return fail(TF24_ERR_ARG, "%s: the statistic needs a z_partial buffer, and only then", fn);
  if (int rc = check_aligned(fn, 4, {p, exp_avg, exp_avg_sq, max_exp_avg_sq, precond_variance, z_partial})) return rc;
  const double bc1 = 1.0 - pow(beta1, (double)step), bc2 = 1.0 - pow(beta2, (double)step);
  StepArgs a;
  a.decay_mul = (float)(1.0 - lr * weight_decay);
  a.beta1 = (float)beta1; a.one_m_beta1 = (float)(1.0 - beta1);
  a.beta2 = (float)beta2; a.one_m_beta2 = (float)(1.0 - beta2);
  a.sqrt_bc2 = (float)sqrt(bc2);
  a.eps = (float)eps;
  a.eps34 = (float)(sqrt(eps) * sqrt(sqrt(eps)));
  a.neg_step_size = (float)(-(lr / bc1));
  a.z_option = z_option;
  hipStream_t s = (hipStream_t)stream;
  switch (grad_dtype) {
    case TF24_F32: return launch<float>(p, grad, exp_avg, exp_avg_sq, max_exp_avg_sq, precond_variance, n, a, z_partial, s);
    case TF24_F16: return launch<f16_t>(p, grad, exp_avg, exp_avg_sq, max_exp_avg_sq, precond_variance, n, a, z_partial, s);
    case TF24_BF16: return launch<bf16_t>(p, grad, exp_avg, exp_avg_sq, max_exp_avg_sq, precond_variance, n, a, z_partial, s);
  }
  return fail(TF24_ERR_DTYPE, "%s: unsupported gradient dtype %d", fn, grad_dtype);
}
