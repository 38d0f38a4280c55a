// AdamW steps as one streaming pass per parameter tensor; nothing is read twice.
//   pico_adamw     fp32 master weights and moments for low-precision parameters: reads the gradient, the master
//                  weight and both moments, writes the three fp32 states plus the bf16 copy of the parameter that the
//                  model computes with.  28 bytes per parameter with a bf16 gradient.
//   pico_adamw_lp  parameter and both moments kept in bf16 and updated in place (what torch.optim.AdamW holds for a
//                  bf16 model): the arithmetic is fp32 and every state is rounded once.  14 bytes per parameter.
#include "common.h"

namespace pico {
namespace {

constexpr int kThreads = 256;
constexpr int kPerThread = 8;  // elements: one 16-byte bf16 vector, two 16-byte fp32 vectors per state

__device__ __forceinline__ void load8(const float* p, float (&out)[8]) {
  const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
#pragma unroll
  for (int i = 0; i < 4; ++i) { out[i] = a[i]; out[4 + i] = b[i]; }
}
__device__ __forceinline__ void store8(float* p, const float (&in)[8]) {
  f32x4 a, b;
#pragma unroll
  for (int i = 0; i < 4; ++i) { a[i] = in[i]; b[i] = in[4 + i]; }
  *reinterpret_cast<f32x4*>(p) = a;
  *reinterpret_cast<f32x4*>(p + 4) = b;
}
__device__ __forceinline__ void load8(const __bf16* p, float (&out)[8]) { io<__bf16>::load(p, out); }
__device__ __forceinline__ void store8(__bf16* p, const float (&in)[8]) { io<__bf16>::store(p, in); }

// The arithmetic follows torch.optim.AdamW's (non-amsgrad) order of operations so that fp32 states match it to
// rounding: p *= 1 - lr*wd;  m = m + (g - m)*(1 - b1);  v = v*b2 + g*g*(1 - b2);
// p -= step_size * m / (sqrt(v) / sqrt(bc2) + eps),  step_size = lr / bc1.
// TS is the type of the three states (the weight that is updated and both moments); param_lp, when given, receives
// a bf16 copy of the updated weight.
template <typename TS, typename TG>
__global__ __launch_bounds__(kThreads) void adamw_kernel(__bf16* __restrict__ param_lp, TS* __restrict__ master,
                                                         const TG* __restrict__ grad, TS* __restrict__ exp_avg,
                                                         TS* __restrict__ exp_avg_sq, int64_t n, float decay,
                                                         float one_minus_b1, float b2, float one_minus_b2,
                                                         float step_size, float inv_sqrt_bc2, float eps,
                                                         float grad_scale) {
  const int64_t i0 = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) * kPerThread;
  if (i0 >= n) return;
  float g[kPerThread], p[kPerThread], m[kPerThread], v[kPerThread];
  if (i0 + kPerThread <= n) {
    load8(grad + i0, g);
    load8(master + i0, p);
    load8(exp_avg + i0, m);
    load8(exp_avg_sq + i0, v);
  } else {
    for (int e = 0; e < kPerThread; ++e) {
      const bool in = i0 + e < n;
      g[e] = in ? static_cast<float>(grad[i0 + e]) : 0.f;
      p[e] = in ? static_cast<float>(master[i0 + e]) : 0.f;
      m[e] = in ? static_cast<float>(exp_avg[i0 + e]) : 0.f;
      v[e] = in ? static_cast<float>(exp_avg_sq[i0 + e]) : 0.f;
    }
  }
#pragma unroll
  for (int e = 0; e < kPerThread; ++e) {
    const float ge = g[e] * grad_scale;
    p[e] = p[e] * decay;
    m[e] = m[e] + (ge - m[e]) * one_minus_b1;
    v[e] = v[e] * b2 + ge * ge * one_minus_b2;
    const float denom = __builtin_sqrtf(v[e]) * inv_sqrt_bc2 + eps;
    p[e] = p[e] - step_size * (m[e] / denom);
  }
  if (i0 + kPerThread <= n) {
    store8(master + i0, p);
    store8(exp_avg + i0, m);
    store8(exp_avg_sq + i0, v);
    if (param_lp) io<__bf16>::store(param_lp + i0, p);
  } else {
    for (int e = 0; e < kPerThread && i0 + e < n; ++e) {
      master[i0 + e] = static_cast<TS>(p[e]);
      exp_avg[i0 + e] = static_cast<TS>(m[e]);
      exp_avg_sq[i0 + e] = static_cast<TS>(v[e]);
      if (param_lp) param_lp[i0 + e] = static_cast<__bf16>(p[e]);
    }
  }
}

}  // namespace
}  // namespace pico

using namespace pico;

namespace {

template <typename TS>
int adamw_launch(const char* who, void* param_lp, TS* master, const void* grad, int grad_dtype, TS* exp_avg,
                 TS* exp_avg_sq, int64_t n, float lr, float beta1, float beta2, float eps, float weight_decay,
                 int64_t step, float grad_scale, void* stream) {
  if (grad_dtype != PICO_BF16 && grad_dtype != PICO_F32)
    return fail(PICO_ERR_DTYPE, "%s: gradient dtype code %d not supported", who, grad_dtype);
  if (n < 0 || step < 1) return fail(PICO_ERR_SHAPE, "%s: n=%lld must be >= 0 and step=%lld >= 1", who,
                                     static_cast<long long>(n), static_cast<long long>(step));
  if (n == 0) return PICO_OK;
  if (!master || !grad || !exp_avg || !exp_avg_sq)
    return fail(PICO_ERR_NULL, "%s: the weight, grad, exp_avg and exp_avg_sq are required", who);
  if (!aligned16(param_lp) || !aligned16(master) || !aligned16(grad) || !aligned16(exp_avg) || !aligned16(exp_avg_sq))
    return fail(PICO_ERR_ALIGN, "%s: pointers must be 16-byte aligned", who);
  // bias corrections in double, as torch computes them on the host
  const double bc1 = 1.0 - __builtin_pow(static_cast<double>(beta1), static_cast<double>(step));
  const double bc2 = 1.0 - __builtin_pow(static_cast<double>(beta2), static_cast<double>(step));
  const float step_size = static_cast<float>(static_cast<double>(lr) / bc1);
  const float inv_sqrt_bc2 = static_cast<float>(1.0 / __builtin_sqrt(bc2));
  const float decay = 1.f - lr * weight_decay;
  const int64_t per_block = static_cast<int64_t>(kThreads) * kPerThread;
  const unsigned grid = static_cast<unsigned>((n + per_block - 1) / per_block);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (grad_dtype == PICO_BF16)
    hipLaunchKernelGGL((adamw_kernel<TS, __bf16>), dim3(grid), dim3(kThreads), 0, s, static_cast<__bf16*>(param_lp),
                       master, static_cast<const __bf16*>(grad), exp_avg, exp_avg_sq, n, decay, 1.f - beta1, beta2,
                       1.f - beta2, step_size, inv_sqrt_bc2, eps, grad_scale);
  else
    hipLaunchKernelGGL((adamw_kernel<TS, float>), dim3(grid), dim3(kThreads), 0, s, static_cast<__bf16*>(param_lp),
                       master, static_cast<const float*>(grad), exp_avg, exp_avg_sq, n, decay, 1.f - beta1, beta2,
                       1.f - beta2, step_size, inv_sqrt_bc2, eps, grad_scale);
  return check_launch(who);
}

}  // namespace

extern "C" int pico_adamw(void* param_lp, float* master, const void* grad, int grad_dtype, float* exp_avg,
                          float* exp_avg_sq, int64_t n, float lr, float beta1, float beta2, float eps,
                          float weight_decay, int64_t step, float grad_scale, void* stream) {
  return adamw_launch<float>("pico_adamw", param_lp, master, grad, grad_dtype, exp_avg, exp_avg_sq, n, lr, beta1, beta2,
                             eps, weight_decay, step, grad_scale, stream);
}

extern "C" int pico_adamw_lp(void* param, const void* grad, int grad_dtype, void* exp_avg, void* exp_avg_sq,
                             int64_t n, int dtype, float lr, float beta1, float beta2, float eps, float weight_decay,
                             int64_t step, float grad_scale, void* stream) {
  if (dtype != PICO_BF16) return fail(PICO_ERR_DTYPE, "pico_adamw_lp: state dtype code %d not supported (bf16 only)", dtype);
  return adamw_launch<__bf16>("pico_adamw_lp", nullptr, static_cast<__bf16*>(param), grad, grad_dtype,
                              static_cast<__bf16*>(exp_avg), static_cast<__bf16*>(exp_avg_sq), n, lr, beta1, beta2, eps,
                              weight_decay, step, grad_scale, stream);
}
