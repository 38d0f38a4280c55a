// AdamW steps as one streaming pass per parameter tensor; nothing is read twice.
//   pico_adamw     fp32 master weights and moments for low-precision parameters: reads the gradient, the master
//                  weight and both moments, writes the three fp32 states plus the bf16 copy of the parameter that the
//                  model computes with.  28 bytes per parameter with a bf16 gradient.
//   pico_adamw_lp  the bf16 parameter is updated in place, no master copy; the moments are fp32 (22 bytes per
//                  parameter) or bf16 (what torch.optim.AdamW holds for a bf16 model; 14 bytes).  The arithmetic is
//                  fp32 and every stored value is rounded once.
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
// TW is the type of the weight that is updated, TM that of both moments; param_lp, when given, receives a bf16 copy
// of the updated weight.
struct Hyper {
  float decay, one_minus_b1, b2, one_minus_b2, step_size, inv_sqrt_bc2, eps, grad_scale;
};

template <typename TW, typename TM, typename TG>
__device__ __forceinline__ void adamw_block(__bf16* __restrict__ param_lp, TW* __restrict__ master,
                                            const TG* __restrict__ grad, TM* __restrict__ exp_avg,
                                            TM* __restrict__ exp_avg_sq, int64_t n, int64_t block, const Hyper& h) {
  const int64_t i0 = (block * kThreads + threadIdx.x) * kPerThread;
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
    const float ge = g[e] * h.grad_scale;
    p[e] = p[e] * h.decay;
    m[e] = m[e] + (ge - m[e]) * h.one_minus_b1;
    v[e] = v[e] * h.b2 + ge * ge * h.one_minus_b2;
    const float denom = __builtin_sqrtf(v[e]) * h.inv_sqrt_bc2 + h.eps;
    p[e] = p[e] - h.step_size * (m[e] / denom);
  }
  if (i0 + kPerThread <= n) {
    store8(master + i0, p);
    store8(exp_avg + i0, m);
    store8(exp_avg_sq + i0, v);
    if (param_lp) io<__bf16>::store(param_lp + i0, p);
  } else {
    for (int e = 0; e < kPerThread && i0 + e < n; ++e) {
      master[i0 + e] = static_cast<TW>(p[e]);
      exp_avg[i0 + e] = static_cast<TM>(m[e]);
      exp_avg_sq[i0 + e] = static_cast<TM>(v[e]);
      if (param_lp) param_lp[i0 + e] = static_cast<__bf16>(p[e]);
    }
  }
}

template <typename TW, typename TM, typename TG>
__global__ __launch_bounds__(kThreads) void adamw_kernel(__bf16* __restrict__ param_lp, TW* __restrict__ master,
                                                         const TG* __restrict__ grad, TM* __restrict__ exp_avg,
                                                         TM* __restrict__ exp_avg_sq, int64_t n, Hyper h) {
  adamw_block<TW, TM, TG>(param_lp, master, grad, exp_avg, exp_avg_sq, n, blockIdx.x, h);
}

// Many tensors in one launch: the pointers travel in the kernel arguments (no table in device memory to keep alive),
// and a workgroup finds its tensor by bisecting the running block count, which is uniform scalar work.
constexpr int kMaxTensors = 48;
struct TensorTable {
  void* weight[kMaxTensors];
  void* param_lp[kMaxTensors];
  const void* grad[kMaxTensors];
  void* exp_avg[kMaxTensors];
  void* exp_avg_sq[kMaxTensors];
  int64_t n[kMaxTensors];
  unsigned block_start[kMaxTensors + 1];
  int count;
};

template <typename TW, typename TM, typename TG>
__global__ __launch_bounds__(kThreads) void adamw_multi_kernel(TensorTable t, Hyper h) {
  const unsigned bid = blockIdx.x;
  int lo = 0, hi = t.count;   // block_start[lo] <= bid < block_start[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (bid >= t.block_start[mid]) lo = mid; else hi = mid;
  }
  adamw_block<TW, TM, TG>(static_cast<__bf16*>(t.param_lp[lo]), static_cast<TW*>(t.weight[lo]),
                          static_cast<const TG*>(t.grad[lo]), static_cast<TM*>(t.exp_avg[lo]),
                          static_cast<TM*>(t.exp_avg_sq[lo]), t.n[lo], bid - t.block_start[lo], h);
}

}  // namespace
}  // namespace pico

using namespace pico;

namespace {

int hyper_check(const char* who, int grad_dtype, int64_t step) {
  if (grad_dtype != PICO_BF16 && grad_dtype != PICO_F32)
    return fail(PICO_ERR_DTYPE, "%s: gradient dtype code %d not supported", who, grad_dtype);
  if (step < 1) return fail(PICO_ERR_SHAPE, "%s: step=%lld must be >= 1", who, static_cast<long long>(step));
  return PICO_OK;
}

Hyper make_hyper(float lr, float beta1, float beta2, float eps, float weight_decay, int64_t step, float grad_scale) {
  // bias corrections in double, as torch computes them on the host
  const double bc1 = 1.0 - __builtin_pow(static_cast<double>(beta1), static_cast<double>(step));
  const double bc2 = 1.0 - __builtin_pow(static_cast<double>(beta2), static_cast<double>(step));
  Hyper h;
  h.decay = 1.f - lr * weight_decay;
  h.one_minus_b1 = 1.f - beta1;
  h.b2 = beta2;
  h.one_minus_b2 = 1.f - beta2;
  h.step_size = static_cast<float>(static_cast<double>(lr) / bc1);
  h.inv_sqrt_bc2 = static_cast<float>(1.0 / __builtin_sqrt(bc2));
  h.eps = eps;
  h.grad_scale = grad_scale;
  return h;
}

constexpr int64_t kPerBlock = static_cast<int64_t>(kThreads) * kPerThread;

template <typename TW, typename TM>
int adamw_launch(const char* who, void* param_lp, TW* master, const void* grad, int grad_dtype, TM* exp_avg,
                 TM* exp_avg_sq, int64_t n, float lr, float beta1, float beta2, float eps, float weight_decay,
                 int64_t step, float grad_scale, void* stream) {
  if (int rc = hyper_check(who, grad_dtype, step)) return rc;
  if (n < 0) return fail(PICO_ERR_SHAPE, "%s: n=%lld must be >= 0", who, static_cast<long long>(n));
  if (n == 0) return PICO_OK;
  if (!master || !grad || !exp_avg || !exp_avg_sq)
    return fail(PICO_ERR_NULL, "%s: the weight, grad, exp_avg and exp_avg_sq are required", who);
  if (!aligned16(param_lp) || !aligned16(master) || !aligned16(grad) || !aligned16(exp_avg) || !aligned16(exp_avg_sq))
    return fail(PICO_ERR_ALIGN, "%s: pointers must be 16-byte aligned", who);
  const Hyper h = make_hyper(lr, beta1, beta2, eps, weight_decay, step, grad_scale);
  const unsigned grid = static_cast<unsigned>((n + kPerBlock - 1) / kPerBlock);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (grad_dtype == PICO_BF16)
    hipLaunchKernelGGL((adamw_kernel<TW, TM, __bf16>), dim3(grid), dim3(kThreads), 0, s, static_cast<__bf16*>(param_lp),
                       master, static_cast<const __bf16*>(grad), exp_avg, exp_avg_sq, n, h);
  else
    hipLaunchKernelGGL((adamw_kernel<TW, TM, float>), dim3(grid), dim3(kThreads), 0, s, static_cast<__bf16*>(param_lp),
                       master, static_cast<const float*>(grad), exp_avg, exp_avg_sq, n, h);
  return check_launch(who);
}

template <typename TW, typename TM>
int adamw_multi_launch(int count, void* const* weights, void* const* param_lps, const void* const* grads,
                       void* const* exp_avgs, void* const* exp_avg_sqs, const int64_t* sizes, int grad_dtype,
                       const Hyper& h, hipStream_t s) {
  const char* who = "pico_adamw_multi";
  // validate everything before the first launch so that a rejected call has changed nothing
  for (int i = 0; i < count; ++i) {
    if (sizes[i] < 0) return fail(PICO_ERR_SHAPE, "%s: tensor %d has n=%lld", who, i, static_cast<long long>(sizes[i]));
    if (sizes[i] == 0) continue;
    if (!weights[i] || !grads[i] || !exp_avgs[i] || !exp_avg_sqs[i])
      return fail(PICO_ERR_NULL, "%s: tensor %d: the weight, grad, exp_avg and exp_avg_sq are required", who, i);
    if (!aligned16(weights[i]) || !aligned16(grads[i]) || !aligned16(exp_avgs[i]) || !aligned16(exp_avg_sqs[i]) ||
        (param_lps && !aligned16(param_lps[i])))
      return fail(PICO_ERR_ALIGN, "%s: tensor %d: pointers must be 16-byte aligned", who, i);
    if ((sizes[i] + kPerBlock - 1) / kPerBlock > 0x7fffffff)
      return fail(PICO_ERR_SHAPE, "%s: tensor %d is too large for one launch", who, i);
  }
  TensorTable t;
  t.count = 0;
  t.block_start[0] = 0;
  auto flush = [&]() -> int {
    if (t.count == 0) return PICO_OK;
    const unsigned grid = t.block_start[t.count];
    if (grad_dtype == PICO_BF16)
      hipLaunchKernelGGL((adamw_multi_kernel<TW, TM, __bf16>), dim3(grid), dim3(kThreads), 0, s, t, h);
    else
      hipLaunchKernelGGL((adamw_multi_kernel<TW, TM, float>), dim3(grid), dim3(kThreads), 0, s, t, h);
    t.count = 0;
    return check_launch(who);
  };
  for (int i = 0; i < count; ++i) {
    if (sizes[i] == 0) continue;
    const uint64_t blocks = static_cast<uint64_t>((sizes[i] + kPerBlock - 1) / kPerBlock);
    if (t.count == kMaxTensors || t.block_start[t.count] + blocks > 0x7fffffffu)
      if (int rc = flush()) return rc;
    const int j = t.count++;
    t.weight[j] = weights[i];
    t.param_lp[j] = param_lps ? param_lps[i] : nullptr;
    t.grad[j] = grads[i];
    t.exp_avg[j] = exp_avgs[i];
    t.exp_avg_sq[j] = exp_avg_sqs[i];
    t.n[j] = sizes[i];
    t.block_start[j + 1] = t.block_start[j] + static_cast<unsigned>(blocks);
  }
  return flush();
}

}  // namespace

extern "C" int pico_adamw_multi(int count, void* const* weights, void* const* param_lps, const void* const* grads,
                                void* const* exp_avgs, void* const* exp_avg_sqs, const int64_t* sizes, int weight_dtype,
                                int state_dtype, int grad_dtype, float lr, float beta1, float beta2, float eps,
                                float weight_decay, int64_t step, float grad_scale, void* stream) {
  const char* who = "pico_adamw_multi";
  if (int rc = hyper_check(who, grad_dtype, step)) return rc;
  if (count < 0) return fail(PICO_ERR_SHAPE, "%s: count=%d must be >= 0", who, count);
  if (count == 0) return PICO_OK;
  if (!weights || !grads || !exp_avgs || !exp_avg_sqs || !sizes)
    return fail(PICO_ERR_NULL, "%s: the pointer tables and sizes are required", who);
  const Hyper h = make_hyper(lr, beta1, beta2, eps, weight_decay, step, grad_scale);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (weight_dtype == PICO_F32 && state_dtype == PICO_F32)
    return adamw_multi_launch<float, float>(count, weights, param_lps, grads, exp_avgs, exp_avg_sqs, sizes, grad_dtype, h, s);
  if (weight_dtype == PICO_BF16 && (state_dtype == PICO_BF16 || state_dtype == PICO_F32)) {
    if (param_lps) return fail(PICO_ERR_NULL, "%s: param_lps must be NULL when the weights are bf16 (they are the parameters)", who);
    if (state_dtype == PICO_BF16)
      return adamw_multi_launch<__bf16, __bf16>(count, weights, nullptr, grads, exp_avgs, exp_avg_sqs, sizes, grad_dtype, h, s);
    return adamw_multi_launch<__bf16, float>(count, weights, nullptr, grads, exp_avgs, exp_avg_sqs, sizes, grad_dtype, h, s);
  }
  return fail(PICO_ERR_DTYPE, "%s: weight dtype code %d with state dtype code %d not supported", who, weight_dtype, state_dtype);
}

extern "C" int pico_adamw(void* param_lp, float* master, const void* grad, int grad_dtype, float* exp_avg,
                          float* exp_avg_sq, int64_t n, float lr, float beta1, float beta2, float eps,
                          float weight_decay, int64_t step, float grad_scale, void* stream) {
  return adamw_launch<float, float>("pico_adamw", param_lp, master, grad, grad_dtype, exp_avg, exp_avg_sq, n, lr, beta1,
                                    beta2, eps, weight_decay, step, grad_scale, stream);
}

extern "C" int pico_adamw_lp(void* param, const void* grad, int grad_dtype, void* exp_avg, void* exp_avg_sq,
                             int64_t n, int param_dtype, int state_dtype, float lr, float beta1, float beta2, float eps,
                             float weight_decay, int64_t step, float grad_scale, void* stream) {
  if (param_dtype != PICO_BF16)
    return fail(PICO_ERR_DTYPE, "pico_adamw_lp: parameter dtype code %d not supported (bf16 only)", param_dtype);
  if (state_dtype == PICO_BF16)
    return adamw_launch<__bf16, __bf16>("pico_adamw_lp", nullptr, static_cast<__bf16*>(param), grad, grad_dtype,
                                        static_cast<__bf16*>(exp_avg), static_cast<__bf16*>(exp_avg_sq), n, lr, beta1,
                                        beta2, eps, weight_decay, step, grad_scale, stream);
  if (state_dtype == PICO_F32)
    return adamw_launch<__bf16, float>("pico_adamw_lp", nullptr, static_cast<__bf16*>(param), grad, grad_dtype,
                                       static_cast<float*>(exp_avg), static_cast<float*>(exp_avg_sq), n, lr, beta1, beta2,
                                       eps, weight_decay, step, grad_scale, stream);
  return fail(PICO_ERR_DTYPE, "pico_adamw_lp: state dtype code %d not supported", state_dtype);
}
