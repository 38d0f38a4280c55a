// Cross-entropy over the vocabulary: one workgroup per token row.
//   forward : lse = logsumexp(row), loss = lse - row[target]      (one read of the logits)
//   backward: dlogits = (exp(row - lse) - onehot(target)) * scale  (one read, one write)
// fp32 arithmetic on bf16 or fp32 logits; rows whose target equals ignore_index -- or lies outside [0, vocab), which
// no load may follow -- contribute nothing: loss 0, gradient row 0.
#include "common.h"

namespace pico {
namespace {

constexpr int kThreads = 512;
constexpr int kWaves = kThreads / kWave;
// The logits of a training step are far larger than the caches, so they are read with streaming loads and dlogits
// leave with streaming stores (forward +13 %, backward +6 % at [4096, 49152]); a thread requests several pieces of its
// row before it uses the first (bytes in flight per thread: forward 2, backward 4 pieces).
constexpr bool kStreamLoads = true, kStreamStores = true;
constexpr int kFwdUnroll = 2, kBwdUnroll = 4;

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void ce_fwd_kernel(const T* __restrict__ logits, const int64_t* __restrict__ targets,
                                                          float* __restrict__ loss, float* __restrict__ lse_out,
                                                          int vocab, int64_t ld, int64_t ignore_index) {
  constexpr int V = io<T>::kVec;
  __shared__ float red_m[kWaves], red_s[kWaves];
  const int64_t row = blockIdx.x;
  const T* x = logits + row * ld;
  const int nvec = vocab / V;
  // online (max, sum of exp) per thread, in the log2 domain
  float m = -INFINITY, s = 0.f;
  auto absorb = [&](const float (&e)[V]) {
    float mx = e[0];
#pragma unroll
    for (int i = 1; i < V; ++i) mx = fmaxf(mx, e[i]);
    mx *= kLog2e;
    if (mx > m) { s *= fast_exp2(m - mx); m = mx; }
#pragma unroll
    for (int i = 0; i < V; ++i) s += fast_exp2(e[i] * kLog2e - m);
  };
  constexpr int U = kFwdUnroll;   // pieces of the row requested together (bytes in flight per thread)
  int v = threadIdx.x;
  for (; v + (U - 1) * kThreads < nvec; v += U * kThreads) {
    float e[U][V];
#pragma unroll
    for (int u = 0; u < U; ++u) load_as<T, kStreamLoads>(x + static_cast<int64_t>(v + u * kThreads) * V, e[u]);
#pragma unroll
    for (int u = 0; u < U; ++u) absorb(e[u]);
  }
  for (; v < nvec; v += kThreads) {
    float e[V];
    load_as<T, kStreamLoads>(x + static_cast<int64_t>(v) * V, e);
    absorb(e);
  }
  for (int j = nvec * V + threadIdx.x; j < vocab; j += kThreads) {  // tail when vocab is not a multiple of V
    const float e = static_cast<float>(x[j]) * kLog2e;
    if (e > m) { s *= fast_exp2(m - e); m = e; }
    s += fast_exp2(e - m);
  }
  const float wm = wave_max(m);
  s = (m == -INFINITY) ? 0.f : s * fast_exp2(m - wm);
  s = wave_sum(s);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (lane == 0) { red_m[wave] = wm; red_s[wave] = s; }
  __syncthreads();
  if (threadIdx.x == 0) {
    float bm = red_m[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) bm = fmaxf(bm, red_m[w]);
    float bs = 0.f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) bs += (red_m[w] == -INFINITY) ? 0.f : red_s[w] * fast_exp2(red_m[w] - bm);
    const float lse = (bm + fast_log2(bs)) * kLn2;
    const int64_t t = targets[row];
    lse_out[row] = lse;
    const bool counts = t != ignore_index && t >= 0 && t < vocab;
    loss[row] = counts ? lse - static_cast<float>(x[t]) : 0.f;
  }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void ce_bwd_kernel(const T* __restrict__ logits, const int64_t* __restrict__ targets,
                                                          const float* __restrict__ lse, const float* __restrict__ scale_ptr,
                                                          T* __restrict__ dlogits, int vocab, int64_t ld, int64_t dld,
                                                          int64_t ignore_index) {
  constexpr int V = io<T>::kVec;
  const int64_t row = blockIdx.x;
  const T* x = logits + row * ld;
  T* d = dlogits + row * dld;
  const int64_t t = targets[row];
  const float scale = (t != ignore_index && t >= 0 && t < vocab) ? *scale_ptr : 0.f;
  const float l2 = lse[row] * kLog2e;
  const int nvec = vocab / V;
  // kCeUnroll pieces of the row per thread are requested before the first is used: one 16-byte load per thread at a
  // time leaves too few bytes in flight to cover the memory latency
  constexpr int U = kBwdUnroll;
  int v = threadIdx.x;
  for (; v + (U - 1) * kThreads < nvec; v += U * kThreads) {
    float e[U][V];
#pragma unroll
    for (int u = 0; u < U; ++u) load_as<T, kStreamLoads>(x + static_cast<int64_t>(v + u * kThreads) * V, e[u]);
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float o[V];
      const int j0 = (v + u * kThreads) * V;
#pragma unroll
      for (int i = 0; i < V; ++i) {
        const float p = fast_exp2(e[u][i] * kLog2e - l2);
        o[i] = (p - ((j0 + i) == t ? 1.f : 0.f)) * scale;
      }
      store_as<T, kStreamStores>(d + static_cast<int64_t>(v + u * kThreads) * V, o);
    }
  }
  for (; v < nvec; v += kThreads) {
    float e[V], o[V];
    load_as<T, kStreamLoads>(x + static_cast<int64_t>(v) * V, e);
    const int j0 = v * V;
#pragma unroll
    for (int i = 0; i < V; ++i) {
      const float p = fast_exp2(e[i] * kLog2e - l2);
      o[i] = (p - ((j0 + i) == t ? 1.f : 0.f)) * scale;
    }
    store_as<T, kStreamStores>(d + static_cast<int64_t>(v) * V, o);
  }
  for (int j = nvec * V + threadIdx.x; j < vocab; j += kThreads) {
    const float p = fast_exp2(static_cast<float>(x[j]) * kLog2e - l2);
    d[j] = static_cast<T>((p - (j == t ? 1.f : 0.f)) * scale);
  }
}

int check_ce(const char* fn, int64_t rows, int64_t vocab, int64_t ld, int dtype) {
  if (dtype != PICO_BF16 && dtype != PICO_F32) return fail(PICO_ERR_DTYPE, "%s: dtype code %d not supported", fn, dtype);
  const int vec = dtype == PICO_BF16 ? 8 : 4;
  if (rows < 0 || vocab <= 0 || vocab > 0x7fffffff) return fail(PICO_ERR_SHAPE, "%s: rows=%lld vocab=%lld", fn,
                                                                static_cast<long long>(rows), static_cast<long long>(vocab));
  if (ld < vocab || ld % vec != 0) return fail(PICO_ERR_STRIDE, "%s: row pitch %lld must be >= vocab and a multiple of %d",
                                               fn, static_cast<long long>(ld), vec);
  return PICO_OK;
}

}  // namespace
}  // namespace pico

using namespace pico;

extern "C" int pico_cross_entropy_fwd(const void* logits, const int64_t* targets, float* loss, float* lse, int64_t rows,
                                      int64_t vocab, int64_t ld, int64_t ignore_index, int dtype, void* stream) {
  if (int rc = check_ce("pico_cross_entropy_fwd", rows, vocab, ld, dtype)) return rc;
  if (rows == 0) return PICO_OK;
  if (!logits || !targets || !loss || !lse) return fail(PICO_ERR_NULL, "pico_cross_entropy_fwd: logits, targets, loss and lse are required");
  if (!aligned16(logits)) return fail(PICO_ERR_ALIGN, "pico_cross_entropy_fwd: logits must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == PICO_BF16)
    hipLaunchKernelGGL(ce_fwd_kernel<__bf16>, dim3(static_cast<unsigned>(rows)), dim3(kThreads), 0, s,
                       static_cast<const __bf16*>(logits), targets, loss, lse, static_cast<int>(vocab), ld, ignore_index);
  else
    hipLaunchKernelGGL(ce_fwd_kernel<float>, dim3(static_cast<unsigned>(rows)), dim3(kThreads), 0, s,
                       static_cast<const float*>(logits), targets, loss, lse, static_cast<int>(vocab), ld, ignore_index);
  return check_launch("pico_cross_entropy_fwd");
}

extern "C" int pico_cross_entropy_bwd(const void* logits, const int64_t* targets, const float* lse, const float* scale,
                                      void* dlogits, int64_t rows, int64_t vocab, int64_t ld, int64_t dld,
                                      int64_t ignore_index, int dtype, void* stream) {
  if (int rc = check_ce("pico_cross_entropy_bwd", rows, vocab, ld, dtype)) return rc;
  if (int rc = check_ce("pico_cross_entropy_bwd", rows, vocab, dld, dtype)) return rc;
  if (rows == 0) return PICO_OK;
  if (!logits || !targets || !lse || !scale || !dlogits)
    return fail(PICO_ERR_NULL, "pico_cross_entropy_bwd: logits, targets, lse, scale and dlogits are required");
  if (!aligned16(logits) || !aligned16(dlogits)) return fail(PICO_ERR_ALIGN, "pico_cross_entropy_bwd: logits and dlogits must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == PICO_BF16)
    hipLaunchKernelGGL(ce_bwd_kernel<__bf16>, dim3(static_cast<unsigned>(rows)), dim3(kThreads), 0, s,
                       static_cast<const __bf16*>(logits), targets, lse, scale, static_cast<__bf16*>(dlogits),
                       static_cast<int>(vocab), ld, dld, ignore_index);
  else
    hipLaunchKernelGGL(ce_bwd_kernel<float>, dim3(static_cast<unsigned>(rows)), dim3(kThreads), 0, s,
                       static_cast<const float*>(logits), targets, lse, scale, static_cast<float*>(dlogits),
                       static_cast<int>(vocab), ld, dld, ignore_index);
  return check_launch("pico_cross_entropy_bwd");
}
