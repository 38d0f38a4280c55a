// RoPE, SwiGLU, the lse merge and the fp32 -> io-dtype conversion: pure streaming kernels.
// Every thread moves 16-byte vectors; index order is chosen on the host so that consecutive
// lanes touch consecutive memory for the layout at hand.
#include "common.h"

namespace pico {
namespace {

constexpr int kThreads = 256;
// Streaming (non-temporal) accesses only where they measured faster: the SwiGLU backward's two outputs (+28 % on warm
// data).  RoPE and the SwiGLU forward are slower with them on the warm data a training step hands these kernels.
constexpr bool kStreamRopeLoads = false, kStreamRopeStores = false, kStreamSwigluLoads = false,
               kStreamSwigluFwdStores = false, kStreamSwigluBwdStores = true;

// ---------------------------------------------------------------------------------- RoPE
// One thread rotates V pairs (x[i], x[i + D/2]).  Work items are numbered (b, o, i, v) with
// v fastest; (o, i) is (s, h) when the h stride is the smaller one ([B,S,H,D] memory) and
// (h, s) otherwise ([B,H,S,D] memory).
template <typename T, typename TT>
__global__ __launch_bounds__(kThreads) void rope_kernel(
    const T* __restrict__ x, T* __restrict__ y, const TT* __restrict__ cos_t, const TT* __restrict__ sin_t,
    int64_t total, int H, int S, int D, int64_t xsb, int64_t xsh, int64_t xss, int64_t ysb, int64_t ysh,
    int64_t yss, int64_t table_ld, int64_t pos_offset, int inverse, int s_outer) {
  constexpr int V = io<T>::kVec;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  const int half = D / 2;
  const int vpr = half / V;  // vectors per half row
  const int v = static_cast<int>(idx % vpr);
  int64_t rest = idx / vpr;
  int h, s;
  if (s_outer) {
    h = static_cast<int>(rest % H); rest /= H;
    s = static_cast<int>(rest % S); rest /= S;
  } else {
    s = static_cast<int>(rest % S); rest /= S;
    h = static_cast<int>(rest % H); rest /= H;
  }
  const int64_t b = rest;
  const T* xp = x + b * xsb + h * xsh + s * xss + v * V;
  T* yp = y + b * ysb + h * ysh + s * yss + v * V;
  float lo[V], hi[V], c[V], sn[V];
  load_as<T, kStreamRopeLoads>(xp, lo);
  load_as<T, kStreamRopeLoads>(xp + half, hi);
  const int64_t trow = (pos_offset + s) * table_ld + v * V;
  if constexpr (io<TT>::kVec == V) {
    io<TT>::load(cos_t + trow, c);
    io<TT>::load(sin_t + trow, sn);
  } else if constexpr (io<TT>::kVec < V) {  // fp32 table, bf16 data: two 16-byte loads per table
    float t0[4], t1[4];
    io<TT>::load(cos_t + trow, t0); io<TT>::load(cos_t + trow + 4, t1);
#pragma unroll
    for (int e = 0; e < 4; ++e) { c[e] = t0[e]; c[e + 4] = t1[e]; }
    io<TT>::load(sin_t + trow, t0); io<TT>::load(sin_t + trow + 4, t1);
#pragma unroll
    for (int e = 0; e < 4; ++e) { sn[e] = t0[e]; sn[e + 4] = t1[e]; }
  } else {  // bf16 table, fp32 data: V = 4 elements = 8 bytes of table
    const u32x2 rc = *reinterpret_cast<const u32x2*>(cos_t + trow);
    const u32x2 rs = *reinterpret_cast<const u32x2*>(sin_t + trow);
#pragma unroll
    for (int e = 0; e < 2; ++e) {
      c[2 * e] = __uint_as_float(rc[e] << 16); c[2 * e + 1] = __uint_as_float(rc[e] & 0xffff0000u);
      sn[2 * e] = __uint_as_float(rs[e] << 16); sn[2 * e + 1] = __uint_as_float(rs[e] & 0xffff0000u);
    }
  }
  float olo[V], ohi[V];
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const float sg = inverse ? -sn[e] : sn[e];
    olo[e] = lo[e] * c[e] - hi[e] * sg;
    ohi[e] = hi[e] * c[e] + lo[e] * sg;
  }
  store_as<T, kStreamRopeStores>(yp, olo);
  store_as<T, kStreamRopeStores>(yp + half, ohi);
}

// ---------------------------------------------------------------------------------- SwiGLU
__device__ __forceinline__ float sigmoidf_fast(float x) { return fast_rcp(1.f + fast_exp2(-x * kLog2e)); }

template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_fwd_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                                              T* __restrict__ y, int64_t total, int vpr,
                                                              int64_t gld, int64_t uld, int64_t yld) {
  constexpr int V = io<T>::kVec;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  const int64_t r = idx / vpr;
  const int64_t c = (idx % vpr) * V;
  float g[V], u[V], o[V];
  load_as<T, kStreamSwigluLoads>(gate + r * gld + c, g);
  load_as<T, kStreamSwigluLoads>(up + r * uld + c, u);
#pragma unroll
  for (int e = 0; e < V; ++e) o[e] = g[e] * sigmoidf_fast(g[e]) * u[e];
  store_as<T, kStreamSwigluFwdStores>(y + r * yld + c, o);
}

template <typename T>
__global__ __launch_bounds__(kThreads) void swiglu_bwd_kernel(const T* __restrict__ dy, const T* __restrict__ gate,
                                                              const T* __restrict__ up, T* __restrict__ dgate,
                                                              T* __restrict__ dup, int64_t total, int vpr,
                                                              int64_t dyld, int64_t gld, int64_t uld, int64_t dgld,
                                                              int64_t duld) {
  constexpr int V = io<T>::kVec;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  const int64_t r = idx / vpr;
  const int64_t c = (idx % vpr) * V;
  float d[V], g[V], u[V], og[V], ou[V];
  load_as<T, kStreamSwigluLoads>(dy + r * dyld + c, d);
  load_as<T, kStreamSwigluLoads>(gate + r * gld + c, g);
  load_as<T, kStreamSwigluLoads>(up + r * uld + c, u);
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const float sg = sigmoidf_fast(g[e]);
    const float silu = g[e] * sg;
    og[e] = d[e] * u[e] * (sg + silu * (1.f - sg));
    ou[e] = d[e] * silu;
  }
  store_as<T, kStreamSwigluBwdStores>(dgate + r * dgld + c, og);
  store_as<T, kStreamSwigluBwdStores>(dup + r * duld + c, ou);
}

// ---------------------------------------------------------------------------------- lse merge
// One thread owns 4 consecutive fp32 elements of an out row.  A row's D/4 threads sit in one wave
// (D/4 divides 64), and the wave reads lse before any of its lanes writes it.
template <typename TB>
__global__ __launch_bounds__(kThreads) void lse_merge_kernel(float* __restrict__ out, float* __restrict__ lse,
                                                             const TB* __restrict__ block_out,
                                                             const float* __restrict__ block_lse, int64_t total,
                                                             int D) {
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  const int vpr = D / 4;
  const int64_t row = idx / vpr;
  const int col = static_cast<int>(idx % vpr) * 4;
  const float l = lse[row];
  const float bl = block_lse[row];
  float o[4], bo[4];
  io<float>::load(out + row * D + col, o);
  if constexpr (sizeof(TB) == 2) {
    const u32x2 raw = *reinterpret_cast<const u32x2*>(block_out + row * D + col);
    bo[0] = __uint_as_float(raw[0] << 16); bo[1] = __uint_as_float(raw[0] & 0xffff0000u);
    bo[2] = __uint_as_float(raw[1] << 16); bo[3] = __uint_as_float(raw[1] & 0xffff0000u);
  } else {
    io<float>::load(block_out + row * D + col, bo);
  }
  // sigmoid(bl - l) and l - logsigmoid(l - bl) = max + log(1 + exp(-|bl - l|)); both sides -inf -> keep
  const float hi = fmaxf(l, bl);
  float w, nl;
  if (hi == -INFINITY) {
    w = 0.f; nl = -INFINITY;
  } else {
    const float el = __expf(l - hi), eb = __expf(bl - hi);
    w = eb / (el + eb);
    nl = hi + __logf(el + eb);
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = o[e] - w * (o[e] - bo[e]);
  io<float>::store(out + row * D + col, o);
  if (col == 0) lse[row] = nl;
}

// ---------------------------------------------------------------------------------- fp32 -> io
template <typename T>
__global__ __launch_bounds__(kThreads) void convert_kernel(const float* __restrict__ src, T* __restrict__ dst,
                                                           int64_t total, int H, int S, int D, int64_t dsb,
                                                           int64_t dsh, int64_t dss, int s_outer) {
  constexpr int V = io<T>::kVec;
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (idx >= total) return;
  const int vpr = D / V;
  const int v = static_cast<int>(idx % vpr);
  int64_t rest = idx / vpr;
  int h, s;
  if (s_outer) {
    h = static_cast<int>(rest % H); rest /= H;
    s = static_cast<int>(rest % S); rest /= S;
  } else {
    s = static_cast<int>(rest % S); rest /= S;
    h = static_cast<int>(rest % H); rest /= H;
  }
  const int64_t b = rest;
  const float* sp = src + ((b * H + h) * S + s) * static_cast<int64_t>(D) + v * V;
  float vals[V];
#pragma unroll
  for (int e = 0; e < V; e += 4) {
    float t[4];
    io<float>::load(sp + e, t);
#pragma unroll
    for (int k = 0; k < 4; ++k) vals[e + k] = t[k];
  }
  io<T>::store(dst + b * dsb + h * dsh + s * dss + v * V, vals);
}

unsigned blocks_for(int64_t total) { return static_cast<unsigned>((total + kThreads - 1) / kThreads); }
bool dtype_ok(int d) { return d == PICO_BF16 || d == PICO_F32; }
int vec_of(int d) { return d == PICO_BF16 ? 8 : 4; }
int64_t elem_size(int d) { return d == PICO_BF16 ? 2 : 4; }
// base pointer 16-byte aligned and every stride a multiple of the vector length
bool strided_ok(const void* p, int dtype, std::initializer_list<int64_t> strides) {
  if (!aligned16(p)) return false;
  for (int64_t s : strides)
    if (s % vec_of(dtype) != 0) return false;
  return true;
}

}  // namespace
}  // namespace pico

using namespace pico;

extern "C" int pico_rope(const void* x, void* y, const void* cos, const void* sin, int64_t B, int64_t H, int64_t S,
                         int64_t D, int64_t xsb, int64_t xsh, int64_t xss, int64_t ysb, int64_t ysh, int64_t yss,
                         int64_t table_ld, int64_t pos_offset, int inverse, int table_dtype, int dtype,
                         void* stream) {
  if (!dtype_ok(dtype) || !dtype_ok(table_dtype))
    return fail(PICO_ERR_DTYPE, "pico_rope: dtype %d / table dtype %d not supported", dtype, table_dtype);
  if (B < 0 || H < 0 || S < 0 || D <= 0 || D > 256 || D % 16 != 0 || pos_offset < 0)
    return fail(PICO_ERR_SHAPE, "pico_rope: B=%lld H=%lld S=%lld D=%lld pos_offset=%lld (D must be a multiple of 16, <= 256)",
                (long long)B, (long long)H, (long long)S, (long long)D, (long long)pos_offset);
  if (B == 0 || H == 0 || S == 0) return PICO_OK;
  if (!x || !y || !cos || !sin) return fail(PICO_ERR_NULL, "pico_rope: x, y, cos and sin are required");
  if (table_ld < D / 2) return fail(PICO_ERR_STRIDE, "pico_rope: table_ld=%lld < D/2", (long long)table_ld);
  if (!strided_ok(x, dtype, {xsb, xsh, xss}) || !strided_ok(y, dtype, {ysb, ysh, yss}))
    return fail(PICO_ERR_ALIGN, "pico_rope: x/y must be 16-byte aligned with strides that are multiples of %d elements",
                vec_of(dtype));
  // a table row must stay vector-aligned for the widest access the kernel makes on it (8 elements)
  if ((reinterpret_cast<uintptr_t>(cos) | reinterpret_cast<uintptr_t>(sin)) % 16 != 0 ||
      (table_ld * elem_size(table_dtype)) % 16 != 0)
    return fail(PICO_ERR_ALIGN, "pico_rope: cos/sin rows must be 16-byte aligned");
  const int64_t total = B * H * S * (D / 2 / vec_of(dtype));
  const int s_outer = (xsh <= xss) ? 1 : 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
#define PICO_ROPE(T, TT)                                                                                       \
  hipLaunchKernelGGL((rope_kernel<T, TT>), dim3(blocks_for(total)), dim3(kThreads), 0, st,                     \
                     static_cast<const T*>(x), static_cast<T*>(y), static_cast<const TT*>(cos),                \
                     static_cast<const TT*>(sin), total, (int)H, (int)S, (int)D, xsb, xsh, xss, ysb, ysh, yss, \
                     table_ld, pos_offset, inverse, s_outer)
  if (dtype == PICO_BF16 && table_dtype == PICO_BF16) PICO_ROPE(__bf16, __bf16);
  else if (dtype == PICO_BF16) PICO_ROPE(__bf16, float);
  else if (table_dtype == PICO_BF16) PICO_ROPE(float, __bf16);
  else PICO_ROPE(float, float);
#undef PICO_ROPE
  return check_launch("pico_rope");
}

extern "C" int pico_swiglu_fwd(const void* gate, const void* up, void* y, int64_t rows, int64_t cols, int64_t gate_ld,
                               int64_t up_ld, int64_t y_ld, int dtype, void* stream) {
  if (!dtype_ok(dtype)) return fail(PICO_ERR_DTYPE, "pico_swiglu_fwd: dtype code %d not supported", dtype);
  if (rows < 0 || cols < 0 || cols % vec_of(dtype) != 0)
    return fail(PICO_ERR_SHAPE, "pico_swiglu_fwd: rows=%lld cols=%lld (cols must be a multiple of %d)", (long long)rows,
                (long long)cols, vec_of(dtype));
  if (rows == 0 || cols == 0) return PICO_OK;
  if (!gate || !up || !y) return fail(PICO_ERR_NULL, "pico_swiglu_fwd: gate, up and y are required");
  if (gate_ld < cols || up_ld < cols || y_ld < cols) return fail(PICO_ERR_STRIDE, "pico_swiglu_fwd: row pitch < cols");
  if (!strided_ok(gate, dtype, {gate_ld}) || !strided_ok(up, dtype, {up_ld}) || !strided_ok(y, dtype, {y_ld}))
    return fail(PICO_ERR_ALIGN, "pico_swiglu_fwd: pointers must be 16-byte aligned, pitches multiples of %d", vec_of(dtype));
  const int vpr = static_cast<int>(cols / vec_of(dtype));
  const int64_t total = rows * vpr;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == PICO_BF16)
    hipLaunchKernelGGL(swiglu_fwd_kernel<__bf16>, dim3(blocks_for(total)), dim3(kThreads), 0, st,
                       static_cast<const __bf16*>(gate), static_cast<const __bf16*>(up), static_cast<__bf16*>(y), total,
                       vpr, gate_ld, up_ld, y_ld);
  else
    hipLaunchKernelGGL(swiglu_fwd_kernel<float>, dim3(blocks_for(total)), dim3(kThreads), 0, st,
                       static_cast<const float*>(gate), static_cast<const float*>(up), static_cast<float*>(y), total,
                       vpr, gate_ld, up_ld, y_ld);
  return check_launch("pico_swiglu_fwd");
}

extern "C" int pico_swiglu_bwd(const void* dy, const void* gate, const void* up, void* dgate, void* dup, int64_t rows,
                               int64_t cols, int64_t dy_ld, int64_t gate_ld, int64_t up_ld, int64_t dgate_ld,
                               int64_t dup_ld, int dtype, void* stream) {
  if (!dtype_ok(dtype)) return fail(PICO_ERR_DTYPE, "pico_swiglu_bwd: dtype code %d not supported", dtype);
  if (rows < 0 || cols < 0 || cols % vec_of(dtype) != 0)
    return fail(PICO_ERR_SHAPE, "pico_swiglu_bwd: rows=%lld cols=%lld (cols must be a multiple of %d)", (long long)rows,
                (long long)cols, vec_of(dtype));
  if (rows == 0 || cols == 0) return PICO_OK;
  if (!dy || !gate || !up || !dgate || !dup) return fail(PICO_ERR_NULL, "pico_swiglu_bwd: all five tensors are required");
  if (dy_ld < cols || gate_ld < cols || up_ld < cols || dgate_ld < cols || dup_ld < cols)
    return fail(PICO_ERR_STRIDE, "pico_swiglu_bwd: row pitch < cols");
  if (!strided_ok(dy, dtype, {dy_ld}) || !strided_ok(gate, dtype, {gate_ld}) || !strided_ok(up, dtype, {up_ld}) ||
      !strided_ok(dgate, dtype, {dgate_ld}) || !strided_ok(dup, dtype, {dup_ld}))
    return fail(PICO_ERR_ALIGN, "pico_swiglu_bwd: pointers must be 16-byte aligned, pitches multiples of %d", vec_of(dtype));
  const int vpr = static_cast<int>(cols / vec_of(dtype));
  const int64_t total = rows * vpr;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dtype == PICO_BF16)
    hipLaunchKernelGGL(swiglu_bwd_kernel<__bf16>, dim3(blocks_for(total)), dim3(kThreads), 0, st,
                       static_cast<const __bf16*>(dy), static_cast<const __bf16*>(gate), static_cast<const __bf16*>(up),
                       static_cast<__bf16*>(dgate), static_cast<__bf16*>(dup), total, vpr, dy_ld, gate_ld, up_ld,
                       dgate_ld, dup_ld);
  else
    hipLaunchKernelGGL(swiglu_bwd_kernel<float>, dim3(blocks_for(total)), dim3(kThreads), 0, st,
                       static_cast<const float*>(dy), static_cast<const float*>(gate), static_cast<const float*>(up),
                       static_cast<float*>(dgate), static_cast<float*>(dup), total, vpr, dy_ld, gate_ld, up_ld, dgate_ld,
                       dup_ld);
  return check_launch("pico_swiglu_bwd");
}

extern "C" int pico_lse_merge(float* out, float* lse, const void* block_out, const float* block_lse, int64_t rows,
                              int64_t D, int block_dtype, void* stream) {
  if (!dtype_ok(block_dtype)) return fail(PICO_ERR_DTYPE, "pico_lse_merge: block dtype code %d not supported", block_dtype);
  if (rows < 0 || D <= 0 || D % 4 != 0 || 64 % (D / 4) != 0)
    return fail(PICO_ERR_SHAPE, "pico_lse_merge: rows=%lld D=%lld (D/4 must divide 64)", (long long)rows, (long long)D);
  if (rows == 0) return PICO_OK;
  if (!out || !lse || !block_out || !block_lse) return fail(PICO_ERR_NULL, "pico_lse_merge: all four tensors are required");
  if (!aligned16(out) || (reinterpret_cast<uintptr_t>(block_out) & 7u))
    return fail(PICO_ERR_ALIGN, "pico_lse_merge: out must be 16-byte and block_out 8-byte aligned");
  if (block_dtype == PICO_F32 && !aligned16(block_out))
    return fail(PICO_ERR_ALIGN, "pico_lse_merge: fp32 block_out must be 16-byte aligned");
  const int64_t total = rows * (D / 4);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (block_dtype == PICO_BF16)
    hipLaunchKernelGGL(lse_merge_kernel<__bf16>, dim3(blocks_for(total)), dim3(kThreads), 0, st, out, lse,
                       static_cast<const __bf16*>(block_out), block_lse, total, (int)D);
  else
    hipLaunchKernelGGL(lse_merge_kernel<float>, dim3(blocks_for(total)), dim3(kThreads), 0, st, out, lse,
                       static_cast<const float*>(block_out), block_lse, total, (int)D);
  return check_launch("pico_lse_merge");
}

extern "C" int pico_convert_f32(const float* src, void* dst, int64_t B, int64_t H, int64_t S, int64_t D,
                                int64_t dsb, int64_t dsh, int64_t dss, int dst_dtype, void* stream) {
  if (!dtype_ok(dst_dtype)) return fail(PICO_ERR_DTYPE, "pico_convert_f32: dtype code %d not supported", dst_dtype);
  if (B < 0 || H < 0 || S < 0 || D <= 0 || D % 8 != 0)
    return fail(PICO_ERR_SHAPE, "pico_convert_f32: B=%lld H=%lld S=%lld D=%lld (D must be a multiple of 8)", (long long)B,
                (long long)H, (long long)S, (long long)D);
  if (B == 0 || H == 0 || S == 0) return PICO_OK;
  if (!src || !dst) return fail(PICO_ERR_NULL, "pico_convert_f32: src and dst are required");
  if (!aligned16(src) || !strided_ok(dst, dst_dtype, {dsb, dsh, dss}))
    return fail(PICO_ERR_ALIGN, "pico_convert_f32: pointers must be 16-byte aligned, strides multiples of %d", vec_of(dst_dtype));
  const int64_t total = B * H * S * (D / vec_of(dst_dtype));
  const int s_outer = (dsh <= dss) ? 1 : 0;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (dst_dtype == PICO_BF16)
    hipLaunchKernelGGL(convert_kernel<__bf16>, dim3(blocks_for(total)), dim3(kThreads), 0, st, src,
                       static_cast<__bf16*>(dst), total, (int)H, (int)S, (int)D, dsb, dsh, dss, s_outer);
  else
    hipLaunchKernelGGL(convert_kernel<float>, dim3(blocks_for(total)), dim3(kThreads), 0, st, src,
                       static_cast<float*>(dst), total, (int)H, (int)S, (int)D, dsb, dsh, dss, s_outer);
  return check_launch("pico_convert_f32");
}
