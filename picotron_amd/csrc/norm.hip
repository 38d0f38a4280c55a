// RMSNorm forward / backward for gfx950.  Bandwidth-bound: every element is moved with 16-byte
// accesses, one row is owned by a wave (hidden <= 64*8 vectors) or by a 256-thread block, the row
// stays in registers between the reduction and the normalisation so HBM is touched once.
#include "common.h"

// Scratch of pico_rmsnorm_bwd_static, the entry point that allocates nothing: the per-block partial sums of dweight
// that pico_rmsnorm_bwd keeps in the caller's workspace.  4 MiB per GPU, held until the process ends.  In host code
// this name is only a handle: the device address comes from hipGetSymbolAddress (static_scratch() below).
constexpr size_t kStaticScratchFloats = size_t(1) << 20;
static __device__ __align__(256) float scratch[kStaticScratchFloats];

namespace pico {
namespace {

// Streaming (non-temporal) accesses where they measured faster: the forward's outputs (+15 % on cold data) and the
// row-per-wave backward's read-once inputs (+5 %); the forward's loads and the backward's stores are plain (streaming
// there is slower on the warm data a training step hands these kernels).
constexpr bool kStreamFwdStores = true, kStreamFwdLoads = false, kStreamBwdStores = false;
__device__ __forceinline__ u32x4 load_raw(const void* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
constexpr int kFwdThreads = 256;
constexpr int kBwdThreads = 512;
constexpr int kMaxBwdBlocks = 512;   // rows of the dweight workspace
constexpr int kBwdWaves = 4;         // waves per block of the row-per-wave backward


template <int G>
__device__ __forceinline__ float group_sum(float v, float* smem /* this group's 4 floats, G == 256 only */) {
  v = wave_sum(v);
  if constexpr (G == kWave) {
    return v;
  } else {
    const int wave = (threadIdx.x % G) / kWave;
    __syncthreads();
    if (threadIdx.x % kWave == 0) smem[wave] = v;
    __syncthreads();
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < G / kWave; ++i) t += smem[i];
    return t;
  }
}

// y = w * round(x * rstd)  (cast_then_scale)  or  round(x * rstd * w)
template <typename T, int G, int NV>
__global__ __launch_bounds__(kFwdThreads) void rmsnorm_fwd_kernel(
    const T* __restrict__ x, const T* __restrict__ w, T* __restrict__ y, float* __restrict__ rstd,
    const T* __restrict__ res_in, T* __restrict__ res_out, int64_t rows, int hidden, float eps,
    int cast_then_scale) {
  constexpr int V = io<T>::kVec;
  __shared__ float smem[8];
  const int gid = threadIdx.x / G;
  const int t = threadIdx.x % G;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * (kFwdThreads / G) + gid;
  const int nvec = hidden / V;
  // G == 256: the block owns one row, so `row < rows` is block-uniform and the barriers inside
  // group_sum are reached by every thread.  G == 64: no barrier is used.
  if (row >= rows) return;
  const T* xr = x + row * hidden;
  float vals[NV][V];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int v = t + j * G;
    if (v < nvec) {
      load_as<T, kStreamFwdLoads>(xr + v * V, vals[j]);
      if (res_in != nullptr) {
        float r[V];
        load_as<T, kStreamFwdLoads>(res_in + row * hidden + v * V, r);
#pragma unroll
        for (int e = 0; e < V; ++e) vals[j][e] += r[e];
        if (res_out != nullptr) store_as<T, kStreamFwdStores>(res_out + row * hidden + v * V, vals[j]);
      }
#pragma unroll
      for (int e = 0; e < V; ++e) ss += vals[j][e] * vals[j][e];
    }
  }
  ss = group_sum<G>(ss, smem + gid * 4);
  const float r = rsqrtf(ss / static_cast<float>(hidden) + eps);
  if (rstd != nullptr && t == 0) rstd[row] = r;
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int v = t + j * G;
    if (v < nvec) {
      float wv[V], o[V];
      io<T>::load(w + v * V, wv);
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float n = vals[j][e] * r;
        o[e] = cast_then_scale ? io<T>::round(n) * wv[e] : n * wv[e];
      }
      store_as<T, kStreamFwdStores>(y + row * hidden + v * V, o);
    }
  }
}

// dx and per-block partial sums of dweight.
template <typename T, int G, int NV>
__global__ __launch_bounds__(kBwdThreads) void rmsnorm_bwd_kernel(
    const T* __restrict__ dy, const T* __restrict__ x, const T* __restrict__ w,
    const float* __restrict__ rstd, const T* dres, T* dx, float* __restrict__ partial,
    int64_t rows, int hidden) {
  constexpr int V = io<T>::kVec;
  constexpr int GPB = kBwdThreads / G;
  extern __shared__ float dw_lds[];  // [hidden] when GPB > 1
  __shared__ float smem[8];
  const int gid = threadIdx.x / G;
  const int t = threadIdx.x % G;
  const int nvec = hidden / V;
  const float inv_h = 1.f / static_cast<float>(hidden);
  float dw[NV][V];
#pragma unroll
  for (int j = 0; j < NV; ++j)
#pragma unroll
    for (int e = 0; e < V; ++e) dw[j][e] = 0.f;
  if constexpr (GPB > 1) {
    for (int i = threadIdx.x; i < hidden; i += kBwdThreads) dw_lds[i] = 0.f;
  }
  // rows are dealt round-robin to groups; with G == 256 (GPB == 2) a group's trip count can differ
  // from its neighbour's, so that variant pads the loop to a block-uniform count for the barriers.
  const int64_t stride = static_cast<int64_t>(gridDim.x) * GPB;
  const int64_t first = static_cast<int64_t>(blockIdx.x) * GPB + gid;
  const int64_t trips = (rows - static_cast<int64_t>(blockIdx.x) * GPB + stride - 1) / stride;  // block-uniform upper bound
  for (int64_t it = 0; it < trips; ++it) {
    const int64_t row = first + it * stride;
    const bool live = row < rows;
    float xh[NV][V], g[NV][V];
    float c = 0.f;
    const float r = live ? rstd[row] : 0.f;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int v = t + j * G;
      if (live && v < nvec) {
        float dyv[V], wv[V];
        io<T>::load(x + row * hidden + v * V, xh[j]);
        io<T>::load(dy + row * hidden + v * V, dyv);
        io<T>::load(w + v * V, wv);
#pragma unroll
        for (int e = 0; e < V; ++e) {
          xh[j][e] *= r;
          g[j][e] = dyv[e] * wv[e];
          c += g[j][e] * xh[j][e];
          dw[j][e] += dyv[e] * xh[j][e];
        }
      }
    }
    c = group_sum<G>(c, smem + gid * 4) * inv_h;
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int v = t + j * G;
      if (live && v < nvec) {
        float o[V];
#pragma unroll
        for (int e = 0; e < V; ++e) o[e] = r * (g[j][e] - xh[j][e] * c);
        if (dres) {  // gradient that reached the residual stream directly; dx may alias it (same thread, same place)
          float dr[V];
          io<T>::load(dres + row * hidden + v * V, dr);
#pragma unroll
          for (int e = 0; e < V; ++e) o[e] += dr[e];
        }
        store_as<T, kStreamBwdStores>(dx + row * hidden + v * V, o);
      }
    }
  }
  float* out = partial + static_cast<int64_t>(blockIdx.x) * hidden;
  if constexpr (GPB > 1) {
    // the groups of the block add their shares one after the other, in group order: the same sum on every run
    // (an atomic add per element would take them in arrival order)
    for (int turn = 0; turn < GPB; ++turn) {
      __syncthreads();
      if (gid == turn) {
#pragma unroll
        for (int j = 0; j < NV; ++j) {
          const int v = t + j * G;
          if (v < nvec) {
#pragma unroll
            for (int e = 0; e < V; ++e) dw_lds[v * V + e] += dw[j][e];
          }
        }
      }
    }
    __syncthreads();
    for (int i = threadIdx.x; i < hidden; i += kBwdThreads) out[i] = dw_lds[i];
  } else {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int v = t + j * G;
      if (v < nvec) {
#pragma unroll
        for (int e = 0; e < V; ++e) out[v * V + e] = dw[j][e];
      }
    }
  }
}

// Row-per-wave backward (hidden <= 64 * NV vectors): a wave keeps the packed x / dy of its row in
// registers and carries its share of dweight in registers across all its rows.  No software prefetch of the
// next row: loads and stores retire in one order, so waiting for a prefetched row also waits for the stores
// of the current one (measured: 3.4 TB/s with the prefetch, 5.2 TB/s -- the rate of a plain copy -- without).  The block's four waves are summed through LDS once at
// the end and the block writes one row of the partial-sum workspace.
template <typename T, int NV, bool kRes, int R, int NWAVE>
__global__ __launch_bounds__(NWAVE * kWave) void rmsnorm_bwd_wave_kernel(
    const T* __restrict__ dy, const T* __restrict__ x, const T* __restrict__ w,
    const float* __restrict__ rstd, const T* dres, T* dx, float* __restrict__ partial,
    int64_t rows, int hidden) {
  constexpr int V = io<T>::kVec;
  extern __shared__ __attribute__((aligned(16))) float red[];  // [NWAVE][hidden]
  const int t = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);   // uniform: row addresses become scalar base + lane offset
  const int nvec = hidden / V;
  const float inv_h = 1.f / static_cast<float>(hidden);
  float dw[NV][V];
  // The weight stays packed (16 bytes per piece) and is unpacked where it is used: unpacked it would double its
  // registers, and registers decide how many rows the GPU has in flight (asm_keep stops the compiler from hoisting the
  // unpacking out of the row loop).
  u32x4 wp[NV];
  // R rows of the wave are in flight together: all their loads are issued before the first is waited for, so a wave
  // that owns R rows pays one memory latency for them, not R
  u32x4 xr[R][NV], dr[R][NV], rr[R][kRes ? NV : 1];  // rr: the residual stream's own gradient (kRes: dres is given)
  float rs[R];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
#pragma unroll
    for (int e = 0; e < V; ++e) dw[j][e] = 0.f;
    const int v = t + j * kWave;
    wp[j] = *reinterpret_cast<const u32x4*>(w + (v < nvec ? v : 0) * V);
  }
  const int64_t stride = static_cast<int64_t>(gridDim.x) * NWAVE;
  int64_t row = static_cast<int64_t>(blockIdx.x) * NWAVE + wave;
  auto fetch = [&](int q, int64_t r) {
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int v = t + j * kWave;
      const int vc = v < nvec ? v : 0;
      xr[q][j] = load_raw(x + r * hidden + vc * V);
      dr[q][j] = load_raw(dy + r * hidden + vc * V);
      if constexpr (kRes) rr[q][j] = load_raw(dres + r * hidden + vc * V);
    }
    rs[q] = rstd[r];
  };
  auto unpack = [&](const u32x4& raw, float (&out)[V]) {
    if constexpr (V == 8) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        out[2 * i] = __uint_as_float(raw[i] << 16);
        out[2 * i + 1] = __uint_as_float(raw[i] & 0xffff0000u);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) out[i] = __uint_as_float(raw[i]);
    }
  };
  for (; row < rows; row += R * stride) {
#pragma unroll
    for (int q = 0; q < R; ++q) {
      const int64_t rq = row + q * stride;
      fetch(q, rq < rows ? rq : row);   // a row past the end re-reads the first one; nothing of it is used
    }
#pragma unroll
    for (int j = 0; j < NV; ++j) asm volatile("" : "+v"(wp[j]));
#pragma unroll
    for (int q = 0; q < R; ++q) {
      const int64_t rq = row + q * stride;
      if (rq >= rows) break;
      const float r = rs[q];
      float c = 0.f;
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        if (t + j * kWave < nvec) {
          float xv[V], dv[V], wv[V];
          unpack(xr[q][j], xv);
          unpack(dr[q][j], dv);
          unpack(wp[j], wv);
#pragma unroll
          for (int e = 0; e < V; ++e) {
            const float xh = xv[e] * r;
            c += dv[e] * wv[e] * xh;
            dw[j][e] += dv[e] * xh;
          }
        }
        __builtin_amdgcn_sched_barrier(0);   // one piece at a time: pieces unpacked side by side cost registers
      }
      c = wave_sum(c) * inv_h;
      // the second pass unpacks the row again: keeping the first pass's products alive for it would cost 2 x the
      // row's share in registers (the empty asm hides from the compiler that the values are the same)
#pragma unroll
      for (int j = 0; j < NV; ++j) asm volatile("" : "+v"(xr[q][j]), "+v"(dr[q][j]), "+v"(wp[j]));
#pragma unroll
      for (int j = 0; j < NV; ++j) {
        const int v = t + j * kWave;
        if (v < nvec) {
          float xv[V], dv[V], wv[V], o[V];
          unpack(xr[q][j], xv);
          unpack(dr[q][j], dv);
          unpack(wp[j], wv);
#pragma unroll
          for (int e = 0; e < V; ++e) o[e] = r * (dv[e] * wv[e] - xv[e] * r * c);
          if constexpr (kRes) {  // dx may alias dres: this lane read its part of the row before it writes it
            float rv[V];
            unpack(rr[q][j], rv);
#pragma unroll
            for (int e = 0; e < V; ++e) o[e] += rv[e];
          }
          store_as<T, kStreamBwdStores>(dx + rq * hidden + v * V, o);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  // block reduction of dweight: every wave parks its share in LDS, then all threads sum columns (a fixed order) and
  // write the block's row of the partial sums
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int v = t + j * kWave;
    if (v < nvec) {
      if constexpr (V == 8) {
        *reinterpret_cast<f32x4*>(&red[wave * hidden + v * V]) = f32x4{dw[j][0], dw[j][1], dw[j][2], dw[j][3]};
        *reinterpret_cast<f32x4*>(&red[wave * hidden + v * V + 4]) = f32x4{dw[j][4], dw[j][5], dw[j][6], dw[j][7]};
      } else {
        *reinterpret_cast<f32x4*>(&red[wave * hidden + v * V]) = f32x4{dw[j][0], dw[j][1], dw[j][2], dw[j][3]};
      }
    }
  }
  __syncthreads();
  float* out = partial + static_cast<int64_t>(blockIdx.x) * hidden;
  for (int c4 = threadIdx.x * 4; c4 < hidden; c4 += NWAVE * kWave * 4) {
    f32x4 acc = *reinterpret_cast<const f32x4*>(&red[c4]);
#pragma unroll
    for (int k = 1; k < NWAVE; ++k) acc += *reinterpret_cast<const f32x4*>(&red[k * hidden + c4]);
    *reinterpret_cast<f32x4*>(&out[c4]) = acc;
  }
}

// dweight[c] = sum_p partial[p][c]; 32 columns x 32 slices per block, every thread's loads issued together.
constexpr int kReduceCols = 32;
constexpr int kReduceSlices = 1024 / kReduceCols;
template <typename TW>
__global__ __launch_bounds__(1024) void rmsnorm_dw_reduce_kernel(
    const float* __restrict__ partial, TW* __restrict__ dweight, int nparts, int hidden) {
  constexpr int kSlices = kReduceSlices, kUnroll = 512 / kSlices;
  __shared__ float red[kSlices][kReduceCols + 1];
  const int c = threadIdx.x % kReduceCols;
  const int col = blockIdx.x * kReduceCols + c;
  const int slice = threadIdx.x / kReduceCols;
  float s = 0.f;
  if (col < hidden) {
    for (int p0 = slice; p0 < nparts; p0 += kSlices * kUnroll) {
      float v[kUnroll];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int p = p0 + u * kSlices;
        v[u] = p < nparts ? partial[static_cast<int64_t>(p) * hidden + col] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) s += v[u];
    }
  }
  red[slice][c] = s;
  __syncthreads();
  if (slice == 0 && col < hidden) {
    float tot = 0.f;
#pragma unroll
    for (int i = 0; i < kSlices; ++i) tot += red[i][c];
    dweight[col] = static_cast<TW>(tot);
  }
}

void launch_dw_reduce(const float* partial, void* dweight, int dweight_dtype, int nparts, int hidden, hipStream_t s) {
  const dim3 grid(static_cast<unsigned>((hidden + kReduceCols - 1) / kReduceCols)), block(1024);
  if (dweight_dtype == PICO_BF16)
    hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel<__bf16>, grid, block, 0, s, partial, static_cast<__bf16*>(dweight), nparts, hidden);
  else
    hipLaunchKernelGGL(rmsnorm_dw_reduce_kernel<float>, grid, block, 0, s, partial, static_cast<float*>(dweight), nparts, hidden);
}

// Blocks of the backward: as many as the rows need, up to a cap that shrinks with the row length -- every block ends by
// writing (and the reduce kernel by reading) one row of the workspace, and at hidden 4096 the 512 blocks that are right
// for hidden 2048 cost 19 % (measured at 4096 rows: 48.7 us with 512 blocks, 39.3 us with 256).
int bwd_blocks(int64_t rows, int gpb, int hidden) {
  int64_t need = (rows + gpb - 1) / gpb;
  if (need < 1) need = 1;
  int cap = (1 << 20) / (hidden > 0 ? hidden : 1);
  cap = cap < 64 ? 64 : (cap > kMaxBwdBlocks ? kMaxBwdBlocks : cap);
  return static_cast<int>(need < cap ? need : cap);
}

// smallest supported NV >= need, or 0
int pick_nv(int need, int max_nv) {
  for (int nv = 1; nv <= max_nv; nv *= 2)
    if (nv >= need) return nv;
  return 0;
}

template <typename T, int G, int NV>
void launch_fwd(const void* x, const void* w, void* y, float* rstd, const void* ri, void* ro, int64_t rows,
                int hidden, float eps, int cts, hipStream_t s) {
  const int gpb = kFwdThreads / G;
  const unsigned grid = static_cast<unsigned>((rows + gpb - 1) / gpb);
  hipLaunchKernelGGL((rmsnorm_fwd_kernel<T, G, NV>), dim3(grid), dim3(kFwdThreads), 0, s,
                     static_cast<const T*>(x), static_cast<const T*>(w), static_cast<T*>(y), rstd,
                     static_cast<const T*>(ri), static_cast<T*>(ro), rows, hidden, eps, cts);
}

template <typename T, int G, int NV>
int launch_bwd(const void* dy, const void* x, const void* w, const float* rstd, const void* dres, void* dx,
               float* partial, int blocks, int64_t rows, int hidden, hipStream_t s) {
  const size_t lds = (kBwdThreads / G > 1) ? static_cast<size_t>(hidden) * sizeof(float) : 0;
  // the longest rows need the whole default LDS allowance for the dweight row plus the kernel's static 32 bytes
  static LdsOnce lds_reserved;
  constexpr size_t kLdsMax = static_cast<size_t>(G) * NV * io<T>::kVec * sizeof(float) + 64;
  if (kLdsMax > 48 * 1024 &&
      !reserve_lds_once(lds_reserved, reinterpret_cast<const void*>(&rmsnorm_bwd_kernel<T, G, NV>), kLdsMax))
    return fail(PICO_ERR_LAUNCH, "pico_rmsnorm_bwd: cannot reserve %zu bytes of LDS", kLdsMax);
  hipLaunchKernelGGL((rmsnorm_bwd_kernel<T, G, NV>), dim3(blocks), dim3(kBwdThreads), lds, s,
                     static_cast<const T*>(dy), static_cast<const T*>(x), static_cast<const T*>(w), rstd,
                     static_cast<const T*>(dres), static_cast<T*>(dx), partial, rows, hidden);
  return PICO_OK;
}

template <typename T>
int dispatch_fwd(const void* x, const void* w, void* y, float* rstd, const void* ri, void* ro, int64_t rows,
                 int hidden, float eps, int cts, hipStream_t s) {
  const int nvec = hidden / io<T>::kVec;
  const int nv_wave = pick_nv((nvec + 63) / 64, 8);
#define PICO_FWD(G, NV) launch_fwd<T, G, NV>(x, w, y, rstd, ri, ro, rows, hidden, eps, cts, s); return PICO_OK
  if (nv_wave) {
    switch (nv_wave) {
      case 1: PICO_FWD(64, 1);
      case 2: PICO_FWD(64, 2);
      case 4: PICO_FWD(64, 4);
      default: PICO_FWD(64, 8);
    }
  }
  switch (pick_nv((nvec + 255) / 256, 16)) {
    case 4: PICO_FWD(256, 4);
    case 8: PICO_FWD(256, 8);
    case 16: PICO_FWD(256, 16);
    default: break;
  }
#undef PICO_FWD
  return fail(PICO_ERR_SHAPE, "pico_rmsnorm_fwd: hidden=%d too large", hidden);
}

template <typename T>
int dispatch_bwd(const void* dy, const void* x, const void* w, const float* rstd, const void* dres, void* dx,
                 float* partial, int64_t rows, int hidden, hipStream_t s, int* blocks_out) {
  const int nvec = hidden / io<T>::kVec;
  const int nv_wave = pick_nv((nvec + 63) / 64, 8);
#define PICO_BWD(G, NV)                                                            \
  {                                                                                \
    const int blocks = bwd_blocks(rows, kBwdThreads / G, hidden);                          \
    *blocks_out = blocks;                                                          \
    return launch_bwd<T, G, NV>(dy, x, w, rstd, dres, dx, partial, blocks, rows, hidden, s); \
  }
#define PICO_BWD_WAVE(NV)                                                                              \
  {                                                                                                    \
    const int blocks = bwd_blocks(rows, kBwdWaves, hidden);                                            \
    *blocks_out = blocks;                                                                              \
    const size_t lds = static_cast<size_t>(kBwdWaves) * hidden * sizeof(float);                        \
    auto go = [&](auto kern, LdsOnce& reserved) -> int {                                               \
      if (lds > 48 * 1024 && !reserve_lds_once(reserved, reinterpret_cast<const void*>(kern),          \
                                               kBwdWaves * 64 * NV * io<T>::kVec * sizeof(float)))     \
        return fail(PICO_ERR_LAUNCH, "pico_rmsnorm_bwd: cannot reserve %zu bytes of LDS",              \
                    static_cast<size_t>(kBwdWaves * 64 * NV * io<T>::kVec * sizeof(float)));           \
      hipLaunchKernelGGL(kern, dim3(blocks), dim3(kBwdWaves * kWave), lds, s,                          \
                         static_cast<const T*>(dy), static_cast<const T*>(x), static_cast<const T*>(w), \
                         rstd, static_cast<const T*>(dres), static_cast<T*>(dx), partial, rows, hidden); \
      return PICO_OK;                                                                                  \
    };                                                                                                 \
    static LdsOnce reserved_res, reserved_res2, reserved_plain;                               \
    /* with dresidual and short rows a wave that owns several rows keeps two in flight (measured at 4096 x 2048: \
       20.2 -> 18.8 us; without dresidual the same costs 0.9 us, with longer rows the registers do not allow it) */ \
    constexpr int kR = NV * io<T>::kVec <= 32 ? 2 : 1;                                                 \
    if (kR == 2 && dres && rows > static_cast<int64_t>(blocks) * kBwdWaves)                            \
      return go(rmsnorm_bwd_wave_kernel<T, NV, true, kR, kBwdWaves>, reserved_res2);                   \
    if (dres) return go(rmsnorm_bwd_wave_kernel<T, NV, true, 1, kBwdWaves>, reserved_res);             \
    return go(rmsnorm_bwd_wave_kernel<T, NV, false, 1, kBwdWaves>, reserved_plain);                    \
  }
  if (nv_wave) {   // rows of at most 64 x 8 vectors: 4 waves x hidden floats of LDS is at most 64 KiB
    switch (nv_wave) {
      case 1: PICO_BWD_WAVE(1);
      case 2: PICO_BWD_WAVE(2);
      case 4: PICO_BWD_WAVE(4);
      default: PICO_BWD_WAVE(8);
    }
  }
  // longer rows: one row per 256 threads, two rows per block.  The two groups add their shares of dweight to the
  // block's LDS row one after the other, in group order (no atomics: the same sum on every run).
  switch (pick_nv((nvec + 255) / 256, 16)) {
    case 4: PICO_BWD(256, 4);
    case 8: PICO_BWD(256, 8);
    case 16: PICO_BWD(256, 16);
    default: break;
  }
#undef PICO_BWD_WAVE
#undef PICO_BWD
  return fail(PICO_ERR_SHAPE, "pico_rmsnorm_bwd: hidden=%d too large", hidden);
}

// Bytes of partial sums one backward launch writes: (blocks it will use) x hidden floats -- the same choice of
// kernel and grid as dispatch_bwd.
int64_t bwd_partial_bytes(int64_t rows, int64_t hidden, int dtype) {
  const int vec = dtype == PICO_BF16 ? 8 : 4;
  const int nvec = static_cast<int>(hidden / vec);
  const int nv_wave = pick_nv((nvec + 63) / 64, 8);
  if (nv_wave) return static_cast<int64_t>(bwd_blocks(rows, kBwdWaves, static_cast<int>(hidden))) * hidden * static_cast<int64_t>(sizeof(float));
  return static_cast<int64_t>(bwd_blocks(rows, kBwdThreads / 256, static_cast<int>(hidden))) * hidden * static_cast<int64_t>(sizeof(float));
}

int check_common(const char* fn, int64_t rows, int64_t hidden, int dtype) {
  if (dtype != PICO_BF16 && dtype != PICO_F32) return fail(PICO_ERR_DTYPE, "%s: dtype code %d not supported", fn, dtype);
  const int vec = dtype == PICO_BF16 ? 8 : 4;
  if (rows < 0 || hidden <= 0 || hidden > 16384 || hidden % vec != 0)
    return fail(PICO_ERR_SHAPE, "%s: rows=%lld hidden=%lld (hidden must be a positive multiple of %d, <= 16384)", fn,
                static_cast<long long>(rows), static_cast<long long>(hidden), vec);
  return PICO_OK;
}

}  // namespace
}  // namespace pico

using namespace pico;

extern "C" int pico_rmsnorm_fwd(const void* x, const void* weight, void* y, float* rstd, const void* residual_in,
                                void* residual_out, int64_t rows, int64_t hidden, float eps, int cast_then_scale,
                                int dtype, void* stream) {
  if (int rc = check_common("pico_rmsnorm_fwd", rows, hidden, dtype)) return rc;
  if (rows == 0) return PICO_OK;
  if (!x || !weight || !y) return fail(PICO_ERR_NULL, "pico_rmsnorm_fwd: x, weight and y are required");
  if (residual_out && !residual_in) return fail(PICO_ERR_NULL, "pico_rmsnorm_fwd: residual_out without residual_in");
  if (!aligned16(x) || !aligned16(weight) || !aligned16(y) || !aligned16(residual_in) || !aligned16(residual_out))
    return fail(PICO_ERR_ALIGN, "pico_rmsnorm_fwd: pointers must be 16-byte aligned");
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc = dtype == PICO_BF16
               ? dispatch_fwd<__bf16>(x, weight, y, rstd, residual_in, residual_out, rows, static_cast<int>(hidden), eps, cast_then_scale, s)
               : dispatch_fwd<float>(x, weight, y, rstd, residual_in, residual_out, rows, static_cast<int>(hidden), eps, cast_then_scale, s);
  if (rc) return rc;
  return check_launch("pico_rmsnorm_fwd");
}

extern "C" int64_t pico_rmsnorm_bwd_workspace_bytes(int64_t rows, int64_t hidden) {
  (void)rows;
  if (hidden <= 0) return 0;
  return static_cast<int64_t>(kMaxBwdBlocks) * hidden * static_cast<int64_t>(sizeof(float));
}

namespace {

// Everything of the backward but the question of where the partial sums live.  `partial_bytes` is what the caller's
// buffer holds; the launch needs bwd_partial_bytes(rows, hidden) of it.
int rmsnorm_bwd_impl(const char* fn, const void* dy, const void* x, const void* weight, const float* rstd,
                     const void* dresidual, void* dx, void* dweight, int dweight_dtype, float* partial,
                     int64_t partial_bytes, int64_t rows, int64_t hidden, int dtype, hipStream_t s) {
  if (int rc = check_common(fn, rows, hidden, dtype)) return rc;
  if (dweight_dtype != PICO_BF16 && dweight_dtype != PICO_F32)
    return fail(PICO_ERR_DTYPE, "%s: dweight dtype code %d not supported", fn, dweight_dtype);
  if (!dweight) return fail(PICO_ERR_NULL, "%s: dweight is required", fn);
  if (rows == 0) {  // empty sum: dweight = 0 (the reduce kernel with no partials writes zeros)
    launch_dw_reduce(nullptr, dweight, dweight_dtype, 0, static_cast<int>(hidden), s);
    return check_launch(fn);
  }
  if (!dy || !x || !weight || !rstd || !dx || !partial)
    return fail(PICO_ERR_NULL, "%s: dy, x, weight, rstd, dx and the partial-sum buffer are required", fn);
  const int64_t need = bwd_partial_bytes(rows, hidden, dtype);
  if (partial_bytes < need)
    return fail(PICO_ERR_WORKSPACE, "%s: the partial-sum buffer has %lld bytes, rows=%lld hidden=%lld need %lld", fn,
                static_cast<long long>(partial_bytes), static_cast<long long>(rows), static_cast<long long>(hidden),
                static_cast<long long>(need));
  if (!aligned16(dy) || !aligned16(x) || !aligned16(weight) || !aligned16(dx) || !aligned16(partial) ||
      !aligned16(dresidual))
    return fail(PICO_ERR_ALIGN, "%s: pointers must be 16-byte aligned", fn);
  int blocks = 0;
  int rc = dtype == PICO_BF16
               ? dispatch_bwd<__bf16>(dy, x, weight, rstd, dresidual, dx, partial, rows, static_cast<int>(hidden), s, &blocks)
               : dispatch_bwd<float>(dy, x, weight, rstd, dresidual, dx, partial, rows, static_cast<int>(hidden), s, &blocks);
  if (rc) return rc;
  if (int lrc = check_launch(fn)) return lrc;
  launch_dw_reduce(partial, dweight, dweight_dtype, blocks, static_cast<int>(hidden), s);
  return check_launch(fn);
}

// Device address of `scratch` on the current GPU, looked up once per device (every GPU holds its own copy of the
// array at its own address).
constexpr int kMaxDevices = 64;
std::atomic<float*> g_scratch_addr[kMaxDevices];

int static_scratch(const char* fn, float** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(PICO_ERR_LAUNCH, "%s: cannot tell the current device", fn);
  float* p = g_scratch_addr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    const hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return fail(PICO_ERR_LAUNCH, "%s: hipGetSymbolAddress(scratch) failed on device %d: %s", fn, dev, hipGetErrorString(e));
    g_scratch_addr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return PICO_OK;
}

}  // namespace

extern "C" int pico_rmsnorm_bwd(const void* dy, const void* x, const void* weight, const float* rstd,
                                const void* dresidual, void* dx, void* dweight, int dweight_dtype, void* workspace,
                                int64_t workspace_bytes, int64_t rows, int64_t hidden, int dtype, void* stream) {
  return rmsnorm_bwd_impl("pico_rmsnorm_bwd", dy, x, weight, rstd, dresidual, dx, dweight, dweight_dtype,
                          static_cast<float*>(workspace), workspace_bytes, rows, hidden, dtype,
                          static_cast<hipStream_t>(stream));
}

extern "C" int64_t pico_rmsnorm_bwd_static_max_bytes(void) {
  return static_cast<int64_t>(kStaticScratchFloats * sizeof(float));
}

extern "C" int pico_rmsnorm_bwd_static(const void* dy, const void* x, const void* weight, const float* rstd,
                                       const void* dresidual, void* dx, void* dweight, int dweight_dtype, int64_t rows,
                                       int64_t hidden, int dtype, void* stream) {
  const char* fn = "pico_rmsnorm_bwd_static";
  if (int rc = check_common(fn, rows, hidden, dtype)) return rc;
  const int64_t need = bwd_partial_bytes(rows, hidden, dtype);
  if (need > pico_rmsnorm_bwd_static_max_bytes())
    return fail(PICO_ERR_WORKSPACE, "%s: rows=%lld hidden=%lld need %lld bytes of partial sums, the static scratch "
                "holds %lld; use pico_rmsnorm_bwd with a workspace", fn, static_cast<long long>(rows),
                static_cast<long long>(hidden), static_cast<long long>(need),
                static_cast<long long>(pico_rmsnorm_bwd_static_max_bytes()));
  float* partial = nullptr;
  if (int rc = static_scratch(fn, &partial)) return rc;
  return rmsnorm_bwd_impl(fn, dy, x, weight, rstd, dresidual, dx, dweight, dweight_dtype, partial,
                          pico_rmsnorm_bwd_static_max_bytes(), rows, hidden, dtype, static_cast<hipStream_t>(stream));
}
