// Attention backward for gfx950 (MFMA bf16): one workgroup owns 128 keys of one kv head, keeps
// dK / dV for them in registers, and walks over the query tiles (and the query heads of a GQA
// group) that can see those keys.
//
// Per 64-query tile:
//   S  = Q K^T, dP = dO V^T          (C tile: lane = key, registers = queries; K, V fragments live
//                                     in registers for the whole kernel)
//   P  = exp2(S*c - lse*log2e),  dS = P * (dP - delta)
//   dV += P^T dO,  dK += dS^T Q      (P / dS feed the MFMA straight from registers as the A operand;
//                                     dO and Q come from the row-major LDS tiles through transposing reads)
//   dS^T -> LDS, barrier
//   dQ  = dS K * scale               (each wave owns 32x32 blocks of the 64 x D tile over all 128 keys; K
//                                     fragments stay in registers, dS comes back through transposing
//                                     LDS reads) -> fp32 atomic adds
#include "attn_common.h"

#include <type_traits>

#if defined(PICO_BWD_TIMING)
__device__ long long pico_dbg[64];
#define PICO_T(i) do { if (blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x == 0 && it == 2) pico_dbg[i] = clock64(); } while (0)
extern "C" int pico_debug_read(long long* out) { return (int)hipMemcpyFromSymbol(out, HIP_SYMBOL(pico_dbg), sizeof(long long) * 64); }
#else
#define PICO_T(i)
#endif

namespace pico {
namespace {

struct BwdParams {
  AttnParams a;
  const __bf16* dout;
  const float* lse;
  const float* delta;
  float* dq_acc;
  void* dk;
  void* dv;
  int dkv_f32;
  int accumulate;
  int64_t dks[3];  // element strides (b, h, s) of dk and dv
};

template <int D>
struct BwdCfg {
  static constexpr int NW = 4;
  static constexpr int kThreads = 64 * NW;
  static constexpr int BN = 32 * NW;  // keys per workgroup
  static constexpr int BM = 64;       // queries per iteration
  static constexpr int LDQ = D + 8;   // pitch of the Q, dO and K tiles
  static constexpr int LDS_ = BM + 8; // pitch of the dS^T tile [BN][BM]
  static constexpr int kVecPerRow = D / 8;
  static constexpr int kQLoads = BM * kVecPerRow / kThreads;
  static constexpr int kKLoads = BN * kVecPerRow / kThreads;
  static constexpr size_t kLdsBytes =
      (2 * BM * LDQ + BN * LDQ + 2 * BN * LDS_) * sizeof(__bf16) + 2 * BM * sizeof(float);
};

template <int D>
__device__ __forceinline__ void attn_bwd_body(const BwdParams& p) {
  using C = BwdCfg<D>;
  constexpr int BM = C::BM, BN = C::BN, LDQ = C::LDQ, LDS_ = C::LDS_;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __bf16* sQ = reinterpret_cast<__bf16*>(smem_raw);
  __bf16* sdO = sQ + BM * LDQ;
  __bf16* sK = sdO + BM * LDQ;
  __bf16* sdS = sK + BN * LDQ;
  float* sL = reinterpret_cast<float*>(sdS + 2 * BN * LDS_);  // sdS is double-buffered
  float* sDelta = sL + BM;

  const AttnParams& a = p.a;
  // grid = (Hkv * B, key tiles): the x index runs fastest in dispatch order, so all heads of key tile 0
  // (the longest under a causal mask) start first and the short tiles fill in behind them; workgroups of
  // one head are a multiple of 8 apart in dispatch order and so share an XCD's L2
  const int ktile = blockIdx.y, hkv = blockIdx.x % a.Hkv, b = blockIdx.x / a.Hkv;
  const int group = a.Hq / a.Hkv;
  const int key0 = ktile * BN;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int n = lane % 32, h = lane / 32;
  const float c = a.sm_scale * kLog2e;

  const __bf16* kbase = a.k + b * a.ks[0] + hkv * a.ks[1];
  const __bf16* vbase = a.v + b * a.vs[0] + hkv * a.vs[1];

  // ---- K, V fragments of this wave's 32 keys (B operand: lane = key, 8 consecutive d per k step)
  bf16x8 kf[D / 16], vf[D / 16];
  {
    const int key = key0 + 32 * wave + n;
    const bool live = key < a.Sk;
#pragma unroll
    for (int s = 0; s < D / 16; ++s) {
      u32x4 rk = {0, 0, 0, 0}, rv = {0, 0, 0, 0};
      if (live) {
        rk = *reinterpret_cast<const u32x4*>(kbase + static_cast<int64_t>(key) * a.ks[2] + 16 * s + 8 * h);
        rv = *reinterpret_cast<const u32x4*>(vbase + static_cast<int64_t>(key) * a.vs[2] + 16 * s + 8 * h);
      }
      kf[s] = __builtin_bit_cast(bf16x8, rk);
      vf[s] = __builtin_bit_cast(bf16x8, rv);
    }
  }
  // ---- K tile -> LDS (row-major, rows past Sk are zero) for the dQ product
#pragma unroll
  for (int i = 0; i < C::kKLoads; ++i) {
    const int idx = tid + i * C::kThreads;
    const int r = idx / C::kVecPerRow, cv = idx % C::kVecPerRow;
    u32x4 raw = {0, 0, 0, 0};
    if (key0 + r < a.Sk) raw = *reinterpret_cast<const u32x4*>(kbase + static_cast<int64_t>(key0 + r) * a.ks[2] + cv * 8);
    *reinterpret_cast<u32x4*>(&sK[r * LDQ + cv * 8]) = raw;
  }

  // ---- K as the B operand of dQ = dS K (B[k = key][n = d]) for the dQ blocks this wave owns: read
  //      once through transposing LDS reads and kept in registers
  constexpr int kDqBlocks = (BM / 32) * (D / 32);
  constexpr int kDqPasses = kDqBlocks / C::NW;
  static_assert(kDqBlocks % C::NW == 0, "dQ blocks must split evenly over the waves");
  bf16x8 ktf[kDqPasses][BN / 16];
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < kDqPasses; ++pass) {
    const int db_w = (pass * C::NW + wave) % (D / 32);
#pragma unroll
    for (int ks = 0; ks < BN / 16; ++ks) {
      const int krow = 16 * ks + 4 * h + (lane % 16) / 4;
      ktf[pass][ks] = lds_read_tr_pair(&sK[krow * LDQ + 32 * db_w + 16 * ((lane / 16) % 2) + 4 * (lane % 4)], LDQ);
    }
  }

  f32x16 dk_acc[D / 32], dv_acc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) { dk_acc[db][i] = 0.f; dv_acc[db][i] = 0.f; }

  // ---- iteration space: (query head of the group) x (query tiles that can see key0)
  const int n_qtiles = (a.Sq + BM - 1) / BM;
  int qt_start = 0;
  if (a.causal) {
    const int first_q = key0 - a.q_offset;  // first query index that sees key0
    qt_start = first_q > 0 ? first_q / BM : 0;
  }
  const int tiles_per_head = n_qtiles > qt_start ? n_qtiles - qt_start : 0;
  const int n_iter = tiles_per_head * group;

  // Global -> register prefetch of the next Q / dO tile (+ lse, delta).  Loads are unconditional (rows
  // past Sq are clamped to the last row and zeroed when they are written to LDS) and nothing here uses a
  // loaded value, so the loop never has to wait for memory inside the prefetch.
  u32x4 qreg[C::kQLoads], doreg[C::kQLoads];
  float lreg = 0.f, dreg = 0.f;
  auto prefetch = [&](int it) {
    const int hq = hkv * group + it / tiles_per_head;
    const int q0 = (qt_start + it % tiles_per_head) * BM;
    const __bf16* qb = a.q + b * a.qs[0] + hq * a.qs[1];
    const __bf16* dob = p.dout + b * a.os[0] + hq * a.os[1];
#pragma unroll
    for (int i = 0; i < C::kQLoads; ++i) {
      const int idx = tid + i * C::kThreads;
      const int r = idx / C::kVecPerRow, cv = idx % C::kVecPerRow;
      const int row = (q0 + r < a.Sq) ? q0 + r : a.Sq - 1;
      qreg[i] = *reinterpret_cast<const u32x4*>(qb + static_cast<int64_t>(row) * a.qs[2] + cv * 8);
      doreg[i] = *reinterpret_cast<const u32x4*>(dob + static_cast<int64_t>(row) * a.os[2] + cv * 8);
    }
    {
      const int r = tid % BM;
      const int row = (q0 + r < a.Sq) ? q0 + r : a.Sq - 1;
      const int64_t gi = (static_cast<int64_t>(b) * a.Hq + hq) * a.Sq + row;
      lreg = p.lse[gi];
      dreg = p.delta[gi];
    }
  };

  if (n_iter > 0) prefetch(0);

  // Software pipeline over the (head, query tile) pairs.  Trip `it` stages tile `it` in LDS and runs its
  // S phase, and first finishes tile `it - 1`: its dS^T sits in the other half of the double-buffered
  // sdS, so the dQ product and its atomics are issued a whole trip before anything waits on memory
  // again, and one barrier per tile disappears.  The prefetch loads are issued after those atomics, so
  // the wait before the next LDS fill covers operations that have had a full trip to complete.
  int prev_hq = 0, prev_q0 = 0;
  for (int it = 0; it <= n_iter; ++it) {
    const bool have_tile = it < n_iter;
    const int hq = hkv * group + (have_tile ? it / tiles_per_head : 0);
    const int q0 = (qt_start + (have_tile ? it % tiles_per_head : 0)) * BM;
    PICO_T(0);
    __syncthreads();  // S phase of tile it-1 is complete: sdS[(it-1)&1] is full, sQ / sdO are free
    PICO_T(1);
    if (have_tile) {
#pragma unroll
      for (int i = 0; i < C::kQLoads; ++i) {
        const int idx = tid + i * C::kThreads;
        const int r = idx / C::kVecPerRow, cv = idx % C::kVecPerRow;
        const bool live = q0 + r < a.Sq;
        const u32x4 zero = {0, 0, 0, 0};
        *reinterpret_cast<u32x4*>(&sQ[r * LDQ + cv * 8]) = live ? qreg[i] : zero;
        *reinterpret_cast<u32x4*>(&sdO[r * LDQ + cv * 8]) = live ? doreg[i] : zero;
      }
      if (tid < BM) {
        // rows past Sq, and rows whose lse is -inf (they saw no key), get lse = +inf so that P = 0
        const bool live = q0 + tid < a.Sq && lreg != -INFINITY;
        sL[tid] = live ? lreg * kLog2e : INFINITY;
        sDelta[tid] = live ? dreg : 0.f;
      }
    }
    PICO_T(2);
    __syncthreads();
    PICO_T(3);

    // ================= dQ of the previous tile: the 64 x D tile is cut into 32 x 32 blocks, NW per pass
#if !defined(PICO_BWD_NO_DQ)
    if (it > 0) {
      const __bf16* sdS_prev = sdS + ((it - 1) & 1) * (BN * LDS_);
#pragma unroll
      for (int pass = 0; pass < kDqPasses; ++pass) {
        const int blk = pass * C::NW + wave;         // block index: query half x d block
        const int qb_w = blk / (D / 32), db_w = blk % (D / 32);
        f32x16 dq;
#pragma unroll
        for (int i = 0; i < 16; ++i) dq[i] = 0.f;
#pragma unroll
        for (int ks = 0; ks < BN / 16; ++ks) {
          // A[m = query][k = key]: slots 4jj+t <- keys 16ks + 8jj + 4h + t, read transposed from dS^T[key][query]
          const int krow = 16 * ks + 4 * h + (lane % 16) / 4;
          const bf16x8 af = lds_read_tr_pair(&sdS_prev[krow * LDS_ + 32 * qb_w + 16 * ((lane / 16) % 2) + 4 * (lane % 4)], LDS_);
          dq = mfma32(af, ktf[pass][ks], dq);
        }
        // rows past Sq add 0 to the last valid row instead of branching around the atomic
        float* dqp = p.dq_acc + ((static_cast<int64_t>(b) * a.Hq + prev_hq) * a.Sq) * D + 32 * db_w + n;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int qrow = prev_q0 + 32 * qb_w + 8 * (i / 4) + 4 * h + (i % 4);
          const bool live = qrow < a.Sq;
          const float val = live ? dq[i] * a.sm_scale : 0.f;
          float* dst = dqp + static_cast<int64_t>(live ? qrow : a.Sq - 1) * D;
#if defined(PICO_BWD_NO_ATOMIC)
          *dst = val;
#else
          unsafeAtomicAdd(dst, val);
#endif
        }
      }
    }
#endif
    PICO_T(4);
    if (!have_tile) break;
    if (it + 1 < n_iter) prefetch(it + 1);
    PICO_T(5);

    // ================= S phase: this wave's 32 keys against the tile's 64 queries
    __bf16* sdS_cur = sdS + (it & 1) * (BN * LDS_);
    const int kw0 = key0 + 32 * wave;
#pragma unroll
    for (int sb = 0; sb < BM / 32; ++sb) {
      const int qs_pos = a.q_offset + q0 + 32 * sb;  // position of the sub-block's first query
      __bf16* ds_dst = &sdS_cur[(32 * wave + n) * LDS_ + 32 * sb + 4 * h];
      if (a.causal && kw0 > qs_pos + 31) {  // every (query, key) pair of this 32x32 block is masked
#pragma unroll
        for (int j = 0; j < 4; ++j) *reinterpret_cast<u32x2*>(ds_dst + 8 * j) = u32x2{0, 0};
        continue;
      }
      f32x16 s_acc, dp_acc;
#pragma unroll
      for (int i = 0; i < 16; ++i) { s_acc[i] = 0.f; dp_acc[i] = 0.f; }
#pragma unroll
      for (int s = 0; s < D / 16; ++s) {
        const bf16x8 qa = *reinterpret_cast<const bf16x8*>(&sQ[(32 * sb + n) * LDQ + 16 * s + 8 * h]);
        const bf16x8 da = *reinterpret_cast<const bf16x8*>(&sdO[(32 * sb + n) * LDQ + 16 * s + 8 * h]);
        s_acc = mfma32(qa, kf[s], s_acc);
        dp_acc = mfma32(da, vf[s], dp_acc);
      }
      // P = exp2(S*c - lse*log2e), dS = P * (dP - delta); the mask test is paid only on the diagonal
      auto softmax_grad = [&](auto mask_c) {
        constexpr bool kMask = decltype(mask_c)::value;
        const int key_rel = kw0 + n - qs_pos - 4 * h;  // key is masked for row (8j + 4h + t) iff key_rel > 8j + t
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const f32x4 l4 = *reinterpret_cast<const f32x4*>(&sL[32 * sb + 8 * j + 4 * h]);
          const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sDelta[32 * sb + 8 * j + 4 * h]);
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int i = 4 * j + t;
            float pv = fast_exp2(s_acc[i] * c - l4[t]);
            if constexpr (kMask) {
              if (key_rel > 8 * j + t) pv = 0.f;
            }
            s_acc[i] = pv;
            dp_acc[i] = pv * (dp_acc[i] - d4[t]);
          }
        }
      };
      if (a.causal && kw0 + 31 > qs_pos) softmax_grad(std::true_type{});
      else softmax_grad(std::false_type{});
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        const bf16x8 pf = pack8(s_acc, 8 * cc);
        const bf16x8 dsf = pack8(dp_acc, 8 * cc);
        // dS^T[key][query]: registers 8cc+4jj+t hold queries 32sb + 16cc + 8jj + 4h + t
        const u32x4 raw = __builtin_bit_cast(u32x4, dsf);
        *reinterpret_cast<u32x2*>(ds_dst + 16 * cc) = u32x2{raw[0], raw[1]};
        *reinterpret_cast<u32x2*>(ds_dst + 16 * cc + 8) = u32x2{raw[2], raw[3]};
        const int qr = 32 * sb + 16 * cc + 4 * h + (lane % 16) / 4;
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          const int col = 32 * db + 16 * ((lane / 16) % 2) + 4 * (lane % 4);
          const bf16x8 dof = lds_read_tr_pair(&sdO[qr * LDQ + col], LDQ);
          const bf16x8 qf = lds_read_tr_pair(&sQ[qr * LDQ + col], LDQ);
          dv_acc[db] = mfma32(pf, dof, dv_acc[db]);
          dk_acc[db] = mfma32(dsf, qf, dk_acc[db]);
        }
      }
    }
    PICO_T(6);
    prev_hq = hq;
    prev_q0 = q0;
  }

  // ---- epilogue: dK (scaled) and dV rows of this wave's keys.  In accumulate mode all reads of a block
  //      are issued before the first write so they overlap instead of serialising on memory latency.
#pragma unroll
  for (int db = 0; db < D / 32; ++db) {
    int64_t off[16];
    bool live[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = key0 + 32 * wave + 8 * (i / 4) + 4 * h + (i % 4);
      live[i] = key < a.Sk;
      off[i] = b * p.dks[0] + hkv * p.dks[1] + static_cast<int64_t>(live[i] ? key : 0) * p.dks[2] + 32 * db + n;
    }
    if (p.dkv_f32) {
      float* pk = static_cast<float*>(p.dk);
      float* pv = static_cast<float*>(p.dv);
      float ok[16], ov[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) { ok[i] = 0.f; ov[i] = 0.f; }
      if (p.accumulate) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (live[i]) { ok[i] = pk[off[i]]; ov[i] = pv[off[i]]; }
      }
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (live[i]) {
          pk[off[i]] = ok[i] + dk_acc[db][i] * a.sm_scale;
          pv[off[i]] = ov[i] + dv_acc[db][i];
        }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i)
        if (live[i]) {
          static_cast<__bf16*>(p.dk)[off[i]] = static_cast<__bf16>(dk_acc[db][i] * a.sm_scale);
          static_cast<__bf16*>(p.dv)[off[i]] = static_cast<__bf16>(dv_acc[db][i]);
        }
    }
  }
}

// D = 64 fits two workgroups per CU (<= 256 registers per lane), which lets one workgroup's MFMA
// work overlap the other's softmax / LDS phases; D = 128 needs the full register file.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_bwd_kernel_d64(const BwdParams p) {
  attn_bwd_body<64>(p);
}
__global__ __launch_bounds__(256) void attn_bwd_kernel_d128(const BwdParams p) { attn_bwd_body<128>(p); }

template <int D> struct BwdKernel;
template <> struct BwdKernel<64> { static constexpr auto fn = &attn_bwd_kernel_d64; };
template <> struct BwdKernel<128> { static constexpr auto fn = &attn_bwd_kernel_d128; };

// delta[row] = sum_d dO * O, one 16-byte vector of each per lane, D/8 lanes per row.
template <int D, typename TO>
__global__ __launch_bounds__(256) void attn_bwd_preprocess_kernel(const __bf16* __restrict__ dout,
                                                                  const TO* __restrict__ out, float* __restrict__ delta,
                                                                  float* __restrict__ dq_acc, int B, int H, int S,
                                                                  int64_t sb, int64_t sh, int64_t ss) {
  constexpr int LPR = D / 8;  // lanes per row
  const int64_t idx = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
  const int64_t rows = static_cast<int64_t>(B) * H * S;
  const int64_t row = idx / LPR;
  const int v = static_cast<int>(idx % LPR);
  float part = 0.f;
  if (row < rows) {
    const int s = static_cast<int>(row % S);
    const int hh = static_cast<int>((row / S) % H);
    const int64_t bb = row / (static_cast<int64_t>(S) * H);
    const int64_t off = bb * sb + hh * sh + s * ss + v * 8;
    float d8[8], o8[8];
    io<__bf16>::load(dout + off, d8);
    if constexpr (sizeof(TO) == 2) {
      io<__bf16>::load(out + off, o8);
    } else {
      float t[4];
      io<float>::load(out + off, t);
#pragma unroll
      for (int e = 0; e < 4; ++e) o8[e] = t[e];
      io<float>::load(out + off + 4, t);
#pragma unroll
      for (int e = 0; e < 4; ++e) o8[4 + e] = t[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) part += d8[e] * o8[e];
    if (dq_acc != nullptr) {
      const f32x4 z = {0.f, 0.f, 0.f, 0.f};
      *reinterpret_cast<f32x4*>(dq_acc + row * D + v * 8) = z;
      *reinterpret_cast<f32x4*>(dq_acc + row * D + v * 8 + 4) = z;
    }
  }
#pragma unroll
  for (int off = LPR / 2; off > 0; off >>= 1) part += __shfl_xor(part, off, kWave);
  if (row < rows && v == 0) delta[row] = part;
}

template <int D>
int launch_bwd(const BwdParams& p, hipStream_t s) {
  using C = BwdCfg<D>;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(BwdKernel<D>::fn),
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(C::kLdsBytes)) != hipSuccess)
      return fail(PICO_ERR_LAUNCH, "pico_attn_bwd: cannot reserve %zu bytes of LDS", C::kLdsBytes);
    attr_set = true;
  }
  const int n_ktiles = (p.a.Sk + C::BN - 1) / C::BN;
  hipLaunchKernelGGL(BwdKernel<D>::fn, dim3(p.a.Hkv * p.a.B, n_ktiles), dim3(C::kThreads), C::kLdsBytes, s, p);
  return PICO_OK;
}

}  // namespace
}  // namespace pico

using namespace pico;

extern "C" int pico_attn_bwd_preprocess(const pico_attn_desc* desc, const void* dout, const void* out, int out_dtype,
                                        float* delta, float* dq_acc, void* stream) {
  if (int rc = check_attn_desc("pico_attn_bwd_preprocess", desc)) return rc;
  if (out_dtype != PICO_BF16 && out_dtype != PICO_F32)
    return fail(PICO_ERR_DTYPE, "pico_attn_bwd_preprocess: out dtype code %d not supported", out_dtype);
  if (desc->B == 0 || desc->Sq == 0) return PICO_OK;
  if (!dout || !out || !delta) return fail(PICO_ERR_NULL, "pico_attn_bwd_preprocess: dout, out and delta are required");
  if (!aligned16(dout) || !aligned16(out) || !aligned16(dq_acc))
    return fail(PICO_ERR_ALIGN, "pico_attn_bwd_preprocess: dout, out and dq_acc must be 16-byte aligned");
  const int64_t rows = static_cast<int64_t>(desc->B) * desc->Hq * desc->Sq;
  const int64_t total = rows * (desc->D / 8);
  const unsigned grid = static_cast<unsigned>((total + 255) / 256);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t* os = desc->o_stride;
#define PICO_PRE(DD, TO)                                                                                   \
  hipLaunchKernelGGL((attn_bwd_preprocess_kernel<DD, TO>), dim3(grid), dim3(256), 0, s,                    \
                     static_cast<const __bf16*>(dout), static_cast<const TO*>(out), delta, dq_acc, desc->B, \
                     desc->Hq, desc->Sq, os[0], os[1], os[2])
  if (desc->D == 64) { if (out_dtype == PICO_BF16) PICO_PRE(64, __bf16); else PICO_PRE(64, float); }
  else               { if (out_dtype == PICO_BF16) PICO_PRE(128, __bf16); else PICO_PRE(128, float); }
#undef PICO_PRE
  return check_launch("pico_attn_bwd_preprocess");
}

extern "C" int pico_attn_bwd(const pico_attn_desc* desc, const void* q, const void* k, const void* v, const void* dout,
                             const float* lse, const float* delta, float* dq_acc, void* dk, void* dv,
                             const int64_t* dkv_stride, int dkv_dtype, int accumulate, void* stream) {
  if (int rc = check_attn_desc("pico_attn_bwd", desc)) return rc;
  if (dkv_dtype != PICO_BF16 && dkv_dtype != PICO_F32)
    return fail(PICO_ERR_DTYPE, "pico_attn_bwd: dk/dv dtype code %d not supported", dkv_dtype);
  if (accumulate && dkv_dtype != PICO_F32) return fail(PICO_ERR_DTYPE, "pico_attn_bwd: accumulate needs fp32 dk/dv");
  if (desc->B == 0 || desc->Sk == 0) return PICO_OK;  // no keys: nothing to add to dq, no dk/dv rows
  if (!k || !v || !dk || !dv || (desc->Sq > 0 && (!q || !dout || !lse || !delta || !dq_acc)))
    return fail(PICO_ERR_NULL, "pico_attn_bwd: q, k, v, dout, lse, delta, dq_acc, dk and dv are required");
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(dout))
    return fail(PICO_ERR_ALIGN, "pico_attn_bwd: q, k, v and dout must be 16-byte aligned");
  BwdParams p;
  p.a = make_params(desc, q, k, v);
  p.dout = static_cast<const __bf16*>(dout);
  p.lse = lse; p.delta = delta; p.dq_acc = dq_acc; p.dk = dk; p.dv = dv;
  p.dkv_f32 = dkv_dtype == PICO_F32;
  p.accumulate = accumulate != 0;
  if (dkv_stride) {
    for (int i = 0; i < 3; ++i) {
      if (dkv_stride[i] < 0) return fail(PICO_ERR_STRIDE, "pico_attn_bwd: negative dk/dv stride");
      p.dks[i] = dkv_stride[i];
    }
  } else {
    p.dks[2] = desc->D;
    p.dks[1] = static_cast<int64_t>(desc->Sk) * desc->D;
    p.dks[0] = p.dks[1] * desc->Hkv;
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc = desc->D == 64 ? launch_bwd<64>(p, s) : launch_bwd<128>(p, s);
  if (rc) return rc;
  return check_launch("pico_attn_bwd");
}
