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
//   dQ  = dS K * scale               (16x16x32 MFMA, each wave takes 16 query rows over all 128 keys;
//                                     both operands through transposing LDS reads) -> fp32 atomic adds
#include "attn_common.h"

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
      (2 * BM * LDQ + BN * LDQ + BN * LDS_) * sizeof(__bf16) + 2 * BM * sizeof(float);
};

template <int D>
__global__ __launch_bounds__(256) void attn_bwd_kernel(const BwdParams p) {
  using C = BwdCfg<D>;
  constexpr int BM = C::BM, BN = C::BN, LDQ = C::LDQ, LDS_ = C::LDS_;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __bf16* sQ = reinterpret_cast<__bf16*>(smem_raw);
  __bf16* sdO = sQ + BM * LDQ;
  __bf16* sK = sdO + BM * LDQ;
  __bf16* sdS = sK + BN * LDQ;
  float* sL = reinterpret_cast<float*>(sdS + BN * LDS_);
  float* sDelta = sL + BM;

  const AttnParams& a = p.a;
  const int ktile = blockIdx.x, hkv = blockIdx.y, b = blockIdx.z;
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

  u32x4 qreg[C::kQLoads], doreg[C::kQLoads];
  float lreg = INFINITY, dreg = 0.f;
  auto prefetch = [&](int it) {
    const int hq = hkv * group + it / tiles_per_head;
    const int q0 = (qt_start + it % tiles_per_head) * BM;
    const __bf16* qb = a.q + b * a.qs[0] + hq * a.qs[1];
    const __bf16* dob = p.dout + b * a.os[0] + hq * a.os[1];
#pragma unroll
    for (int i = 0; i < C::kQLoads; ++i) {
      const int idx = tid + i * C::kThreads;
      const int r = idx / C::kVecPerRow, cv = idx % C::kVecPerRow;
      u32x4 zq = {0, 0, 0, 0}, zo = {0, 0, 0, 0};
      if (q0 + r < a.Sq) {
        zq = *reinterpret_cast<const u32x4*>(qb + static_cast<int64_t>(q0 + r) * a.qs[2] + cv * 8);
        zo = *reinterpret_cast<const u32x4*>(dob + static_cast<int64_t>(q0 + r) * a.os[2] + cv * 8);
      }
      qreg[i] = zq;
      doreg[i] = zo;
    }
    if (tid < BM) {
      // rows past Sq (and rows whose lse is -inf: they saw no key) get lse = +inf so that P = 0
      lreg = INFINITY;
      dreg = 0.f;
      if (q0 + tid < a.Sq) {
        const int64_t row = (static_cast<int64_t>(b) * a.Hq + hq) * a.Sq + q0 + tid;
        const float l = p.lse[row];
        lreg = (l == -INFINITY) ? INFINITY : l * kLog2e;
        dreg = p.delta[row];
      }
    }
  };

  if (n_iter > 0) prefetch(0);

  for (int it = 0; it < n_iter; ++it) {
    const int hq = hkv * group + it / tiles_per_head;
    const int q0 = (qt_start + it % tiles_per_head) * BM;
    __syncthreads();  // previous dQ phase has finished with sdS; previous S phase with sQ / sdO
#pragma unroll
    for (int i = 0; i < C::kQLoads; ++i) {
      const int idx = tid + i * C::kThreads;
      const int r = idx / C::kVecPerRow, cv = idx % C::kVecPerRow;
      *reinterpret_cast<u32x4*>(&sQ[r * LDQ + cv * 8]) = qreg[i];
      *reinterpret_cast<u32x4*>(&sdO[r * LDQ + cv * 8]) = doreg[i];
    }
    if (tid < BM) { sL[tid] = lreg; sDelta[tid] = dreg; }
    __syncthreads();
    if (it + 1 < n_iter) prefetch(it + 1);

    // ================= S phase: this wave's 32 keys against the tile's 64 queries
    const int kw0 = key0 + 32 * wave;
#pragma unroll
    for (int sb = 0; sb < BM / 32; ++sb) {
      const int qs_pos = a.q_offset + q0 + 32 * sb;  // position of the sub-block's first query
      __bf16* ds_dst = &sdS[(32 * wave + n) * LDS_ + 32 * sb + 4 * h];
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
      const bool need_mask = a.causal && (kw0 + 31 > qs_pos);
      const int key = kw0 + n;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(&sL[32 * sb + 8 * j + 4 * h]);
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sDelta[32 * sb + 8 * j + 4 * h]);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int i = 4 * j + t;
          float pv = fast_exp2(s_acc[i] * c - l4[t]);
          if (need_mask && key > qs_pos + 8 * j + 4 * h + t) pv = 0.f;
          s_acc[i] = pv;
          dp_acc[i] = pv * (dp_acc[i] - d4[t]);
        }
      }
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
    __syncthreads();

    // ================= dQ phase: 16 query rows per wave, all 128 keys
    {
      const int m16 = lane % 16, g = lane / 16;
      f32x4 dq[D / 16];
#pragma unroll
      for (int nb = 0; nb < D / 16; ++nb) dq[nb] = f32x4{0.f, 0.f, 0.f, 0.f};
      typedef __attribute__((ext_vector_type(8))) short s16x8;
#pragma unroll
      for (int ks = 0; ks < BN / 32; ++ks) {
        // A[m = query][k = key]: slots e<4 -> keys 32ks + 8g + e, e>=4 -> +4
        const int krow = 32 * ks + 8 * g + m16 / 4;
        const __bf16* pa = &sdS[krow * LDS_ + 16 * wave + 4 * (m16 % 4)];
        const s16x4 a_lo = lds_read_tr(pa);
        const s16x4 a_hi = lds_read_tr(pa + 4 * LDS_);
        const bf16x8 af = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(a_lo, a_hi, 0, 1, 2, 3, 4, 5, 6, 7));
#pragma unroll
        for (int nb = 0; nb < D / 16; ++nb) {
          const __bf16* pb = &sK[krow * LDQ + 16 * nb + 4 * (m16 % 4)];
          const s16x4 b_lo = lds_read_tr(pb);
          const s16x4 b_hi = lds_read_tr(pb + 4 * LDQ);
          const bf16x8 bf = __builtin_bit_cast(bf16x8, (s16x8)__builtin_shufflevector(b_lo, b_hi, 0, 1, 2, 3, 4, 5, 6, 7));
          dq[nb] = mfma16(af, bf, dq[nb]);
        }
      }
      float* dqp = p.dq_acc + ((static_cast<int64_t>(b) * a.Hq + hq) * a.Sq) * D;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int qrow = q0 + 16 * wave + 4 * g + i;
        if (qrow < a.Sq) {
#pragma unroll
          for (int nb = 0; nb < D / 16; ++nb)
            unsafeAtomicAdd(dqp + static_cast<int64_t>(qrow) * D + 16 * nb + m16, dq[nb][i] * a.sm_scale);
        }
      }
    }
  }

  // ---- epilogue: dK (scaled) and dV rows of this wave's keys
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int key = key0 + 32 * wave + 8 * (i / 4) + 4 * h + (i % 4);
      if (key >= a.Sk) continue;
      const int64_t off = ((static_cast<int64_t>(b) * a.Hkv + hkv) * a.Sk + key) * D + 32 * db + n;
      const float vk = dk_acc[db][i] * a.sm_scale, vv = dv_acc[db][i];
      if (p.dkv_f32) {
        float* pk = static_cast<float*>(p.dk) + off;
        float* pv = static_cast<float*>(p.dv) + off;
        if (p.accumulate) { *pk += vk; *pv += vv; } else { *pk = vk; *pv = vv; }
      } else {
        static_cast<__bf16*>(p.dk)[off] = static_cast<__bf16>(vk);
        static_cast<__bf16*>(p.dv)[off] = static_cast<__bf16>(vv);
      }
    }
}

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
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_bwd_kernel<D>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(C::kLdsBytes)) != hipSuccess)
      return fail(PICO_ERR_LAUNCH, "pico_attn_bwd: cannot reserve %zu bytes of LDS", C::kLdsBytes);
    attr_set = true;
  }
  const int n_ktiles = (p.a.Sk + C::BN - 1) / C::BN;
  hipLaunchKernelGGL((attn_bwd_kernel<D>), dim3(n_ktiles, p.a.Hkv, p.a.B), dim3(C::kThreads), C::kLdsBytes, s, p);
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
                             const float* lse, const float* delta, float* dq_acc, void* dk, void* dv, int dkv_dtype,
                             int accumulate, void* stream) {
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
  hipStream_t s = static_cast<hipStream_t>(stream);
  int rc = desc->D == 64 ? launch_bwd<64>(p, s) : launch_bwd<128>(p, s);
  if (rc) return rc;
  return check_launch("pico_attn_bwd");
}
