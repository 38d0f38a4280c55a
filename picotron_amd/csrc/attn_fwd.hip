// Flash-style attention forward for gfx950: S^T = K Q^T and O^T = V^T P^T on MFMA 32x32x16 bf16.
//
// Computing the TRANSPOSED score tile puts one query in each lane (column n of the C tile) and
// the keys in its registers, so the online-softmax max/sum are in-register reductions plus one
// exchange between the two wave halves, the per-query rescale factor is a per-lane scalar for the
// O^T accumulator, and the probabilities can be fed to the second MFMA as its B operand without
// leaving registers.  K and V tiles are staged row-major in LDS once per workgroup; K is read with
// 16-byte loads, V with transposing LDS reads (the contraction index of P V is V's row).
#include "attn_common.h"

namespace pico {
namespace {

struct FwdParams {
  AttnParams a;
  void* out;
  float* lse;
  int out_f32;
  int merge;
  int pair_order;  // dispatch order of the query tiles, see the kernel
  RopeArgs rope;   // rope.cos != nullptr: q arrives un-rotated and is rotated in the prologue (k is rotated already)
  __bf16* q_rot;   // ... and, if given, the rotated q is written here for the backward
  int64_t qrs[3];  // element strides (b, h, s) of q_rot
};

// KS > 1 splits the keys of a staged tile over KS waves that share the same queries (NW / KS waves cover the queries):
// for launches with about one wave per SIMD, where a wave's S -> softmax -> PV chain per key tile is not hidden by
// anything, this multiplies the waves in flight and divides each chain's length by KS.  The KS partial (m, l, O)
// states of a query meet in LDS at the end.
template <int D, int QB, int NW, int KT, int KS = 1>
struct FwdCfg {
  static constexpr int kThreads = 64 * NW;
  static constexpr int kQWaves = NW / KS;        // waves that cover different queries
  static constexpr int BM = 32 * QB * kQWaves;   // queries per workgroup
  static_assert(NW % KS == 0 && (KS == 1 || KT == 64 * KS), "one 64-key step of every staged tile per key-split wave");
  static_assert(KS == 1 || QB == 1, "key split is built for one query block per wave");
  static constexpr int BN = 64;            // keys per compute step
  static constexpr int kKT = KT;           // keys per staged LDS tile (a multiple of BN), double-buffered
  static constexpr int kKDepth = D >= 128 ? 2 : 0;  // K fragments in flight from LDS ahead of the MFMA that uses them (0: compiler's order)
  static constexpr int LDK = D + 8;        // K tile pitch: 16-byte row reads hit distinct banks
  // V tile pitch for the 4-row transposing reads.  At head_dim 128: 16 (mod 32) words, so that the 16-word pieces of 4
  // consecutive rows tile the 64 LDS banks (2 requests per bank, the minimum for an 8-byte read; a pitch of D + 8 gives
  // 3-4): -3 %.  At head_dim 64 the kernel's time does not depend on it, and the smaller tile lets two key-split
  // workgroups (128 staged keys each) share a CU.
  static constexpr int LDV = D + (D >= 128 ? 32 : 8);
  static constexpr int kVecPerRow = D / 8;
  static constexpr int kLoads = KT * kVecPerRow / kThreads;  // 16-byte loads per thread per tensor
  static constexpr int kTileElems = KT * (LDK + LDV);
  static constexpr size_t kLdsBytes = 2 * kTileElems * sizeof(__bf16);
  static_assert(NW * QB * kRowRegionBytes <= kLdsBytes, "the epilogue reuses the tile buffers");
  // exchange of partial states between key-split waves: per wave O^T accumulators (D/32 x 16 registers x 64 lanes) + m + l
  static constexpr size_t kExchangeBytes = (D / 32) * 16 * 64 * 4 + 2 * 64 * 4;
  static_assert(KS == 1 || NW * kExchangeBytes <= kLdsBytes, "the exchange reuses the tile buffers");
  static_assert(NW * QB * WaveTile<D>::kRegionBytes <= kLdsBytes, "the Q fragments pass through the tile buffers");
  static_assert(KT % BN == 0 && (KT * kVecPerRow) % kThreads == 0, "tile must split evenly over the threads");
};

template <int D, int QB, int NW, int KT, int KS = 1>
__global__ __launch_bounds__(64 * NW) void attn_fwd_kernel(const FwdParams p) {
  using C = FwdCfg<D, QB, NW, KT, KS>;
  constexpr int BM = C::BM, BN = C::BN, LDK = C::LDK, LDV = C::LDV;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __bf16* smem = reinterpret_cast<__bf16*>(smem_raw);

  const AttnParams& a = p.a;
  const int n_qtiles = (a.Sq + BM - 1) / BM;
  // grid = (Hq * B, query tiles): x runs fastest in dispatch order, so every head's last query tile (the
  // longest under a causal mask) starts first and the short tiles fill in behind.  When the whole launch is
  // resident at once (pair_order), workgroups j and j + (half the grid) share a CU, so the second half runs
  // the short tiles in ASCENDING order: every CU then holds a long and a short tile of equal total length.
  const int y = static_cast<int>(blockIdx.y), half = (n_qtiles + 1) / 2;
  const int qtile = (p.pair_order && y >= half) ? y - half : n_qtiles - 1 - y;
  const int hq = blockIdx.x % a.Hq, b = blockIdx.x / a.Hq;
  const int hkv = hq / (a.Hq / a.Hkv);
  const int q0 = qtile * BM;
  const int tid = threadIdx.x, lane = tid % 64;
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64);   // uniform over the wave: lets wave-dependent tests be scalar branches
  const int n = lane % 32, h = lane / 32;
  const int qw = wave % C::kQWaves, ks = wave / C::kQWaves;   // which queries, which 64-key step of a staged tile

  const __bf16* qbase = a.q + b * a.qs[0] + hq * a.qs[1];

  // ---- Q fragments (B operand of S^T): lane = query, 8 consecutive d per 16-wide k step; fetched row-major and
  //      turned into fragments through the wave's piece of LDS (the tile buffers are filled only after the
  //      barrier below)
  bf16x8 qf[QB][D / 16];
  int qrow[QB];
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const int row0 = q0 + (qw * QB + qb) * 32;
    qrow[qb] = row0 + n;
    WaveTile<D> qt;
    qt.issue(make_buffer(qbase + static_cast<int64_t>(row0) * a.qs[2], span_bytes(a.Sq - row0, a.qs[2], D)), a.qs[2], lane);
    qt.fragments(smem_raw + (wave * QB + qb) * WaveTile<D>::kRegionBytes, lane, qf[qb]);
    if (p.rope.cos != nullptr) {
      // RoPE on the wave's own queries, once per query in the whole launch (every query belongs to one wave)
      const bool qlive = qrow[qb] < a.Sq;
      rope_rotate_fragments<D>(qf[qb], p.rope, qlive ? p.rope.q_pos0 + qrow[qb] : 0, h);
      if (p.q_rot != nullptr && qlive && (KS == 1 || ks == 0)) {
        __bf16* dst = p.q_rot + b * p.qrs[0] + hq * p.qrs[1] + static_cast<int64_t>(qrow[qb]) * p.qrs[2];
#pragma unroll
        for (int s = 0; s < D / 16; ++s) *reinterpret_cast<bf16x8*>(dst + 16 * s + 8 * h) = qf[qb][s];
      }
    }
  }

  // ---- running state: m in the log2 domain (scores scaled by sm_scale*log2e), l split over the halves
  const float c = a.sm_scale * kLog2e;
  float m_run[QB], l_run[QB];
  f32x16 o[QB][D / 32];
  const int64_t lse_row0 = (static_cast<int64_t>(b) * a.Hq + hq) * a.Sq;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[qb][db][i] = 0.f;
    if (p.merge && ks == 0 && qrow[qb] < a.Sq) {
      // continue from (out, lse) of the earlier blocks: m = lse, l = 1, acc = out
      const float prev = p.lse[lse_row0 + qrow[qb]];
      if (prev != -INFINITY) {
        m_run[qb] = prev * kLog2e;
        l_run[qb] = (h == 0) ? 1.f : 0.f;
        const float* po = static_cast<const float*>(p.out) + b * a.os[0] + hq * a.os[1] +
                          static_cast<int64_t>(qrow[qb]) * a.os[2];
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const f32x4 v4 = *reinterpret_cast<const f32x4*>(po + 32 * db + 8 * j + 4 * h);
#pragma unroll
            for (int t = 0; t < 4; ++t) o[qb][db][4 * j + t] = v4[t];
          }
      }
    }
  }

  // ---- key range of this query tile
  const int q_hi = (q0 + BM < a.Sq ? q0 + BM : a.Sq);           // one past the last live query
  int kv_end = a.Sk;
  if (a.causal) {
    const int vis = a.q_offset + q_hi;                            // keys < vis can be seen by some query
    kv_end = vis < a.Sk ? vis : a.Sk;
    if (kv_end < 0) kv_end = 0;
  }
  const int ntiles = (kv_end + KT - 1) / KT;

  // ---- global -> register -> LDS staging of one K/V tile of KT keys, with buffer loads: a wave-uniform
  //      resource per tile (first key row, bytes left in the sequence) plus per-lane byte offsets that are
  //      computed once; rows past Sk read as zeros.  The loop body holds no wait for memory other than the
  //      one in front of the LDS fill, a whole tile after the loads were issued.
  u32x4 kreg[C::kLoads], vreg[C::kLoads];
  uint32_t k_off[C::kLoads], v_off[C::kLoads];
#pragma unroll
  for (int i = 0; i < C::kLoads; ++i) {
    const int idx = tid + i * C::kThreads;
    const int r = idx / C::kVecPerRow, cv = idx % C::kVecPerRow;
    k_off[i] = static_cast<uint32_t>((static_cast<int64_t>(r) * a.ks[2] + cv * 8) * 2);
    v_off[i] = static_cast<uint32_t>((static_cast<int64_t>(r) * a.vs[2] + cv * 8) * 2);
  }
  // a cursor walks the key tiles in order (and from chunk to chunk): stepping it is a few scalar adds
  KvCursor<D> cur;
  cur.open(a, 0, b, hkv, KT);
  auto load_tile = [&]() {  // the next tile of KT keys
    const buffer_rsrc kb = make_buffer(cur.k, cur.k_left), vb = make_buffer(cur.v, cur.v_left);
#pragma unroll
    for (int i = 0; i < C::kLoads; ++i) {
      kreg[i] = buffer_load_b128(kb, k_off[i]);
      vreg[i] = buffer_load_b128(vb, v_off[i]);
    }
    cur.next(a);
  };
  auto store_tile = [&](int buf) {
    __bf16* sK = smem + buf * C::kTileElems;
    __bf16* sV = sK + KT * LDK;
#pragma unroll
    for (int i = 0; i < C::kLoads; ++i) {
      const int idx = tid + i * C::kThreads;
      const int r = idx / C::kVecPerRow, cv = idx % C::kVecPerRow;
      *reinterpret_cast<u32x4*>(&sK[r * LDK + cv * 8]) = kreg[i];
      *reinterpret_cast<u32x4*>(&sV[r * LDV + cv * 8]) = vreg[i];
    }
  };

  if (ntiles > 0) load_tile();
  __syncthreads();  // every wave has its Q fragments: the tile buffers may be filled
  if (ntiles > 0) store_tile(0);
  // Every load issued so far (Q fragments, the merge state, tile 0) is complete on each path that enters the
  // loop, because the LDS fill waited for the newest of them -- but not on the static path that skips the
  // fill.  Saying so here keeps the compiler from putting a vmcnt(0) wait in front of the loop's first MFMAs,
  // where it would wait for the prefetch of the NEXT tile on every trip.
  __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);
  if (ntiles > 1) load_tile();
  __syncthreads();

  for (int t = 0; t < ntiles; ++t) {
    // stage tile t+1 into the other buffer (its readers finished before the barrier that ended trip t-1)
    if (t + 1 < ntiles) {
      store_tile((t + 1) & 1);
      if (t + 2 < ntiles) load_tile();
    }
    const __bf16* sK = smem + (t & 1) * C::kTileElems;
    const __bf16* sV = sK + KT * LDK;

#pragma unroll
    for (int sub = 0; sub < KT / BN; ++sub) {
      if (KS > 1 && sub != ks) continue;
      const int k0 = t * KT + sub * BN;
      if (k0 >= kv_end) break;
      const __bf16* sKs = sK + sub * BN * LDK;
      const __bf16* sVs = sV + sub * BN * LDV;
#pragma unroll
      for (int qb = 0; qb < QB; ++qb) {
        const int blk_q_lo = a.q_offset + q0 + (qw * QB + qb) * 32;  // position of the block's first query
        if (a.causal && k0 > blk_q_lo + 31) continue;                  // whole 32x64 block is in the future
        // ---- S^T[key][query] for 64 keys x 32 queries
        f32x16 s_acc[BN / 32];
        // Where no order is pinned by hand (head_dim 64), the compiler's scheduler is asked for its MFMA / LDS-read
        // interleaving of this block (-1 % with 8 waves, -5 % with 4; the key-split variant is better off without)
        if constexpr (C::kKDepth == 0 && KS == 1) __builtin_amdgcn_iglp_opt(0);
        // D = 128: the K fragments are fetched from LDS a fixed number of MFMAs ahead of their use.  An LDS read
        // takes several MFMA times to come back, so a read issued right before its MFMA leaves the matrix pipe
        // waiting for it (measured: +5 %).  At D = 64 the softmax arithmetic, not this wait, paces the loop, and the
        // compiler's own order is 2 % faster.
        if constexpr (C::kKDepth > 0) {
          constexpr int kSteps = (BN / 32) * (D / 16), kDepth = C::kKDepth < kSteps ? C::kKDepth : kSteps;
          bf16x8 kf[kSteps];
#pragma unroll
          for (int j = 0; j < kSteps; ++j)
            kf[j] = *reinterpret_cast<const bf16x8*>(&sKs[(32 * (j / (D / 16)) + n) * LDK + 16 * (j % (D / 16)) + 8 * h]);
#pragma unroll
          for (int mb = 0; mb < BN / 32; ++mb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s_acc[mb][i] = 0.f;
#pragma unroll
            for (int s = 0; s < D / 16; ++s) s_acc[mb] = mfma32(kf[mb * (D / 16) + s], qf[qb][s], s_acc[mb]);
          }
          // scheduling groups: kDepth LDS reads, then one MFMA and one read in turn, then the last kDepth MFMAs
          __builtin_amdgcn_sched_group_barrier(0x100, kDepth, 0);
#pragma unroll
          for (int j = 0; j < kSteps - kDepth; ++j) {
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
          }
          __builtin_amdgcn_sched_group_barrier(0x008, kDepth, 0);
        } else {
#pragma unroll
          for (int mb = 0; mb < BN / 32; ++mb) {
#pragma unroll
            for (int i = 0; i < 16; ++i) s_acc[mb][i] = 0.f;
#pragma unroll
            for (int s = 0; s < D / 16; ++s) {
              const bf16x8 kf = *reinterpret_cast<const bf16x8*>(&sKs[(32 * mb + n) * LDK + 16 * s + 8 * h]);
              s_acc[mb] = mfma32(kf, qf[qb][s], s_acc[mb]);
            }
          }
        }
        // ---- mask (only for tiles that straddle the diagonal or the end of K)
        const bool need_mask = (a.causal && k0 + BN - 1 > blk_q_lo) || (k0 + BN > a.Sk);
        if (need_mask) {
          // the asm statement keeps this a real (wave-uniform) branch: without it the compiler turns the
          // block into per-element selects that every tile pays for
          asm volatile("; masked tile" ::: "memory");
          const int qpos = a.causal ? a.q_offset + qrow[qb] : 0x7fffffff;
#pragma unroll
          for (int mb = 0; mb < BN / 32; ++mb)
#pragma unroll
            for (int i = 0; i < 16; ++i) {
              const int key = k0 + 32 * mb + 8 * (i / 4) + 4 * h + (i % 4);
              if (key > qpos || key >= a.Sk) s_acc[mb][i] = -INFINITY;
            }
        }
        // ---- online softmax.  The running maximum is only raised (and O, l rescaled) when some query of
        //      the wave saw its maximum grow by more than 2^kTau; until then exp2(s - m) may exceed 1 by at
        //      most that factor, which fp32 accumulators and bf16 probabilities hold without loss.
        constexpr float kTau = 8.f;
        float mx = s_acc[0][0];
#pragma unroll
        for (int mb = 0; mb < BN / 32; ++mb)
#pragma unroll
          for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s_acc[mb][i]);
        mx = half_max(mx) * c;
        if (__any(mx > m_run[qb] + kTau)) {
          const float m_new = fmaxf(m_run[qb], mx);
          const float alpha = (m_new == -INFINITY) ? 1.f : fast_exp2(m_run[qb] - m_new);
          m_run[qb] = m_new;
#pragma unroll
          for (int db = 0; db < D / 32; ++db)
#pragma unroll
            for (int i = 0; i < 16; ++i) o[qb][db][i] *= alpha;
          l_run[qb] *= alpha;
        }
        const float m_use = (m_run[qb] == -INFINITY) ? 0.f : m_run[qb];
        float psum = 0.f;
#pragma unroll
        for (int mb = 0; mb < BN / 32; ++mb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const float pv = fast_exp2(s_acc[mb][i] * c - m_use);
            s_acc[mb][i] = pv;
            psum += pv;
          }
        l_run[qb] += psum;
        // ---- O^T[d][query] += V^T[d][key] P^T[key][query]
#pragma unroll
        for (int mb = 0; mb < BN / 32; ++mb)
#pragma unroll
          for (int cc = 0; cc < 2; ++cc) {
            const bf16x8 pf = pack8(s_acc[mb], 8 * cc);
            const int krow = 32 * mb + 16 * cc + 4 * h + (lane % 16) / 4;
#pragma unroll
            for (int db = 0; db < D / 32; ++db) {
              const int col = 32 * db + 16 * ((lane / 16) % 2) + 4 * (lane % 4);
              const bf16x8 vf = lds_read_tr_pair(&sVs[krow * LDV + col], LDV);
              o[qb][db] = mfma32(vf, pf, o[qb][db]);
            }
          }
      }
    }
    __syncthreads();  // all waves are done with buffer t&1 (it is refilled in trip t+1) and tile t+1 is visible
  }

  // ---- key split: the waves ks > 0 hand their partial state to the wave ks == 0 of the same queries through LDS
  //      (the loop ended on a barrier, so the tile buffers are free).  States with different reference maxima m
  //      combine as O = sum_i 2^(m_i - m) O_i, l = sum_i 2^(m_i - m) l_i with m = max_i m_i.
  if constexpr (KS > 1) {
    float* xo = reinterpret_cast<float*>(smem_raw + wave * C::kExchangeBytes);
    float* xm = xo + (D / 32) * 16 * 64;
    if (ks > 0) {
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) xo[(db * 16 + i) * 64 + lane] = o[0][db][i];
      xm[lane] = m_run[0];
      xm[64 + lane] = l_run[0];
    }
    __syncthreads();
    if (ks > 0) return;
    float m_all = m_run[0];
#pragma unroll
    for (int j = 1; j < KS; ++j) {
      const float* om = reinterpret_cast<const float*>(smem_raw + (qw + j * C::kQWaves) * C::kExchangeBytes) + (D / 32) * 16 * 64;
      m_all = fmaxf(m_all, om[lane]);
    }
    const float a0 = (m_run[0] == -INFINITY) ? 0.f : fast_exp2(m_run[0] - m_all);
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[0][db][i] *= a0;
    l_run[0] *= a0;
#pragma unroll
    for (int j = 1; j < KS; ++j) {
      const float* oo = reinterpret_cast<const float*>(smem_raw + (qw + j * C::kQWaves) * C::kExchangeBytes);
      const float* om = oo + (D / 32) * 16 * 64;
      const float mj = om[lane];
      const float aj = (mj == -INFINITY) ? 0.f : fast_exp2(mj - m_all);
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[0][db][i] += aj * oo[(db * 16 + i) * 64 + lane];
      l_run[0] += aj * om[64 + lane];
    }
    m_run[0] = m_all;
    // (the rows below leave through the first kQWaves * kRowRegionBytes of LDS, which no exchange area of a ks > 0 wave
    // overlaps)
    static_assert(C::kQWaves * kRowRegionBytes <= C::kQWaves * C::kExchangeBytes, "store pieces lie below the exchange areas read above");
  }

  // ---- epilogue: lse per query; the wave's 32 output rows leave through its piece of LDS as whole lines
  //      (the loop ended on a barrier, so the tile buffers are free)
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    const float l_tot = half_sum(l_run[qb]);
    const bool live = qrow[qb] < a.Sq;
    const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
    if (live && h == 0)
      p.lse[lse_row0 + qrow[qb]] = l_tot > 0.f ? (m_run[qb] + fast_log2(l_tot)) * kLn2 : -INFINITY;
    // normalise in place: 1 / l differs per lane (row), the store helper applies one scale to all
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[qb][db][i] *= inv;
    unsigned char* region = smem_raw + (wave * QB + qb) * kRowRegionBytes;
    const int row0 = q0 + (qw * QB + qb) * 32;
    const int64_t off = b * a.os[0] + hq * a.os[1] + static_cast<int64_t>(row0) * a.os[2];
    if (p.out_f32)
      wave_store_rows<D, true>(region, o[qb], 1.f, static_cast<float*>(p.out) + off, a.os[2], a.Sq - row0, lane, false, false);
    else
      wave_store_rows<D, false>(region, o[qb], 1.f, static_cast<__bf16*>(p.out) + off, a.os[2], a.Sq - row0, lane, false, false);
  }
}

template <int D, int QB, int NW, int KT, int KS = 1>
int launch(const FwdParams& p, hipStream_t s) {
  using C = FwdCfg<D, QB, NW, KT, KS>;
  static LdsOnce lds_reserved;
  if (!reserve_lds_once(lds_reserved, reinterpret_cast<const void*>(&attn_fwd_kernel<D, QB, NW, KT, KS>), C::kLdsBytes))
    return fail(PICO_ERR_LAUNCH, "pico_attn_fwd: cannot reserve %zu bytes of LDS", C::kLdsBytes);
  const int n_qtiles = (p.a.Sq + C::BM - 1) / C::BM;
  FwdParams q = p;
  // (the pairing needs two workgroups per CU: at head_dim 128 the eight-wave kernel has one, the launch is two
  // generations of workgroups and longest-first is the better order -- 160 -> 137 us at B1 H32 S4096)
  constexpr bool kTwoPerCu = !(D >= 128 && NW == 8);
  q.pair_order = kTwoPerCu && p.a.causal && n_qtiles >= 2 && static_cast<int64_t>(p.a.Hq) * p.a.B * n_qtiles <= 512;
  hipLaunchKernelGGL((attn_fwd_kernel<D, QB, NW, KT, KS>), dim3(p.a.Hq * p.a.B, n_qtiles), dim3(C::kThreads), C::kLdsBytes, s, q);
  return PICO_OK;
}

}  // namespace

int check_attn_desc(const char* fn, const pico_attn_desc* d) {
  if (!d) return fail(PICO_ERR_NULL, "%s: descriptor is NULL", fn);
  if (d->D != 64 && d->D != 128) return fail(PICO_ERR_SHAPE, "%s: head_dim %d not supported (64 or 128)", fn, d->D);
  if (d->B < 0 || d->Hq <= 0 || d->Hkv <= 0 || d->Sq < 0 || d->Sk < 0)
    return fail(PICO_ERR_SHAPE, "%s: negative size (B=%d Hq=%d Hkv=%d Sq=%d Sk=%d)", fn, d->B, d->Hq, d->Hkv, d->Sq, d->Sk);
  if (d->Hq % d->Hkv != 0) return fail(PICO_ERR_SHAPE, "%s: Hq=%d is not a multiple of Hkv=%d", fn, d->Hq, d->Hkv);
  if (static_cast<int64_t>(d->B) * d->Hq > 0x7fffffffLL) return fail(PICO_ERR_SHAPE, "%s: B * Hq too large", fn);
  if (d->q_offset < 0) return fail(PICO_ERR_SHAPE, "%s: q_offset=%d must be >= 0", fn, d->q_offset);
  if (!(d->sm_scale > 0.f)) return fail(PICO_ERR_SHAPE, "%s: sm_scale must be positive", fn);
  const int64_t* all[4] = {d->q_stride, d->k_stride, d->v_stride, d->o_stride};
  for (const int64_t* st : all)
    for (int i = 0; i < 3; ++i)
      if (st[i] < 0 || st[i] % 8 != 0)
        return fail(PICO_ERR_STRIDE, "%s: strides must be non-negative multiples of 8 elements", fn);
  // the kernels address one head's rows through 32-bit byte offsets (the key side is checked per chunk, set_chunks)
  const int64_t spans[2] = {(d->Sq - 1) * d->q_stride[2], (d->Sq - 1) * d->o_stride[2]};
  for (int64_t span : spans)
    if ((span + d->D) * 2 >= (1LL << 32))
      return fail(PICO_ERR_STRIDE, "%s: the rows of one head must span less than 4 GiB", fn);
  return PICO_OK;
}

int check_rope_tables(const char* fn, const pico_rope_tables* t, int D, int64_t last_pos) {
  if (!t || !t->cos || !t->sin) return fail(PICO_ERR_NULL, "%s: cos / sin tables are required", fn);
  if (t->dtype != PICO_BF16 && t->dtype != PICO_F32) return fail(PICO_ERR_DTYPE, "%s: table dtype code %d not supported", fn, t->dtype);
  if (t->pitch < D / 2 || t->pitch % 4 != 0 || !aligned16(t->cos) || !aligned16(t->sin) ||
      (t->dtype == PICO_BF16 && t->pitch % 8 != 0))
    return fail(PICO_ERR_STRIDE, "%s: table rows must hold D/2 columns, start 16-byte aligned and lie a multiple of 16 bytes apart", fn);
  if (last_pos >= t->rows) return fail(PICO_ERR_SHAPE, "%s: positions up to %lld needed, the tables have %d rows", fn,
                                       static_cast<long long>(last_pos), t->rows);
  return PICO_OK;
}

AttnParams make_params(const pico_attn_desc* d, const void* q, const void* k, const void* v) {
  AttnParams a;
  a.q = static_cast<const __bf16*>(q);
  for (int c = 0; c < kMaxChunks; ++c) a.kv.k[c] = a.kv.v[c] = nullptr;
  a.kv.k[0] = static_cast<const __bf16*>(k);
  a.kv.v[0] = static_cast<const __bf16*>(v);
  a.kv.count = 1;
  a.kv.len = d->Sk;
  a.B = d->B; a.Hq = d->Hq; a.Hkv = d->Hkv; a.Sq = d->Sq; a.Sk = d->Sk;
  a.causal = d->causal != 0;
  a.q_offset = d->q_offset;
  a.sm_scale = d->sm_scale;
  for (int i = 0; i < 3; ++i) {
    a.qs[i] = d->q_stride[i]; a.ks[i] = d->k_stride[i]; a.vs[i] = d->v_stride[i]; a.os[i] = d->o_stride[i];
  }
  return a;
}

int set_chunks(const char* fn, const pico_attn_desc* d, const pico_kv_chunks* kv, AttnParams& a, bool need_kv) {
  if (!kv) return fail(PICO_ERR_NULL, "%s: the chunk list is NULL", fn);
  if (kv->count < 1 || kv->count > kMaxChunks)
    return fail(PICO_ERR_SHAPE, "%s: %d chunks (1 to %d supported)", fn, kv->count, kMaxChunks);
  if (kv->chunk_len < 0 || static_cast<int64_t>(kv->count) * kv->chunk_len != d->Sk)
    return fail(PICO_ERR_SHAPE, "%s: %d chunks of %d keys do not make Sk=%d", fn, kv->count, kv->chunk_len, d->Sk);
  if (kv->count > 1 && kv->chunk_len % 128 != 0)
    return fail(PICO_ERR_SHAPE, "%s: with several chunks the chunk length (%d) must be a multiple of 128", fn, kv->chunk_len);
  // a chunk is addressed through the same 32-bit window as a whole tensor
  if (((kv->chunk_len - 1) * std::max(d->k_stride[2], d->v_stride[2]) + d->D) * 2 >= (1LL << 32))
    return fail(PICO_ERR_STRIDE, "%s: the rows of one head must span less than 4 GiB", fn);
  for (int c = 0; c < kv->count; ++c) {
    if (need_kv && (!kv->k[c] || !kv->v[c])) return fail(PICO_ERR_NULL, "%s: k / v of chunk %d are NULL", fn, c);
    if (!aligned16(kv->k[c]) || !aligned16(kv->v[c]) || !aligned16(kv->dk[c]) || !aligned16(kv->dv[c]))
      return fail(PICO_ERR_ALIGN, "%s: chunk %d: k, v, dk and dv must be 16-byte aligned", fn, c);
    a.kv.k[c] = static_cast<const __bf16*>(kv->k[c]);
    a.kv.v[c] = static_cast<const __bf16*>(kv->v[c]);
  }
  a.kv.count = kv->count;
  a.kv.len = kv->chunk_len;
  return PICO_OK;
}

}  // namespace pico

using namespace pico;

namespace {

// rows of [B, H, S, D] memory addressed by `st` must not overlap: every stride spans what lies inside it
bool rows_disjoint(const int64_t* st, int B, int H, int S, int D) {
  struct Dim { int64_t stride; int extent; } dims[3] = {{st[0], B}, {st[1], H}, {st[2], S}};
  std::sort(dims, dims + 3, [](const Dim& x, const Dim& y) { return x.stride < y.stride; });
  int64_t span = D;   // elements covered by the dimensions handled so far
  for (const Dim& d : dims) {
    if (d.extent <= 1) continue;
    if (d.stride < span) return false;
    span = d.stride * (d.extent - 1) + span;
  }
  return true;
}

int run_fwd(const char* fn, const pico_attn_desc* desc, const void* q, const pico_kv_chunks* kv, void* out, float* lse,
            int out_dtype, int merge, const pico_rope_tables* rope, int q_pos_offset, void* q_rot,
            const int64_t* q_rot_stride, void* stream) {
  if (int rc = check_attn_desc(fn, desc)) return rc;
  if (out_dtype != PICO_BF16 && out_dtype != PICO_F32)
    return fail(PICO_ERR_DTYPE, "%s: out dtype code %d not supported", fn, out_dtype);
  if (merge && out_dtype != PICO_F32) return fail(PICO_ERR_DTYPE, "%s: merge needs an fp32 running out", fn);
  FwdParams p;
  p.a = make_params(desc, q, nullptr, nullptr);
  if (int rc = set_chunks(fn, desc, kv, p.a, desc->B > 0 && desc->Sq > 0 && desc->Sk > 0)) return rc;
  if (desc->B == 0 || desc->Sq == 0) return PICO_OK;
  if (!q || !out || !lse) return fail(PICO_ERR_NULL, "%s: q, out and lse are required", fn);
  if (!aligned16(q) || !aligned16(out) || !aligned16(q_rot))
    return fail(PICO_ERR_ALIGN, "%s: q, out and q_rot must be 16-byte aligned", fn);
  p.out = out;
  p.lse = lse;
  p.out_f32 = out_dtype == PICO_F32;
  p.merge = merge != 0;
  p.rope = RopeArgs{nullptr, nullptr, 0, 0, 0, 0};
  p.q_rot = nullptr;
  p.qrs[0] = p.qrs[1] = p.qrs[2] = 0;
  if (rope) {
    if (q_pos_offset < 0) return fail(PICO_ERR_SHAPE, "%s: q_pos_offset=%d must be >= 0", fn, q_pos_offset);
    if (int rc = check_rope_tables(fn, rope, desc->D, static_cast<int64_t>(q_pos_offset) + desc->Sq - 1)) return rc;
    p.rope = RopeArgs{rope->cos, rope->sin, rope->pitch, rope->dtype == PICO_F32, q_pos_offset, 0};
    if (q_rot) {
      if (!q_rot_stride) return fail(PICO_ERR_NULL, "%s: q_rot needs its strides", fn);
      for (int i = 0; i < 3; ++i) {
        if (q_rot_stride[i] < 0 || q_rot_stride[i] % 8 != 0)
          return fail(PICO_ERR_STRIDE, "%s: q_rot strides must be non-negative multiples of 8 elements", fn);
        p.qrs[i] = q_rot_stride[i];
      }
      if (!rows_disjoint(q_rot_stride, desc->B, desc->Hq, desc->Sq, desc->D))
        return fail(PICO_ERR_STRIDE, "%s: q_rot strides make rows overlap (every stride must span what lies inside it)", fn);
      p.q_rot = static_cast<__bf16*>(q_rot);
    }
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Tile choice for D = 64: more waves per workgroup share each staged K/V tile (fewer barriers and
  // global loads per MFMA), but the launch still has to fill 256 CUs, so small problems get small tiles.
  int rc;
  if (desc->D == 64) {
    const int64_t heads = static_cast<int64_t>(desc->B) * desc->Hq;
    auto groups = [&](int bm) { return heads * ((desc->Sq + bm - 1) / bm); };
    const int64_t visible_keys = desc->causal ? std::min<int64_t>(desc->Sk, static_cast<int64_t>(desc->q_offset) + desc->Sq) : desc->Sk;
    // a launch whose queries all see at least as many keys as they are themselves (a rank's share of a ring, a dense
    // block): the waves of a workgroup then do nearly equal work, and workgroups of eight waves, which share every
    // staged tile among twice as many waves, pay even where the launch has few of them
    const bool rectangular = !desc->causal || desc->q_offset >= desc->Sq;
    if (groups(256) >= 512) rc = launch<64, 1, 8, 64>(p, s);
    else if (groups(128) >= 512) {
      // (measured at B8, 256 queries x 1024 keys of every head: 26.9 us with eight waves, 30.1 us with four)
      if (rectangular && groups(256) >= 256) rc = launch<64, 1, 8, 64>(p, s);
      else rc = launch<64, 1, 4, 64>(p, s);
    }
    // few waves in all: two waves per 32 queries, 64 keys of every 128 each -- in workgroups of eight waves (128 queries)
    // when those still cover the CUs and the launch is rectangular (one rank's share of configs[1]: 19.8 -> 16.9 us for
    // rank 3 of 4; on a whole causal sequence, or with 256 keys, the smaller workgroups are a few percent faster)
    else if (groups(128) >= 256 && rectangular && visible_keys >= 512) rc = launch<64, 1, 8, 128, 2>(p, s);
    else rc = launch<64, 1, 4, 128, 2>(p, s);
  } else {
    const int64_t heads = static_cast<int64_t>(desc->B) * desc->Hq;
    // (64-key staged tiles: 0.5-4 % faster than 128-key ones at every size measured)
    if (heads * ((desc->Sq + 255) / 256) >= 256) rc = launch<128, 1, 8, 64>(p, s);
    else rc = launch<128, 1, 4, 64>(p, s);
  }
  if (rc) return rc;
  return check_launch(fn);
}

pico_kv_chunks one_chunk(const pico_attn_desc* desc, const void* k, const void* v) {
  pico_kv_chunks kv = {};
  kv.count = 1;
  kv.chunk_len = desc ? desc->Sk : 0;
  kv.k[0] = k;
  kv.v[0] = v;
  return kv;
}

}  // namespace

extern "C" int pico_attn_fwd(const pico_attn_desc* desc, const void* q, const void* k, const void* v, void* out,
                             float* lse, int out_dtype, int merge, void* stream) {
  const pico_kv_chunks kv = one_chunk(desc, k, v);
  return run_fwd("pico_attn_fwd", desc, q, &kv, out, lse, out_dtype, merge, nullptr, 0, nullptr, nullptr, stream);
}

extern "C" int pico_attn_fwd_rope(const pico_attn_desc* desc, const void* q, const void* k_rot, const void* v, void* out,
                                  float* lse, int out_dtype, int merge, const pico_rope_tables* rope, int q_pos_offset,
                                  void* q_rot, const int64_t* q_rot_stride, void* stream) {
  if (!rope) return fail(PICO_ERR_NULL, "pico_attn_fwd_rope: the tables are required");
  const pico_kv_chunks kv = one_chunk(desc, k_rot, v);
  return run_fwd("pico_attn_fwd_rope", desc, q, &kv, out, lse, out_dtype, merge, rope, q_pos_offset, q_rot, q_rot_stride, stream);
}

extern "C" int pico_attn_fwd_chunks(const pico_attn_desc* desc, const void* q, const pico_kv_chunks* kv, void* out,
                                    float* lse, int out_dtype, int merge, const pico_rope_tables* rope, int q_pos_offset,
                                    void* q_rot, const int64_t* q_rot_stride, void* stream) {
  return run_fwd("pico_attn_fwd_chunks", desc, q, kv, out, lse, out_dtype, merge, rope, q_pos_offset, q_rot, q_rot_stride, stream);
}
