// Attention backward for gfx950 (MFMA bf16), split into two kernels so that no gradient needs atomics:
//
//  dK/dV kernel: one workgroup owns 128 keys of one kv head (32 per wave), keeps their K / V fragments and
//    the dK / dV accumulators in registers, and walks over the 64-query tiles (and the query heads of a
//    GQA group) that can see those keys:
//      S = Q K^T, dP = dO V^T   (C tile: lane = key, registers = queries)
//      P = exp2(S*c - lse*log2e),  dS = P * (dP - delta)
//      dV += P^T dO,  dK += dS^T Q   (P / dS feed the MFMA straight from registers as A operands; dO and Q
//                                     come from the row-major LDS tiles through transposing reads)
//  dQ kernel: one workgroup owns 32 queries per wave, keeps Q / dO fragments, lse and delta in registers and
//    walks over the K/V tiles like the forward kernel, in the transposed orientation (lane = query):
//      S^T = K Q^T, dP^T = V dO^T,  dS^T = P^T * (dP^T - delta)  (lse / delta are per-lane scalars)
//      dQ^T += K^T dS^T            (dS^T goes from the C registers into the B operand; K^T is read from the
//                                   row-major K tile through transposing LDS reads)
//
// Recomputing S and dP in the second kernel costs 2 of 7 MFMA products; a single-kernel version that
// accumulated dQ with fp32 atomics was bound by the atomic rate of the memory system (measured).
#include "attn_common.h"

#include <type_traits>

namespace pico {
namespace {

struct BwdParams {
  AttnParams a;
  const __bf16* dout;
  const float* lse;
  const float* delta;
  const __bf16* out;   // fused-delta mode of the dQ kernel: the forward output, addressed like dout
  float* delta_w;      //   ... and where that kernel writes delta = sum_d dO * O for the dK/dV kernel
  void* dq;
  void* dk[kMaxChunks];      // per K / V chunk; nullptr: that chunk's gradient is not wanted
  void* dv[kMaxChunks];
  __bf16* dk_final[kMaxChunks];   // per chunk, optional: the chunk's total (fp32 dk[c] if its accumulate bit is set, plus this
  __bf16* dv_final[kMaxChunks];   //   launch's block) leaves here in bf16; dk[c] / dv[c] are only read
  int64_t dkfs[3];                // element strides (b, h, s) of dk_final / dv_final
  uint32_t dkv_accumulate;   // bit c: chunk c's dk / dv are added to (fp32)
  int dq_f32, dq_accumulate;
  int dkv_f32;
  int pair_ktiles;  // dK/dV kernel: a workgroup takes key tile t and then tile n-1-t (equal work under a causal mask)
  int64_t dqs[3];  // element strides (b, h, s) of dq
  int64_t dks[3];  // element strides (b, h, s) of dk and dv
  RopeArgs rope;   // rope.cos != nullptr: q and k are rotated tensors; dq and dk leave un-rotated (RoPE's backward)
};

// =====================================================================================  dK / dV
// bf16 gradients leave with streaming (non-temporal) stores: nothing on this GPU reads them back soon
constexpr bool kStreamGrads = true;
// PAIR: eight waves instead of four; waves w and w + 4 (they share a SIMD) own the same 32 keys and split every
// 64-query tile between them, one 32-query sub-block each, with accumulators of their own that are added through LDS
// at the end of the key tile.  A wave then holds one sub-block's S / dP tiles instead of two, which is what lets the
// head_dim 128 kernel fit 256 registers, i.e. two waves per SIMD.
constexpr int kPairKRegs = 4;   // PAIR: K fragments (of D / 16) that stay in registers; the others are read from LDS

template <int D, bool PAIR = false>
struct KvCfg {
  static constexpr int NW = PAIR ? 8 : 4;
  static constexpr int kKeyWaves = 4;          // waves that own different keys
  static constexpr int kThreads = 64 * NW;
  static constexpr int BN = 32 * kKeyWaves;  // keys per workgroup
  static constexpr int BM = 64;       // queries per trip
  // Q and dO tiles: rows of D elements at a pitch of LDQ elements, plus kSkew elements after every 4 rows.  Every
  // tile is read both by rows (16 bytes per lane, 32 consecutive rows per instruction) and transposed (8 bytes per
  // lane: 4 rows x 32 bytes per 16 lanes, rows 4 apart for the two wave halves).  An LDS instruction takes as many
  // cycles as its busiest bank (64 banks of 4 bytes) has requests.  With the pitch = 16 (mod 32) words the 16-word
  // pieces of 4 consecutive rows tile the banks (transposed reads at their minimum of 2 requests per bank; at a pitch
  // of D + 8 they take 3-4), and the 4-word skew per 4 rows spreads 16 consecutive rows over all multiples of 4 words
  // (row reads at their minimum of 4).
  static constexpr int LDQ = D + 32;
  static constexpr int kSkew = 8;
  static constexpr int kTileElems = BM * LDQ + kSkew * (BM / 4);       // one tile
  static constexpr int kTrStep = 8 * LDQ + 2 * kSkew;                  // 8 rows further down
  static constexpr int kVecPerRow = D / 8;
  static constexpr int kQLoads = BM * kVecPerRow / kThreads;
  static constexpr int kBufElems = 2 * kTileElems;                     // Q + dO tile of one stage (bf16)
  static constexpr size_t kBufBytes = kBufElems * sizeof(__bf16) + 2 * BM * sizeof(float);
  static constexpr size_t kTileBytes = 2 * kBufBytes;  // the two Q / dO tile buffers
  // PAIR: the K and V fragments of the four key waves stay in LDS behind the tile buffers instead of in registers
  static constexpr size_t kKvBytes = PAIR ? static_cast<size_t>(kKeyWaves) * 2 * WaveTile<D>::kRegionBytes : 0;
  static constexpr size_t kLdsBytes = kTileBytes + kKvBytes;
  static_assert(NW * kRowRegionBytes <= kTileBytes, "the epilogue reuses the tile buffers");
  static_assert(PAIR || NW * WaveTile<D>::kRegionBytes <= kBufBytes, "the K / V fragments pass through the second tile buffer");
  // PAIR: one accumulator set (D/32 x 16 registers x 64 lanes of fp32) per key wave passes through LDS at a time
  static constexpr size_t kPairExchangeBytes = static_cast<size_t>(D / 32) * 16 * 64 * 4;
  static_assert(!PAIR || kKeyWaves * kPairExchangeBytes <= kTileBytes, "the pair exchange reuses the tile buffers");
};

template <int D, bool PAIR = false>
__device__ __forceinline__ void attn_bwd_dkdv_tile(const BwdParams& p, const int ktile) {
  using C = KvCfg<D, PAIR>;
  constexpr int BM = C::BM, BN = C::BN;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  auto tile_row = [](int r) { return r * C::LDQ + C::kSkew * (r >> 2); };   // element offset of a tile row

  const AttnParams& a = p.a;
  const int hkv = blockIdx.x % a.Hkv, b = blockIdx.x / a.Hkv;
  const int group = a.Hq / a.Hkv;
  const int key0 = ktile * BN;                     // position of the tile's first key in the launch
  const int chunk = a.kv.count > 1 ? key0 / a.kv.len : 0;
  const int crow0 = key0 - chunk * a.kv.len;       // ... and its row in the chunk that holds it
  if (p.dk[chunk] == nullptr && p.dk_final[chunk] == nullptr) return;   // this chunk's gradient is not wanted (uniform over the workgroup)
  const int tid = threadIdx.x, wave_id = tid / 64, lane = tid % 64;
  // wave: which 32 keys of the tile; pair_sb (PAIR only): which 32-query sub-block of every query tile
  const int wave = PAIR ? __builtin_amdgcn_readfirstlane(wave_id % C::kKeyWaves) : wave_id;
  const int pair_sb = PAIR ? __builtin_amdgcn_readfirstlane(wave_id / C::kKeyWaves) : 0;
  const int n = lane % 32, h = lane / 32;
  const float c = a.sm_scale * kLog2e;

  const __bf16* kbase = a.kv.k[chunk] + b * a.ks[0] + hkv * a.ks[1];
  const __bf16* vbase = a.kv.v[chunk] + b * a.vs[0] + hkv * a.vs[1];

  // ---- K, V fragments of this wave's 32 keys (B operand: lane = key, 8 consecutive d per k step), fetched
  //      row-major and turned into fragments through the wave's piece of the SECOND tile buffer, which nothing
  //      else writes before the end of the first trip, a barrier later.  The loads are issued here; the first
  //      Q / dO tile's loads follow them further down before anything waits, so that the two latencies overlap.
  bf16x8 kf[D / 16], vf[D / 16];
  constexpr int kFragPitch = (D + 8) * 2;   // WaveTile's row pitch in bytes
  unsigned char* const pair_k = smem_raw + C::kTileBytes + wave * 2 * WaveTile<D>::kRegionBytes;   // (PAIR only)
  unsigned char* const pair_v = pair_k + WaveTile<D>::kRegionBytes;
  const bool loads_kv = !PAIR || pair_sb == 0;
  WaveTile<D> kt, vt;
  if (loads_kv) {
    // (the wave index read as a scalar: the buffer windows below are then built in scalar registers; from the
    // per-lane value the compiler cannot tell that they are the same in all lanes and loops over the lanes' values)
    const int row0 = crow0 + 32 * __builtin_amdgcn_readfirstlane(wave);
    kt.issue(make_buffer(kbase + static_cast<int64_t>(row0) * a.ks[2], span_bytes(a.kv.len - row0, a.ks[2], D)), a.ks[2], lane);
    vt.issue(make_buffer(vbase + static_cast<int64_t>(row0) * a.vs[2], span_bytes(a.kv.len - row0, a.vs[2], D)), a.vs[2], lane);
  }

  f32x16 dk_acc[D / 32], dv_acc[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) { dk_acc[db][i] = 0.f; dv_acc[db][i] = 0.f; }

  // ---- trip space: (query head of the group) x (query tiles that can see key0)
  const int n_qtiles = (a.Sq + BM - 1) / BM;
  int qt_start = 0;
  if (a.causal) {
    const int first_q = key0 - a.q_offset;  // first query index that sees key0
    qt_start = first_q > 0 ? first_q / BM : 0;
  }
  const int tiles_per_head = n_qtiles > qt_start ? n_qtiles - qt_start : 0;
  const int n_iter = tiles_per_head * group;

  // Global -> register prefetch of a Q / dO tile (+ lse, delta) with buffer loads.  A cursor (wave-uniform:
  // it lives in scalar registers) walks the trip space; stepping to the next tile of the same head is a few
  // scalar adds, only a change of head recomputes addresses.  The per-lane byte offsets are computed once,
  // and rows past Sq read as zeros because they lie past the end of the buffer window.  Every instruction
  // of a wave costs an issue slot, scalar ones included, so the per-trip bookkeeping is kept this small.
  u32x4 qreg[C::kQLoads], doreg[C::kQLoads];
  float lreg = 0.f, dreg = 0.f;
  uint32_t q_off[C::kQLoads], do_off[C::kQLoads];
#pragma unroll
  for (int i = 0; i < C::kQLoads; ++i) {
    const int idx = tid + i * C::kThreads;
    const int r = idx / C::kVecPerRow, cv = idx % C::kVecPerRow;
    q_off[i] = static_cast<uint32_t>((static_cast<int64_t>(r) * a.qs[2] + cv * 8) * 2);
    do_off[i] = static_cast<uint32_t>((static_cast<int64_t>(r) * a.os[2] + cv * 8) * 2);
  }
  const uint32_t row_off = static_cast<uint32_t>((tid % BM) * 4);
  const uint32_t q_step = static_cast<uint32_t>(BM * a.qs[2] * 2), do_step = static_cast<uint32_t>(BM * a.os[2] * 2);
  struct Cursor {
    int tile, head;                  // query tile within the head, query head
    const char *q, *dout;            // first row of the tile
    const float *lse, *delta;
    uint32_t q_left, do_left, rows_left;  // bytes from there to the end of the head's rows
  } cur;
  auto seek = [&](int head, int tile) {
    const int q0 = tile * BM;
    cur.tile = tile;
    cur.head = head;
    cur.q = reinterpret_cast<const char*>(a.q + b * a.qs[0] + head * a.qs[1] + static_cast<int64_t>(q0) * a.qs[2]);
    cur.dout = reinterpret_cast<const char*>(p.dout + b * a.os[0] + head * a.os[1] + static_cast<int64_t>(q0) * a.os[2]);
    const int64_t row0 = (static_cast<int64_t>(b) * a.Hq + head) * a.Sq + q0;
    cur.lse = p.lse + row0;
    cur.delta = p.delta + row0;
    cur.q_left = span_bytes(a.Sq - q0, a.qs[2], D);
    cur.do_left = span_bytes(a.Sq - q0, a.os[2], D);
    cur.rows_left = static_cast<uint32_t>(a.Sq - q0) * 4u;
  };
  auto advance = [&]() {
    if (cur.tile + 1 == n_qtiles) {
      seek(cur.head + 1, qt_start);
    } else {
      ++cur.tile;
      cur.q += q_step;  cur.q_left -= q_step;
      cur.dout += do_step;  cur.do_left -= do_step;
      cur.lse += BM;  cur.delta += BM;  cur.rows_left -= BM * 4;
    }
  };
  auto prefetch = [&]() {  // the tile under the cursor
    const buffer_rsrc qb = make_buffer(cur.q, cur.q_left), dob = make_buffer(cur.dout, cur.do_left);
    const buffer_rsrc lb = make_buffer(cur.lse, cur.rows_left), db = make_buffer(cur.delta, cur.rows_left);
#pragma unroll
    for (int i = 0; i < C::kQLoads; ++i) {
      qreg[i] = buffer_load_b128(qb, q_off[i]);
      doreg[i] = buffer_load_b128(dob, do_off[i]);
    }
    lreg = buffer_load_f32(lb, row_off);
    dreg = buffer_load_f32(db, row_off);
  };
  auto stage = [&](int buf) {  // the prefetched tile (still under the cursor) goes to LDS buffer `buf`
    __bf16* sQ = reinterpret_cast<__bf16*>(smem_raw + buf * C::kBufBytes);
    __bf16* sdO = sQ + C::kTileElems;
    float* sL = reinterpret_cast<float*>(sdO + C::kTileElems);
    float* sDelta = sL + BM;
#pragma unroll
    for (int i = 0; i < C::kQLoads; ++i) {
      const int idx = tid + i * C::kThreads;
      const int r = idx / C::kVecPerRow, cv = idx % C::kVecPerRow;
      *reinterpret_cast<u32x4*>(&sQ[tile_row(r) + cv * 8]) = qreg[i];
      *reinterpret_cast<u32x4*>(&sdO[tile_row(r) + cv * 8]) = doreg[i];
    }
    if (tid < BM) {
      // rows past Sq, and rows whose lse is -inf (they saw no key), get lse = +inf so that P = 0
      const bool live = static_cast<uint32_t>(tid) * 4u < cur.rows_left && lreg != -INFINITY;
      sL[tid] = live ? lreg * kLog2e : INFINITY;
      sDelta[tid] = -dreg;   // stored negated: it is loaded straight into the dP accumulator (0 past Sq)
    }
  };

  if (n_iter > 0) {
    seek(hkv * group, qt_start);
    prefetch();
  }
  if (loads_kv) {
    if constexpr (!PAIR) {
      unsigned char* region = smem_raw + C::kBufBytes + wave * WaveTile<D>::kRegionBytes;
      kt.fragments(region, lane, kf);
      vt.fragments(region, lane, vf);
    } else {
      // the first wave of each pair leaves both tiles in the pair's piece of LDS
      kt.fragments(pair_k, lane, kf);
      vt.fragments(pair_v, lane, vf);
    }
  }
  if constexpr (PAIR) {
    __syncthreads();
    // the first few K fragments stay in registers (as many as fit beside the accumulators)
#pragma unroll
    for (int j = 0; j < kPairKRegs; ++j) kf[j] = *reinterpret_cast<const bf16x8*>(pair_k + n * kFragPitch + (16 * j + 8 * h) * 2);
  }
  if (n_iter > 0) stage(0);
  // The K / V fragment loads above are complete by now on every path that enters the loop (the LDS fill
  // waited for all loads), but not on the static path that skips the fill; saying so here keeps the compiler
  // from putting a vmcnt(0) wait in front of the loop's first MFMAs, where it would wait for the prefetch
  // of the NEXT tile on every trip.
  __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);
  __syncthreads();
  // PAIR: the tile after the one being computed goes to LDS at the TOP of a trip, from loads that
  // were issued at the top of the trip before; the registers are then reloaded with the tile after that.  The LDS
  // writes are off the end of the trip (where every wave of the workgroup would wait for them in front of the barrier)
  // and a load has a whole trip to arrive.
  constexpr bool kStageTop = PAIR;
  if constexpr (kStageTop) {
    if (n_iter > 1) { advance(); prefetch(); }
  }

  const int kw0 = key0 + 32 * wave;
  int tile = qt_start;       // query tile (within its head) of the trip being computed
  uint32_t buf_off = 0;      // byte offset of the LDS buffer being read
  for (int it = 0; it < n_iter; ++it) {
    // tile it+1 travels global -> registers while this trip computes; it goes to the other LDS buffer at
    // the end of the trip (that buffer's readers finished before the barrier that ended trip it-1)
    const bool has_next = it + 1 < n_iter;
    if constexpr (kStageTop) {
      if (has_next) {
        stage(buf_off == 0);   // tile it+1 (the cursor is on it)
        if (it + 2 < n_iter) { advance(); prefetch(); }
      }
    } else {
      if (has_next) advance();
    }
    const int q0 = tile * BM;
    const __bf16* sQ = reinterpret_cast<const __bf16*>(smem_raw + buf_off);
    const __bf16* sdO = sQ + C::kTileElems;
    const float* sL = reinterpret_cast<const float*>(sdO + C::kTileElems);
    const float* sDelta = sL + BM;

    // The three phases of a 32-query sub-block.
    // products(): S = Q K^T and dP = dO V^T (C tile: lane = key, registers = queries); the dP accumulator starts at
    // -delta of its row (sDelta holds the negated value), so dP - delta comes out of the MFMA.
    auto products = [&](int sb, f32x16& s_acc, f32x16& dp_acc) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sDelta[32 * sb + 8 * j + 4 * h]);
#pragma unroll
        for (int t = 0; t < 4; ++t) { s_acc[4 * j + t] = 0.f; dp_acc[4 * j + t] = d4[t]; }
      }
      if constexpr (PAIR) {
        // both operands of every MFMA come from LDS: they are requested kAhead steps before the MFMAs that use them, and
        // the scheduling barriers keep that order (left alone, the compiler reuses one set of registers and every MFMA
        // waits for an LDS round trip)
        constexpr int kSteps = D / 16, kAhead = 1;
        bf16x8 qa[kSteps], da[kSteps], kb[kSteps], vb[kSteps];
        auto fetch = [&](int j) {
          qa[j] = *reinterpret_cast<const bf16x8*>(&sQ[tile_row(32 * sb + n) + 16 * j + 8 * h]);
          if (j >= kPairKRegs) kb[j] = *reinterpret_cast<const bf16x8*>(pair_k + n * kFragPitch + (16 * j + 8 * h) * 2);
          da[j] = *reinterpret_cast<const bf16x8*>(&sdO[tile_row(32 * sb + n) + 16 * j + 8 * h]);
          vb[j] = *reinterpret_cast<const bf16x8*>(pair_v + n * kFragPitch + (16 * j + 8 * h) * 2);
        };
#pragma unroll
        for (int j = 0; j < kAhead; ++j) fetch(j);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < kSteps; ++j) {
          if (j + kAhead < kSteps) fetch(j + kAhead);
          s_acc = mfma32(qa[j], j < kPairKRegs ? kf[j] : kb[j], s_acc);
          dp_acc = mfma32(da[j], vb[j], dp_acc);
          __builtin_amdgcn_sched_barrier(0);
        }
      } else {
#pragma unroll
        for (int s = 0; s < D / 16; ++s) {
          const bf16x8 qa = *reinterpret_cast<const bf16x8*>(&sQ[tile_row(32 * sb + n) + 16 * s + 8 * h]);
          const bf16x8 da = *reinterpret_cast<const bf16x8*>(&sdO[tile_row(32 * sb + n) + 16 * s + 8 * h]);
          s_acc = mfma32(qa, kf[s], s_acc);
          dp_acc = mfma32(da, vf[s], dp_acc);
        }
      }
    };
    // softmax_grad(): P = exp2(S*c - lse*log2e), dS = P * (dP - delta) [already in the accumulator]; the mask test
    // is compiled in only for sub-blocks on the diagonal.
    auto softmax_grad = [&](int sb, f32x16& s_acc, f32x16& dp_acc, auto mask_c) {
      constexpr bool kMask = decltype(mask_c)::value;
      const int qs_pos = a.q_offset + q0 + 32 * sb;
      const int key_rel = kw0 + n - qs_pos - 4 * h;  // key is masked for row (8j + 4h + t) iff key_rel > 8j + t
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const f32x4 l4 = *reinterpret_cast<const f32x4*>(&sL[32 * sb + 8 * j + 4 * h]);
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const int i = 4 * j + t;
          float pv = fast_exp2(s_acc[i] * c - l4[t]);
          if constexpr (kMask) {
            if (key_rel > 8 * j + t) pv = 0.f;
          }
          s_acc[i] = pv;
          dp_acc[i] = pv * dp_acc[i];
        }
      }
    };
    // accumulate(): the transposed products dV^T += dO^T P and dK^T += Q^T dS (lane = key, registers = 4 consecutive
    // d, which is what lets the epilogue write whole 16-byte pieces of a row); P / dS come from the registers,
    // dO^T / Q^T from the row-major LDS tiles through transposing reads.
    auto accumulate = [&](int sb, const f32x16& s_acc, const f32x16& dp_acc) {
      if constexpr (PAIR) {
        constexpr int kSlots = 2 * (D / 32), kAhead = 2;
        bf16x8 dof[kSlots], qf[kSlots];
        auto fetch = [&](int idx) {
          const int cc = idx / (D / 32), db = idx % (D / 32);
          const int qr = 32 * sb + 16 * cc + 4 * h + (lane % 16) / 4;
          const int col = 32 * db + 16 * ((lane / 16) % 2) + 4 * (lane % 4);
          dof[idx] = lds_read_tr_pair_step(&sdO[tile_row(qr) + col], C::kTrStep);
          qf[idx] = lds_read_tr_pair_step(&sQ[tile_row(qr) + col], C::kTrStep);
        };
#pragma unroll
        for (int j = 0; j < kAhead; ++j) fetch(j);
        bf16x8 pf = pack8(s_acc, 0), dsf = pack8(dp_acc, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int idx = 0; idx < kSlots; ++idx) {
          const int db = idx % (D / 32);
          if (idx + kAhead < kSlots) fetch(idx + kAhead);
          dv_acc[db] = mfma32(dof[idx], pf, dv_acc[db]);
          dk_acc[db] = mfma32(qf[idx], dsf, dk_acc[db]);
          if (idx + 1 == D / 32) { pf = pack8(s_acc, 8); dsf = pack8(dp_acc, 8); }
          __builtin_amdgcn_sched_barrier(0);
        }
        return;
      }
#pragma unroll
      for (int cc = 0; cc < 2; ++cc) {
        // registers 8cc+4jj+t hold queries 32sb + 16cc + 8jj + 4h + t: fetch dO / Q rows in that order
        const bf16x8 pf = pack8(s_acc, 8 * cc);
        const bf16x8 dsf = pack8(dp_acc, 8 * cc);
        const int qr = 32 * sb + 16 * cc + 4 * h + (lane % 16) / 4;
#pragma unroll
        for (int db = 0; db < D / 32; ++db) {
          const int col = 32 * db + 16 * ((lane / 16) % 2) + 4 * (lane % 4);
          const bf16x8 dof = lds_read_tr_pair_step(&sdO[tile_row(qr) + col], C::kTrStep);
          const bf16x8 qf = lds_read_tr_pair_step(&sQ[tile_row(qr) + col], C::kTrStep);
          dv_acc[db] = mfma32(dof, pf, dv_acc[db]);
          dk_acc[db] = mfma32(qf, dsf, dk_acc[db]);
        }
      }
    };

    const bool off_diagonal = !PAIR && (!a.causal || kw0 + 31 <= a.q_offset + q0);
    if (!kStageTop && has_next && !off_diagonal) prefetch();
    if (off_diagonal) {
      // Every pair of this trip is visible to this wave (all trips off the diagonal): straight-line code in an order
      // that lets the wave's own phases overlap -- the matrix pipe works on the second sub-block's S / dP while the
      // vector pipe does the first one's softmax, and on the first one's dV / dK during the second one's softmax.
      f32x16 s0, d0, s1, d1;
      // Four stages; in the middle two, every pair of MFMAs is followed in program order by a share of the OTHER
      // sub-block's softmax arithmetic and by the LDS reads of a later pair.  A wave issues in order: vector
      // instructions that merely follow a batch of MFMAs start when the batch has been issued, i.e. when the matrix
      // pipe is nearly done with it, while an MFMA followed by a few vector instructions keeps both pipes busy
      // (measured on this GPU with one wave per SIMD: 16 MFMAs then 64 fma + 16 exp take 1.63x the time of the same
      // work dealt out one MFMA at a time).  The scheduling barriers pin that order slot by slot (+5 % at head_dim 128,
      // one wave per SIMD; +2.5 % at head_dim 64, where the second wave of the SIMD fills most gaps already).  The
      // head_dim 64 kernel has 256 registers: fragments are fetched one pair ahead and lse rows one slot ahead so
      // that nothing spills.
      constexpr int kPairs = D / 16;        // (S, dP) MFMA pairs per sub-block
      constexpr int kSlots = 2 * (D / 32);  // (dV, dK) MFMA pairs per sub-block
      auto softmax_part = [&](f32x16& s_acc, f32x16& dp_acc, const f32x4 (&l4)[4], int first, int count) {
#pragma unroll
        for (int i = first; i < first + count; ++i) {
          const float pv = fast_exp2(s_acc[i] * c - l4[i / 4][i % 4]);
          s_acc[i] = pv;
          dp_acc[i] = pv * dp_acc[i];
        }
      };
      // stage A: products of sub-block 0
      products(0, s0, d0);
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(1);
      // stage B: products of sub-block 1, softmax of sub-block 0 between them
      {
        // lse rows of sub-block 0 are fetched a slot ahead of the elements that need them (kPer elements per slot)
        constexpr int kPer = 16 / kPairs;
        f32x4 l4[4];
        auto lse_row = [&](int r) {
          l4[r] = *reinterpret_cast<const f32x4*>(&sL[8 * r + 4 * h]);
        };
        lse_row(0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const f32x4 d4 = *reinterpret_cast<const f32x4*>(&sDelta[32 + 8 * j + 4 * h]);
#pragma unroll
          for (int t = 0; t < 4; ++t) { s1[4 * j + t] = 0.f; d1[4 * j + t] = d4[t]; }
        }
        bf16x8 qa[kPairs], da[kPairs];
        auto fetch = [&](int j) {
          qa[j] = *reinterpret_cast<const bf16x8*>(&sQ[tile_row(32 + n) + 16 * j + 8 * h]);
          da[j] = *reinterpret_cast<const bf16x8*>(&sdO[tile_row(32 + n) + 16 * j + 8 * h]);
        };
        constexpr int kAhead = D >= 128 ? 2 : 1;   // fragment pairs in flight ahead of their MFMAs
#pragma unroll
        for (int j = 0; j < kAhead; ++j) fetch(j);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < kPairs; ++j) {
          if (j + kAhead < kPairs) fetch(j + kAhead);
          if (((j + 1) * kPer) % 4 == 0 && (j + 1) * kPer < 16) lse_row((j + 1) * kPer / 4);
          s1 = mfma32(qa[j], kf[j], s1);
          d1 = mfma32(da[j], vf[j], d1);
          softmax_part(s0, d0, l4, j * kPer, kPer);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // stage C: dV / dK of sub-block 0, softmax of sub-block 1 between them
      {
        constexpr int kPer = 16 / kSlots;
        f32x4 l4[4];
        auto lse_row = [&](int r) {
          l4[r] = *reinterpret_cast<const f32x4*>(&sL[32 + 8 * r + 4 * h]);
        };
        lse_row(0);
        bf16x8 dof[kSlots], qf[kSlots];
        auto fetch = [&](int idx) {
          const int cc = idx / (D / 32), db = idx % (D / 32);
          const int qr = 16 * cc + 4 * h + (lane % 16) / 4;
          const int col = 32 * db + 16 * ((lane / 16) % 2) + 4 * (lane % 4);
          dof[idx] = lds_read_tr_pair_step(&sdO[tile_row(qr) + col], C::kTrStep);
          qf[idx] = lds_read_tr_pair_step(&sQ[tile_row(qr) + col], C::kTrStep);
        };
        fetch(0);
        bf16x8 pf = pack8(s0, 0), dsf = pack8(d0, 0);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int idx = 0; idx < kSlots; ++idx) {
          const int db = idx % (D / 32);
          if (idx + 1 < kSlots) fetch(idx + 1);
          dv_acc[db] = mfma32(dof[idx], pf, dv_acc[db]);
          dk_acc[db] = mfma32(qf[idx], dsf, dk_acc[db]);
          if (idx + 1 == D / 32) { pf = pack8(s0, 8); dsf = pack8(d0, 8); }
          if (((idx + 1) * kPer) % 4 == 0 && (idx + 1) * kPer < 16) lse_row((idx + 1) * kPer / 4);
          softmax_part(s1, d1, l4, idx * kPer, kPer);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
      // stage D: dV / dK of sub-block 1; the next tile's global loads are issued here, not at the top of the trip:
      // their registers are free until now
      __builtin_amdgcn_s_setprio(0);
      if (has_next) prefetch();
      accumulate(1, s1, d1);
    } else {
#pragma unroll
      for (int sbi = 0; sbi < (PAIR ? 1 : BM / 32); ++sbi) {
        const int sb = PAIR ? pair_sb : sbi;
        const int qs_pos = a.q_offset + q0 + 32 * sb;       // position of the sub-block's first query
        if (a.causal && kw0 > qs_pos + 31) continue;        // every (query, key) pair of this block is masked
        f32x16 s_acc, dp_acc;
        products(sb, s_acc, dp_acc);
        if (a.causal && kw0 + 31 > qs_pos) softmax_grad(sb, s_acc, dp_acc, std::true_type{});
        else softmax_grad(sb, s_acc, dp_acc, std::false_type{});
        accumulate(sb, s_acc, dp_acc);
      }
    }
    buf_off ^= static_cast<uint32_t>(C::kBufBytes);
    if (!kStageTop && has_next) stage(buf_off != 0);
    tile = tile + 1 == n_qtiles ? qt_start : tile + 1;
    __syncthreads();  // all waves are done with the buffer just read (refilled in the next trip) and the next tile is visible
  }

  // ---- epilogue: dK (scaled) and dV rows of this wave's 32 keys, through the wave's piece of LDS (free now:
  //      the loop ended on a barrier).  bf16 gradients are written with streaming stores: nothing on this
  //      GPU reads them back soon, and lines left dirty in L2 are only written back when the kernel ends.
  if constexpr (PAIR) {
    // the second wave of each pair hands its sums over, dK then dV (the loop ended on a barrier, or never ran)
    float* xch = reinterpret_cast<float*>(smem_raw + wave * C::kPairExchangeBytes);
#pragma unroll
    for (int which = 0; which < 2; ++which) {
      f32x16 (&acc)[D / 32] = which == 0 ? dk_acc : dv_acc;
      if (pair_sb == 1) {
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
          for (int i = 0; i < 16; i += 4)
            *reinterpret_cast<f32x4*>(&xch[((db * 4 + i / 4) * 64 + lane) * 4]) = f32x4{acc[db][i], acc[db][i + 1], acc[db][i + 2], acc[db][i + 3]};
      }
      __syncthreads();
      if (pair_sb == 0) {
#pragma unroll
        for (int db = 0; db < D / 32; ++db)
#pragma unroll
          for (int i = 0; i < 16; i += 4) {
            const f32x4 o = *reinterpret_cast<const f32x4*>(&xch[((db * 4 + i / 4) * 64 + lane) * 4]);
#pragma unroll
            for (int t = 0; t < 4; ++t) acc[db][i + t] += o[t];
          }
      }
      __syncthreads();
    }
  }
  if (!PAIR || pair_sb == 0) {
    unsigned char* region = smem_raw + wave * kRowRegionBytes;
    const int row0 = crow0 + 32 * wave;          // first row of the wave inside its chunk
    const int rows_live = a.kv.len - row0;
    const int64_t off = b * p.dks[0] + hkv * p.dks[1] + static_cast<int64_t>(row0) * p.dks[2];
    // gradient w.r.t. the un-rotated k: rotate the lane's row of dK back (linear, so the scale and the sum can follow)
    if (p.rope.cos != nullptr) rope_unrotate_acc<D>(dk_acc, p.rope, n < rows_live ? p.rope.k_pos0 + kw0 + n : 0, h);
    const bool accumulate = (p.dkv_accumulate >> chunk) & 1u;
    if (p.dk_final[chunk] != nullptr) {
      // the last block this chunk's gradient was waiting for: total = travelling sums + this block, rounded once
      const int64_t foff = b * p.dkfs[0] + hkv * p.dkfs[1] + static_cast<int64_t>(row0) * p.dkfs[2];
      wave_store_rows_total<D>(region, dk_acc, a.sm_scale, accumulate ? static_cast<const float*>(p.dk[chunk]) + off : nullptr, p.dks[2],
                               p.dk_final[chunk] + foff, p.dkfs[2], rows_live, lane);
      wave_store_rows_total<D>(region, dv_acc, 1.f, accumulate ? static_cast<const float*>(p.dv[chunk]) + off : nullptr, p.dks[2],
                               p.dv_final[chunk] + foff, p.dkfs[2], rows_live, lane);
    } else if (p.dkv_f32) {
      wave_store_rows<D, true>(region, dk_acc, a.sm_scale, static_cast<float*>(p.dk[chunk]) + off, p.dks[2], rows_live, lane, accumulate, false);
      wave_store_rows<D, true>(region, dv_acc, 1.f, static_cast<float*>(p.dv[chunk]) + off, p.dks[2], rows_live, lane, accumulate, false);
    } else {
      wave_store_rows<D, false>(region, dk_acc, a.sm_scale, static_cast<__bf16*>(p.dk[chunk]) + off, p.dks[2], rows_live, lane, false, kStreamGrads);
      wave_store_rows<D, false>(region, dv_acc, 1.f, static_cast<__bf16*>(p.dv[chunk]) + off, p.dks[2], rows_live, lane, false, kStreamGrads);
    }
  }
}

// grid = (Hkv * B, key tiles or pairs of key tiles): the x index runs fastest in dispatch order, so all heads of
// key tile 0 (the longest under a causal mask) start first and the short tiles fill in behind them; workgroups
// of one head are a multiple of 8 apart in dispatch order and so share an XCD's L2.  With pair_ktiles a
// workgroup takes tile t and then tile n-1-t: under a causal mask every pair is the same amount of work, so a
// launch whose pairs fill the GPU once ends without a tail of short workgroups and pays the start-up of a
// workgroup (kernel arguments, first loads) half as often.
template <int D, bool PAIR = false>
__device__ __forceinline__ void attn_bwd_dkdv_body(const BwdParams& p) {
  const int n_ktiles = (p.a.Sk + KvCfg<D, PAIR>::BN - 1) / KvCfg<D, PAIR>::BN;
  const int first = blockIdx.y;
  attn_bwd_dkdv_tile<D, PAIR>(p, first);
  const int second = n_ktiles - 1 - first;
  if (p.pair_ktiles && second != first) {
    __syncthreads();  // the epilogue's pieces of LDS are the next tile's buffers
    attn_bwd_dkdv_tile<D, PAIR>(p, second);
  }
}

// D = 64 fits two workgroups per CU (<= 256 registers per lane), which lets one workgroup's MFMA
// work overlap the other's softmax / LDS phases; D = 128 needs the full register file.
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void attn_bwd_dkdv_kernel_d64(const BwdParams p) {
  attn_bwd_dkdv_body<64>(p);
}
// D = 128: eight waves, two per key block (see KvCfg), 256 registers each
__global__ __launch_bounds__(512) void attn_bwd_dkdv_kernel_d128(const BwdParams p) {
  attn_bwd_dkdv_body<128, true>(p);
}

template <int D> struct KvKernel;
template <> struct KvKernel<64> { static constexpr auto fn = &attn_bwd_dkdv_kernel_d64; };
template <> struct KvKernel<128> { static constexpr auto fn = &attn_bwd_dkdv_kernel_d128; };

// =====================================================================================  dQ
// KS > 1: KS waves share the same 32 queries and each takes one 64-key step of every staged tile (see the forward
// kernel); their dQ partial sums meet in LDS at the end.
template <int D, int NW, int KT, int KS = 1>
struct DqCfg {
  static constexpr int kThreads = 64 * NW;
  static constexpr int kQWaves = NW / KS;
  static constexpr int BM = 32 * kQWaves;  // queries per workgroup (32 per query wave)
  static_assert(NW % KS == 0 && (KS == 1 || KT == 64 * KS), "one 64-key step of every staged tile per key-split wave");
  static constexpr int BN = 64;            // keys per compute step
  static constexpr int LDK = D + 8;        // pitch of the K and V tiles
  static constexpr int kVecPerRow = D / 8;
  static constexpr int kLoads = KT * kVecPerRow / kThreads;
  static constexpr int kTileElems = 2 * KT * LDK;
  static constexpr size_t kLdsBytes = 2 * kTileElems * sizeof(__bf16);  // double-buffered
  static_assert(NW * kRowRegionBytes <= kLdsBytes, "the epilogue reuses the tile buffers");
  static_assert(NW * WaveTile<D>::kRegionBytes <= kLdsBytes, "the Q / dO fragments pass through the tile buffers");
  static_assert(KT % BN == 0 && (KT * kVecPerRow) % kThreads == 0, "tile must split evenly over the threads");
  static constexpr size_t kExchangeBytes = (D / 32) * 16 * 64 * 4;   // a wave's dQ^T accumulators
  static_assert(KS == 1 || NW * kExchangeBytes <= kLdsBytes, "the exchange reuses the tile buffers");
};

// (small workgroups are built for two of them per CU: at most 256 registers per lane)
template <int D, int NW, int KT, bool kDelta, int KS = 1>
__global__ __launch_bounds__(64 * NW, (NW <= 4 && D <= 64) ? 2 : 1) void attn_bwd_dq_kernel(const BwdParams p) {
  using C = DqCfg<D, NW, KT, KS>;
  constexpr int BM = C::BM, BN = C::BN, LDK = C::LDK;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  __bf16* smem = reinterpret_cast<__bf16*>(smem_raw);

  const AttnParams& a = p.a;
  const int n_qtiles = (a.Sq + BM - 1) / BM;
  // same dispatch order as the forward kernel: every head's last (longest) query tile first
  const int qtile = n_qtiles - 1 - static_cast<int>(blockIdx.y);
  const int hq = blockIdx.x % a.Hq, b = blockIdx.x / a.Hq;
  const int hkv = hq / (a.Hq / a.Hkv);
  const int q0 = qtile * BM;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int n = lane % 32, h = lane / 32;
  const int qw = wave % C::kQWaves, ks = wave / C::kQWaves;   // which queries, which 64-key step of a staged tile
  const float c = a.sm_scale * kLog2e;

  // ---- per-lane query: Q and dO fragments (B operands: fetched row-major, turned into fragments through the
  //      wave's piece of LDS; the tile buffers are filled only after the barrier below), lse and delta
  const int qrow = q0 + qw * 32 + n;
  const bool qlive = qrow < a.Sq;
  bf16x8 qf[D / 16], dof[D / 16];
  float lse2 = INFINITY, delta = 0.f;
  {
    const int row0 = q0 + qw * 32;
    WaveTile<D> qt, dt;
    qt.issue(make_buffer(a.q + b * a.qs[0] + hq * a.qs[1] + static_cast<int64_t>(row0) * a.qs[2],
                         span_bytes(a.Sq - row0, a.qs[2], D)), a.qs[2], lane);
    dt.issue(make_buffer(p.dout + b * a.os[0] + hq * a.os[1] + static_cast<int64_t>(row0) * a.os[2],
                         span_bytes(a.Sq - row0, a.os[2], D)), a.os[2], lane);
    WaveTile<D> ot;
    if constexpr (kDelta)
      ot.issue(make_buffer(p.out + b * a.os[0] + hq * a.os[1] + static_cast<int64_t>(row0) * a.os[2],
                           span_bytes(a.Sq - row0, a.os[2], D)), a.os[2], lane);
    const int64_t gi = (static_cast<int64_t>(b) * a.Hq + hq) * a.Sq + qrow;
    if (qlive) {
      const float l = p.lse[gi];
      lse2 = (l == -INFINITY) ? INFINITY : l * kLog2e;  // a row that saw no key contributes nothing
      if constexpr (!kDelta) delta = p.delta[gi];
    }
    unsigned char* region = smem_raw + wave * WaveTile<D>::kRegionBytes;
    qt.fragments(region, lane, qf);
    dt.fragments(region, lane, dof);
    if constexpr (kDelta) {
      // delta = sum_d dO * O of the lane's row (context_parallel.py:145): each half of the wave holds half of the
      // row's columns in its fragments; the dK/dV kernel, launched after this one, reads the result from memory
      bf16x8 of[D / 16];
      ot.fragments(region, lane, of);
      float part = 0.f;
#pragma unroll
      for (int s = 0; s < D / 16; ++s)
#pragma unroll
        for (int e = 0; e < 8; ++e) part += static_cast<float>(dof[s][e]) * static_cast<float>(of[s][e]);
      delta = half_sum(part);
      if (qlive && h == 0 && ks == 0) p.delta_w[gi] = delta;
    }
  }

  f32x16 dq[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int i = 0; i < 16; ++i) dq[db][i] = 0.f;

  // ---- key range of this query tile
  const int q_hi = (q0 + BM < a.Sq ? q0 + BM : a.Sq);
  int kv_end = a.Sk;
  if (a.causal) {
    const int vis = a.q_offset + q_hi;
    kv_end = vis < a.Sk ? vis : a.Sk;
    if (kv_end < 0) kv_end = 0;
  }
  const int ntiles = (kv_end + KT - 1) / KT;

  // K / V tiles travel global -> registers -> LDS with buffer loads (wave-uniform resource per tile, per-lane
  // byte offsets computed once, rows past Sk read as zeros)
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
      *reinterpret_cast<u32x4*>(&sV[r * LDK + cv * 8]) = vreg[i];
    }
  };

  if (ntiles > 0) load_tile();
  __syncthreads();  // every wave has its Q / dO fragments: the tile buffers may be filled
  if (ntiles > 0) store_tile(0);
  // all loads so far are complete on every path into the loop (the LDS fill waited for the newest); stating
  // it keeps a vmcnt(0) wait, which would hit the next tile's prefetch, out of the loop body
  __builtin_amdgcn_s_waitcnt(kWaitVmcnt0);
  if (ntiles > 1) load_tile();
  __syncthreads();

  const int blk_q_lo = a.q_offset + q0 + qw * 32;  // position of this wave's first query
  const int qpos = a.q_offset + qrow;
  for (int t = 0; t < ntiles; ++t) {
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
      if (a.causal && k0 > blk_q_lo + 31) continue;  // the wave's whole 32x64 block is in the future
      const __bf16* sKs = sK + sub * BN * LDK;
      const __bf16* sVs = sV + sub * BN * LDK;
      f32x16 s_acc[BN / 32], dp_acc[BN / 32];
      // the compiler's scheduler is asked for its MFMA / LDS-read interleaving of this block (-1 to -5 %; the key-split
      // variant is better off without)
      if constexpr (KS == 1) __builtin_amdgcn_iglp_opt(0);
#pragma unroll
      for (int mb = 0; mb < BN / 32; ++mb) {
        // dP - delta comes out of the MFMA
#pragma unroll
        for (int i = 0; i < 16; ++i) { s_acc[mb][i] = 0.f; dp_acc[mb][i] = -delta; }
#pragma unroll
        for (int s = 0; s < D / 16; ++s) {
          const bf16x8 ka = *reinterpret_cast<const bf16x8*>(&sKs[(32 * mb + n) * LDK + 16 * s + 8 * h]);
          const bf16x8 va = *reinterpret_cast<const bf16x8*>(&sVs[(32 * mb + n) * LDK + 16 * s + 8 * h]);
          s_acc[mb] = mfma32(ka, qf[s], s_acc[mb]);
          dp_acc[mb] = mfma32(va, dof[s], dp_acc[mb]);
        }
      }
      // dS^T = P^T * (dP^T - delta); keys past the diagonal are masked only in tiles that straddle it
      // (rows of K / V past Sk are zero, so those keys add nothing to dQ)
      const bool need_mask = a.causal && (k0 + BN - 1 > blk_q_lo);
      if (need_mask) {
        // the asm statement keeps this a real (wave-uniform) branch instead of per-element selects
        asm volatile("; masked tile" ::: "memory");
#pragma unroll
        for (int mb = 0; mb < BN / 32; ++mb)
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            const int key = k0 + 32 * mb + 8 * (i / 4) + 4 * h + (i % 4);
            if (key > qpos) s_acc[mb][i] = -INFINITY;   // exp2(-inf) = 0
          }
      }
#pragma unroll
      for (int mb = 0; mb < BN / 32; ++mb)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const float pv = fast_exp2(s_acc[mb][i] * c - lse2);
          dp_acc[mb][i] = pv * dp_acc[mb][i];
        }
      // ---- dQ^T[d][query] += K^T[d][key] dS^T[key][query]
#pragma unroll
      for (int mb = 0; mb < BN / 32; ++mb)
#pragma unroll
        for (int cc = 0; cc < 2; ++cc) {
          const bf16x8 dsf = pack8(dp_acc[mb], 8 * cc);
          const int krow = 32 * mb + 16 * cc + 4 * h + (lane % 16) / 4;
#pragma unroll
          for (int db = 0; db < D / 32; ++db) {
            const int col = 32 * db + 16 * ((lane / 16) % 2) + 4 * (lane % 4);
            const bf16x8 ktf = lds_read_tr_pair(&sKs[krow * LDK + col], LDK);
            dq[db] = mfma32(ktf, dsf, dq[db]);
          }
        }
    }
    __syncthreads();
  }

  // ---- key split: the partial sums of the waves ks > 0 are added to the wave ks == 0 of the same queries through LDS
  //      (the loop ended on a barrier: the tile buffers are free; the store pieces used below lie in front of the
  //      exchange areas of the ks > 0 waves)
  if constexpr (KS > 1) {
    float* xo = reinterpret_cast<float*>(smem_raw + wave * C::kExchangeBytes);
    if (ks > 0) {
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) xo[(db * 16 + i) * 64 + lane] = dq[db][i];
    }
    __syncthreads();
    if (ks > 0) return;
#pragma unroll
    for (int j = 1; j < KS; ++j) {
      const float* oo = reinterpret_cast<const float*>(smem_raw + (qw + j * C::kQWaves) * C::kExchangeBytes);
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int i = 0; i < 16; ++i) dq[db][i] += oo[(db * 16 + i) * 64 + lane];
    }
    static_assert(kRowRegionBytes <= C::kExchangeBytes, "store pieces lie below the exchange areas read above");
  }

  // ---- epilogue: the wave's 32 dQ rows leave through its piece of LDS as whole lines (the loop ended on a barrier)
  {
    unsigned char* region = smem_raw + wave * kRowRegionBytes;
    const int row0 = q0 + qw * 32;
    const int64_t off = b * p.dqs[0] + hq * p.dqs[1] + static_cast<int64_t>(row0) * p.dqs[2];
    if (p.rope.cos != nullptr) rope_unrotate_acc<D>(dq, p.rope, qlive ? p.rope.q_pos0 + qrow : 0, h);
    if (p.dq_f32)
      wave_store_rows<D, true>(region, dq, a.sm_scale, static_cast<float*>(p.dq) + off, p.dqs[2], a.Sq - row0, lane, p.dq_accumulate, false);
    else
      wave_store_rows<D, false>(region, dq, a.sm_scale, static_cast<__bf16*>(p.dq) + off, p.dqs[2], a.Sq - row0, lane, false, kStreamGrads);
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
int launch_dkdv(const BwdParams& p, hipStream_t s) {
  using C = KvCfg<D, D == 128>;
  static LdsOnce lds_reserved;
  if (!reserve_lds_once(lds_reserved, reinterpret_cast<const void*>(KvKernel<D>::fn), C::kLdsBytes))
    return fail(PICO_ERR_LAUNCH, "pico_attn_bwd(dk/dv): cannot reserve %zu bytes of LDS", C::kLdsBytes);
  const int n_ktiles = (p.a.Sk + C::BN - 1) / C::BN;
  // pairs only when they still fill most of the GPU (two workgroups per CU for D = 64, one for D = 128; at D = 64 three
  // quarters of the places are enough: rank 2 of 4 at configs[1], 384 pairs, 21.2 -> 20.3 us; with 256 pairs single tiles
  // are up to 30 % faster)
  BwdParams q = p;
  const int64_t slots = D == 64 ? 384 : 256;
  q.pair_ktiles = p.a.causal && n_ktiles >= 2 && static_cast<int64_t>(p.a.Hkv) * p.a.B * ((n_ktiles + 1) / 2) >= slots;
  const int grid_y = q.pair_ktiles ? (n_ktiles + 1) / 2 : n_ktiles;
  hipLaunchKernelGGL(KvKernel<D>::fn, dim3(p.a.Hkv * p.a.B, grid_y), dim3(C::kThreads), C::kLdsBytes, s, q);
  return PICO_OK;
}

template <int D, int NW, int KT, bool kDelta, int KS>
int launch_dq_impl(const BwdParams& p, hipStream_t s) {
  using C = DqCfg<D, NW, KT, KS>;
  static LdsOnce lds_reserved;
  if (!reserve_lds_once(lds_reserved, reinterpret_cast<const void*>(&attn_bwd_dq_kernel<D, NW, KT, kDelta, KS>), C::kLdsBytes))
    return fail(PICO_ERR_LAUNCH, "pico_attn_bwd(dq): cannot reserve %zu bytes of LDS", C::kLdsBytes);
  const int n_qtiles = (p.a.Sq + C::BM - 1) / C::BM;
  hipLaunchKernelGGL((attn_bwd_dq_kernel<D, NW, KT, kDelta, KS>), dim3(p.a.Hq * p.a.B, n_qtiles), dim3(C::kThreads), C::kLdsBytes, s, p);
  return PICO_OK;
}

template <int D, int NW, int KT, int KS = 1>
int launch_dq(const BwdParams& p, hipStream_t s) {
  return p.out ? launch_dq_impl<D, NW, KT, true, KS>(p, s) : launch_dq_impl<D, NW, KT, false, KS>(p, s);
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

namespace {

// Shared body of the backward entry points.  With `out` (bf16 forward output) the dQ kernel computes delta itself,
// writes it to `delta_w`, and runs BEFORE the dK/dV kernel, which reads it from there.
int run_bwd(const char* fn, const pico_attn_desc* desc, const void* q, const pico_kv_chunks* kv, const void* dout,
            const float* lse, const float* delta, const void* out, float* delta_w, void* dq, const int64_t* dq_stride,
            int dq_dtype, int dq_accumulate, const int64_t* dkv_stride, int dkv_dtype, void* stream,
            const RopeArgs* rope = nullptr) {
  if ((dkv_dtype != PICO_BF16 && dkv_dtype != PICO_F32) || (dq_dtype != PICO_BF16 && dq_dtype != PICO_F32))
    return fail(PICO_ERR_DTYPE, "%s: gradient dtype codes %d / %d not supported", fn, dq_dtype, dkv_dtype);
  if (dq_accumulate && dq_dtype != PICO_F32) return fail(PICO_ERR_DTYPE, "%s: accumulate needs fp32 gradients", fn);
  BwdParams p;
  p.a = make_params(desc, q, nullptr, nullptr);
  if (int rc = set_chunks(fn, desc, kv, p.a, false)) return rc;
  if (desc->B == 0) return PICO_OK;
  // a gradient that is not wanted is passed as NULL and its kernel (or its chunk's workgroups) is skipped
  bool want_dkv = false;
  p.dkv_accumulate = 0;
  for (int c = 0; c < kMaxChunks; ++c) {
    p.dk[c] = p.dv[c] = nullptr;
    p.dk_final[c] = p.dv_final[c] = nullptr;
  }
  bool any_final = false;
  for (int c = 0; c < kv->count; ++c) {
    if ((kv->dk[c] == nullptr) != (kv->dv[c] == nullptr) || (kv->dk_final[c] == nullptr) != (kv->dv_final[c] == nullptr))
      return fail(PICO_ERR_NULL, "%s: dk and dv (and dk_final and dv_final) must be given together (chunk %d)", fn, c);
    if (!aligned16(kv->dk_final[c]) || !aligned16(kv->dv_final[c]))
      return fail(PICO_ERR_ALIGN, "%s: chunk %d: dk_final and dv_final must be 16-byte aligned", fn, c);
    p.dk[c] = kv->dk[c];
    p.dv[c] = kv->dv[c];
    p.dk_final[c] = static_cast<__bf16*>(kv->dk_final[c]);
    p.dv_final[c] = static_cast<__bf16*>(kv->dv_final[c]);
    const bool acc = kv->dk[c] && ((kv->accumulate_mask >> c) & 1u);
    if (kv->dk[c] || kv->dk_final[c]) want_dkv = true;
    if (acc) p.dkv_accumulate |= 1u << c;
    if (kv->dk_final[c]) {
      any_final = true;
      if (acc && dkv_dtype != PICO_F32)
        return fail(PICO_ERR_DTYPE, "%s: chunk %d: the sums that dk_final completes must be fp32", fn, c);
    }
  }
  for (int i = 0; i < 3; ++i) {
    p.dkfs[i] = any_final ? kv->final_stride[i] : 0;
    if (any_final && (p.dkfs[i] < 0 || p.dkfs[i] % 4 != 0))
      return fail(PICO_ERR_STRIDE, "%s: final_stride must hold non-negative multiples of 4 elements", fn);
  }
  if (p.dkv_accumulate && dkv_dtype != PICO_F32) return fail(PICO_ERR_DTYPE, "%s: accumulate needs fp32 gradients", fn);
  const bool want_dq = dq != nullptr;
  const bool have_q = desc->Sq > 0 && want_dq, have_k = desc->Sk > 0 && want_dkv;
  if ((have_q || have_k) && desc->Sq > 0 && (!q || !dout || !lse || !delta))
    return fail(PICO_ERR_NULL, "%s: q, dout, lse and delta are required", fn);
  if ((have_q || have_k) && desc->Sk > 0)
    for (int c = 0; c < kv->count; ++c)
      if (!kv->k[c] || !kv->v[c]) return fail(PICO_ERR_NULL, "%s: k / v of chunk %d are NULL", fn, c);
  if (!aligned16(q) || !aligned16(dout) || !aligned16(dq) || !aligned16(out))
    return fail(PICO_ERR_ALIGN, "%s: q, dout, out and dq must be 16-byte aligned", fn);
  p.dout = static_cast<const __bf16*>(dout);
  p.lse = lse; p.delta = delta; p.dq = dq;
  p.out = static_cast<const __bf16*>(out);
  p.delta_w = delta_w;
  p.dq_f32 = dq_dtype == PICO_F32;
  p.dq_accumulate = dq_accumulate != 0;
  p.dkv_f32 = dkv_dtype == PICO_F32;
  p.pair_ktiles = 0;
  p.rope = rope ? *rope : RopeArgs{nullptr, nullptr, 0, 0, 0, 0};
  auto strides = [&](const int64_t* given, int heads, int seq, int64_t (&st)[3], int align) -> bool {
    if (given) {
      for (int i = 0; i < 3; ++i) {
        if (given[i] < 0 || given[i] % align != 0) return false;
        st[i] = given[i];
      }
    } else {
      st[2] = desc->D;
      st[1] = static_cast<int64_t>(seq) * desc->D;
      st[0] = st[1] * heads;
    }
    return true;
  };
  if (!strides(dq_stride, desc->Hq, desc->Sq, p.dqs, p.dq_f32 ? 4 : 8) || !strides(dkv_stride, desc->Hkv, kv->chunk_len, p.dks, 8))
    return fail(PICO_ERR_STRIDE, "%s: dq strides must be non-negative multiples of 4 (fp32) or 8 (bf16), dk/dv strides of 8", fn);
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto run_dkdv = [&]() -> int {
    if (!have_k) return PICO_OK;
    // without queries the dK/dV kernel still runs: it writes (or adds) zeros
    if (int rc = desc->D == 64 ? launch_dkdv<64>(p, s) : launch_dkdv<128>(p, s)) return rc;
    return check_launch("pico_attn_bwd(dk/dv)");
  };
  auto run_dq = [&]() -> int {
    if (!have_q) return PICO_OK;
    // without keys the dQ kernel still runs: it writes (or adds) zeros
    int rc;
    const int64_t heads = static_cast<int64_t>(desc->B) * desc->Hq;
    if (desc->D == 64) {
      auto groups = [&](int bm) { return heads * ((desc->Sq + bm - 1) / bm); };
      const int64_t visible_keys = desc->causal ? std::min<int64_t>(desc->Sk, static_cast<int64_t>(desc->q_offset) + desc->Sq) : desc->Sk;
      // the forward's rules: eight waves per workgroup also for rectangular launches (every query sees at least as many
      // keys as there are queries) with fewer workgroups than the square ones need
      const bool rectangular = !desc->causal || desc->q_offset >= desc->Sq;
      // several generations of workgroups over short key ranges (a few trips each): two four-wave workgroups per CU hide
      // each other's prologues and epilogues, which one eight-wave workgroup per CU cannot (B8 S768 51.3 -> 44.3 us,
      // B16 S512 54.4 -> 48.1, B8 S1024 78.5 -> 72.9, B8 S1536 147.8 -> 144.3; from S2048 on, and with 512 workgroups,
      // the eight-wave kernel is level or ahead)
      if (groups(256) >= 768 && visible_keys <= 1536) rc = launch_dq<64, 4, 64>(p, s);
      else if (groups(256) >= 512) rc = launch_dq<64, 8, 64>(p, s);
      else if (groups(128) >= 512) {
        if (rectangular && groups(256) >= 256) rc = launch_dq<64, 8, 64>(p, s);
        else rc = launch_dq<64, 4, 64>(p, s);
      }
      // few waves in all: two waves per 32 queries, 64 keys of every 128 each (rank 3 of 4 at configs[1] with eight waves
      // per workgroup: 18.8 -> 17.9 us)
      else if (groups(128) >= 256 && rectangular && visible_keys >= 512) rc = launch_dq<64, 8, 128, 2>(p, s);
      else rc = launch_dq<64, 4, 128, 2>(p, s);
    } else {
      if (heads * ((desc->Sq + 255) / 256) >= 256) rc = launch_dq<128, 8, 64>(p, s);
      else rc = launch_dq<128, 4, 64>(p, s);
    }
    if (rc) return rc;
    return check_launch("pico_attn_bwd(dq)");
  };
  if (p.out) {  // the dQ kernel produces delta for the dK/dV kernel
    if (int rc = run_dq()) return rc;
    return run_dkdv();
  }
  if (int rc = run_dkdv()) return rc;
  return run_dq();
}

pico_kv_chunks one_chunk(const pico_attn_desc* desc, const void* k, const void* v, void* dk, void* dv, int accumulate) {
  pico_kv_chunks kv = {};
  kv.count = 1;
  kv.chunk_len = desc->Sk;
  kv.k[0] = k;
  kv.v[0] = v;
  kv.dk[0] = dk;
  kv.dv[0] = dv;
  kv.accumulate_mask = accumulate ? 1u : 0u;
  return kv;
}

// delta inside the dQ kernel needs that kernel to run and a bf16 out; otherwise the pre-pass computes it
int run_bwd_with_out(const char* fn, const pico_attn_desc* desc, const void* q, const pico_kv_chunks* kv, const void* dout,
                     const void* out, int out_dtype, const float* lse, float* delta, void* dq, const int64_t* dq_stride,
                     int dq_dtype, int dq_accumulate, const int64_t* dkv_stride, int dkv_dtype, void* stream,
                     const RopeArgs* rope) {
  if (out_dtype != PICO_BF16 && out_dtype != PICO_F32)
    return fail(PICO_ERR_DTYPE, "%s: out dtype code %d not supported", fn, out_dtype);
  if (desc->B == 0) return PICO_OK;
  if (desc->Sq > 0 && (!out || !delta)) return fail(PICO_ERR_NULL, "%s: out and delta are required", fn);
  const bool in_kernel = out_dtype == PICO_BF16 && dq != nullptr && desc->Sq > 0;
  if (!in_kernel) {
    if (int rc = pico_attn_bwd_preprocess(desc, dout, out, out_dtype, delta, nullptr, stream)) return rc;
    return run_bwd(fn, desc, q, kv, dout, lse, delta, nullptr, nullptr, dq, dq_stride, dq_dtype, dq_accumulate, dkv_stride,
                   dkv_dtype, stream, rope);
  }
  return run_bwd(fn, desc, q, kv, dout, lse, delta, out, delta, dq, dq_stride, dq_dtype, dq_accumulate, dkv_stride, dkv_dtype,
                 stream, rope);
}

int rope_args(const char* fn, const pico_attn_desc* desc, const pico_rope_tables* rope, int q_pos_offset, int k_pos_offset,
              RopeArgs& r) {
  if (q_pos_offset < 0 || k_pos_offset < 0) return fail(PICO_ERR_SHAPE, "%s: position offsets must be >= 0", fn);
  const int64_t last = std::max(static_cast<int64_t>(q_pos_offset) + desc->Sq, static_cast<int64_t>(k_pos_offset) + desc->Sk) - 1;
  if (int rc = check_rope_tables(fn, rope, desc->D, last)) return rc;
  r = RopeArgs{rope->cos, rope->sin, rope->pitch, rope->dtype == PICO_F32, q_pos_offset, k_pos_offset};
  return PICO_OK;
}

}  // namespace

extern "C" int pico_attn_bwd(const pico_attn_desc* desc, const void* q, const void* k, const void* v, const void* dout,
                             const float* lse, const float* delta, void* dq, const int64_t* dq_stride, int dq_dtype,
                             int dq_accumulate, void* dk, void* dv, const int64_t* dkv_stride, int dkv_dtype,
                             int dkv_accumulate, void* stream) {
  if (int rc = check_attn_desc("pico_attn_bwd", desc)) return rc;
  if (dkv_accumulate && dkv_dtype != PICO_F32) return fail(PICO_ERR_DTYPE, "pico_attn_bwd: accumulate needs fp32 gradients");
  const pico_kv_chunks kv = one_chunk(desc, k, v, dk, dv, dkv_accumulate);
  return run_bwd("pico_attn_bwd", desc, q, &kv, dout, lse, delta, nullptr, nullptr, dq, dq_stride, dq_dtype, dq_accumulate,
                 dkv_stride, dkv_dtype, stream);
}

extern "C" int pico_attn_bwd_fused(const pico_attn_desc* desc, const void* q, const void* k, const void* v,
                                   const void* dout, const void* out, int out_dtype, const float* lse, float* delta,
                                   void* dq, const int64_t* dq_stride, int dq_dtype, int dq_accumulate, void* dk, void* dv,
                                   const int64_t* dkv_stride, int dkv_dtype, int dkv_accumulate, void* stream) {
  const char* fn = "pico_attn_bwd_fused";
  if (int rc = check_attn_desc(fn, desc)) return rc;
  if (dkv_accumulate && dkv_dtype != PICO_F32) return fail(PICO_ERR_DTYPE, "%s: accumulate needs fp32 gradients", fn);
  const pico_kv_chunks kv = one_chunk(desc, k, v, dk, dv, dkv_accumulate);
  return run_bwd_with_out(fn, desc, q, &kv, dout, out, out_dtype, lse, delta, dq, dq_stride, dq_dtype, dq_accumulate,
                          dkv_stride, dkv_dtype, stream, nullptr);
}

extern "C" int pico_attn_bwd_rope(const pico_attn_desc* desc, const void* q_rot, const void* k_rot, const void* v,
                                  const void* dout, const void* out, const float* lse, float* delta, void* dq,
                                  const int64_t* dq_stride, int dq_dtype, int dq_accumulate, void* dk, void* dv,
                                  const int64_t* dkv_stride, int dkv_dtype, int dkv_accumulate,
                                  const pico_rope_tables* rope, int q_pos_offset, int k_pos_offset, void* stream) {
  const char* fn = "pico_attn_bwd_rope";
  if (int rc = check_attn_desc(fn, desc)) return rc;
  if (desc->B == 0) return PICO_OK;
  RopeArgs r;
  if (int rc = rope_args(fn, desc, rope, q_pos_offset, k_pos_offset, r)) return rc;
  if (!dq || !dk || !dv) return fail(PICO_ERR_NULL, "%s: dq, dk and dv are required", fn);
  if (dkv_accumulate && dkv_dtype != PICO_F32) return fail(PICO_ERR_DTYPE, "%s: accumulate needs fp32 gradients", fn);
  const pico_kv_chunks kv = one_chunk(desc, k_rot, v, dk, dv, dkv_accumulate);
  return run_bwd_with_out(fn, desc, q_rot, &kv, dout, out, PICO_BF16, lse, delta, dq, dq_stride, dq_dtype, dq_accumulate,
                          dkv_stride, dkv_dtype, stream, &r);
}

extern "C" int pico_attn_bwd_chunks(const pico_attn_desc* desc, const void* q, const pico_kv_chunks* kv, const void* dout,
                                    const void* out, int out_dtype, const float* lse, float* delta, void* dq,
                                    const int64_t* dq_stride, int dq_dtype, int dq_accumulate, const int64_t* dkv_stride,
                                    int dkv_dtype, const pico_rope_tables* rope, int q_pos_offset, int k_pos_offset,
                                    void* stream) {
  const char* fn = "pico_attn_bwd_chunks";
  if (int rc = check_attn_desc(fn, desc)) return rc;
  if (!kv) return fail(PICO_ERR_NULL, "%s: the chunk list is NULL", fn);
  if (desc->B == 0) return PICO_OK;
  RopeArgs r;
  if (rope) {
    if (int rc = rope_args(fn, desc, rope, q_pos_offset, k_pos_offset, r)) return rc;
  }
  if (out)
    return run_bwd_with_out(fn, desc, q, kv, dout, out, out_dtype, lse, delta, dq, dq_stride, dq_dtype, dq_accumulate, dkv_stride,
                            dkv_dtype, stream, rope ? &r : nullptr);
  return run_bwd(fn, desc, q, kv, dout, lse, delta, nullptr, nullptr, dq, dq_stride, dq_dtype, dq_accumulate, dkv_stride,
                 dkv_dtype, stream, rope ? &r : nullptr);
}
