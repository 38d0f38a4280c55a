// Pieces shared by the attention forward and backward kernels (gfx950, wave64, MFMA 32x32x16 bf16).
//
// MFMA 32x32x16 operand layout (verified on hardware): lane l, half h = l / 32, n = l % 32
//   A[m][k]  : lane holds m = n, k = 8h .. 8h+7          (8 bf16)
//   B[k][n]  : lane holds n,     k = 8h .. 8h+7          (8 bf16)
//   C[m][n]  : lane holds column n, register i holds row 8*(i/4) + 4h + i%4   (16 fp32)
// The sum over k does not care which physical index sits in slot k as long as A and B agree, so a
// C tile can be fed back as the k-operand of the next MFMA straight from registers: registers
// 8c .. 8c+7 of a lane hold rows {16c + 8jj + 4h + t : jj < 2, t < 4}, and the partner operand is
// fetched with that same row order.
//
// ds_read_b64_tr_b16 (verified on hardware): within a group of 16 lanes, lane p supplies the address
// of 4 consecutive 16-bit elements; lane p receives element p%4 of lanes {p/4, 4 + p/4, 8 + p/4, 12 + p/4}.
// With lane p pointing at tile[row0 + p/4][col0 + 4*(p%4)] every lane p ends up with
// tile[row0 .. row0+3][col0 + p]: a 4-deep column of a row-major tile, which is what an MFMA operand
// needs when the contraction index is the tile's row.
#pragma once
#include "common.h"

namespace pico {

typedef __attribute__((address_space(3))) s16x4 lds_s16x4;

__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}

// 4 rows x 1 column of a row-major bf16 tile in LDS, transposed into the lane (see header comment).
// `p` must point at tile[row0 + (lane%16)/4][col0 + 4*(lane%4)].
__device__ __forceinline__ s16x4 lds_read_tr(const __bf16* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4*)(p));
}

// Two transposed reads -> the 8 k-slots of an MFMA operand.  Slots 0-3 come from rows
// row0 .. row0+3, slots 4-7 from rows row0+8 .. row0+11 (the register order of a C tile).
__device__ __forceinline__ bf16x8 lds_read_tr_pair(const __bf16* p, int ld) {
  s16x4 lo = lds_read_tr(p);
  s16x4 hi = lds_read_tr(p + 8 * ld);
  typedef __attribute__((ext_vector_type(8))) short s16x8;
  s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

// the same with the second read `step` elements after the first (tiles whose rows are not evenly spaced)
__device__ __forceinline__ bf16x8 lds_read_tr_pair_step(const __bf16* p, int step) {
  s16x4 lo = lds_read_tr(p);
  s16x4 hi = lds_read_tr(p + step);
  typedef __attribute__((ext_vector_type(8))) short s16x8;
  s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

// s_waitcnt immediate for "vmcnt(0)" with the other counters left at their maxima (gfx9 encoding:
// vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14])
constexpr int kWaitVmcnt0 = 0x0F70;

// ---- buffer loads.  A buffer resource (4 SGPRs: base, byte count) plus a 32-bit per-lane byte offset replaces
// 64-bit per-lane addresses; a lane whose offset is past the byte count reads zeros, which is how tile rows
// past the end of a sequence become zero rows without clamps or selects.
using buffer_rsrc = __amdgpu_buffer_rsrc_t;
// `bytes` is the exact size of the window: the entry points reject tensors whose rows of one head span 4 GiB or more
__device__ __forceinline__ buffer_rsrc make_buffer(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, static_cast<int>(bytes), 0x00020000);
}
// bytes from the first element of row 0 to the end of row rows-1, for rows of D bf16 elements `stride` elements apart
__device__ __forceinline__ uint32_t span_bytes(int rows, int64_t stride, int D) {
  return rows <= 0 ? 0u : static_cast<uint32_t>((static_cast<int64_t>(rows - 1) * stride + D) * 2);
}
__device__ __forceinline__ u32x4 buffer_load_b128(buffer_rsrc r, uint32_t byte_off) {
  return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>(byte_off), 0, 0));
}
__device__ __forceinline__ float buffer_load_f32(buffer_rsrc r, uint32_t byte_off) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, static_cast<int>(byte_off), 0, 0));
}

__device__ __forceinline__ bf16x8 pack8(const f32x16& c, int base) {
  bf16x8 r;
#pragma unroll
  for (int e = 0; e < 8; ++e) r[e] = static_cast<__bf16>(c[base + e]);
  return r;
}

// max / sum of a value across the two 32-lane halves of a wave (lane l with lane l^32)
__device__ __forceinline__ float half_max(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float half_sum(float v) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// ---- reading a wave's 32 x D operand tile as MFMA fragments.  Fetched straight in fragment layout (lane =
// row, 16 bytes per lane) one instruction touches 32 different lines; fetched row-major -- 16 bytes per lane,
// 8 or 16 consecutive lanes per row -- the same bytes arrive in a quarter of the line requests, and a detour
// through a 32 x (D + 8) piece of LDS private to the wave turns them into fragments: lane n gets row n % 32,
// and for k step s the elements 16s + 8h ..+7 (h = lane / 32).  Rows past the end of the window read as zeros.
template <int D>
struct WaveTile {
  static constexpr int kChunks = D / 16;                 // 16-byte pieces per lane
  static constexpr int kRegionBytes = 32 * (D + 8) * 2;
  u32x4 raw[kChunks];
  __device__ __forceinline__ void issue(buffer_rsrc window, int64_t row_stride, int lane) {
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      const int idx = lane + 64 * i, r = idx / (D / 8), cv = idx % (D / 8);
      raw[i] = buffer_load_b128(window, static_cast<uint32_t>((static_cast<int64_t>(r) * row_stride + cv * 8) * 2));
    }
  }
  __device__ __forceinline__ void fragments(unsigned char* region, int lane, bf16x8 (&frag)[D / 16]) const {
    constexpr int kPitch = (D + 8) * 2;
#pragma unroll
    for (int i = 0; i < kChunks; ++i) {
      const int idx = lane + 64 * i, r = idx / (D / 8), cv = idx % (D / 8);
      *reinterpret_cast<u32x4*>(region + r * kPitch + cv * 16) = raw[i];
    }
    const int n = lane % 32, h = lane / 32;
#pragma unroll
    for (int s = 0; s < D / 16; ++s)
      frag[s] = *reinterpret_cast<const bf16x8*>(region + n * kPitch + (16 * s + 8 * h) * 2);
  }
};

// ---- writing a wave's 32 result rows.  The accumulators of the transposed products hold, per lane, one row
// (lane % 32) and, in registers 4j..4j+3 of block db, columns 32db + 8j + 4h ..+3 (h = lane / 32).  Stored
// straight from that layout a wave would touch 32 different 128-byte lines with 8 or 16 bytes each per
// instruction; instead the rows take a detour through a 32 x 144-byte piece of LDS that belongs to the wave
// (the caller guarantees that every wave of the workgroup is done with the tile buffers) and leave as whole
// 128-byte lines, 16 bytes per lane.  One pass moves 128 bytes of every row: 32 fp32 or 64 bf16 columns.
//   dst_row0: address of column 0 of the wave's first row; row_stride in elements; rows_live rows exist.
//   accumulate (fp32 only) adds to what is there; all its reads are issued before the first write.
//   streaming marks bf16 stores non-temporal (the data is not read again by the kernels that follow soon).
constexpr int kRowRegionBytes = 32 * 144;
template <int D, bool kF32>
__device__ __forceinline__ void wave_store_rows(unsigned char* region, const f32x16 (&acc)[D / 32], float scale,
                                                void* dst_row0, int64_t row_stride, int rows_live, int lane,
                                                bool accumulate, bool streaming) {
  constexpr int kPitch = 144;
  constexpr int kColsPerPass = kF32 ? 32 : 64;
  const int n = lane % 32, h = lane / 32;
#pragma unroll
  for (int c0 = 0; c0 < D; c0 += kColsPerPass) {
#pragma unroll
    for (int db = c0 / 32; db < (c0 + kColsPerPass) / 32; ++db)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int col = 32 * db + 8 * j + 4 * h - c0;
        if constexpr (kF32) {
          f32x4 v4;
#pragma unroll
          for (int t = 0; t < 4; ++t) v4[t] = acc[db][4 * j + t] * scale;
          *reinterpret_cast<f32x4*>(region + n * kPitch + col * 4) = v4;
        } else {
          bf16x4 v4;
#pragma unroll
          for (int t = 0; t < 4; ++t) v4[t] = static_cast<__bf16>(acc[db][4 * j + t] * scale);
          *reinterpret_cast<bf16x4*>(region + n * kPitch + col * 2) = v4;
        }
      }
    // 32 rows x 8 pieces of 16 bytes = 4 pieces per lane; 8 consecutive lanes cover one row's line
    unsigned char* g[4];
    u32x4 v[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int idx = lane + 64 * t, r = idx / 8, ch = idx % 8;
      v[t] = *reinterpret_cast<const u32x4*>(region + r * kPitch + ch * 16);
      g[t] = r < rows_live ? static_cast<unsigned char*>(dst_row0) +
                                 (static_cast<int64_t>(r) * row_stride + c0) * (kF32 ? 4 : 2) + ch * 16
                           : nullptr;
    }
    if constexpr (kF32) {
      f32x4 old[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) old[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (accumulate) {
#pragma unroll
        for (int t = 0; t < 4; ++t)
          if (g[t]) old[t] = *reinterpret_cast<const f32x4*>(g[t]);
      }
#pragma unroll
      for (int t = 0; t < 4; ++t)
        if (g[t]) *reinterpret_cast<f32x4*>(g[t]) = __builtin_bit_cast(f32x4, v[t]) + old[t];
    } else {
#pragma unroll
      for (int t = 0; t < 4; ++t)
        if (g[t]) {
          if (streaming) __builtin_nontemporal_store(v[t], reinterpret_cast<u32x4*>(g[t]));
          else *reinterpret_cast<u32x4*>(g[t]) = v[t];
        }
    }
  }
}

// The same rows as the sum of an fp32 buffer and the accumulators, rounded once to bf16 and written somewhere else:
// the last block of a ring adds itself to the travelling fp32 sums (`old_row0`, nullptr: nothing to add) and hands
// the total back in the dtype of the inputs.  32 columns per pass (fp32 staging), 8-byte bf16 pieces per lane.
template <int D>
__device__ __forceinline__ void wave_store_rows_total(unsigned char* region, const f32x16 (&acc)[D / 32], float scale,
                                                      const float* old_row0, int64_t old_stride, __bf16* dst_row0,
                                                      int64_t dst_stride, int rows_live, int lane) {
  constexpr int kPitch = 144;
  const int n = lane % 32, h = lane / 32;
#pragma unroll
  for (int c0 = 0; c0 < D; c0 += 32) {
    const int db = c0 / 32;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f32x4 v4;
#pragma unroll
      for (int t = 0; t < 4; ++t) v4[t] = acc[db][4 * j + t] * scale;
      *reinterpret_cast<f32x4*>(region + n * kPitch + (8 * j + 4 * h) * 4) = v4;
    }
    f32x4 v[4], old[4];
    int row[4], piece[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int idx = lane + 64 * t;
      row[t] = idx / 8;
      piece[t] = idx % 8;
      v[t] = *reinterpret_cast<const f32x4*>(region + row[t] * kPitch + piece[t] * 16);
      old[t] = f32x4{0.f, 0.f, 0.f, 0.f};
      if (old_row0 != nullptr && row[t] < rows_live)
        old[t] = *reinterpret_cast<const f32x4*>(old_row0 + static_cast<int64_t>(row[t]) * old_stride + c0 + piece[t] * 4);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t)
      if (row[t] < rows_live) {
        bf16x4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = static_cast<__bf16>(v[t][e] + old[t][e]);
        __builtin_nontemporal_store(__builtin_bit_cast(u32x2, o),
                                    reinterpret_cast<u32x2*>(dst_row0 + static_cast<int64_t>(row[t]) * dst_stride + c0 + piece[t] * 4));
      }
  }
}

// ---- RoPE inside the attention kernels (non-interleaved: column d pairs with d + D/2; model.py:12-19).
// Tables are [rows, >= D/2 columns] with `pitch` elements between rows, bf16 or fp32; row index = position.
struct RopeArgs {
  const void* cos;   // nullptr: no rotation
  const void* sin;
  int64_t pitch;
  int f32;
  int q_pos0, k_pos0;   // position of query row 0 / key row 0
};
// n (4 or 8) consecutive table entries starting at column `col` of row `pos`
template <int N>
__device__ __forceinline__ void rope_load(const RopeArgs& r, const void* table, int pos, int col, float (&out)[N]) {
  if (r.f32) {
    const float* t = static_cast<const float*>(table) + static_cast<int64_t>(pos) * r.pitch + col;
#pragma unroll
    for (int e = 0; e < N; e += 4) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(t + e);
#pragma unroll
      for (int u = 0; u < 4; ++u) out[e + u] = v[u];
    }
  } else {
    const __bf16* t = static_cast<const __bf16*>(table) + static_cast<int64_t>(pos) * r.pitch + col;
#pragma unroll
    for (int e = 0; e < N; e += 4) {
      const u32x2 v = *reinterpret_cast<const u32x2*>(t + e);
      out[e] = __uint_as_float(v[0] << 16);  out[e + 1] = __uint_as_float(v[0] & 0xffff0000u);
      out[e + 2] = __uint_as_float(v[1] << 16);  out[e + 3] = __uint_as_float(v[1] & 0xffff0000u);
    }
  }
}
// Rotates a lane's operand fragments in place: fragment s holds columns 16 s + 8 h ..+7 of the lane's row, its partner
// (column + D/2) is fragment s + D/32.  fp32 arithmetic, one rounding, the formula of the stand-alone kernel.
template <int D>
__device__ __forceinline__ void rope_rotate_fragments(bf16x8 (&f)[D / 16], const RopeArgs& r, int pos, int h) {
#pragma unroll
  for (int s = 0; s < D / 32; ++s) {
    float c[8], sn[8];
    rope_load<8>(r, r.cos, pos, 16 * s + 8 * h, c);
    rope_load<8>(r, r.sin, pos, 16 * s + 8 * h, sn);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float lo = static_cast<float>(f[s][e]), hi = static_cast<float>(f[s + D / 32][e]);
      f[s][e] = static_cast<__bf16>(lo * c[e] - hi * sn[e]);
      f[s + D / 32][e] = static_cast<__bf16>(hi * c[e] + lo * sn[e]);
    }
  }
}
// Un-rotates (rotation by the negative angle: the backward of RoPE) a lane's row of a transposed-product accumulator:
// registers 4j..4j+3 of block db hold columns 32 db + 8 j + 4 h ..+3; the partner of block db is block db + D/64.
template <int D>
__device__ __forceinline__ void rope_unrotate_acc(f32x16 (&acc)[D / 32], const RopeArgs& r, int pos, int h) {
#pragma unroll
  for (int db = 0; db < D / 64; ++db)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float c[4], sn[4];
      rope_load<4>(r, r.cos, pos, 32 * db + 8 * j + 4 * h, c);
      rope_load<4>(r, r.sin, pos, 32 * db + 8 * j + 4 * h, sn);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const float lo = acc[db][4 * j + t], hi = acc[db + D / 64][4 * j + t];
        acc[db][4 * j + t] = lo * c[t] + hi * sn[t];
        acc[db + D / 64][4 * j + t] = hi * c[t] - lo * sn[t];
      }
    }
}

// K / V as a list of equally long chunks that lie one after another along the key axis: key j of the launch is row
// j % len of chunk j / len.  One chunk of len = Sk is the plain case.  With several chunks len is a multiple of every
// kernel's staged key tile (128), so no tile straddles two chunks.
constexpr int kMaxChunks = PICO_MAX_KV_CHUNKS;
struct KvChunks {
  const __bf16* k[kMaxChunks];
  const __bf16* v[kMaxChunks];
  int count, len;
};

struct AttnParams {
  const __bf16* q;
  KvChunks kv;
  int B, Hq, Hkv, Sq, Sk;
  int causal, q_offset;
  float sm_scale;
  int64_t qs[3], ks[3], vs[3], os[3];
};

// A cursor over the key tiles of KT keys, in order, across the chunks: wave-uniform, so it lives in scalar registers;
// stepping inside a chunk is four adds, a new chunk re-reads its base addresses from the kernel arguments.
template <int D>
struct KvCursor {
  const char *k, *v;            // first row of the next tile
  uint32_t k_left, v_left;      // bytes from there to the end of the chunk's rows of this head
  uint32_t k_step, v_step;
  int tiles_left, chunk, tiles_per_chunk;
  int64_t k_head, v_head;       // element offset of the (batch, kv head) inside every chunk
  __device__ __forceinline__ void open(const AttnParams& a, int chunk_, int b, int hkv, int KT) {
    chunk = chunk_;
    k_head = b * a.ks[0] + hkv * a.ks[1];
    v_head = b * a.vs[0] + hkv * a.vs[1];
    k_step = static_cast<uint32_t>(KT * a.ks[2] * 2);
    v_step = static_cast<uint32_t>(KT * a.vs[2] * 2);
    tiles_per_chunk = (a.kv.len + KT - 1) / KT;
    enter(a);
  }
  __device__ __forceinline__ void enter(const AttnParams& a) {
    k = reinterpret_cast<const char*>(a.kv.k[chunk] + k_head);
    v = reinterpret_cast<const char*>(a.kv.v[chunk] + v_head);
    k_left = span_bytes(a.kv.len, a.ks[2], D);
    v_left = span_bytes(a.kv.len, a.vs[2], D);
    tiles_left = tiles_per_chunk;
  }
  __device__ __forceinline__ void next(const AttnParams& a) {
    if (--tiles_left == 0 && chunk + 1 < a.kv.count) {
      ++chunk;
      enter(a);
    } else {
      k += k_step;  k_left -= k_step;
      v += v_step;  v_left -= v_step;
    }
  }
};

int check_attn_desc(const char* fn, const pico_attn_desc* d);
// tables usable for head_dim D and positions 0 .. last_pos?
int check_rope_tables(const char* fn, const pico_rope_tables* t, int D, int64_t last_pos);
// one chunk of d->Sk keys
AttnParams make_params(const pico_attn_desc* d, const void* q, const void* k, const void* v);
// the chunk list checked against the descriptor (count, length, tile multiple, alignment; with need_kv also that no
// k / v pointer is NULL) and copied into `a`
int set_chunks(const char* fn, const pico_attn_desc* d, const pico_kv_chunks* kv, AttnParams& a, bool need_kv);

}  // namespace pico
