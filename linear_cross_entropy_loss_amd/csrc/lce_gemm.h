// Shared MFMA tile machinery for the gfx950 kernels of the fused
// linear + cross-entropy operator.
//
// Every heavy kernel here is the same contraction
//     D[p][q] = sum_k P[p][k] * Q[q][k]
// on a 256 x 256 output tile with a 64-deep K step, computed by
// v_mfma_f32_32x32x16 (bf16 or f16 operands, fp32 accumulate).  P is the MFMA
// "A" operand, so the P index of D runs along accumulator registers (four
// consecutive p per register quad); Q is the "B" operand, so the Q index runs
// along lanes (q = lane % 32).  Kernels choose P/Q so that the quantity they
// reduce or store contiguously lies along P.
//
// An operand tile is staged in LDS in one of two layouts:
//   KC  source is K-contiguous  ([rows][k]); fragments are read with
//       ds_read_b128 (8 consecutive k per lane).
//   MC  source is row-contiguous along the P/Q index ([k][cols]); fragments
//       are read with ds_read_b64_tr_b16, the gfx950 LDS transpose load,
//       which hands each lane 4 consecutive k for its column.
// Both layouts are XOR-swizzled so that neither the 16-byte stores that fill
// them nor the fragment reads collide on LDS banks.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lce {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) short s16x4_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4_t;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2_t;

#define LCE_DEV __device__ __forceinline__
#define LCE_LDS(T) __attribute__((address_space(3))) T

constexpr int kTile = 256;     // output tile edge (both P and Q)
constexpr int kBK = 64;        // K depth of one LDS stage
constexpr int kThreads = 256;  // 4 waves, 2 x 2, each owning a 128 x 128 sub-tile
constexpr int kWaveTile = 128;
constexpr int kBlk = 32;                 // MFMA block edge
constexpr int kNB = kWaveTile / kBlk;    // 4 blocks per wave per dimension
constexpr int kTileBytes = kTile * kBK * 2;        // 32 KiB per operand per stage
constexpr int kStageBytes = 2 * kTileBytes;        // P + Q
constexpr int kMainloopLds = 2 * kStageBytes;      // double buffered: 128 KiB

struct BF16 {};
struct F16 {};

template <class T> struct elem_of;
template <> struct elem_of<BF16> { typedef __bf16 type; };
template <> struct elem_of<F16> { typedef _Float16 type; };

template <class T> LCE_DEV f32x16_t mfma32(s16x8_t a, s16x8_t b, f32x16_t c);
template <> LCE_DEV f32x16_t mfma32<BF16>(s16x8_t a, s16x8_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                 __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}
template <> LCE_DEV f32x16_t mfma32<F16>(s16x8_t a, s16x8_t b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

// float -> 16-bit compute type, round to nearest even, returned as raw bits.
template <class T> LCE_DEV unsigned short to_bits(float f) {
  typename elem_of<T>::type h = (typename elem_of<T>::type)f;
  return __builtin_bit_cast(unsigned short, h);
}
// Two floats -> one dword of the 16-bit type (a single v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32).
template <class T> LCE_DEV unsigned int pack2(float lo, float hi) {
  typedef float f32x2_t __attribute__((ext_vector_type(2)));
  typedef typename elem_of<T>::type e2_t __attribute__((ext_vector_type(2)));
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(unsigned int, __builtin_convertvector(v, e2_t));
}
// fp32 operands are carried as two bf16 numbers, v = hi + lo with hi = bf16(v) and lo = bf16(v - hi): 16
// bits of mantissa instead of 8.  A product a*b is then taken as a_hi*b_hi + a_hi*b_lo + a_lo*b_hi (the
// a_lo*b_lo term is of relative order 2^-18 and dropped), which the kernels get by running along a K axis
// that is three times as long, over copies of the operands laid out as [hi | hi | lo] and [hi | lo | hi].
LCE_DEV float bf16_hi(float v) {
  return __builtin_bit_cast(float, (unsigned)to_bits<BF16>(v) << 16);
}
LCE_DEV float bf16_lo(float v) { return v - bf16_hi(v); }  // exact in fp32; rounded to bf16 when stored

// threadIdx.x behind an optimisation barrier.  Epilogues that run inside a
// persistent tile loop derive their per-lane indices from this, so that the
// compiler recomputes them per tile instead of hoisting them out of the loop
// and keeping them alive (in scarce vector registers) across the main loop.
LCE_DEV int opaque_tid() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// ---------------------------------------------------------------------------
// Workgroup -> tile mapping.  Workgroups are dealt round-robin to the 8 XCDs,
// each with its own L2, so consecutive ids are first regrouped per XCD and
// then walked in bands of `band` P-tiles with Q fastest: the 32 workgroups an
// XCD runs at a time then cover a compact (band x 32/band) patch of tiles.
//
// `live`: how many bands the 8 XCDs work on at the same time.  8 (the plain regrouping: every XCD walks its
// own eighth of the ids, so each is in a band of its own) keeps 8 P bands in flight; each is re-read once
// per round from the 256 MB Infinity Cache, and with a long K they no longer fit there together (a band of
// 8 P-tiles is 32 MiB at K = 8192: the forward ran 7 % slower on 128 vocabulary tiles than on 32).  With
// live = 4, 2 or 1 the bands are taken `live` at a time and 8 / live XCDs share a band, each walking its own
// part of the band's Q range.  Needs tiles_p to be a multiple of band * live (else the plain regrouping).
// ---------------------------------------------------------------------------
LCE_DEV void tile_coords(int bid, int nblocks, int tiles_p, int tiles_q, int band, int live, int& tp, int& tq) {
  int id = bid;
  if ((nblocks & 7) == 0) {
    const int xcd = bid & 7, seq = bid >> 3;
    if (live >= 8 || tiles_p % (band * live) != 0) {
      id = xcd * (nblocks >> 3) + seq;
    } else {
      const int per = 8 / live;                      // XCDs per band
      const int band_ids = band * tiles_q;
      const int share = band_ids / per;              // ids of a band that one XCD walks (band * tiles_q * live / 8)
      const int step = seq / share, r = seq - step * share;
      id = (step * live + xcd / per) * band_ids + (xcd % per) * share + r;
    }
  }
  const int per_band = band * tiles_q;
  const int b = id / per_band;
  const int within = id - b * per_band;
  const int p0 = b * band;
  const int rem = tiles_p - p0;
  const int width = rem < band ? rem : band;
  tq = within / width;
  tp = p0 + (within - tq * width);
}

// ---------------------------------------------------------------------------
// Fragment readers: per-lane LDS offsets for the four 32-wide blocks of this
// wave's 128-wide slice of an operand tile.
// ---------------------------------------------------------------------------
template <bool KC> struct FragReader;

template <> struct FragReader<true> {
  int off[4];  // byte offset per k-step (block 0); blocks add 32 rows = 4096 bytes
  LCE_DEV void init(int wave_off /* first row of the wave's slice */) {
    const int l = threadIdx.x & 63;
    const int r = l & 31;
    const int sw = (r & 7) ^ ((r >> 3) & 1);
    const int t0 = (l >> 5) ^ sw;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) off[ks] = (wave_off + r) * 128 + (((2 * ks) ^ t0) << 4);
  }
  LCE_DEV s16x8_t read(const char* tile, int blk, int ks) const {
    return *reinterpret_cast<const s16x8_t*>(tile + off[ks] + blk * 4096);
  }
};

template <> struct FragReader<false> {
  int off[4];  // byte offset per block at k-step 0, first half
  LCE_DEV void init(int wave_off /* first column of the wave's slice */) {
    const int l = threadIdx.x & 63;
    const int g = l >> 4, s = l & 15, j = s >> 2, c = s & 3;
    const int mask = ((j & 1) << 7) | ((j >> 1) << 6) | ((j & 1) << 5);
    const int krow = 8 * (g >> 1) + j;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const int colbyte = (wave_off + b * 32 + 16 * (g & 1) + 4 * c) * 2;
      off[b] = krow * 512 + (colbyte ^ mask);
    }
  }
  LCE_DEV s16x8_t read(const char* tile, int blk, int ks) const {
    const char* p = tile + off[blk] + ks * (16 * 512);
    const s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LCE_LDS(s16x4_t)*)(p));
    const s16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LCE_LDS(s16x4_t)*)(p + 4 * 512));
    s16x8_t v;
    v[0] = lo[0]; v[1] = lo[1]; v[2] = lo[2]; v[3] = lo[3];
    v[4] = hi[0]; v[5] = hi[1]; v[6] = hi[2]; v[7] = hi[3];
    return v;
  }
};

// Accumulator layout shared by all kernels: the wave at (wp, wq) of the 2 x 2 wave
// grid owns P rows [wp*128, +128) and Q rows [wq*128, +128) of the tile, and
// element r of block (pb, qb) in lane l is
//     p = wp*128 + pb*32 + 8*(r/4) + 4*(l/32) + r%4,   q = wq*128 + qb*32 + l%32.

}  // namespace lce
