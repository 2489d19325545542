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
template <class T> LCE_DEV unsigned int pack2(float lo, float hi) {
  return (unsigned int)to_bits<T>(lo) | ((unsigned int)to_bits<T>(hi) << 16);
}
// threadIdx.x behind an optimisation barrier.  Epilogues that run inside a
// persistent tile loop derive their per-lane indices from this, so that the
// compiler recomputes them per tile instead of hoisting them out of the loop
// and keeping them alive (in scarce vector registers) across the main loop.
LCE_DEV int opaque_tid() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// Bit pattern -> float.  Takes the word by value on purpose: bit-casting a
// vector element expression directly reads element 0 for every index.
LCE_DEV float as_f32(unsigned int u) { return __builtin_bit_cast(float, u); }

// ---------------------------------------------------------------------------
// Workgroup -> tile mapping.  Workgroups are dealt round-robin to the 8 XCDs,
// each with its own L2, so consecutive ids are first regrouped per XCD and
// then walked in bands of `band` P-tiles with Q fastest: the 32 workgroups an
// XCD runs at a time then cover a compact (band x 32/band) patch of tiles.
// ---------------------------------------------------------------------------
LCE_DEV void tile_coords(int bid, int nblocks, int tiles_p, int tiles_q, int band, int& tp, int& tq) {
  int id = bid;
  if ((nblocks & 7) == 0) id = (bid & 7) * (nblocks >> 3) + (bid >> 3);
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
// Global -> register -> LDS staging of one operand tile.
// SrcT is the element type in memory: 2 bytes (already the compute type) or
// float (converted to the compute type on the way into LDS).
// ---------------------------------------------------------------------------
template <class T, class SrcT, bool KC> struct TileStager {
  static constexpr bool kWide = sizeof(SrcT) == 4;
  // 16-byte chunks of 8 compute elements; 2048 chunks per tile, 8 per thread.
  static constexpr int kIter = kTile * kBK / 8 / kThreads;
  u32x4_t raw[kIter * (kWide ? 2 : 1)];
  const SrcT* gptr;     // this thread's first chunk of the current K tile
  int64_t iter_stride;  // elements between this thread's consecutive chunks
  int64_t k_stride;     // elements between consecutive K tiles
  int lds_off;          // byte offset of the first chunk inside the operand tile

  // origin: element (row0, k=0) for KC, (k=0, col0) for MC; ld = row stride.
  LCE_DEV void init(const SrcT* origin, int64_t ld) {
    const int t = threadIdx.x;
    if (KC) {
      const int c = t & 7, r = t >> 3;  // 8 chunks per 64-element row, 32 rows per pass
      gptr = origin + (int64_t)r * ld + c * 8;
      iter_stride = 32 * ld;
      k_stride = kBK;
      const int sw = (r & 7) ^ ((r >> 3) & 1);
      lds_off = r * 128 + ((c ^ sw) << 4);
    } else {
      const int c = t & 31, k = t >> 5;  // 32 chunks per 256-element row, 8 k-rows per pass
      gptr = origin + (int64_t)k * ld + c * 8;
      iter_stride = 8 * ld;
      k_stride = kBK * ld;
      const int j = k & 3;
      const int mask = ((j & 1) << 7) | ((j >> 1) << 6) | ((j & 1) << 5);
      lds_off = k * 512 + ((c << 4) ^ mask);
    }
  }
  LCE_DEV void load() {
#pragma unroll
    for (int i = 0; i < kIter; ++i) {
      const u32x4_t* p = reinterpret_cast<const u32x4_t*>(gptr + i * iter_stride);
      if (kWide) {
        raw[2 * i] = p[0];
        raw[2 * i + 1] = p[1];
      } else {
        raw[i] = p[0];
      }
    }
    gptr += k_stride;
  }
  LCE_DEV void store(char* tile) const {
    constexpr int step = KC ? 32 * 128 : 8 * 512;
#pragma unroll
    for (int i = 0; i < kIter; ++i) {
      u32x4_t v;
      if (kWide) {
        const u32x4_t a = raw[2 * i], b = raw[2 * i + 1];
        v[0] = pack2<T>(as_f32(a[0]), as_f32(a[1]));
        v[1] = pack2<T>(as_f32(a[2]), as_f32(a[3]));
        v[2] = pack2<T>(as_f32(b[0]), as_f32(b[1]));
        v[3] = pack2<T>(as_f32(b[2]), as_f32(b[3]));
      } else {
        v = raw[i];
      }
      *reinterpret_cast<u32x4_t*>(tile + lds_off + i * step) = v;
    }
  }
};

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

// ---------------------------------------------------------------------------
// Main loop: acc[pb][qb] += P-block x Q-block over `ktiles` K tiles.
// The wave at (wp, wq) of the 2 x 2 wave grid owns P rows [wp*128, +128) and
// Q rows [wq*128, +128) of the tile.  Accumulator element r of block
// (pb, qb) in lane l is
//     p = wp*128 + pb*32 + 8*(r/4) + 4*(l/32) + r%4,   q = wq*128 + qb*32 + l%32.
// ---------------------------------------------------------------------------
template <class T, class PSrc, bool P_KC, class QSrc, bool Q_KC>
LCE_DEV void gemm_mainloop(f32x16_t (&acc)[kNB][kNB], const PSrc* p_origin, int64_t ldp,
                           const QSrc* q_origin, int64_t ldq, int ktiles, char* lds) {
  const int wave = threadIdx.x >> 6;
  const int wp = wave & 1, wq = wave >> 1;

  TileStager<T, PSrc, P_KC> ps;
  TileStager<T, QSrc, Q_KC> qs;
  ps.init(p_origin, ldp);
  qs.init(q_origin, ldq);
  FragReader<P_KC> pr;
  FragReader<Q_KC> qr;
  pr.init(wp * kWaveTile);
  qr.init(wq * kWaveTile);

#pragma unroll
  for (int i = 0; i < kNB; ++i)
#pragma unroll
    for (int j = 0; j < kNB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  ps.load();
  qs.load();
  ps.store(lds);
  qs.store(lds + kTileBytes);
  __syncthreads();

  for (int kt = 0; kt < ktiles; ++kt) {
    const char* cur = lds + (kt & 1) * kStageBytes;
    char* nxt = lds + ((kt + 1) & 1) * kStageBytes;
    const bool more = kt + 1 < ktiles;
    if (more) {
      ps.load();
      qs.load();
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      s16x8_t pf[kNB], qf[kNB];
#pragma unroll
      for (int b = 0; b < kNB; ++b) pf[b] = pr.read(cur, b, ks);
#pragma unroll
      for (int b = 0; b < kNB; ++b) qf[b] = qr.read(cur + kTileBytes, b, ks);
#pragma unroll
      for (int i = 0; i < kNB; ++i)
#pragma unroll
        for (int j = 0; j < kNB; ++j) acc[i][j] = mfma32<T>(pf[i], qf[j], acc[i][j]);
    }
    if (more) {
      ps.store(nxt);
      qs.store(nxt + kTileBytes);
    }
    __syncthreads();
  }
}

}  // namespace lce
