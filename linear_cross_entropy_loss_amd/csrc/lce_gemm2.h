// Software-pipelined main loop for 16-bit operands (both tiles already in the
// compute type in memory).
//
// Compared with gemm_mainloop (lce_gemm.h), which it matches bit for bit:
//   * two register staging sets keep two K tiles of global loads in flight, so
//     a load has about 1.5 iterations (~3000 cycles) to arrive;
//   * the LDS store of tile t+1 and the global loads of tile t+3 are issued
//     between the MFMAs of tile t instead of after them;
//   * MFMA fragments are double buffered: the reads for k-step s+1 are issued
//     before the MFMAs of step s, and the reads for the next tile's first step
//     are issued right after the (single) barrier, under the last 8 MFMAs;
//   * the loop is unrolled by two so that the staging set and the LDS stage are
//     compile-time constants, and sched_group_barrier pins the interleaving.
#pragma once

#include "lce_gemm.h"

namespace lce {

// 8 x 16-byte chunks per thread per operand tile.
struct StageRegs {
  u32x4_t v[8];
};

// Operand tiles are fetched with buffer loads: the resource descriptor (in
// SGPRs) points at the current K tile, each thread contributes one 32-bit byte
// offset, and the stride between a thread's 8 chunks is a scalar offset, so a
// load costs one instruction and no address arithmetic in vector registers.
template <bool KC> struct Stager2 {
  const char* base;     // uniform: first byte of the current K tile of this operand
  unsigned voff;        // per-thread byte offset of its first chunk
  unsigned iter_stride; // uniform: bytes between this thread's consecutive chunks
  int64_t k_stride;     // bytes between consecutive K tiles
  int lds_off;          // per-thread byte offset of chunk 0 inside the operand tile

  LCE_DEV void init(const void* origin, int64_t ld) {
    const int t = threadIdx.x;
    base = reinterpret_cast<const char*>(origin);
    if (KC) {
      const int c = t & 7, r = t >> 3;
      voff = (unsigned)(((int64_t)r * ld + c * 8) * 2);
      iter_stride = (unsigned)(32 * ld * 2);
      k_stride = kBK * 2;
      const int sw = (r & 7) ^ ((r >> 3) & 1);
      lds_off = r * 128 + ((c ^ sw) << 4);
    } else {
      const int c = t & 31, k = t >> 5;
      voff = (unsigned)(((int64_t)k * ld + c * 8) * 2);
      iter_stride = (unsigned)(8 * ld * 2);
      k_stride = (int64_t)kBK * ld * 2;
      const int j = k & 3;
      const int mask = ((j & 1) << 7) | ((j >> 1) << 6) | ((j & 1) << 5);
      lds_off = k * 512 + ((c << 4) ^ mask);
    }
  }
  // chunks [i0, i1) of the current K tile; advance() moves on to the next tile
  LCE_DEV void load(StageRegs& r, int i0 = 0, int i1 = 8) const {
    // 0x00020000: raw 32-bit data format; the range check is left wide open
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base), 0, 0x7fffffff, 0x00020000);
#pragma unroll
    for (int i = i0; i < i1; ++i)
      r.v[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff, (int)(i * iter_stride), 0);
  }
  LCE_DEV void advance() { base += k_stride; }
  LCE_DEV void store(const StageRegs& r, char* tile, int i0 = 0, int i1 = 8) const {
    constexpr int step = KC ? 32 * 128 : 8 * 512;
#pragma unroll
    for (int i = i0; i < i1; ++i) *reinterpret_cast<u32x4_t*>(tile + lds_off + i * step) = r.v[i];
  }
};

// scheduling-group masks of __builtin_amdgcn_sched_group_barrier
#define LCE_SG_MFMA 0x008
#define LCE_SG_VMEM_RD 0x020
#define LCE_SG_DS_RD 0x100
#define LCE_SG_DS_WR 0x200

template <class T, bool P_KC, bool Q_KC> struct Pipe2 {
  Stager2<P_KC> ps;
  Stager2<Q_KC> qs;
  FragReader<P_KC> pr;
  FragReader<Q_KC> qr;
  s16x8_t pf[2][kNB], qf[2][kNB];
  char* lds;

  static constexpr int kPReads = P_KC ? 4 : 8;  // LDS read instructions per k-step per operand
  static constexpr int kQReads = Q_KC ? 4 : 8;

  LCE_DEV void read_frags(int buf, const char* stage, int ks) {
#pragma unroll
    for (int b = 0; b < kNB; ++b) pf[buf][b] = pr.read(stage, b, ks);
#pragma unroll
    for (int b = 0; b < kNB; ++b) qf[buf][b] = qr.read(stage + kTileBytes, b, ks);
  }
  LCE_DEV void mfma_rows(f32x16_t (&acc)[kNB][kNB], int buf, int i0, int i1) {
#pragma unroll
    for (int i = i0; i < i1; ++i)
#pragma unroll
      for (int j = 0; j < kNB; ++j) acc[i][j] = mfma32<T>(pf[buf][i], qf[buf][j], acc[i][j]);
  }

  // Chunks 0..7 of a staged K tile belong to P, 8..15 to Q.
  LCE_DEV void store_chunks(const StageRegs& sp, const StageRegs& sq, char* stage, int c0, int c1) {
    if (c0 < 8) ps.store(sp, stage, c0, c1 < 8 ? c1 : 8);
    if (c1 > 8) qs.store(sq, stage + kTileBytes, c0 > 8 ? c0 - 8 : 0, c1 - 8);
  }
  LCE_DEV void load_chunks(StageRegs& sp, StageRegs& sq, int c0, int c1) {
    if (c0 < 8) ps.load(sp, c0, c1 < 8 ? c1 : 8);
    if (c1 > 8) qs.load(sq, c0 > 8 ? c0 - 8 : 0, c1 - 8);
  }

  // One K tile.  STAGE = LDS stage holding this tile; the staging set passed in
  // holds tile t+1 (written to the other stage here when WRITE) and is refilled
  // with tile t+3 (when LOAD).  NEXT: another tile follows (barrier + fragment
  // prefetch).  All four waves leave a barrier in lockstep, so LDS stores and
  // global loads are spread over the k-steps instead of being issued in one
  // burst that would oversubscribe the LDS port.
  template <int STAGE, bool WRITE, bool LOAD, bool NEXT>
  LCE_DEV void tile(f32x16_t (&acc)[kNB][kNB], StageRegs& sp, StageRegs& sq) {
    const char* cur = lds + STAGE * kStageBytes;
    char* nxt = lds + (STAGE ^ 1) * kStageBytes;
    constexpr int kReads = kPReads + kQReads;

    // k-step 0: MFMAs on buffer 0, fragment reads for step 1, LDS stores 0..5 of tile t+1
    read_frags(1, cur, 1);
    if (WRITE) store_chunks(sp, sq, nxt, 0, 6);
    mfma_rows(acc, 0, 0, kNB);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      __builtin_amdgcn_sched_group_barrier(LCE_SG_MFMA, 1, 0);
      if (i < kReads) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_RD, 1, 0);
      if (WRITE && i >= 4 && i < 16 && (i & 1) == 0) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_WR, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);

    // k-step 1: MFMAs on buffer 1, reads for step 2, stores 6..10, global loads 0..5 of tile t+3
    read_frags(0, cur, 2);
    if (WRITE) store_chunks(sp, sq, nxt, 6, 11);
    if (LOAD) load_chunks(sp, sq, 0, 6);
    mfma_rows(acc, 1, 0, kNB);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      __builtin_amdgcn_sched_group_barrier(LCE_SG_MFMA, 1, 0);
      if (i < kReads) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_RD, 1, 0);
      if (WRITE && i >= 1 && i < 11 && (i & 1) == 1) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_WR, 1, 0);
      if (LOAD && i >= 4 && (i & 1) == 0) __builtin_amdgcn_sched_group_barrier(LCE_SG_VMEM_RD, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);

    // k-step 2: MFMAs on buffer 0, reads for step 3, stores 11..15, global loads 6..10
    read_frags(1, cur, 3);
    if (WRITE) store_chunks(sp, sq, nxt, 11, 16);
    if (LOAD) load_chunks(sp, sq, 6, 11);
    mfma_rows(acc, 0, 0, kNB);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      __builtin_amdgcn_sched_group_barrier(LCE_SG_MFMA, 1, 0);
      if (i < kReads) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_RD, 1, 0);
      if (WRITE && i >= 1 && i < 11 && (i & 1) == 1) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_WR, 1, 0);
      if (LOAD && i >= 6 && (i & 1) == 0) __builtin_amdgcn_sched_group_barrier(LCE_SG_VMEM_RD, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);

    // k-step 3: first half of the MFMAs with global loads 11..15, barrier, reads for the next
    // tile's step 0, second half
    if (LOAD) {
      load_chunks(sp, sq, 11, 16);
      ps.advance();
      qs.advance();
    }
    mfma_rows(acc, 1, 0, kNB / 2);
    if (LOAD) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        __builtin_amdgcn_sched_group_barrier(LCE_SG_MFMA, 1, 0);
        if (i < 5) __builtin_amdgcn_sched_group_barrier(LCE_SG_VMEM_RD, 1, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
    if (NEXT) {
      __syncthreads();
      read_frags(0, nxt, 0);
    }
    mfma_rows(acc, 1, kNB / 2, kNB);
    if (NEXT) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        __builtin_amdgcn_sched_group_barrier(LCE_SG_MFMA, 1, 0);
        if (i < 4) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_RD, (kReads + 3) / 4, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
};

// Same contract as gemm_mainloop; ktiles must be a multiple of 4 (it is: every
// contraction length here is a multiple of 256).
template <class T, class PSrc, bool P_KC, class QSrc, bool Q_KC>
LCE_DEV void gemm_mainloop2(f32x16_t (&acc)[kNB][kNB], const PSrc* p_origin, int64_t ldp,
                            const QSrc* q_origin, int64_t ldq, int ktiles, char* lds) {
  static_assert(sizeof(PSrc) == 2 && sizeof(QSrc) == 2, "16-bit operands only");
  const int wave = threadIdx.x >> 6;
  const int wp = wave & 1, wq = wave >> 1;

  Pipe2<T, P_KC, Q_KC> pipe;
  pipe.lds = lds;
  pipe.ps.init(p_origin, ldp);
  pipe.qs.init(q_origin, ldq);
  pipe.pr.init(wp * kWaveTile);
  pipe.qr.init(wq * kWaveTile);

#pragma unroll
  for (int i = 0; i < kNB; ++i)
#pragma unroll
    for (int j = 0; j < kNB; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  StageRegs p0, q0, p1, q1;  // set 0 stages even tiles, set 1 odd tiles
  pipe.ps.load(p0);
  pipe.qs.load(q0);
  pipe.ps.advance();
  pipe.qs.advance();
  pipe.ps.load(p1);
  pipe.qs.load(q1);
  pipe.ps.advance();
  pipe.qs.advance();
  pipe.ps.store(p0, lds);
  pipe.qs.store(q0, lds + kTileBytes);
  pipe.ps.load(p0);  // tile 2
  pipe.qs.load(q0);
  pipe.ps.advance();
  pipe.qs.advance();
  __syncthreads();
  pipe.read_frags(0, lds, 0);

  // steady state: tiles t and t+1, all with a successor to write (t+1) and one to load (t+3)
  int t = 0;
  for (; t < ktiles - 4; t += 2) {
    pipe.template tile<0, true, true, true>(acc, p1, q1);
    pipe.template tile<1, true, true, true>(acc, p0, q0);
  }
  // last four tiles: KT-4 (loads KT-1), KT-3, KT-2 (no loads), KT-1 (nothing follows)
  pipe.template tile<0, true, true, true>(acc, p1, q1);
  pipe.template tile<1, true, false, true>(acc, p0, q0);
  pipe.template tile<0, true, false, true>(acc, p1, q1);
  pipe.template tile<1, false, false, false>(acc, p0, q0);
  __syncthreads();  // LDS is free for the caller's epilogue
}

// Picks the pipelined loop when both operands are 16-bit in memory, and the
// simple loop (which converts fp32 sources on the way into LDS) otherwise.
// Both produce identical accumulators for identical 16-bit operand values.
template <class T, class PSrc, bool P_KC, class QSrc, bool Q_KC>
LCE_DEV void gemm_tile(f32x16_t (&acc)[kNB][kNB], const PSrc* p_origin, int64_t ldp,
                       const QSrc* q_origin, int64_t ldq, int ktiles, char* lds) {
  if constexpr (sizeof(PSrc) == 2 && sizeof(QSrc) == 2) {
    gemm_mainloop2<T, PSrc, P_KC, QSrc, Q_KC>(acc, p_origin, ldp, q_origin, ldq, ktiles, lds);
  } else {
    gemm_mainloop<T, PSrc, P_KC, QSrc, Q_KC>(acc, p_origin, ldp, q_origin, ldq, ktiles, lds);
  }
}

}  // namespace lce
