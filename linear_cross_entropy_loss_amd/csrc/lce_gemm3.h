// Persistent, software-pipelined contraction of 16-bit operands (fp32 inputs are
// rounded to the compute type by copy kernels before a tile kernel sees them).
//
// One workgroup per CU walks a list of 256 x 256 output tiles.  The operand
// fetch is one continuous stream of K tiles that runs THROUGH output-tile
// boundaries: while the last K tiles of output tile A are being multiplied,
// the first K tiles of output tile B are already in flight, so B starts
// without a load bubble and A's epilogue overlaps B's memory latency.
//
// Per K tile (64 deep) each wave issues 64 MFMAs and, between them,
//   * the LDS reads of the next k-step's fragments (double buffered),
//   * the LDS stores of K tile t+1 (from the register staging set),
//   * the buffer loads of K tile t+2 (each chunk into the register just stored),
// spread over the k-steps so the four waves, which leave the single barrier
// in lockstep, never oversubscribe the LDS port.  A load therefore has one K
// tile (~2000 cycles) to arrive; a second staging set (two K tiles of slack)
// measured less than 1 % faster and cost 64 registers, i.e. spills.  The LDS
// stage is a compile-time constant (the loop is unrolled by two); the
// accumulator of an output tile starts from a zero C operand.
//
// Across an epilogue the staging set (K tile 1 of the next output tile) stays in
// flight but no fragments, which leaves the epilogue ~180 vector registers.
//
// K tiles per output tile (`ktiles`) must be a multiple of 2 and at least 4, so
// that the first K tile of every output tile lands in LDS stage 0.
#pragma once

#include "lce_gemm.h"

namespace lce {

// Register staging of one operand tile: 8 chunks of 8 elements (one 16-byte register quad) per thread.
// Operands are always 16-bit in memory: fp32 activations and weights are rounded to the compute type by
// copy kernels before the tile kernels run.
struct StageRegs {
  u32x4_t v[8];
};

#define LCE_SG_VALU 0x002
#define LCE_SG_TRANS 0x400
#define LCE_SG_MFMA 0x008
#define LCE_SG_VMEM_RD 0x020
#define LCE_SG_DS_RD 0x100
#define LCE_SG_DS_WR 0x200

// Operand tiles are fetched with buffer loads: the resource descriptor (in
// SGPRs) points at the current K tile, each thread contributes one 32-bit byte
// offset, and the stride between a thread's 8 chunks is a scalar offset, so a
// load costs one instruction and no vector address arithmetic.
// KMASK = false compiles the K mask out, for launches whose K tiles cover the K extent exactly.
template <class T, class SrcT, bool KC, bool KMASK> struct Stager3 {
  static_assert(sizeof(SrcT) == 2, "operands are staged as 16-bit data");
  static constexpr int kEs = (int)sizeof(SrcT);
  typedef StageRegs Regs;
  const char* base;      // uniform: first byte of the K tile being loaded
  const char* end;       // uniform: one past the last valid byte of the operand (loads beyond return 0)
  unsigned range;        // uniform: bytes from `base` to `end`, clamped to [0, 2^31)
  unsigned voff;         // per-thread byte offset of its first chunk
  unsigned voff_cur;     // voff, or an always-out-of-range offset when this thread's k lies past the K extent
  int kpos;              // KC only: first k (element index inside a K tile) this thread loads
  unsigned iter_stride;  // uniform: bytes between this thread's consecutive chunks
  int64_t k_stride;      // bytes between consecutive K tiles
  int lds_off;           // per-thread byte offset of chunk 0 inside the operand tile

  LCE_DEV void init(int64_t ld) {
    const int t = threadIdx.x;
    if (KC) {
      const int c = t & 7, r = t >> 3;
      voff = (unsigned)(((int64_t)r * ld + c * 8) * kEs);
      iter_stride = (unsigned)(32 * ld * kEs);
      k_stride = kBK * kEs;
      const int sw = (r & 7) ^ ((r >> 3) & 1);
      lds_off = r * 128 + ((c ^ sw) << 4);
      kpos = c * 8;
    } else {
      const int c = t & 31, k = t >> 5;
      voff = (unsigned)(((int64_t)k * ld + c * 8) * kEs);
      iter_stride = (unsigned)(8 * ld * kEs);
      k_stride = (int64_t)kBK * ld * kEs;
      const int j = k & 3;
      const int mask = ((j & 1) << 7) | ((j >> 1) << 6) | ((j & 1) << 5);
      lds_off = k * 512 + ((c << 4) ^ mask);
      kpos = 0;
    }
    voff_cur = voff;
    base = end = nullptr;
    range = 0;
  }
  // The operand is stored in blocks of 256 rows x 64 columns, [rows / 256][cols / 64][256][64] (the staged dz, see
  // BwdArgs::dz), instead of row-major.  KC (its columns are the K index): the 256 rows x 64 k of a K tile are one
  // contiguous block of 128-byte rows, and the next K tile is the next block.  Otherwise (its rows are the K
  // index): the tile's 256 columns are four consecutive blocks, each thread stays in one; a K tile is 64 rows of
  // them, and after four K tiles the stream moves on to the next row of blocks (Pipe3::stream_advance).
  LCE_DEV void init_blocked() {
    init(kBK);
    if (KC) {
      k_stride = kTile * (kBK * kEs);
    } else {
      const int t = threadIdx.x, c = t & 31, k = t >> 5;
      voff = (unsigned)((c >> 3) * (kTile * kBK * kEs) + k * (kBK * kEs) + (c & 7) * 16);
      voff_cur = voff;
      iter_stride = (unsigned)(8 * kBK * kEs);
      k_stride = (int64_t)kBK * kBK * kEs;
    }
  }
  // Called whenever `base` moves.  `k_rem` = valid k elements from the start of
  // this K tile on.  Along K a K-contiguous operand runs on into the next row, so
  // its threads past the K extent are switched to an out-of-range offset; a
  // row-contiguous operand has K as its slow index and simply runs off `end`.
  LCE_DEV void retarget(int k_rem) {
    // clamp(end - base, 0, 2^31 - 1), on 32-bit halves so that it stays on the scalar unit
    const int64_t left = end - base;
    int hi = (int)(left >> 32);
    unsigned lo = (unsigned)left;
    asm("" : "+s"(hi), "+s"(lo));  // keeps the compiler from fusing the halves back into 64-bit vector compares
    const unsigned low = lo < 0x7fffffffu ? lo : 0x7fffffffu;
    const unsigned capped = hi != 0 ? 0x7fffffffu : low;
    range = hi < 0 ? 0u : capped;
    if (KC && KMASK) voff_cur = kpos < k_rem ? voff : 0x80000000u;
  }
  LCE_DEV void load(Regs& r, int i0, int i1) const {
    // 0x00020000: raw 32-bit data format.  The hardware returns 0 for every
    // dword at or beyond `range` bytes (voffset + soffset are both checked), which
    // zero-fills rows past the end of the operand and, with range == 0, turns
    // every load into a no-op once the stream is past the last output tile.
    const __amdgpu_buffer_rsrc_t rsrc =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(base), 0, (int)range, 0x00020000);
#pragma unroll
    for (int i = i0; i < i1; ++i)
      r.v[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff_cur, (int)(i * iter_stride), 0);
  }
  LCE_DEV void store(const Regs& r, char* tile, int i0, int i1) const {
    constexpr int step = KC ? 32 * 128 : 8 * 512;
#pragma unroll
    for (int i = i0; i < i1; ++i) *reinterpret_cast<u32x4_t*>(tile + lds_off + i * step) = r.v[i];
  }
};

// One past the last byte the loads of a row-major matrix may touch.  The range
// check of a buffer load works on whole dwords, so for 16-bit elements the last
// row is taken to end on a dword boundary: with an odd row length the element
// after the last one is read (it lies in the stride padding, must be finite and
// never reaches a valid output).
template <class S> LCE_DEV const void* matrix_end(const void* base, int64_t rows, int64_t ld, int64_t cols) {
  const int64_t c = sizeof(S) == 2 ? (cols + 1) & ~(int64_t)1 : cols;
  return reinterpret_cast<const S*>(base) + (rows - 1) * ld + c;
}

// What a kernel plugs into the persistent loop.
//   int  num_tiles()                              output tiles in this launch
//   void origins(int tile, const void*& p, const void*& q)
//        first element of the P / Q operand of that output tile:
//        (row0, k=0) for a KC operand, (k=0, col0) for an MC operand
//   const void* p_end(), q_end()                  one past the last valid byte of each operand
//   static constexpr bool kVarK                   true if work items differ in their number of K tiles; then
//   int  item_ktiles(int tile)                    gives it (even, at least 4) -- otherwise run() is told once
//   static constexpr bool kSwapAB                 false: P fragments feed the A side of the matrix instruction (the P index
//        runs along accumulator registers, Q along lanes); true: the Q fragments do (acc[i][j] is still the block
//        of P block i and Q block j, with Q along its registers and P along its lanes)
//   void prefetch(int tile)                       called three K tiles before the tile's epilogue: the place to issue loads
//        of per-row data the epilogue starts with (kept in members), so that their latency is not exposed there
//   static constexpr bool kQBlocked               true if the Q operand is stored in blocks of 256 rows x 64 columns
//        (Stager3::init_blocked); run() then takes the column groups per row of blocks in place of the Q row stride, and
//   int  q_phase(int tile)                        (rows are the K index) says which of the four K tiles of a row of blocks
//        the tile's first K tile is
//   static constexpr bool kKMask                  false if `ktiles * 64 == k_valid` for every tile of the launch
//   int  k_valid(int tile)                        K extent of that tile's contraction; the K tiles of the
//        loop may run past it (`ktiles * 64 >= k_valid`), the excess contributes exact zeros
//   static constexpr bool kColumnEpilogue          true if the epilogue works through the accumulator one block column
//        (Q block: 32 lanes' worth of Q rows, all 128 P rows of the wave) at a time, in 16 slots of straight-line
//        vector ALU code per column:
//          void epilogue_begin(int tile, char* extra)     per-tile scalars, kept in members
//          template <int J> void epilogue_slot(int tile, acc, int slot, char* extra)   slot 0..15 of column J
//          (acc[0..3][J]); no branches, no barriers; state between slots in members
//          void epilogue_end(int tile, acc, char* extra)  whatever is rare and branchy, after the last column
//        The last K tile of an output tile is then multiplied column by column, and slot k of column j runs
//        behind the k-th matrix instruction of column j + 1 (step_last_columns).  `extra`: LDS behind the two stages
//        (the launch must provide it), which the main loop never touches.  Otherwise:
//   void epilogue(int tile, acc, char* scratch)
//        consumes the finished accumulator; may use `scratch`, 96 KiB of LDS
//        that the pipeline does not touch until the next barrier it issues
//        itself -- the epilogue must end with all its LDS traffic complete
//        (a __syncthreads() if it used scratch).
template <class T, class PSrc, bool P_KC, class QSrc, bool Q_KC, class Problem> struct Pipe3 {
  typedef Stager3<T, PSrc, P_KC, Problem::kKMask> PStager;
  typedef Stager3<T, QSrc, Q_KC, Problem::kKMask> QStager;
  typedef typename PStager::Regs PRegs;
  typedef typename QStager::Regs QRegs;
  PStager ps;
  QStager qs;
  FragReader<P_KC> pr;
  FragReader<Q_KC> qr;
  s16x8_t pf[2][kNB], qf[2][kNB];
  char* lds;
  Problem& prob;
  int ktiles;
  int load_tile;  // output tile the fetch stream is in
  int k_rem;      // valid k elements left from the K tile the stream points at
  int q_phase;    // blocked Q operand with rows as its K index: K tile of the current row of blocks, 0..3
  int64_t q_jump; // and the bytes from the last K tile of a row of blocks to the first of the next
  static constexpr bool kQRowBlocks = Problem::kQBlocked && !Q_KC;

  static constexpr int kPReads = P_KC ? 4 : 8;  // LDS read instructions per k-step
  static constexpr int kQReads = Q_KC ? 4 : 8;
  static constexpr int kReads = kPReads + kQReads;
  // Fragment reads of the next K step go out early in the current one, so that their data is
  // back before its first matrix instruction: a quarter of them (2, 3 or 4) after each of the
  // first four MFMAs.  (One per MFMA, or all of them in one go, both measure slower.)
  static constexpr int kReadsPerSlot = kReads / 4;
  // Rows of MFMAs of the last K step that run before the workgroup barrier.  The earlier the
  // barrier, the more time the first fragment reads of the next K tile have; with 16 of them
  // (both operands transposed) the barrier opens the step, otherwise one row precedes it.
  static constexpr int kPreRows = kReads > 12 ? 0 : 1;

  LCE_DEV Pipe3(Problem& p) : prob(p) {}

  LCE_DEV void stream_begin(int tile) {
    load_tile = tile;
    if (tile < prob.num_tiles()) {
      const void *p, *q;
      prob.origins(tile, p, q);
      ps.base = reinterpret_cast<const char*>(p);
      qs.base = reinterpret_cast<const char*>(q);
      ps.end = reinterpret_cast<const char*>(prob.p_end());
      qs.end = reinterpret_cast<const char*>(prob.q_end());
    } else {
      ps.end = ps.base;  // nothing left to fetch: every load returns 0
      qs.end = qs.base;
    }
    k_rem = prob.k_valid(tile);
    if constexpr (kQRowBlocks) q_phase = tile < prob.num_tiles() ? prob.q_phase(tile) : 0;
    ps.retarget(k_rem);
    qs.retarget(k_rem);
  }
  LCE_DEV void stream_advance() {
    ps.base += ps.k_stride;
    if constexpr (kQRowBlocks) {
      qs.base += q_phase == 3 ? q_jump : qs.k_stride;
      q_phase = (q_phase + 1) & 3;
    } else {
      qs.base += qs.k_stride;
    }
    k_rem -= kBK;
    ps.retarget(k_rem);
    qs.retarget(k_rem);
  }
  // chunks 0..7 of a staged K tile belong to P, 8..15 to Q
  LCE_DEV void store_chunks(const PRegs& sp, const QRegs& sq, char* stage, int c0, int c1) {
    if (c0 < 8) ps.store(sp, stage, c0, c1 < 8 ? c1 : 8);
    if (c1 > 8) qs.store(sq, stage + kTileBytes, c0 > 8 ? c0 - 8 : 0, c1 - 8);
  }
  LCE_DEV void load_chunks(PRegs& sp, QRegs& sq, int c0, int c1) {
    if (c0 < 8) ps.load(sp, c0, c1 < 8 ? c1 : 8);
    if (c1 > 8) qs.load(sq, c0 > 8 ? c0 - 8 : 0, c1 - 8);
  }
  // The order of the two operands' reads is a measured choice (about 1 % either way).
  LCE_DEV void read_frags(int buf, const char* stage, int ks) {
    if (kReads > 12) {
#pragma unroll
      for (int b = 0; b < kNB; ++b) pf[buf][b] = pr.read(stage, b, ks);
    }
#pragma unroll
    for (int b = 0; b < kNB; ++b) qf[buf][b] = qr.read(stage + kTileBytes, b, ks);
    if (kReads <= 12) {
#pragma unroll
      for (int b = 0; b < kNB; ++b) pf[buf][b] = pr.read(stage, b, ks);
    }
  }
  // The accumulator blocks of a row are visited left to right in even rows and right to left in odd ones, so
  // that consecutive matrix instructions always differ in exactly one operand (measured 0.1-0.3 % faster than
  // restarting every row on the left, where both operands change at a row change).
  template <bool ZERO> LCE_DEV void mfma_rows(f32x16_t (&acc)[kNB][kNB], int buf, int i0, int i1) {
#pragma unroll
    for (int i = i0; i < i1; ++i)
#pragma unroll
      for (int jj = 0; jj < kNB; ++jj) {
        const int j = (i & 1) ? kNB - 1 - jj : jj;
        f32x16_t c;
        if (ZERO) {
#pragma unroll
          for (int r = 0; r < 16; ++r) c[r] = 0.f;
        } else {
          c = acc[i][j];
        }
        acc[i][j] = Problem::kSwapAB ? mfma32<T>(qf[buf][j], pf[buf][i], c) : mfma32<T>(pf[buf][i], qf[buf][j], c);
      }
  }

  // One K tile t, held in LDS stage STAGE.  The staging set holds K tile t+1: it is
  // stored to the other LDS stage and, chunk by chunk, refilled with K tile t+2.
  // FIRST  first K tile of an output tile: zero C operand.
  // WRAP   K tile t+2 is the last of this output tile: the stream moves on afterwards.
  // LAST   last K tile of an output tile: no fragment prefetch (the epilogue follows).
  template <int STAGE, bool FIRST, bool WRAP, bool LAST>
  LCE_DEV void step(f32x16_t (&acc)[kNB][kNB], PRegs& sp, QRegs& sq) {
    const char* cur = lds + STAGE * kStageBytes;
    char* nxt = lds + (STAGE ^ 1) * kStageBytes;

    // k-step 0: MFMAs on buffer 0; fragment reads for step 1; LDS stores 0..5
    read_frags(1, cur, 1);
    store_chunks(sp, sq, nxt, 0, 6);
    mfma_rows<FIRST>(acc, 0, 0, kNB);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      __builtin_amdgcn_sched_group_barrier(LCE_SG_MFMA, 1, 0);
      if (i < 4) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_RD, kReadsPerSlot, 0);
      if (i >= 4 && (i & 1) == 0) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_WR, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);

    // k-step 1: MFMAs on buffer 1; reads for step 2; stores 6..11 (in slots the reads leave free); loads 0..5
    read_frags(0, cur, 2);
    store_chunks(sp, sq, nxt, 6, 12);
    load_chunks(sp, sq, 0, 6);
    mfma_rows<false>(acc, 1, 0, kNB);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      __builtin_amdgcn_sched_group_barrier(LCE_SG_MFMA, 1, 0);
      if (i < 4) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_RD, kReadsPerSlot, 0);
      if (i >= 5 && (i & 1) == 1) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_WR, 1, 0);
      if (i >= 4 && (i & 1) == 0) __builtin_amdgcn_sched_group_barrier(LCE_SG_VMEM_RD, 1, 0);  // chunks 0..5: P
    }
    __builtin_amdgcn_sched_barrier(0);

    // k-step 2: MFMAs on buffer 0; reads for step 3; stores 12..15; loads 6..10
    read_frags(1, cur, 3);
    store_chunks(sp, sq, nxt, 12, 16);
    load_chunks(sp, sq, 6, 11);
    mfma_rows<false>(acc, 0, 0, kNB);
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      __builtin_amdgcn_sched_group_barrier(LCE_SG_MFMA, 1, 0);
      if (i < 4) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_RD, kReadsPerSlot, 0);
      if (i >= 4 && i < 12 && (i & 1) == 0) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_WR, 1, 0);
      if (i >= 5 && i < 9 && (i & 1) == 1) __builtin_amdgcn_sched_group_barrier(LCE_SG_VMEM_RD, 1, 0);  // chunks 6, 7: P
      if (i >= 9 && i < 15 && (i & 1) == 1) __builtin_amdgcn_sched_group_barrier(LCE_SG_VMEM_RD, 1, 0);  // chunks 8..10: Q
    }
    __builtin_amdgcn_sched_barrier(0);

    // k-step 3: kPreRows rows of MFMAs with loads 11..; barrier; reads for the next K tile's step 0; the rest
    constexpr int kPre = 4 * kPreRows, kPreLoads = kPre < 5 ? kPre : 5;
    load_chunks(sp, sq, 11, 11 + kPreLoads);
    mfma_rows<false>(acc, 1, 0, kPreRows);
#pragma unroll
    for (int i = 0; i < kPre; ++i) {
      __builtin_amdgcn_sched_group_barrier(LCE_SG_MFMA, 1, 0);
      if (i < kPreLoads) __builtin_amdgcn_sched_group_barrier(LCE_SG_VMEM_RD, 1, 0);  // chunks 11..: Q
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    if (!LAST) read_frags(0, nxt, 0);
    load_chunks(sp, sq, 11 + kPreLoads, 16);
    // The fetch stream moves on to K tile t+3 (first needed by the next step's loads).  Its scalar
    // address / range arithmetic sits in this region so that it issues between the MFMAs below.
    if (WRAP) {
      stream_begin(load_tile + (int)gridDim.x);
    } else {
      stream_advance();
    }
    mfma_rows<false>(acc, 1, kPreRows, kNB);
#pragma unroll
    for (int i = 0; i < 16 - kPre; ++i) {
      __builtin_amdgcn_sched_group_barrier(LCE_SG_MFMA, 1, 0);
      if (!LAST && i < 4) __builtin_amdgcn_sched_group_barrier(LCE_SG_DS_RD, kReadsPerSlot, 0);
      if (i >= 4 && i < 4 + 5 - kPreLoads) __builtin_amdgcn_sched_group_barrier(LCE_SG_VMEM_RD, 1, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  }


  // The last K tile of an output tile, for a problem whose epilogue works column by column
  // (Problem::kColumnEpilogue), with that epilogue.  The 64 matrix instructions of the K tile are issued one
  // block column of the accumulator after the other (all four k-steps of column 0, then of column 1, ...):
  // column j is final when column j + 1 starts, and its epilogue -- vector ALU work that would otherwise run
  // with the matrix pipe idle -- is cut into 16 slots, one behind each matrix instruction of column j + 1.  Only
  // the last column's epilogue runs on its own.  The order is fixed in the source, slot by slot (a scheduling
  // barrier after each): left to the compiler, with or without scheduling groups, the matrix instructions end
  // up in a row ahead of the epilogue.  The K tile's 16 P fragments stay in registers once read (64 VGPRs, where the
  // steady-state loop double-buffers 8 + 8 fragments), the Q fragments come one k-step ahead of their use.
  // Everything else is as in step<1, false, false, true>: the staging set (K tile 0 of the next output tile) goes to
  // LDS stage 0 (one chunk per slot of column 0) and is refilled with its K tile 1 (one chunk per slot of column
  // 1); one workgroup barrier.  Each accumulator block still sums its k-steps in the same order, so the result
  // is bit-identical to the row-by-row order.
  template <int J>
  LCE_DEV void last_column(f32x16_t (&acc)[kNB][kNB], PRegs& sp, QRegs& sq, s16x8_t (&pa)[4][kNB], s16x8_t (&qk)[2],
                           int tile) {
    const char* cur = lds + kStageBytes;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      const int n = 4 * J + ks, nn = n + 1;  // Q fragment of k-step n = 4 * column + ks lives in buffer n & 1
      // one k-step ahead: the Q fragment of the next k-step (of the next column after the last) and, in column 0,
      // the P fragments of the next k-step, which then stay for the other columns
      if (nn < 16) qk[nn & 1] = qr.read(cur + kTileBytes, nn >> 2, nn & 3);
      if (J == 0 && ks < 3) {
#pragma unroll
        for (int b = 0; b < kNB; ++b) pa[ks + 1][b] = pr.read(cur, b, ks + 1);
      }
#pragma unroll
      for (int i = 0; i < kNB; ++i) {
        const int slot = 4 * ks + i;
        acc[i][J] = Problem::kSwapAB ? mfma32<T>(qk[n & 1], pa[ks][i], acc[i][J])
                                     : mfma32<T>(pa[ks][i], qk[n & 1], acc[i][J]);
        if (J == 0) store_chunks(sp, sq, lds, slot, slot + 1);
        if (J == 1) load_chunks(sp, sq, slot, slot + 1);
        if constexpr (J > 0) prob.template epilogue_slot<J - 1>(tile, acc, slot, lds + kMainloopLds);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
  LCE_DEV void step_last_columns(f32x16_t (&acc)[kNB][kNB], PRegs& sp, QRegs& sq, int tile) {
    s16x8_t pa[4][kNB], qk[2];  // the K tile's P fragments [k-step][block]; two Q fragments
#pragma unroll
    for (int b = 0; b < kNB; ++b) pa[0][b] = pf[0][b];
    qk[0] = qf[0][0];
    prob.epilogue_begin(tile, lds + kMainloopLds);
    last_column<0>(acc, sp, sq, pa, qk, tile);
    last_column<1>(acc, sp, sq, pa, qk, tile);
    stream_advance();
    last_column<2>(acc, sp, sq, pa, qk, tile);
    last_column<3>(acc, sp, sq, pa, qk, tile);
    // the barrier: every wave's part of the next K tile is in LDS stage 0, and no wave reads this stage any more
    __syncthreads();
#pragma unroll
    for (int slot = 0; slot < 16; ++slot) {
      prob.template epilogue_slot<3>(tile, acc, slot, lds + kMainloopLds);
      __builtin_amdgcn_sched_barrier(0);
    }
    prob.epilogue_end(tile, acc, lds + kMainloopLds);
  }

  LCE_DEV void run(int64_t ldp, int64_t ldq, int ktiles_, char* lds_) {
    lds = lds_;
    ktiles = ktiles_;
    const int wave = threadIdx.x >> 6;
    ps.init(ldp);
    if constexpr (Problem::kQBlocked) {
      qs.init_blocked();
      // (ldq: column groups per row of blocks) what takes a stream whose K index is the rows from the last K tile of
      // a row of blocks to the first of the next
      q_jump = ldq * (kTile * kBK * QStager::kEs) - 3 * qs.k_stride;
    } else {
      qs.init(ldq);
    }
    pr.init((wave & 1) * kWaveTile);
    qr.init((wave >> 1) * kWaveTile);

    PRegs sp;
    QRegs sq;
    stream_begin((int)blockIdx.x);
    load_chunks(sp, sq, 0, 16);
    stream_advance();
    store_chunks(sp, sq, lds, 0, 16);
    load_chunks(sp, sq, 0, 16);
    stream_advance();
    __syncthreads();

    f32x16_t acc[kNB][kNB];
    for (int tile = (int)blockIdx.x; tile < prob.num_tiles(); tile += (int)gridDim.x) {
      if constexpr (Problem::kVarK) ktiles = prob.item_ktiles(tile);
      read_frags(0, lds, 0);
      step<0, true, false, false>(acc, sp, sq);
      if (ktiles > 4) {
        step<1, false, false, false>(acc, sp, sq);
        for (int t = 2; t < ktiles - 4; t += 2) {
          step<0, false, false, false>(acc, sp, sq);
          step<1, false, false, false>(acc, sp, sq);
        }
        step<0, false, false, false>(acc, sp, sq);
      }
      prob.prefetch(tile);  // three K tiles ahead of the epilogue
      step<1, false, true, false>(acc, sp, sq);
      step<0, false, false, false>(acc, sp, sq);
      if constexpr (Problem::kColumnEpilogue) {
        step_last_columns(acc, sp, sq, tile);
      } else {
        step<1, false, false, true>(acc, sp, sq);
        prob.epilogue(tile, acc, lds + kStageBytes);
      }
    }
  }
};

}  // namespace lce
