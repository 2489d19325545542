// Backward, step 1: recompute a 256(v) x 256(token) logit tile with the same
// MFMA main loop as the forward (so the logits are bit-identical to the ones
// the saved lse was built from) and turn it, in registers, into
//     dz = softmax * (1 + 2*z_reg*lse) - onehot(y),   0 for ignored tokens
// (times 2^dz_shift, a power of two that keeps small probabilities in fp16's normal range)
// (linear_cross_entropy/ops.py:309-314 and 415-422), rounded once to the
// 16-bit compute type exactly where the reference casts dz before its dot
// products (ops.py:314, 422).  The staging buffer of the current vocabulary slab
// is laid out in groups of 64 columns (BwdArgs::dz): a token's 64 columns of a
// group are one 128-byte line, and dz leaves the compute unit as whole lines,
// transposed through a small LDS area that the main loop does not use.
// The kernel is persistent (one workgroup per CU, operand stream pipelined across tiles).
#include "lce_gemm3.h"
#include "lce_internal.h"

namespace lce {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kGroup = 64;               // columns per group of the stage
constexpr int kPieceBytes = kBlk * kGroup * 2;   // 32 tokens x 64 columns: what a wave stages at a time
constexpr int kWaveLds = 2 * kPieceBytes;        // two pieces per wave (the two column groups of its slice)
constexpr int kLdsBytes = kMainloopLds + 4 * kWaveLds;  // the main loop's stages, then the epilogue's pieces
static_assert(kLdsBytes <= 160 * 1024, "a compute unit has 160 KiB of LDS");
#ifndef LCE_DZ_STORE_AUX
#define LCE_DZ_STORE_AUX 2
#endif
constexpr int kDzStoreAux = LCE_DZ_STORE_AUX;  // cache policy of the dz stores: 2 = nt (streaming)

// Turns the finished logit tile (tp, tq) into dz and writes it out.
//
// Each lane owns 4 tokens (columns of the accumulator) x 64 vocabulary entries
// per token, four consecutive entries per register quad; lanes l and l+32 hold
// the two halves of every run of 8 entries.  One v_permlane32_swap per pair of
// register quads hands each lane a full run of 8 (16 bytes in the 16-bit
// staging type).  A wave stages 32 tokens x 64 columns at a time (a piece: the
// tokens of one accumulator block, one column group) in its own LDS area and
// reads the piece back as whole 128-byte lines, 8 consecutive tokens (1 KiB of
// the stage) per store instruction; measured against storing the 16-byte runs
// straight from the registers (32-byte sectors of 32 different lines per
// instruction): 3 % of the kernel in favour of whole lines, 10 % with streaming
// stores.  Lines of a piece have their 16-byte chunk index XOR-ed by
// (line & 7) ^ ((line >> 3) & 1), the swizzle of the K-contiguous operand tiles,
// for the 16-byte writes (32 lines per instruction) and the line reads (8 lines
// per instruction).  The area lies behind the main loop's stages and only its
// own wave touches it: no barrier, a wave that is done moves on by itself.
//   * ignored tokens use lse = +inf, which makes every exp2 an exact +0;
//   * the "- onehot" is applied afterwards by the one lane that owns the target
//     column: it waits for the wave's stores, then overwrites the staged
//     softmax value with the rounding of the fp32 (p - 1) (one rounding, as in
//     ops.py:313-314).  A wave meets a target in about one tile out of eight at
//     a vocabulary of 131072, so the wait is rare.
//
// VTAIL is the variant for the one tile column that straddles the end of the
// vocabulary: every run of 8 columns (a pair of register quads in lanes l, l+32)
// but at most one is inside or outside as a whole, uniformly over the wave; the
// one run that V cuts through is handled element by element.  Columns outside
// are written as exact zeros.
//
// SPLIT (fp32 tensors carried as bf16 pairs, lce_gemm.h): dz is staged as hi = bf16(dz) and lo = bf16(dz - hi)
// in three parts of Np rows, [hi ; lo ; hi], each lane storing its 16-byte runs itself (this
// path serves accuracy, not speed).
// `pf_y`, `pf_lse`: label and lse of this lane's four tokens (DzProblem::prefetch), ignore_index / 0 for rows that do not exist.
//
// FUSE (launch_fwd_stage: the logits are computed once, for the loss and for the gradients): the tile leaves
// e = 2^dz_shift * exp(z - m) instead, m = the largest logit of the token within this wave's 128 columns, for
// every row, whatever its label; the wave also writes the forward's partials of its slice (m and
// m + log sum exp(z - m)) and the target logit.  `pf_lse` is not used, and there is no gain to apply: under FUSE the
// switch ZREG stands for the monitoring values instead (the slice's sum softmax * z and sum z^2, as lce_fwd.hip forms them).
constexpr int kNoLabel = -0x7fffffff - 1;  // ignore_index, or no such row
constexpr int kOffLabel = -1;              // a label that is no column of W (V <= 2^30): matches nothing
template <class T, bool ZREG, bool VTAIL, bool SPLIT, bool FUSE>
LCE_DEV void dz_epilogue_impl(const BwdArgs& a, const int (&pf_y)[kNB], const float (&pf_lse)[kNB],
                              f32x16_t (&acc)[kNB][kNB], int tp, int tq, char* pieces) {
  typedef typename elem_of<T>::type E;
  const int64_t v0 = a.v0 + (int64_t)tp * kTile, t0 = (int64_t)tq * kTile;
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  const int half = lane >> 5;
  const int64_t slice_v0 = v0 + wp * kWaveTile;
  const float c1 = a.scale * kLog2e;
  // columns of this wave's slice that exist: nq whole runs of 8, then `cut` more columns
  const int64_t left = a.v0 + a.vw - slice_v0;
  const int vrem = VTAIL ? (int)(left < 0 ? 0 : (left > kWaveTile ? kWaveTile : left)) : kWaveTile;
  const int nq = vrem >> 3, cut = vrem & 7;
  const int cut_mine = cut - 4 * half;  // elements of this lane's quad of the cut run that exist (<= 0: none)
  // This wave's 128 columns are two column groups (accumulator blocks 0, 1 and 2, 3), neighbouring blocks of the
  // stage; `row` = this lane's token row of block qb = 0 in the first of them.
  constexpr int64_t grp = kDzBlockElems;  // elements from a block of the stage to the next column group's
  const int wpu = __builtin_amdgcn_readfirstlane(wp), wqu = __builtin_amdgcn_readfirstlane(wq);  // (uniform, for the scalar unit)
  E* wave_base = reinterpret_cast<E*>(a.dz) + dz_block_offset(tq, tp * (kTile / kGroup) + wpu * (kWaveTile / kGroup), a.vs) +
                 wqu * kWaveTile * kGroup;
  E* row = wave_base + (lane & 31) * kGroup;
  constexpr bool MON = FUSE && ZREG;
  const int64_t blk = a.Np * a.vs;  // SPLIT: elements between the three parts of the stage
  // Stores go through a buffer descriptor over this wave's part of the stage (scalar base, one 32-bit offset per
  // lane, the block's offset as a scalar): no 64-bit vector address arithmetic.  All offsets stay below 2^31
  // (one block for the second column group, plus two parts of a bf16-pair stage).
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(wave_base, 0, 0x7fffffff, 0x00020000);
  const unsigned lane_off = (unsigned)((lane & 31) * (kGroup * 2) + half * 16);
  // staging: this lane's line of a piece when it writes (its token), and line / chunk when it reads back: 8 lines
  // per instruction, 8 lanes each; the upper 32 lanes take their four lines in the order 5, 4, 7, 6 so that lanes
  // l and l+32 always sit in lines of opposite parity (opposite bank halves)
  char* mine = pieces + wave * kWaveLds;
  const int wline = lane & 31, wsw = (wline & 7) ^ ((wline >> 3) & 1);
  const int rline = (lane >> 3) + ((lane >> 5) ? 1 - 2 * ((lane >> 3) & 1) : 0), rchunk = lane & 7;

  // per-token scalars of this lane's four tokens
  float nlse[kNB], gain[kNB];
  int ykey[kNB];
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    // (rows past the last one are staged as zeros, like ignored tokens)
    const int yy = pf_y[qb];  // the label as DzProblem::prefetch keeps it: kNoLabel, or the column (kOffLabel: none of W's)
    const int64_t rel = (int64_t)yy - slice_v0;
    const bool valid = yy != kNoLabel;
    const float l = FUSE ? 0.f : pf_lse[qb];
    // (the power-of-two factor of the staged dz rides along in the exponent)
    nlse[qb] = valid ? fmaf(-l, kLog2e, (float)a.dz_shift) : -INFINITY;  // (FUSE: set per block below)
    gain[qb] = 1.f + 2.f * a.z_reg * l;
    // (with the staging factor 2^10 of fp16 in place: |dz| * 2^10 <= 63 * 2^10 stays finite in fp16 whatever lse is)
    if (a.dz_shift != 0) gain[qb] = fminf(fmaxf(gain[qb], -63.f), 63.f);
    // target column inside this wave's slice, only in the lane half that holds it
    ykey[qb] = (valid && rel >= 0 && rel < kWaveTile && ((rel >> 2) & 1) == half) ? (int)rel : -1;
  }

#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    float m = -INFINITY, ssum = 0.f, mpz = 0.f, msq = 0.f;
    if constexpr (FUSE) {
      // the largest of this token's logits in the slice: this lane's 64, then the other half's
#pragma unroll
      for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq)
          if (!VTAIL || pb * 4 + rq < nq) {
#pragma unroll
            for (int j = 0; j < 4; ++j) m = fmaxf(m, acc[pb][qb][rq * 4 + j]);
          } else if (pb * 4 + rq == nq && cut != 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) m = j < cut_mine ? fmaxf(m, acc[pb][qb][rq * 4 + j]) : m;
          }
      m = fmaxf(m, __shfl_xor(m, 32));
      // (a slice with no column inside the vocabulary: every e below is an exact zero, whatever this is)
      nlse[qb] = fmaf(-m, c1, (float)a.dz_shift);
    }
#pragma unroll
    for (int pb = 0; pb < kNB; ++pb) {
      const unsigned blk_off = (unsigned)((pb >> 1) * grp * 2) + qb * (kBlk * kGroup * 2);  // bytes, uniform
#pragma unroll
      for (int g = 0; g < 4; g += 2) {
        float d[8];
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          if (!VTAIL || pb * 4 + g + h2 < nq) {
#pragma unroll
            for (int i = 4 * h2; i < 4 * h2 + 4; ++i) {
              const float zr = acc[pb][qb][g * 4 + i];
              d[i] = __builtin_amdgcn_exp2f(fmaf(zr, c1, nlse[qb]));
              if (ZREG && !FUSE) d[i] *= gain[qb];
              if constexpr (MON) {
                const float z = zr * a.scale;
                mpz = fmaf(d[i], z, mpz);
                msq = fmaf(z, z, msq);
              }
            }
          } else if (pb * 4 + g + h2 == nq && cut != 0) {
#pragma unroll
            for (int i = 4 * h2; i < 4 * h2 + 4; ++i) {
              const float zr = acc[pb][qb][g * 4 + i];
              d[i] = __builtin_amdgcn_exp2f(fmaf(zr, c1, nlse[qb]));
              if (ZREG && !FUSE) d[i] *= gain[qb];
              d[i] = (i - 4 * h2) < cut_mine ? d[i] : 0.f;
              if constexpr (MON) {
                const float z = zr * a.scale;
                mpz = fmaf(d[i], z, mpz);
                msq = (i - 4 * h2) < cut_mine ? fmaf(z, z, msq) : msq;
              }
            }
          } else {
#pragma unroll
            for (int i = 4 * h2; i < 4 * h2 + 4; ++i) d[i] = 0.f;
          }
        }
        if constexpr (FUSE) ssum += ((d[0] + d[1]) + (d[2] + d[3])) + ((d[4] + d[5]) + (d[6] + d[7]));
#pragma unroll
        for (int part = 0; part < (SPLIT ? 2 : 1); ++part) {
          if (part == 1) {
#pragma unroll
            for (int i = 0; i < 8; ++i) d[i] = bf16_lo(d[i]);
          }
          const unsigned x0 = pack2<T>(d[0], d[1]), x1 = pack2<T>(d[2], d[3]);
          const unsigned y0 = pack2<T>(d[4], d[5]), y1 = pack2<T>(d[6], d[7]);
          // lanes 0..31 keep their quad g and receive the partner's quad g; lanes
          // 32..63 receive the partner's quad g+1 and keep their own
          const auto s0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
          const auto s1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
          u32x4_t o;
          o[0] = s0[0];
          o[1] = s1[0];
          o[2] = s0[1];
          o[3] = s1[1];
          // streaming stores (aux 2 = nt): dz (1 GiB per slab) is read back from memory by the next kernels anyway,
          // and a normal store would evict the W / x tiles the following main loop is about to reuse from L2
          if constexpr (SPLIT) {
            const unsigned voff = lane_off + (pb & 1) * (kBlk * 2) + g * 16;
            const unsigned soff = blk_off + (part == 1 ? (unsigned)(blk * 2) : 0u);
            __builtin_amdgcn_raw_buffer_store_b128(o, rsrc, (int)voff, (int)soff, kDzStoreAux);
            if (part == 0) __builtin_amdgcn_raw_buffer_store_b128(o, rsrc, (int)voff, (int)(soff + (unsigned)(blk * 4)), kDzStoreAux);
          } else {
            const int chunk = (pb & 1) * 4 + g + half;  // 16-byte chunk of the token's line
            *reinterpret_cast<u32x4_t*>(mine + (pb >> 1) * kPieceBytes + wline * (kGroup * 2) + ((chunk ^ wsw) << 4)) = o;
          }
        }
      }
    }
    if constexpr (!SPLIT) {
      // read the two pieces back as 128-byte lines and send them out
#pragma unroll
      for (int gi = 0; gi < 2; ++gi)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int line = i * 8 + rline;
          const u32x4_t v = *reinterpret_cast<const u32x4_t*>(mine + gi * kPieceBytes + line * (kGroup * 2) +
                                                              ((rchunk ^ (line & 7) ^ ((line >> 3) & 1)) << 4));
          const unsigned soff = (unsigned)(gi * grp * 2) + qb * (kBlk * kGroup * 2);
          __builtin_amdgcn_raw_buffer_store_b128(v, rsrc, line * (kGroup * 2) + rchunk * 16, (int)soff, kDzStoreAux);
        }
    }
    // The target column of this lane's token, if it lies in this wave's slice: the staged softmax value is
    // replaced by the rounding of the fp32 (p - 1), once the wave's stores above have reached memory (the
    // 16-byte piece that holds the column may have been another lane's store).  (These rare branches also keep
    // the compiler from gathering the accumulator reads of all four blocks at the top, which spills.)
    const int yl = ykey[qb];
    if constexpr (FUSE) {
      // the forward's partials of this slice for the token, and its target logit if it lies here
      ssum += __shfl_xor(ssum, 32);
      const int64_t tokl = t0 + wq * kWaveTile + qb * kBlk + (lane & 31);
      const int64_t o = (slice_v0 / kChunkV) * a.nc + tokl;
      if (lane < 32) {
        // (no column of the slice inside the vocabulary: m = -inf, ssum = 0 -> -inf, nothing to add to the lse)
        a.part_max[o] = m * a.scale;
        a.part_lse[o] = ssum > 0.f ? fmaf(m, a.scale, (__builtin_amdgcn_logf(ssum) - (float)a.dz_shift) * 0.6931471805599453f)
                                   : -INFINITY;
      }
      if constexpr (MON) {
        mpz += __shfl_xor(mpz, 32);
        msq += __shfl_xor(msq, 32);
        if (lane < 32) {
          a.part_pz[o] = ssum > 0.f ? mpz / ssum : 0.f;  // (both sums carry the factor 2^dz_shift)
          a.part_sq[o] = msq;
        }
      }
      if (yl >= 0) {
        const int want = (yl >> 5) * 16 + ((yl >> 3) & 3) * 4 + (yl & 3);  // (block, register) index
        float zt = 0.f;
#pragma unroll
        for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            float v;
            asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(acc[pb][qb][r]));
            if (want == pb * 16 + r) zt = v;
          }
        a.tgt[tokl] = zt * a.scale;
      }
    } else if (yl >= 0) {
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      const int want = (yl >> 5) * 16 + ((yl >> 3) & 3) * 4 + (yl & 3);  // (block, register) index
      float zt = 0.f;
#pragma unroll
      for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          // (a volatile read: the compiler would otherwise hoist the 64 accumulator reads above the branch)
          float v;
          asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(v) : "a"(acc[pb][qb][r]));
          if (want == pb * 16 + r) zt = v;
        }
      float p = __builtin_amdgcn_exp2f(fmaf(zt, c1, nlse[qb]));
      if (ZREG) p *= gain[qb];
      const float tv = p - __builtin_bit_cast(float, (127 + a.dz_shift) << 23);  // the one, times 2^dz_shift
      E* at = row + (yl >> 6) * grp + qb * (kBlk * kGroup) + (yl & (kGroup - 1));
      *reinterpret_cast<unsigned short*>(at) = to_bits<T>(tv);
      if (SPLIT) {
        *reinterpret_cast<unsigned short*>(at + 2 * blk) = to_bits<T>(tv);
        *reinterpret_cast<unsigned short*>(at + blk) = to_bits<T>(bf16_lo(tv));
      }
    }
  }
}

// ZREG (z_regularization != 0) is a compile-time switch of the kernels rather than a
// branch inside them: with a branch the compiler hoists the accumulator reads of
// both arms above it and needs every vector register at once.
// The launch covers `tiles_p` tile columns of the slab starting at column tile
// `tp0`: all the full ones, or (VTAIL) those from the one straddling the end
// of the vocabulary to the end of the padded slab -- or, with BwdArgs::vtail_all, every column (the VTAIL code
// is right for full columns too, only slower).
// WVH: the weight is stored (V, H) row-major, so that the P operand runs along K in memory like x does.
template <class T, bool ZREG, bool VTAIL, bool KMASK, bool SPLIT, bool WVH, bool FUSE = false> struct DzProblem {
  typedef typename elem_of<T>::type E;
  static constexpr bool kKMask = KMASK;
  static constexpr bool kSwapAB = false;
  static constexpr bool kVarK = false;
  static constexpr bool kQBlocked = false;
  static constexpr bool kColumnEpilogue = false;
  const BwdArgs& a;
  int64_t rows, ldx;  // token rows: all of x, or the packed rows (see BwdArgs)
  const E* x;
  int tp0, tiles_p, tiles_q;
  LCE_DEV DzProblem(const BwdArgs& a_)
      : a(a_), tp0(VTAIL && !a_.vtail_all ? (int)(a_.vw / kTile) : 0),
        tiles_p(VTAIL ? (int)(a_.vs / kTile) - (a_.vtail_all ? 0 : (int)(a_.vw / kTile)) : (int)(a_.vw / kTile)) {
    rows = packed_rows(a.n_rows, a.N);
    const bool packed = rows != a.N;
    x = reinterpret_cast<const E*>(packed ? a.xc : a.x);
    ldx = packed ? a.ldxc : a.ldx;
    // SPLIT: the dW contraction runs through all Np rows of each of the three blocks of the stage, so every
    // token tile is written (rows past the last kept token as zeros), not only those that hold kept tokens
    tiles_q = SPLIT ? (int)(a.Np / kTile) : (int)((rows + kTile - 1) / kTile);
  }
  LCE_DEV int num_tiles() const { return tiles_p * tiles_q; }
  LCE_DEV void coords(int tile, int& tp, int& tq) const {
    tile_coords(tile, num_tiles(), tiles_p, tiles_q, 8, a.live, tp, tq);
    tp += tp0;
  }
  LCE_DEV void origins(int tile, const void*& p, const void*& q) const {
    int tp, tq;
    coords(tile, tp, tq);
    const int64_t v = (a.v0 - a.wv0) + (int64_t)tp * kTile;  // first column of the tile inside the buffer `w`
    p = reinterpret_cast<const E*>(a.w) + (WVH ? v * a.ldw : v);
    q = x + (int64_t)tq * kTile * ldx;
  }
  LCE_DEV const void* p_end() const {
    return WVH ? matrix_end<E>(a.w, a.Vw, a.ldw, a.H) : matrix_end<E>(a.w, a.H, a.ldw, a.Vw);
  }
  LCE_DEV const void* q_end() const { return matrix_end<E>(x, rows, ldx, a.H); }
  LCE_DEV int k_valid(int) const { return (int)a.H; }
  // The epilogue starts with the label and lse of each of this lane's four tokens: fetched while the last K tiles
  // of the tile are still being multiplied, instead of one exposed round trip to memory per tile.
  int pf_y[kNB];  // kNoLabel / kOffLabel / the column: four registers held over the last K tiles instead of eight
  float pf_lse[kNB];
  LCE_DEV void prefetch(int tile) {
    int tp, tq;
    coords(tile, tp, tq);
    const int lane = threadIdx.x & 63, wq = threadIdx.x >> 7;
#pragma unroll
    for (int qb = 0; qb < kNB; ++qb) {
      const int64_t tok = (int64_t)tq * kTile + wq * kWaveTile + qb * kBlk + (lane & 31);
      const bool exists = tok < rows;
      const int64_t yy = exists ? a.y[tok] : a.ignore_index;
      pf_y[qb] = yy == a.ignore_index ? kNoLabel : (yy >= 0 && yy < a.V ? (int)yy : kOffLabel);
      pf_lse[qb] = exists && !FUSE ? a.lse[tok] : 0.f;
    }
  }
  LCE_DEV void epilogue(int tile, f32x16_t (&acc)[kNB][kNB], char* scratch) const {
    int tp, tq;
    coords(tile, tp, tq);
    dz_epilogue_impl<T, ZREG, VTAIL, SPLIT, FUSE>(a, pf_y, pf_lse, acc, tp, tq, scratch + kStageBytes);  // (behind the main loop's stages)
  }
};

template <class T, bool ZREG, bool VTAIL, bool KMASK, bool SPLIT, bool WVH, bool FUSE>
__global__ __launch_bounds__(kThreads) void bwd_dz_persistent_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  typedef typename elem_of<T>::type E;
  DzProblem<T, ZREG, VTAIL, KMASK, SPLIT, WVH, FUSE> prob(a);
  Pipe3<T, E, WVH, E, true, DzProblem<T, ZREG, VTAIL, KMASK, SPLIT, WVH, FUSE>> pipe(prob);
  pipe.run(a.ldw, prob.ldx, (int)(padded_k(a.H) / kBK), lds);
}

template <class T, bool ZREG, bool VTAIL, bool KMASK, bool SPLIT, bool WVH, bool FUSE = false>
hipError_t launch_one(const BwdArgs& a, int64_t tiles, hipStream_t s) {
  auto kern = bwd_dz_persistent_kernel<T, ZREG, VTAIL, KMASK, SPLIT, WVH, FUSE>;
  static LdsOptIn optin;
  hipError_t e = optin.ensure(reinterpret_cast<const void*>(kern), kLdsBytes);
  if (e != hipSuccess) return e;
  const int grid = (int)(tiles < a.num_cus ? tiles : a.num_cus);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), kLdsBytes, s, a);
  return hipGetLastError();
}

// All full tile columns of the slab, then the column that straddles the end of the vocabulary.
template <class T, bool ZREG, bool SPLIT, bool WVH, bool FUSE = false>
hipError_t launch_persistent_z(const BwdArgs& a, hipStream_t s) {
  const int64_t tq = a.Np / kTile, full = a.vw / kTile, tail = a.vs / kTile - full;
  const bool exact_k = padded_k(a.H) == a.H;  // the K tiles cover H exactly: no K mask needed
  if (full > 0) {
    hipError_t e;
    if constexpr (FUSE && ZREG) {
      // (the monitoring sums on top of the K mask do not fit the registers in the kernel for full columns: a hidden
      // size that is not a multiple of 128 sends every column through the kernel for the last one, which has both)
      if (!exact_k) {
        BwdArgs all = a;
        all.vtail_all = 1;
        return launch_one<T, ZREG, true, true, SPLIT, WVH, FUSE>(all, (a.vs / kTile) * tq, s);
      }
      e = launch_one<T, ZREG, false, false, SPLIT, WVH, FUSE>(a, full * tq, s);
    } else {
      e = exact_k ? launch_one<T, ZREG, false, false, SPLIT, WVH, FUSE>(a, full * tq, s)
                  : launch_one<T, ZREG, false, true, SPLIT, WVH, FUSE>(a, full * tq, s);
    }
    if (e != hipSuccess) return e;
  }
  if (tail > 0) return launch_one<T, ZREG, true, true, SPLIT, WVH, FUSE>(a, tail * tq, s);
  return hipSuccess;
}

template <class T, bool SPLIT, bool WVH> hipError_t launch_persistent(const BwdArgs& a, hipStream_t s) {
  return a.z_reg != 0.f ? launch_persistent_z<T, true, SPLIT, WVH>(a, s)
                        : launch_persistent_z<T, false, SPLIT, WVH>(a, s);
}

}  // namespace

hipError_t launch_bwd_dz(const BwdArgs& a, hipStream_t s) {
  if (a.w_vh) {  // (never with bf16 pairs)
    if (a.split) return hipErrorInvalidValue;
    if (a.x_dtype == DT_BF16 && a.w_dtype == DT_BF16) return launch_persistent<BF16, false, true>(a, s);
    if (a.x_dtype == DT_F16 && a.w_dtype == DT_F16) return launch_persistent<F16, false, true>(a, s);
    return hipErrorInvalidValue;
  }
  if (a.x_dtype == DT_BF16 && a.w_dtype == DT_BF16)
    return a.split ? launch_persistent<BF16, true, false>(a, s) : launch_persistent<BF16, false, false>(a, s);
  if (a.x_dtype == DT_F16 && a.w_dtype == DT_F16) return launch_persistent<F16, false, false>(a, s);
  // (an fp32 weight arrives here as a 16-bit slab copy, fp32 activations as bf16 pairs with split set)
  return hipErrorInvalidValue;
}

template <class T, bool WVH> hipError_t launch_stage(const BwdArgs& a, hipStream_t s) {
  // (the second template argument: the monitoring values, see dz_epilogue_impl)
  return a.part_pz != nullptr ? launch_persistent_z<T, true, false, WVH, true>(a, s)
                              : launch_persistent_z<T, false, false, WVH, true>(a, s);
}

hipError_t launch_fwd_stage(const BwdArgs& a, hipStream_t s) {
  if (a.split || a.part_lse == nullptr || a.part_max == nullptr || a.tgt == nullptr) return hipErrorInvalidValue;
  if ((a.part_pz == nullptr) != (a.part_sq == nullptr)) return hipErrorInvalidValue;
  if (a.x_dtype == DT_BF16 && a.w_dtype == DT_BF16) return a.w_vh ? launch_stage<BF16, true>(a, s) : launch_stage<BF16, false>(a, s);
  if (a.x_dtype == DT_F16 && a.w_dtype == DT_F16) return a.w_vh ? launch_stage<F16, true>(a, s) : launch_stage<F16, false>(a, s);
  return hipErrorInvalidValue;
}

}  // namespace lce
