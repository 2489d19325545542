// Backward, step 1: recompute a 256(v) x 256(token) logit tile with the same
// MFMA main loop as the forward (so the logits are bit-identical to the ones
// the saved lse was built from) and turn it, in registers, into
//     dz = softmax * (1 + 2*z_reg*lse) - onehot(y),   0 for ignored tokens
// (times 2^dz_shift, a power of two that keeps small probabilities in fp16's normal range)
// (linear_cross_entropy/ops.py:309-314 and 415-422), rounded once to the
// 16-bit compute type exactly where the reference casts dz before its dot
// products (ops.py:314, 422).  The tile is transposed through LDS and written
// to the row-major staging buffer dz[N][vs] of the current vocabulary slab as
// full 128-byte lines.  The kernel is persistent (one workgroup per CU, operand
// stream pipelined across tiles); fp32 operands are converted on the way into LDS.
#include "lce_gemm3.h"
#include "lce_internal.h"

namespace lce {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kPassCols = 64;                        // columns staged per pass
constexpr int kSliceBytes = kWaveTile * kPassCols * 2;  // one wave's staging slice: 128 rows of 128 bytes
constexpr int kLdsBytes = kMainloopLds;  // the epilogue stages through main-loop stage 1, idle by then
static_assert(4 * kSliceBytes <= kLdsBytes - kStageBytes, "four wave slices must fit beside one stage");

// Turns the finished logit tile (tp, tq) into dz and writes it out.
//
// Each lane owns 4 tokens (columns of the accumulator) x 64 vocabulary entries
// per token, four consecutive entries per register quad; lanes l and l+32 hold
// the two halves of every run of 8 entries.  One v_permlane32_swap per pair of
// register quads hands each lane a full run of 8 (16 bytes in the 16-bit
// staging type).  A wave stages its own 128(token) x 128(v) sub-tile through a
// private slice of `scratch` in two passes of 64 columns and reads it back as
// whole 128-byte rows, so dz leaves the CU as full lines; no other wave is
// involved, hence no workgroup barrier until the very end.  Staging rows are
// 128 bytes with the 16-byte chunk index XOR-ed by (row & 7) ^ ((row >> 3) & 1),
// the swizzle of the K-contiguous operand tiles, for the 16-byte writes (32
// rows per instruction) and the row reads (8 rows per instruction).
//   * ignored tokens use lse = +inf, which makes every exp2 an exact +0;
//   * the "- onehot" is applied by the one lane that owns the target column,
//     from the fp32 value, onto the staged pass (one rounding, as in
//     ops.py:313-314).
//
// VTAIL is the variant for the one tile column that straddles the end of the
// vocabulary: every run of 8 columns (a pair of register quads in lanes l, l+32)
// but at most one is inside or outside as a whole, uniformly over the wave; the
// one run that V cuts through is handled element by element.  Columns outside
// are written as exact zeros.
//
// SPLIT (fp32 tensors carried as bf16 pairs, lce_gemm.h): dz is staged as hi = bf16(dz) and lo = bf16(dz - hi)
// in three blocks of Np rows, [hi ; lo ; hi].  The staging sequence simply runs twice, once per part (this
// path serves accuracy, not speed).
// `pf_y`, `pf_lse`: label and lse of this lane's four tokens (DzProblem::prefetch), ignore_index / 0 for rows that do not exist.
template <class T, bool ZREG, bool VTAIL, bool SPLIT>
LCE_DEV void dz_epilogue_impl(const BwdArgs& a, const int64_t (&pf_y)[kNB], const float (&pf_lse)[kNB],
                              f32x16_t (&acc)[kNB][kNB], int tp, int tq, char* scratch) {
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
  char* mine = scratch + wave * kSliceBytes;
  E* out = reinterpret_cast<E*>(a.dz) + (t0 + wq * kWaveTile) * a.vs + (int64_t)tp * kTile + wp * kWaveTile;

  // per-token scalars of this lane's four tokens
  float nlse[kNB], gain[kNB];
  int ykey[kNB];
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    const int64_t yy = pf_y[qb];  // (rows past the last one are staged as zeros, like ignored tokens)
    const int64_t rel = yy - slice_v0;
    const bool valid = yy != a.ignore_index;
    const float l = pf_lse[qb];
    // (the power-of-two factor of the staged dz rides along in the exponent)
    nlse[qb] = valid ? fmaf(-l, kLog2e, (float)a.dz_shift) : -INFINITY;
    gain[qb] = 1.f + 2.f * a.z_reg * l;
    // target column inside this wave's slice, only in the lane half that holds it
    ykey[qb] = (valid && rel >= 0 && rel < kWaveTile && ((rel >> 2) & 1) == half) ? (int)rel : -1;
  }

  const int64_t blk = a.Np * a.vs;  // SPLIT: elements between the three blocks of the stage
#pragma unroll
  for (int part = 0; part < (SPLIT ? 2 : 1); ++part) {
  // (SPLIT: an opaque copy of the scale per part, so that the compiler recomputes the exponentials of part 1 instead of
  // keeping all 256 of part 0 alive across the staging of that part, which spilled 2 KiB per lane)
  float c1p = c1;
  if (SPLIT) asm volatile("" : "+v"(c1p));
#pragma unroll
  for (int ph = 0; ph < 2; ++ph) {
#pragma unroll
    for (int qb = 0; qb < kNB; ++qb) {
      const int row = qb * kBlk + (lane & 31);
      char* lrow = mine + row * (kPassCols * 2);
      const int sw = (row & 7) ^ ((row >> 3) & 1);
#pragma unroll
      for (int pp = 0; pp < 2; ++pp) {
        const int pb = 2 * ph + pp;
#pragma unroll
        for (int g = 0; g < 4; g += 2) {
          float d[8];
#pragma unroll
          for (int h2 = 0; h2 < 2; ++h2) {
            if (!VTAIL || pb * 4 + g + h2 < nq) {
#pragma unroll
              for (int i = 4 * h2; i < 4 * h2 + 4; ++i) {
                d[i] = __builtin_amdgcn_exp2f(fmaf(acc[pb][qb][g * 4 + i], c1p, nlse[qb]));
                if (ZREG) d[i] *= gain[qb];
              }
            } else if (pb * 4 + g + h2 == nq && cut != 0) {
#pragma unroll
              for (int i = 4 * h2; i < 4 * h2 + 4; ++i) {
                d[i] = __builtin_amdgcn_exp2f(fmaf(acc[pb][qb][g * 4 + i], c1p, nlse[qb]));
                if (ZREG) d[i] *= gain[qb];
                d[i] = (i - 4 * h2) < cut_mine ? d[i] : 0.f;
              }
            } else {
#pragma unroll
              for (int i = 4 * h2; i < 4 * h2 + 4; ++i) d[i] = 0.f;
            }
          }
          if (SPLIT && part == 1) {
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
          const int chunk = pp * 4 + g + half;  // 16-byte chunk of the 64-column pass
          *reinterpret_cast<u32x4_t*>(lrow + ((chunk ^ sw) << 4)) = o;
        }
      }
      // the target column, if it falls into this pass: overwrite the staged value
      // with the rounding of the fp32 (p - 1), as ops.py:313-314 rounds once
      const int yl = ykey[qb] - ph * kPassCols;
      if (yl >= 0 && yl < kPassCols) {
        const int want = (yl >> 5) * 16 + ((yl >> 3) & 3) * 4 + (yl & 3);  // (pp, register) index
        float zt = 0.f;
#pragma unroll
        for (int pp = 0; pp < 2; ++pp)
#pragma unroll
          for (int r = 0; r < 16; ++r)
            if (want == pp * 16 + r) zt = acc[2 * ph + pp][qb][r];
        float p = __builtin_amdgcn_exp2f(fmaf(zt, c1p, nlse[qb]));
        if (ZREG) p *= gain[qb];
        float tv = p - __builtin_bit_cast(float, (127 + a.dz_shift) << 23);  // the one, times 2^dz_shift
        if (SPLIT && part == 1) tv = bf16_lo(tv);
        *reinterpret_cast<unsigned short*>(lrow + (((yl >> 3) ^ sw) << 4) + (yl & 7) * 2) = to_bits<T>(tv);
      }
      // keep the register footprint small: an operand tile is in flight across this function
      __builtin_amdgcn_sched_barrier(0);
    }
    // read the pass back as 128-byte rows and send it out
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      // 8 rows per instruction, 8 lanes each; the upper 32 lanes take their four rows in the order
      // 5, 4, 7, 6 so that lanes l and l+32 always sit in rows of opposite parity (opposite bank halves)
      const int row = i * 8 + (lane >> 3) + ((lane >> 5) ? 1 - 2 * ((lane >> 3) & 1) : 0), chunk = lane & 7;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(mine + row * (kPassCols * 2) + ((chunk ^ (row & 7) ^ ((row >> 3) & 1)) << 4));
      // streaming store: dz (1 GiB per slab) is read back from HBM by the next kernels anyway, and a
      // normal store would evict the W / x tiles the following main loop is about to reuse from L2
      E* dst = out + (int64_t)row * a.vs + ph * kPassCols + chunk * 8 + (SPLIT && part == 1 ? blk : 0);
      __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>(dst));
      if (SPLIT && part == 0) __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>(dst + 2 * blk));
      if ((i & 3) == 3) __builtin_amdgcn_sched_barrier(0);  // at most 4 rows in registers at a time
    }
  }
  }
  __syncthreads();  // scratch is handed back to the main loop
}

// ZREG (z_regularization != 0) is a compile-time switch of the kernels rather than a
// branch inside them: with a branch the compiler hoists the accumulator reads of
// both arms above it and needs every vector register at once.
// The launch covers `tiles_p` tile columns of the slab starting at column tile
// `tp0`: all the full ones, or (VTAIL) those from the one straddling the end
// of the vocabulary to the end of the padded slab.
// WVH: the weight is stored (V, H) row-major, so that the P operand runs along K in memory like x does.
template <class T, bool ZREG, bool VTAIL, bool KMASK, bool SPLIT, bool WVH> struct DzProblem {
  typedef typename elem_of<T>::type E;
  static constexpr bool kKMask = KMASK;
  static constexpr bool kSwapAB = false;
  static constexpr bool kVarK = false;
  const BwdArgs& a;
  int64_t rows, ldx;  // token rows: all of x, or the packed rows (see BwdArgs)
  const E* x;
  int tp0, tiles_p, tiles_q;
  LCE_DEV DzProblem(const BwdArgs& a_)
      : a(a_), tp0(VTAIL ? (int)(a_.vw / kTile) : 0),
        tiles_p(VTAIL ? (int)(a_.vs / kTile - a_.vw / kTile) : (int)(a_.vw / kTile)) {
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
  int64_t pf_y[kNB];
  float pf_lse[kNB];
  LCE_DEV void prefetch(int tile) {
    int tp, tq;
    coords(tile, tp, tq);
    const int lane = threadIdx.x & 63, wq = threadIdx.x >> 7;
#pragma unroll
    for (int qb = 0; qb < kNB; ++qb) {
      const int64_t tok = (int64_t)tq * kTile + wq * kWaveTile + qb * kBlk + (lane & 31);
      const bool exists = tok < rows;
      pf_y[qb] = exists ? a.y[tok] : a.ignore_index;
      pf_lse[qb] = exists ? a.lse[tok] : 0.f;
    }
  }
  LCE_DEV void epilogue(int tile, f32x16_t (&acc)[kNB][kNB], char* scratch) const {
    int tp, tq;
    coords(tile, tp, tq);
    dz_epilogue_impl<T, ZREG, VTAIL, SPLIT>(a, pf_y, pf_lse, acc, tp, tq, scratch);
  }
};

template <class T, bool ZREG, bool VTAIL, bool KMASK, bool SPLIT, bool WVH>
__global__ __launch_bounds__(kThreads) void bwd_dz_persistent_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  typedef typename elem_of<T>::type E;
  DzProblem<T, ZREG, VTAIL, KMASK, SPLIT, WVH> prob(a);
  Pipe3<T, E, WVH, E, true, DzProblem<T, ZREG, VTAIL, KMASK, SPLIT, WVH>> pipe(prob);
  pipe.run(a.ldw, prob.ldx, (int)(padded_k(a.H) / kBK), lds);
}

template <class T, bool ZREG, bool VTAIL, bool KMASK, bool SPLIT, bool WVH>
hipError_t launch_one(const BwdArgs& a, int64_t tiles, hipStream_t s) {
  auto kern = bwd_dz_persistent_kernel<T, ZREG, VTAIL, KMASK, SPLIT, WVH>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes);
  if (e != hipSuccess) return e;
  const int grid = (int)(tiles < a.num_cus ? tiles : a.num_cus);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), kLdsBytes, s, a);
  return hipGetLastError();
}

// All full tile columns of the slab, then the column that straddles the end of the vocabulary.
template <class T, bool ZREG, bool SPLIT, bool WVH> hipError_t launch_persistent_z(const BwdArgs& a, hipStream_t s) {
  const int64_t tq = a.Np / kTile, full = a.vw / kTile, tail = a.vs / kTile - full;
  const bool exact_k = padded_k(a.H) == a.H;  // the K tiles cover H exactly: no K mask needed
  if (full > 0) {
    hipError_t e = exact_k ? launch_one<T, ZREG, false, false, SPLIT, WVH>(a, full * tq, s)
                           : launch_one<T, ZREG, false, true, SPLIT, WVH>(a, full * tq, s);
    if (e != hipSuccess) return e;
  }
  if (tail > 0) return launch_one<T, ZREG, true, true, SPLIT, WVH>(a, tail * tq, s);
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

}  // namespace lce
