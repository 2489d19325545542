// Forward of the fused linear + cross-entropy operator on gfx950.
//
// fwd_tiles_kernel computes one 256(v) x 256(token) tile of the scaled logits
// z = logit_scale * x W with MFMA and reduces it, in registers, to per-token
// partials over each 128-column slice: logsumexp, and when monitoring is on
// the slice max, sum softmax*z and sum z^2.  The logit of the target column is
// written by the one lane that holds it.  No logits reach memory.  (The
// reference kernel, linear_cross_entropy/ops.py:190-236, computes the same
// per-tile lse but also stores the fp32 logits, ops.py:216.)
//
// fwd_rows_kernel merges the slice partials of each token into its lse and
// forms the per-token loss terms (ops.py:753-761); fwd_final_kernel sums them
// in a fixed order into the five scalars of ops.py:802 and the valid-label
// count of ops.py:705.  All reductions are order-deterministic.
#include "lce_gemm3.h"
#include "lce_internal.h"

namespace lce {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f;

LCE_DEV float fast_exp2(float v) { return __builtin_amdgcn_exp2f(v); }
LCE_DEV float fast_log(float v) { return __builtin_amdgcn_logf(v) * kLn2; }

// Reduces the finished 256(v) x 256(token) accumulator of tile (tp, tq) to the
// per-slice partials.  Accumulator rows (v) lie along registers and columns
// (tokens) along lanes, so each lane reduces its own tokens in registers and
// meets the other half of the vocabulary slice in lane ^ 32.
//
// VTAIL is the variant for the one tile column that straddles V (V % 256 != 0).
// A register quad covers 4 columns of a run of 8 (lanes l and l+32 hold the two
// halves), so every run but at most one is inside or outside the vocabulary as a
// whole, uniformly over the wave, and is taken or skipped with a scalar branch;
// the one run that V cuts through is handled element by element.
// MON: the monitoring partials (slice max, sum softmax*z, sum z^2) are formed as well.
template <class T, bool VTAIL, bool MON>
LCE_DEV void fwd_epilogue(const FwdArgs& a, int64_t rows, f32x16_t (&acc)[kNB][kNB], int tp, int tq) {
  const int64_t v0 = (int64_t)tp * kTile, t0 = (int64_t)tq * kTile;  // t0: inside the chunk of rows of this launch
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  const int64_t slice_v0 = v0 + wp * kWaveTile;
  // columns of this wave's slice inside the vocabulary: nq whole runs of 8, then `cut` more columns
  const int64_t left = a.V - slice_v0;
  const int vrem = VTAIL ? (int)(left < 0 ? 0 : (left > kWaveTile ? kWaveTile : left)) : kWaveTile;
  const int nq = vrem >> 3, cut = vrem & 7;
  const int mine = cut - 4 * (lane >> 5);  // elements of this lane's quad of the cut run that exist (<= 0: none)

  const float c1 = a.scale * kLog2e;
  const int64_t slice = slice_v0 / kChunkV;
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    const int64_t tokl = t0 + wq * kWaveTile + qb * kBlk + (lane & 31);  // row inside the chunk
    const int64_t tok = a.row0 + tokl;
    const int64_t o = slice * a.nc + tokl;
    if (VTAIL && vrem == 0) {  // nothing of this slice exists
      if (lane < 32) {
        a.part_lse[o] = -INFINITY;
        if (MON) {
          a.part_max[o] = -INFINITY;
          a.part_pz[o] = 0.f;
          a.part_sq[o] = 0.f;
        }
      }
      continue;
    }
    // Column of the target inside this wave's 128-wide slice, or -1.
    const int64_t yy = tok < rows ? a.y[tok] : a.ignore_index;
    const int64_t rel = yy - slice_v0;
    const int yl = (yy != a.ignore_index && rel >= 0 && rel < kWaveTile) ? (int)rel : -1;

    float m = -INFINITY;
#pragma unroll
    for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq)
        if (!VTAIL || pb * 4 + rq < nq) {
#pragma unroll
          for (int j = 0; j < 4; ++j) m = fmaxf(m, acc[pb][qb][rq * 4 + j]);
        } else if (pb * 4 + rq == nq && cut != 0) {
#pragma unroll
          for (int j = 0; j < 4; ++j) m = j < mine ? fmaxf(m, acc[pb][qb][rq * 4 + j]) : m;
        }
    m = fmaxf(m, __shfl_xor(m, 32));
    m *= a.scale;  // logit_scale > 0, so max commutes with the scaling
    const float mo = m * kLog2e;
    float s = 0.f, pz = 0.f, sq = 0.f;
    if (MON) {
#pragma unroll
      for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq)
          if (!VTAIL || pb * 4 + rq < nq) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const float e = fast_exp2(fmaf(acc[pb][qb][rq * 4 + j], c1, -mo));
              const float z = acc[pb][qb][rq * 4 + j] * a.scale;
              s += e;
              pz = fmaf(e, z, pz);
              sq = fmaf(z, z, sq);
            }
          } else if (pb * 4 + rq == nq && cut != 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const float e = fast_exp2(fmaf(acc[pb][qb][rq * 4 + j], c1, -mo));
              const float z = acc[pb][qb][rq * 4 + j] * a.scale;
              s += j < mine ? e : 0.f;
              pz = j < mine ? fmaf(e, z, pz) : pz;
              sq = j < mine ? fmaf(z, z, sq) : sq;
            }
          }
      pz += __shfl_xor(pz, 32);
      sq += __shfl_xor(sq, 32);
    } else {
#pragma unroll
      for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq)
          if (!VTAIL || pb * 4 + rq < nq) {
#pragma unroll
            for (int j = 0; j < 4; ++j) s += fast_exp2(fmaf(acc[pb][qb][rq * 4 + j], c1, -mo));
          } else if (pb * 4 + rq == nq && cut != 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              const float e = fast_exp2(fmaf(acc[pb][qb][rq * 4 + j], c1, -mo));
              s += j < mine ? e : 0.f;
            }
          }
    }
    s += __shfl_xor(s, 32);
    if (lane < 32) {
      a.part_lse[o] = m + fast_log(s);
      if (MON) {
        a.part_max[o] = m;
        a.part_pz[o] = pz / s;
        a.part_sq[o] = sq;
      }
    }
    if (yl >= 0 && ((yl >> 2) & 1) == (lane >> 5)) {
      const int want_pb = yl >> 5, want_r = ((yl >> 3) & 3) * 4 + (yl & 3);
      float zt = 0.f;
#pragma unroll
      for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (pb == want_pb && r == want_r) zt = acc[pb][qb][r];
      a.tgt[tok] = zt * a.scale;
    }
  }
}


// The logit of the target column, written by the one lane that holds it (rare: a wave holds the target of
// one token in a thousand at a vocabulary of 131072).  `yl`: the column inside this wave's 128-wide slice if
// this lane's half holds it, else -1.
LCE_DEV void fwd_store_target(const FwdArgs& a, f32x16_t (&acc)[kNB][kNB], int64_t tok, int qb, int yl) {
  if (yl >= 0) {
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
    a.tgt[tok] = zt * a.scale;
  }
}

// The same reduction for the kernels whose last K tile is multiplied column by column (Pipe3::step_last_columns:
// all but the tile column that straddles V): one block column of the accumulator at a time -- 32 tokens along the lanes, this
// wave's 128 vocabulary entries of each token in 4 x 16 registers of lanes l and l + 32 -- cut into 16 slots of
// straight-line code that run behind the matrix instructions of the next column.  A lane folds its 64 values
// in two chunks of 32 (slots 8c .. 8c + 7 of chunk c) into a running (max, sum of exp2) pair, so that only 32
// accumulator values are in vector registers at a time, and meets the other half of the slice in lane ^ 32.
struct FwdColumnState {
  float v[32];   // the chunk being summed
  float m, s;    // running max (unscaled logits) and sum of exp2(scaled logit - scaled max)
  float mo;      // scaled max of the chunk being summed
  float e[4], f; // exponentials of the last slot, not yet added; factor for the sum at a chunk change
  float pz, sq;  // monitoring: sum exp2(..) * scaled logit (moves with the max like s) and sum of squared scaled logits
};
// Slot 0..15 of block column QB: the running (max, sum) of this lane's 64 values -- and, MON, the two monitoring
// sums, which leave the arithmetic on (max, sum) as it is, so that the loss does not depend on the monitoring flag
// bit for bit.  The exponentials of a slot are added up in the next one, when they are there.
template <int QB, bool MON>
LCE_DEV void fwd_slot_sum(const FwdArgs& a, FwdColumnState& st, f32x16_t (&acc)[kNB][kNB], int slot) {
  const float c1 = a.scale * kLog2e;
  const int c = slot >> 3, sub = slot & 7;  // chunk c: accumulator blocks 2c, 2c + 1, slots 8c .. 8c + 7
  if (slot > 0) {
    st.s += (st.e[0] + st.e[1]) + (st.e[2] + st.e[3]);
    if (MON) {
      const int prev = 4 * ((slot - 1) & 7);  // (the chunk of the previous slot is still in st.v)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float z = st.v[prev + r] * a.scale;
        st.pz = fmaf(st.e[r], z, st.pz);
        st.sq = fmaf(z, z, st.sq);
      }
    }
  }
  if (sub == 0) {
#pragma unroll
    for (int r = 0; r < 32; ++r) st.v[r] = acc[2 * c + (r >> 4)][QB][r & 15];
    float cm = st.v[0];
#pragma unroll
    for (int r = 1; r < 32; ++r) cm = fmaxf(cm, st.v[r]);
    const float mn = c == 0 ? cm : fmaxf(st.m, cm);
    st.mo = mn * c1;  // logit_scale > 0, so max commutes with the scaling
    if (c == 0) {
      st.s = 0.f;
      if (MON) st.pz = st.sq = 0.f;
    } else {
      st.f = fast_exp2(fmaf(st.m, c1, -st.mo));  // moves the sums to the new max
      st.s *= st.f;
      if (MON) st.pz *= st.f;
    }
    st.m = mn;
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) st.e[r] = fast_exp2(fmaf(st.v[4 * sub + r], c1, -st.mo));
  if (slot == 15) {
    st.s += (st.e[0] + st.e[1]) + (st.e[2] + st.e[3]);
    if (MON) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float z = st.v[28 + r] * a.scale;
        st.pz = fmaf(st.e[r], z, st.pz);
        st.sq = fmaf(z, z, st.sq);
      }
    }
  }
}
// After slot 15: the other half of the slice.  Leaves the slice's max (unscaled) in st.m, its sum of exp2 in st.s
// and, MON, the slice's monitoring sums in st.pz, st.sq.
template <bool MON>
LCE_DEV void fwd_merge_halves(const FwdArgs& a, FwdColumnState& st) {
  const float c1 = a.scale * kLog2e;
  // after the swaps both lanes of a pair hold the lower lane's value in [0] and the upper lane's in [1]
  const unsigned mb = __builtin_bit_cast(unsigned, st.m), sb = __builtin_bit_cast(unsigned, st.s);
  const auto mm = __builtin_amdgcn_permlane32_swap(mb, mb, false, false);
  const auto ss = __builtin_amdgcn_permlane32_swap(sb, sb, false, false);
  // (elements copied to scalars first: a bit cast applied to a vector element reads element 0 whichever is named)
  const unsigned m0u = mm[0], m1u = mm[1], s0u = ss[0], s1u = ss[1];
  const float m0 = __builtin_bit_cast(float, m0u), m1 = __builtin_bit_cast(float, m1u);
  const float s0 = __builtin_bit_cast(float, s0u), s1 = __builtin_bit_cast(float, s1u);
  const float mt = fmaxf(m0, m1), mo = mt * c1;
  const float f0 = fast_exp2(fmaf(m0, c1, -mo)), f1 = fast_exp2(fmaf(m1, c1, -mo));
  st.s = s0 * f0 + s1 * f1;
  st.m = mt;
  if (MON) {
    const unsigned pb = __builtin_bit_cast(unsigned, st.pz), qb = __builtin_bit_cast(unsigned, st.sq);
    const auto pp = __builtin_amdgcn_permlane32_swap(pb, pb, false, false);
    const auto qq = __builtin_amdgcn_permlane32_swap(qb, qb, false, false);
    const unsigned p0u = pp[0], p1u = pp[1], q0u = qq[0], q1u = qq[1];
    st.pz = __builtin_bit_cast(float, p0u) * f0 + __builtin_bit_cast(float, p1u) * f1;
    st.sq = __builtin_bit_cast(float, q0u) + __builtin_bit_cast(float, q1u);
  }
}
template <class T, int QB, bool MON>
LCE_DEV void fwd_epilogue_slot(const FwdArgs& a, FwdColumnState& st, f32x16_t (&acc)[kNB][kNB], int tp, int tq, int slot) {
  fwd_slot_sum<QB, MON>(a, st, acc, slot);
  if (slot == 15) {
    fwd_merge_halves<MON>(a, st);
    // one store per token and partial: the upper lanes get an offset that the range check of the buffer store drops
    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int64_t slice = ((int64_t)tp * kTile + (wave & 1) * kWaveTile) / kChunkV;
    const int64_t o = slice * a.nc + (int64_t)tq * kTile + (wave >> 1) * kWaveTile + QB * kBlk;
    const int voff = lane < 32 ? lane * 4 : (int)0x80000000;
    auto store = [&](float* base, float v) {
      const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(base + o, 0, kBlk * 4, 0x00020000);
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), rsrc, voff, 0, 0);
    };
    store(a.part_lse, fmaf(st.m, a.scale, fast_log(st.s)));
    if (MON) {
      store(a.part_max, st.m * a.scale);
      store(a.part_pz, st.pz / st.s);
      store(a.part_sq, st.sq);
    }
  }
}

// Persistent workgroups, operand stream pipelined across output tiles.  The
// launch covers `tiles_p` tile columns of the vocabulary window [v0, v0 + vw)
// starting at its column tile `tp0` (all full columns, or the one straddling V
// for the VTAIL variant).  The token rows are those of x, or -- when the tokens with ignored
// labels were packed away -- the first `rows` rows of the packed copy (the count lives on the device).
// WVH: the weight is stored (V, H) row-major, so that the P operand runs along K in memory like x does.
template <class T, bool VTAIL, bool KMASK, bool WVH, bool MON> struct FwdProblem {
  typedef typename elem_of<T>::type E;
  static constexpr bool kKMask = KMASK;
  static constexpr bool kSwapAB = false;
  static constexpr bool kVarK = false;
  static constexpr bool kQBlocked = false;
  static constexpr bool kColumnEpilogue = !VTAIL;
  const FwdArgs& a;
  int64_t rows, ldx;
  const E* x;
  int tp0, tiles_p, tiles_q;
  LCE_DEV FwdProblem(const FwdArgs& a_)
      : a(a_), tp0(VTAIL ? (int)(a_.vw / kTile) : 0), tiles_p(VTAIL ? 1 : (int)(a_.vw / kTile)) {
    rows = a.n_rows ? packed_rows(a.n_rows, a.N) : a.N;
    const bool packed = rows != a.N;
    x = reinterpret_cast<const E*>(packed ? a.xc : a.x);
    ldx = packed ? a.ldxc : a.ldx;
    // rows of this launch's chunk that exist
    int64_t here = rows - a.row0;
    here = here < 0 ? 0 : (here > a.nc ? a.nc : here);
    tiles_q = (int)((here + kTile - 1) / kTile);
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
    q = x + (a.row0 + (int64_t)tq * kTile) * ldx;
  }
  LCE_DEV const void* p_end() const {
    return WVH ? matrix_end<E>(a.w, a.Vw, a.ldw, a.H) : matrix_end<E>(a.w, a.H, a.ldw, a.Vw);
  }
  LCE_DEV const void* q_end() const { return matrix_end<E>(x, rows, ldx, a.H); }
  LCE_DEV int k_valid(int) const { return (int)a.H; }
  // Column epilogue: the labels of this lane's four tokens are fetched three K tiles ahead.
  int64_t pf_y[kNB];
  int etp, etq;
  LCE_DEV void prefetch(int tile) {
    if constexpr (kColumnEpilogue) {
      int tp, tq;
      coords(tile, tp, tq);
      const int lane = threadIdx.x & 63, wq = threadIdx.x >> 7;
#pragma unroll
      for (int qb = 0; qb < kNB; ++qb) {
        const int64_t tok = a.row0 + (int64_t)tq * kTile + wq * kWaveTile + qb * kBlk + (lane & 31);
        pf_y[qb] = tok < rows ? a.y[tok] : a.ignore_index;
      }
    }
  }
  LCE_DEV void epilogue_begin(int tile, char*) {
    coords(tile, etp, etq);
    etp += (int)(a.v0 / kTile);
  }
  FwdColumnState est;
  template <int J> LCE_DEV void epilogue_slot(int, f32x16_t (&acc)[kNB][kNB], int slot, char*) {
    fwd_epilogue_slot<T, J, MON>(a, est, acc, etp, etq, slot);
  }
  LCE_DEV void epilogue_end(int, f32x16_t (&acc)[kNB][kNB], char*) const {
    const int tid = opaque_tid();
    const int lane = tid & 63, wave = tid >> 6;
    const int64_t slice_v0 = (int64_t)etp * kTile + (wave & 1) * kWaveTile;
#pragma unroll
    for (int qb = 0; qb < kNB; ++qb) {
      const int64_t tok = a.row0 + (int64_t)etq * kTile + (wave >> 1) * kWaveTile + qb * kBlk + (lane & 31);
      const int64_t yy = pf_y[qb], rel = yy - slice_v0;
      const bool here = yy != a.ignore_index && rel >= 0 && rel < kWaveTile && ((rel >> 2) & 1) == (lane >> 5);
      fwd_store_target(a, acc, tok, qb, here ? (int)rel : -1);
    }
  }
  LCE_DEV void epilogue(int tile, f32x16_t (&acc)[kNB][kNB], char*) const {
    int tp, tq;
    coords(tile, tp, tq);
    fwd_epilogue<T, VTAIL, MON>(a, rows, acc, (int)(a.v0 / kTile) + tp, tq);
  }
};

template <class T, bool VTAIL, bool KMASK, bool WVH, bool MON>
__global__ __launch_bounds__(kThreads) void fwd_tiles_persistent_kernel(const FwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  typedef typename elem_of<T>::type E;
  FwdProblem<T, VTAIL, KMASK, WVH, MON> prob(a);
  Pipe3<T, E, WVH, E, true, FwdProblem<T, VTAIL, KMASK, WVH, MON>> pipe(prob);
  pipe.run(a.ldw, prob.ldx, (int)(padded_k(a.H) / kBK), lds);
}

// One workgroup = 64 tokens x 4 strided groups of slices.
__global__ __launch_bounds__(256) void fwd_rows_kernel(const FwdArgs a) {
  __shared__ float sh_m[4][kMergeRows], sh_s[4][kMergeRows], sh_lse[kMergeRows];
  __shared__ float sh_pz[4][kMergeRows], sh_sq[4][kMergeRows], sh_mx[4][kMergeRows];
  __shared__ double sh_red[7][kMergeRows];
  const int r = threadIdx.x & 63, g = threadIdx.x >> 6;
  const int64_t tokl = (int64_t)blockIdx.x * kMergeRows + r;  // row inside the chunk of this launch
  const int64_t tok = a.row0 + tokl;  // < Np; rows that do not exist only keep the block sums aligned
  const int64_t rows = a.n_rows ? packed_rows(a.n_rows, a.N) : a.N;
  const bool exists = tok < rows;
  // packed rows: lse goes back to the token's own place; tokens that were dropped get 0 (as every token with an
  // ignored label does, below)
  if (a.perm != nullptr && g == 1 && tok < a.N && a.y0[tok] == a.ignore_index) a.lse[tok] = 0.f;
  const int nslices = (int)(a.Vp / kChunkV);

  // Online (max, sum) merge of this group's slices, 8 at a time so that the loads of a
  // batch are in flight together (a slice without a single valid column holds -inf and
  // contributes exp2(-inf) = 0).
  float M = -INFINITY, S = 0.f;
  for (int c0 = g; c0 < nslices; c0 += 32) {
    float l[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int c = c0 + 4 * u;
      l[u] = c < nslices ? a.part_lse[(int64_t)c * a.nc + tokl] : -INFINITY;
    }
    float mb = l[0];
#pragma unroll
    for (int u = 1; u < 8; ++u) mb = fmaxf(mb, l[u]);
    if (mb == -INFINITY) continue;
    float sb = 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) sb += fast_exp2((l[u] - mb) * kLog2e);
    const float Mn = fmaxf(M, mb);
    S = S * fast_exp2((M - Mn) * kLog2e) + sb * fast_exp2((mb - Mn) * kLog2e);
    M = Mn;
  }
  sh_m[g][r] = M;
  sh_s[g][r] = S;
  __syncthreads();
  if (g == 0) {
    float Mt = fmaxf(fmaxf(sh_m[0][r], sh_m[1][r]), fmaxf(sh_m[2][r], sh_m[3][r]));
    float St = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (sh_s[i][r] != 0.f) St += sh_s[i][r] * fast_exp2((sh_m[i][r] - Mt) * kLog2e);
    const float lse = Mt + fast_log(St);
    sh_lse[r] = lse;
    if (a.lse_rows != nullptr) a.lse_rows[tok] = lse;
    // lse[i] of a token with an ignored label is 0, whether its row was computed (all rows are when they are not
    // packed) or not: a caller sees one thing.  (sh_lse keeps the value: logit_entropy is taken over valid rows only,
    // and the backward never looks at the lse of such a token.)
    if (exists) a.lse[a.perm != nullptr ? packed_token(a.perm, tok, a.N) : tok] = a.y[tok] != a.ignore_index ? lse : 0.f;
  }
  __syncthreads();
  const float lse = sh_lse[r];
  if (a.monitoring) {
    float pz = 0.f, sq = 0.f, mx = -INFINITY;
    for (int c0 = g; c0 < nslices; c0 += 32) {
      float pl[8], pp[8], ps[8], pm[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int c = c0 + 4 * u;
        const bool in = c < nslices;
        const int64_t o = (int64_t)(in ? c : 0) * a.nc + tokl;
        pl[u] = in ? a.part_lse[o] : -INFINITY;
        pp[u] = in ? a.part_pz[o] : 0.f;
        ps[u] = in ? a.part_sq[o] : 0.f;
        pm[u] = in ? a.part_max[o] : -INFINITY;
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        pz = fmaf(pp[u], fast_exp2((pl[u] - lse) * kLog2e), pz);
        sq += ps[u];
        mx = fmaxf(mx, pm[u]);
      }
    }
    sh_pz[g][r] = pz;
    sh_sq[g][r] = sq;
    sh_mx[g][r] = mx;
  }
  __syncthreads();
  if (g == 0) {
    const bool valid = exists && a.y[tok] != a.ignore_index;
    const double l = (double)lse;
    double ent = 0.0, nrm = 0.0, mx = -INFINITY;
    if (a.monitoring && exists) {
      const float pz = (sh_pz[0][r] + sh_pz[1][r]) + (sh_pz[2][r] + sh_pz[3][r]);
      const float sq = (sh_sq[0][r] + sh_sq[1][r]) + (sh_sq[2][r] + sh_sq[3][r]);
      mx = (double)fmaxf(fmaxf(sh_mx[0][r], sh_mx[1][r]), fmaxf(sh_mx[2][r], sh_mx[3][r]));
      ent = valid ? (double)(lse - pz) : 0.0;
      nrm = (double)sqrtf(sq);
    }
    // tgt[tok] is written by the one tile that holds the target column; it is only read for a valid
    // label (for a valid label outside [0, V) nothing wrote it -- and the loss is NaN anyway)
    sh_red[0][r] = valid ? l - (double)a.tgt[tok] : 0.0;
    sh_red[1][r] = valid ? l * l : 0.0;
    sh_red[2][r] = ent;
    sh_red[3][r] = nrm;
    sh_red[4][r] = mx;
    sh_red[5][r] = valid ? 1.0 : 0.0;
    // a label that is neither ignore_index nor a column of W: poisons the loss (see fwd_final_kernel)
    sh_red[6][r] = (valid && (a.y[tok] < 0 || a.y[tok] >= a.V)) ? 1.0 : 0.0;
  }
  __syncthreads();
  if (threadIdx.x < 7) {
    const int q = threadIdx.x;
    double acc = sh_red[q][0];
    for (int i = 1; i < kMergeRows; ++i) acc = (q == 4) ? fmax(acc, sh_red[q][i]) : acc + sh_red[q][i];
    reinterpret_cast<double*>(a.blk)[(a.row0 / kMergeRows + (int64_t)blockIdx.x) * 8 + q] = acc;
  }
}

__global__ __launch_bounds__(256) void fwd_final_kernel(const FwdArgs a) {
  __shared__ double sh[7][256];
  const int nblk = (int)(a.Np / kMergeRows);
  const double* blk = reinterpret_cast<const double*>(a.blk);
  double v[7] = {0, 0, 0, 0, -INFINITY, 0, 0};
  for (int b = threadIdx.x; b < nblk; b += 256) {
#pragma unroll
    for (int q = 0; q < 7; ++q) {
      const double t = blk[(int64_t)b * 8 + q];
      v[q] = (q == 4) ? fmax(v[q], t) : v[q] + t;
    }
  }
#pragma unroll
  for (int q = 0; q < 7; ++q) sh[q][threadIdx.x] = v[q];
  __syncthreads();
  for (int w = 128; w > 0; w >>= 1) {
    if (threadIdx.x < w) {
#pragma unroll
      for (int q = 0; q < 7; ++q) {
        const double t = sh[q][threadIdx.x + w];
        sh[q][threadIdx.x] = (q == 4) ? fmax(sh[q][threadIdx.x], t) : sh[q][threadIdx.x] + t;
      }
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    const double R = sh[5][0];  // 0 valid labels -> 0/0 = NaN, as F.cross_entropy gives
    const double ce = sh[0][0] / R, zr = sh[1][0] / R;
    // Labels outside [0, V) that are not ignore_index have no column to match; the reference lets
    // them contribute lse alone, silently.  Here they turn the loss into NaN (F.cross_entropy
    // raises a device-side assert for them) -- visible to the caller, no synchronisation needed.
    const bool bad_labels = sh[6][0] != 0.0;
    a.out5[0] = bad_labels ? __builtin_nanf("") : (float)(ce + (double)a.z_reg * zr);
    a.out5[1] = (float)zr;
    a.out5[2] = a.monitoring ? (float)sh[4][0] : 0.f;
    a.out5[3] = a.monitoring ? (float)(sh[2][0] / R) : 0.f;
    a.out5[4] = a.monitoring ? (float)(sh[3][0] / (double)a.N) : 0.f;
    a.n_valid[0] = (int64_t)R;
  }
}

template <class T, bool VTAIL, bool KMASK, bool WVH, bool MON>
hipError_t launch_one(const FwdArgs& a, int64_t tiles, hipStream_t s) {
  auto kern = fwd_tiles_persistent_kernel<T, VTAIL, KMASK, WVH, MON>;
  static LdsOptIn optin;
  hipError_t e = optin.ensure(reinterpret_cast<const void*>(kern), kMainloopLds);
  if (e != hipSuccess) return e;
  const int grid = (int)(tiles < a.num_cus ? tiles : a.num_cus);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), kMainloopLds, s, a);
  return hipGetLastError();
}

// All full tile columns of the vocabulary, then the column that straddles V.
template <class T, bool WVH, bool MON> hipError_t launch_persistent(const FwdArgs& a, hipStream_t s) {
  const int64_t left = a.Np - a.row0;  // token tiles of this chunk at most
  const int64_t tq = (left < a.nc ? left : a.nc) / kTile, full = a.vw / kTile;
  const bool exact_k = padded_k(a.H) == a.H;  // the K tiles cover H exactly: no K mask needed
  if (full > 0) {
    hipError_t e = exact_k ? launch_one<T, false, false, WVH, MON>(a, full * tq, s)
                           : launch_one<T, false, true, WVH, MON>(a, full * tq, s);
    if (e != hipSuccess) return e;
  }
  if (a.vw % kTile) return launch_one<T, true, true, WVH, MON>(a, tq, s);
  return hipSuccess;
}

template <class T, bool WVH> hipError_t launch_layout(const FwdArgs& a, hipStream_t s) {
  return a.monitoring ? launch_persistent<T, WVH, true>(a, s) : launch_persistent<T, WVH, false>(a, s);
}

}  // namespace

hipError_t launch_fwd_tiles(const FwdArgs& a, hipStream_t s) {
  if (a.x_dtype == DT_BF16 && a.w_dtype == DT_BF16)
    return a.w_vh ? launch_layout<BF16, true>(a, s) : launch_layout<BF16, false>(a, s);
  if (a.x_dtype == DT_F16 && a.w_dtype == DT_F16)
    return a.w_vh ? launch_layout<F16, true>(a, s) : launch_layout<F16, false>(a, s);
  // (an fp32 weight arrives here as a 16-bit slab copy, fp32 activations as the bf16 packed copy)
  return hipErrorInvalidValue;
}

hipError_t launch_fwd_rows(const FwdArgs& a, hipStream_t s) {
  const int64_t left = a.Np - a.row0;
  hipLaunchKernelGGL(fwd_rows_kernel, dim3((unsigned)((left < a.nc ? left : a.nc) / kMergeRows)), dim3(256), 0, s, a);
  return hipGetLastError();
}

hipError_t launch_fwd_final(const FwdArgs& a, hipStream_t s) {
  hipLaunchKernelGGL(fwd_final_kernel, dim3(1), dim3(256), 0, s, a);
  return hipGetLastError();
}

}  // namespace lce
