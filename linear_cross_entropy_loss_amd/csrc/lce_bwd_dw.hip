// Backward, step 3: dW[h][v] = coef * sum_token x[token][h] * dz[token][v] for
// the columns of one vocabulary slab (the contraction of
// linear_cross_entropy/ops.py:424).  K = token, so both operands are read
// through the LDS transpose path.  A workgroup owns its dW tile over ALL tokens
// (the rows that are left after tokens with an ignored label were packed away):
// the fp32 accumulator never leaves registers and the result is written once
// in the output dtype after scaling by grad_out * logit_scale / n_valid
// (ops.py:443-447, 810).  Only the tiles of a mostly idle last round of
// workgroups are cut along K instead and summed by a second kernel (DwPlan).
#include "lce_gemm3.h"
#include "lce_internal.h"

namespace lce {

namespace {

// `part` != null: this is a K segment of a tail tile (see DwPlan); its raw fp32 sum goes to that
// 256(h) x 256(v) block, through the statements of the fp32 output path (another destination, row
// stride and factor, no bounds) -- a separate code path behind a branch would read the accumulator twice.
template <class T>
LCE_DEV void dw_epilogue(const BwdArgs& a, float* part, f32x16_t (&acc)[kNB][kNB], int tp, int tq) {
  typedef typename elem_of<T>::type E;
  const int64_t vl0 = (int64_t)tp * kTile, h0 = (int64_t)tq * kTile;
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  const bool tail = part != nullptr;
  const float coef = tail ? 1.f : final_factor_of(a);
  // fp32 destination addressed as [h][v] with v counted over the whole vocabulary
  float* f32dst = tail ? part - (h0 * kTile + a.v0 + vl0) : reinterpret_cast<float*>(a.dw);
  const int64_t f32ld = tail ? kTile : a.lddw;
  const int half = lane >> 5;
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    const int64_t h = h0 + wq * kWaveTile + qb * kBlk + (lane & 31);
    const bool row_exists = h < a.H;
#pragma unroll
    for (int pb = 0; pb < kNB; ++pb) {
      const int64_t vb = a.v0 + vl0 + wp * kWaveTile + pb * kBlk;
      // Pieces (4 columns in fp32, 8 in the 16-bit types) that start at or past V are not
      // stored; one that V cuts through is written whole, into the stride padding of its row.
      if (a.dw_dtype == DT_F32 || tail) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          if (!tail && (vb + 8 * rq + 4 * half >= a.V || !row_exists)) continue;
          f32x4_t o;
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = acc[pb][qb][rq * 4 + j] * coef;
          *reinterpret_cast<f32x4_t*>(f32dst + h * f32ld + vb + 8 * rq + 4 * half) = o;
        }
      } else {
        // Lanes l and l+32 hold the two halves of every run of 8 columns; one
        // lane-half swap per pair of register quads gives each lane a whole run,
        // so a store writes 32 contiguous bytes (a full sector) per row of dW.
#pragma unroll
        for (int g = 0; g < 4; g += 2) {
          float d[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) d[i] = acc[pb][qb][g * 4 + i] * coef;
          const unsigned x0 = pack2<T>(d[0], d[1]), x1 = pack2<T>(d[2], d[3]);
          const unsigned y0 = pack2<T>(d[4], d[5]), y1 = pack2<T>(d[6], d[7]);
          const auto s0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
          const auto s1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
          u32x4_t o;
          o[0] = s0[0];
          o[1] = s1[0];
          o[2] = s0[1];
          o[3] = s1[1];
          if (vb + 8 * (g + half) < a.V && row_exists)
            *reinterpret_cast<u32x4_t*>(reinterpret_cast<E*>(a.dw) + h * a.lddw + vb + 8 * (g + half)) = o;
        }
      }
    }
  }
}

// How one launch divides its work: as for dx (lce_bwd_dx.hip).  The T = (vs/256) x (Hp/256) output tiles
// go to G persistent workgroups in rounds; a last round with r <= G/2 tiles is cut along K = tokens into
// `nseg` segments of `kseg` K tiles (r * nseg <= G, at least 16 K tiles each), whose fp32 sums meet in
// 256 x 256 blocks of dw_part and are added, in segment order, by dw_tail_kernel.  With few tiles in all
// (a small vocabulary slab times a small hidden size) every tile is a tail tile.  The K extent comes from
// the row count on the device, so the plan is made there; a last segment that runs past the rows reads zeros.
struct DwPlan {
  int tiles, full, tail_tiles, nseg, kseg, kt;
};
LCE_DEV DwPlan dw_plan(const BwdArgs& a, int64_t rows) {
  DwPlan p;
  const int G = a.dw_grid;
  const int64_t kt2 = (rows + 2 * kBK - 1) / (2 * kBK) * 2;  // K tiles: an even number, at least four, covering the rows
  p.kt = (int)(kt2 < 4 ? 4 : kt2);
  p.tiles = (int)(a.vs / kTile) * (int)(a.Hp / kTile);
  p.full = p.tiles / G * G;
  const int r = p.tiles - p.full, cap = G < kTailBlocks ? G : kTailBlocks;
  int s = 1;
  if (r > 0 && a.dw_part != nullptr)  // (no blocks for partial sums: nothing is split)
    while (r * s * 2 <= cap && p.kt / (s * 2) >= 16) s *= 2;
  if (s == 1) {
    p.full = p.tiles;
    p.tail_tiles = 0;
    p.nseg = 1;
    p.kseg = p.kt;
  } else {
    const int seg = ((p.kt + s - 1) / s + 1) & ~1;  // even
    p.tail_tiles = r;
    p.kseg = seg;
    p.nseg = (p.kt + seg - 1) / seg;
  }
  return p;
}

template <class T> struct DwProblem {
  static constexpr bool kVarK = true;    // whole tiles and segment items have different K extents
  static constexpr bool kKMask = false;  // both operands have K as their slow index: nothing to mask
  typedef typename elem_of<T>::type E;
  const BwdArgs& a;
  int64_t rows, ldx;  // token rows (the K extent): all of x, or the packed rows (see BwdArgs)
  const E* x;
  int tiles_p, tiles_q;
  DwPlan plan;
  LCE_DEV DwProblem(const BwdArgs& a_) : a(a_), tiles_p((int)(a_.vs / kTile)), tiles_q((int)(a_.Hp / kTile)) {
    rows = packed_rows(a.n_rows, a.N);
    const bool packed = rows != a.N;
    x = reinterpret_cast<const E*>(packed ? a.xc : a.x);
    ldx = packed ? a.ldxc : a.ldx;
    plan = dw_plan(a, rows);
  }
  LCE_DEV int num_tiles() const { return plan.full + plan.tail_tiles * plan.nseg; }
  // seg < 0: a whole tile
  LCE_DEV void decode(int item, int& tp, int& tq, int& seg) const {
    int tile = item;
    seg = -1;
    if (item >= plan.full) {
      const int j = item - plan.full;
      tile = plan.full + j / plan.nseg;
      seg = j % plan.nseg;
    }
    tile_coords(tile, plan.tiles, tiles_p, tiles_q, 8, tp, tq);
  }
  LCE_DEV int item_ktiles(int item) const { return item < plan.full ? plan.kt : plan.kseg; }
  LCE_DEV void origins(int item, const void*& p, const void*& q) const {
    int tp, tq, seg;
    decode(item, tp, tq, seg);
    const int64_t k0 = seg < 0 ? 0 : (int64_t)seg * plan.kseg * kBK;  // first token of the segment
    p = reinterpret_cast<const E*>(a.dz) + k0 * a.vs + (int64_t)tp * kTile;
    q = x + k0 * ldx + (int64_t)tq * kTile;
  }
  // dz is written for whole token tiles; x rows past the last one read as zeros
  LCE_DEV const void* p_end() const {
    return reinterpret_cast<const E*>(a.dz) + (rows + kTile - 1) / kTile * kTile * a.vs;
  }
  LCE_DEV const void* q_end() const { return matrix_end<E>(x, rows, ldx, a.H); }
  LCE_DEV int k_valid(int) const { return (int)a.Np; }
  LCE_DEV void epilogue(int item, f32x16_t (&acc)[kNB][kNB], char*) const {
    int tp, tq, seg;
    decode(item, tp, tq, seg);
    float* part = seg >= 0 ? a.dw_part + (int64_t)(item - plan.full) * kTile * kTile : nullptr;
    dw_epilogue<T>(a, part, acc, tp, tq);
  }
};

template <class T>
__global__ __launch_bounds__(kThreads) void bwd_dw_persistent_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  typedef typename elem_of<T>::type E;
  DwProblem<T> prob(a);
  Pipe3<T, E, false, E, false, DwProblem<T>> pipe(prob);
  pipe.run(a.vs, prob.ldx, prob.plan.kt, lds);
}

// Second step for the tail tiles: kTailParts workgroups share tail tile b (16 rows of h each) -- they sum
// its segments in order, scale, and store dW[:, slab] in the output dtype.
constexpr int kTailParts = 16;
template <class T>
__global__ __launch_bounds__(256) void dw_tail_kernel(const BwdArgs a) {
  typedef typename elem_of<T>::type E;
  const DwPlan plan = dw_plan(a, packed_rows(a.n_rows, a.N));
  const int b = (int)blockIdx.x / kTailParts, piece = (int)blockIdx.x % kTailParts;
  if (b >= plan.tail_tiles) return;
  int tp, tq;
  tile_coords(plan.full + b, plan.tiles, (int)(a.vs / kTile), (int)(a.Hp / kTile), 8, tp, tq);
  const float coef = final_factor_of(a);
  const float* part = a.dw_part + (int64_t)b * plan.nseg * kTile * kTile;
  constexpr int kQuads = kTile * kTile / 4 / kTailParts;
  for (int i = piece * kQuads + threadIdx.x; i < (piece + 1) * kQuads; i += 256) {
    const int row = i / (kTile / 4), vl = (i - row * (kTile / 4)) * 4;
    const int64_t h = (int64_t)tq * kTile + row, v = a.v0 + (int64_t)tp * kTile + vl;
    if (h >= a.H || v >= a.V) continue;  // a quad that V cuts through is written whole, into the stride padding of its row
    f32x4_t acc = *reinterpret_cast<const f32x4_t*>(part + row * kTile + vl);
#pragma unroll 4
    for (int s = 1; s < plan.nseg; ++s)
      acc += *reinterpret_cast<const f32x4_t*>(part + (int64_t)s * kTile * kTile + row * kTile + vl);
    if (a.dw_dtype == DT_F32) {
      *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(a.dw) + h * a.lddw + v) = acc * coef;
    } else {
      u32x2_t o;
      o[0] = pack2<T>(acc[0] * coef, acc[1] * coef);
      o[1] = pack2<T>(acc[2] * coef, acc[3] * coef);
      *reinterpret_cast<u32x2_t*>(reinterpret_cast<E*>(a.dw) + h * a.lddw + v) = o;
    }
  }
}

template <class T> hipError_t launch_persistent(const BwdArgs& a, hipStream_t s) {
  auto kern = bwd_dw_persistent_kernel<T>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kMainloopLds);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3(a.dw_grid), dim3(kThreads), kMainloopLds, s, a);
  e = hipGetLastError();
  if (e != hipSuccess) return e;
  if (a.dw_part == nullptr || dw_tail_blocks(a.Np, a.Hp, a.vs) == 0) return hipSuccess;  // this launch cannot have a split tail
  // (the tile count does not depend on the rows: no second kernel when the last round is not split)
  if (!has_split_tail((a.vs / kTile) * (a.Hp / kTile), a.dw_grid)) return hipSuccess;
  // at most dw_grid / 2 tail tiles can be split (two segments each)
  const unsigned tail_most = (unsigned)(a.dw_grid / 2 > 0 ? a.dw_grid / 2 : 1);
  hipLaunchKernelGGL(dw_tail_kernel<T>, dim3(tail_most * kTailParts), dim3(256), 0, s, a);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_bwd_dw(const BwdArgs& a, hipStream_t s) {
  if (a.x_dtype == DT_BF16) return launch_persistent<BF16>(a, s);
  if (a.x_dtype == DT_F16) return launch_persistent<F16>(a, s);
  return hipErrorInvalidValue;
}

}  // namespace lce
