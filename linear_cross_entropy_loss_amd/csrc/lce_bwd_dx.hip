// Backward, step 2: dx[token][h] (+)= sum_v dz[token][v] * W[h][v] over one
// vocabulary slab (the contraction of linear_cross_entropy/ops.py:317).  Both
// operands are K-contiguous (K = v).  The running sum over slabs is kept in
// fp32; the factor grad_out * logit_scale / n_valid is applied once, after the
// last slab, as the reference does after its accumulation (ops.py:332, 810).
// The token rows are those left after tokens with an ignored label were packed
// away; the tiles of a mostly idle last round of workgroups are cut along K
// and summed by a second kernel (DxPlan).
#include "lce_gemm3.h"
#include "lce_internal.h"

namespace lce {

namespace {

// The running sum lives in a padded [Np][Hp] fp32 buffer and needs no bounds.
// The final result goes out through range-checked buffer stores: the descriptor
// ends at the last element of dx, so rows past N are dropped by the hardware,
// and quads of hidden indices that start at or past H are given an
// out-of-range offset (a quad that H cuts through is written whole: the row
// stride is a multiple of 4, so it stays inside its row).
// `out` / `ldo` / `rows`: dx itself, or the packed copy when tokens were dropped (see BwdArgs).  `perm` != null
// (packed rows, dx smaller than 2 GiB): the rows go straight to their tokens' places in dx instead.
//
// What happens to a tile is fixed at compile time (a kernel per case): with the cases behind run-time branches
// the compiler emitted one load - wait - add - store round trip per register quad, 64 in a row per tile
// (about 30 us of latency; a step has up to 8 such tiles per workgroup at the headline shape, 1024 at
// N = 65536, H = 8192).  Here the 8 quads of two accumulator blocks are fetched together before any is used.
//   ADD    add the running sum of the earlier slabs (every slab but the first)
//   FINAL  scale and store in the output dtype (last slab), else store the fp32 running sum
template <class T, bool ADD, bool FINAL>
LCE_DEV void dx_epilogue(const BwdArgs& a, int64_t rows, void* out, int64_t ldo, const int* perm,
                         f32x16_t (&acc)[kNB][kNB], int tp, int tq) {
  typedef typename elem_of<T>::type E;
  const int64_t h0 = (int64_t)tp * kTile, t0 = (int64_t)tq * kTile;
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  const float coef = final_factor_of(a);
  const int es = a.dx_dtype == DT_F32 ? 4 : 2;
  // descriptor over the rows of this tile: base = first row, range = bytes to the end of dx
  // (scattered rows: base = dx, all of it in range; rows that do not exist get an out-of-range offset below)
  const char* tile_base = reinterpret_cast<const char*>(out) + (perm != nullptr ? 0 : t0 * ldo * es);
  // whole dwords: with 16-bit data and an odd H the last row ends one element into its stride padding
  const int64_t hcols = es == 2 ? (a.H + 1) & ~(int64_t)1 : a.H;
  const int64_t last_row = perm != nullptr ? a.N : rows;
  const int64_t left = (reinterpret_cast<const char*>(out) + ((last_row - 1) * ldo + hcols) * es) - tile_base;
  const unsigned range = left <= 0 ? 0u : (left > 0x7fffffff ? 0x7fffffffu : (unsigned)left);
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(tile_base), 0, (int)range, 0x00020000);
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    const int row = wq * kWaveTile + qb * kBlk + (lane & 31);  // row inside the tile
    const int64_t tok = t0 + row;
    unsigned row_off = (unsigned)(row * ldo * es);
    if (FINAL && perm != nullptr) row_off = tok < rows ? (unsigned)(packed_token(perm, tok, a.N) * ldo * es) : 0x80000000u;
    float* sum_row = a.dx_acc + tok * a.Hp + h0 + wp * kWaveTile + 4 * (lane >> 5);  // this lane's quads of the running sum
#pragma unroll
    for (int pb2 = 0; pb2 < kNB; pb2 += 2) {
      f32x4_t old[2][4];
      if (ADD) {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int rq = 0; rq < 4; ++rq)
            old[u][rq] = *reinterpret_cast<const f32x4_t*>(sum_row + (pb2 + u) * kBlk + 8 * rq);
      }
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          const int pb = pb2 + u;
          f32x4_t v;
#pragma unroll
          for (int j = 0; j < 4; ++j) v[j] = acc[pb][qb][rq * 4 + j];
          if (ADD) v += old[u][rq];
          if (!FINAL) {
            *reinterpret_cast<f32x4_t*>(sum_row + pb * kBlk + 8 * rq) = v;
          } else {
            const int64_t h = h0 + wp * kWaveTile + pb * kBlk + 8 * rq + 4 * (lane >> 5);
            const unsigned off = (h < a.H && row_off != 0x80000000u) ? row_off + (unsigned)(h * es) : 0x80000000u;
            if (a.dx_dtype == DT_F32) {
              const f32x4_t o = v * coef;
              u32x4_t bits;
#pragma unroll
              for (int j = 0; j < 4; ++j) bits[j] = __builtin_bit_cast(unsigned, (float)o[j]);
              __builtin_amdgcn_raw_buffer_store_b128(bits, rsrc, (int)off, 0, 0);
            } else {
              u32x2_t o;
              o[0] = pack2<T>(v[0] * coef, v[1] * coef);
              o[1] = pack2<T>(v[2] * coef, v[3] * coef);
              __builtin_amdgcn_raw_buffer_store_b64(o, rsrc, (int)off, 0, 0);
            }
          }
        }
    }
  }
}

// A K segment of a tail tile: its raw fp32 sum goes to its 256 x 256 block of dx_part, [token][hidden].
LCE_DEV void dx_store_segment(float* part, f32x16_t (&acc)[kNB][kNB]) {
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    float* prow = part + (wq * kWaveTile + qb * kBlk + (lane & 31)) * kTile + wp * kWaveTile + 4 * (lane >> 5);
#pragma unroll
    for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        f32x4_t v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = acc[pb][qb][rq * 4 + j];
        *reinterpret_cast<f32x4_t*>(prow + pb * kBlk + 8 * rq) = v;
      }
  }
}

// How one launch divides its work.  The output tiles (T of them, from the row count on the device) go to G
// persistent workgroups in rounds of G.  A last round that would keep only r < G workgroups busy is cut along K
// instead: its r tiles are split into `nseg` segments of `kseg` K tiles each (a power of two, r * nseg <= G, at
// least 16 K tiles per segment), one work item per (tile, segment), so that the round is 1/nseg as long and
// nearly all workgroups take part.  The segments' fp32 partial sums go to dx_part, one 256 x 256 block per
// item, and dx_tail_kernel adds them in segment order -- deterministic, no atomics.  With few tiles in total
// (small token counts) every tile is such a tail tile.
struct DxPlan {
  int tiles, full, tail_tiles, nseg, kseg;  // items [0, full) are whole tiles, then tail_tiles * nseg segment items
};
LCE_DEV DxPlan dx_plan(const BwdArgs& a, int tiles) {
  DxPlan p;
  const int G = a.dx_grid, kt = (int)(a.vs / kBK);
  p.tiles = tiles;
  p.full = tiles / G * G;
  const int r = tiles - p.full, cap = G < kTailBlocks ? G : kTailBlocks;
  int s = 1;
  if (r > 0 && a.dx_part != nullptr)  // (no blocks for partial sums: nothing is split)
    while (r * s * 2 <= cap && kt / (s * 2) >= 16) s *= 2;
  if (s == 1) {
    p.full = tiles;
    p.tail_tiles = 0;
    p.nseg = 1;
    p.kseg = kt;
  } else {
    // an even number of K tiles per segment; a last segment that runs past the slab is masked (K mask)
    p.tail_tiles = r;
    p.kseg = ((kt + s - 1) / s + 1) & ~1;
    p.nseg = (kt + p.kseg - 1) / p.kseg;
  }
  return p;
}

// Which work items of the plan a launch covers and what becomes of a tile (see dx_epilogue): whole tiles of the
// first / a middle / the last / the only slab, or the K segments of the tail tiles (a launch of their own).
enum { kDxFirst = 0, kDxMiddle = 1, kDxLast = 2, kDxOnly = 3, kDxTails = 4 };

// WVH: the weight is stored (V, H) row-major: the P tile then has K = v as its slow index (read through the
// LDS transpose path) and only dz, the K-contiguous operand, carries the K mask.
template <class T, bool KMASK, bool WVH, int MODE> struct DxProblem {
  static constexpr bool kKMask = KMASK;
  static constexpr bool kSwapAB = false;
  static constexpr bool kVarK = MODE == kDxTails;  // segment items have their own K extent
  static constexpr bool kQBlocked = true;          // dz is staged in blocks of 256 rows x 64 columns (BwdArgs::dz)
  static constexpr bool kColumnEpilogue = false;
  typedef typename elem_of<T>::type E;
  const BwdArgs& a;
  int64_t rows;  // token rows: all, or the packed ones (see BwdArgs)
  int tiles_p, tiles_q;
  DxPlan plan;
  int first, count;  // this launch's items of the plan: [first, first + count)
  LCE_DEV DxProblem(const BwdArgs& a_) : a(a_), rows(packed_rows(a_.n_rows, a_.N)), tiles_p((int)(a_.Hp / kTile)) {
    tiles_q = (int)((rows + kTile - 1) / kTile);
    plan = dx_plan(a, tiles_p * tiles_q);
    first = MODE == kDxTails ? plan.full : 0;
    count = MODE == kDxTails ? plan.tail_tiles * plan.nseg : plan.full;
  }
  LCE_DEV int num_tiles() const { return count; }
  // `local` counts this launch's items; seg < 0: a whole tile
  LCE_DEV void decode(int local, int& item, int& tp, int& tq, int& seg) const {
    item = first + local;
    int tile = item;
    seg = -1;
    if (item >= plan.full) {
      const int j = item - plan.full;
      tile = plan.full + j / plan.nseg;
      seg = j % plan.nseg;
    }
    tile_coords(tile, plan.tiles, tiles_p, tiles_q, 8, 8, tp, tq);
  }
  LCE_DEV int item_ktiles(int) const { return plan.kseg; }
  LCE_DEV void prefetch(int) {}
  LCE_DEV int64_t k0_of(int seg) const { return seg < 0 ? 0 : (int64_t)seg * plan.kseg * kBK; }
  LCE_DEV void origins(int local, const void*& p, const void*& q) const {
    int item, tp, tq, seg;
    decode(local, item, tp, tq, seg);
    const int64_t k0 = k0_of(seg);
    p = WVH ? reinterpret_cast<const E*>(a.w) + ((a.v0 - a.wv0) + k0) * a.ldw + (int64_t)tp * kTile
            : reinterpret_cast<const E*>(a.w) + (int64_t)tp * kTile * a.ldw + (a.v0 - a.wv0) + k0;
    q = reinterpret_cast<const E*>(a.dz) + dz_block_offset(tq, k0 / kBK, a.vs);  // (k0 is a multiple of 64)
  }
  LCE_DEV const void* p_end() const {
    return WVH ? matrix_end<E>(a.w, a.Vw, a.ldw, a.H) : matrix_end<E>(a.w, a.H, a.ldw, a.Vw);
  }
  // (only whole token tiles that were written are read.  K tiles past the slab -- the last segment of a split tail
  // tile may have some -- lie in the next row of blocks, or past the stage: the K mask gives those threads an
  // out-of-range offset, the other operand's are zeros)
  LCE_DEV const void* q_end() const { return reinterpret_cast<const E*>(a.dz) + a.dz_rows * a.vs; }
  LCE_DEV int k_valid(int local) const {
    int item, tp, tq, seg;
    decode(local, item, tp, tq, seg);
    const int64_t left = a.vw - k0_of(seg);
    return (int)(left < 0 ? 0 : left);
  }
  LCE_DEV void epilogue(int local, f32x16_t (&acc)[kNB][kNB], char*) const {
    int item, tp, tq, seg;
    decode(local, item, tp, tq, seg);
    if (MODE == kDxTails) {
      dx_store_segment(a.dx_part + (int64_t)(item - plan.full) * kTile * kTile, acc);
    } else {
      const bool packed = rows != a.N || a.perm_always != 0, copy = packed && a.dxc != nullptr;
      dx_epilogue<T, MODE == kDxMiddle || MODE == kDxLast, MODE == kDxLast || MODE == kDxOnly>(
          a, rows, copy ? a.dxc : a.dx, copy ? a.lddxc : a.lddx, packed && !copy ? a.perm : nullptr, acc, tp, tq);
    }
  }
};

template <class T, bool KMASK, bool WVH, int MODE>
__global__ __launch_bounds__(kThreads) void bwd_dx_persistent_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  typedef typename elem_of<T>::type E;
  DxProblem<T, KMASK, WVH, MODE> prob(a);
  Pipe3<T, E, !WVH, E, true, DxProblem<T, KMASK, WVH, MODE>> pipe(prob);
  pipe.run(a.ldw, a.vs / kBK, MODE == kDxTails ? prob.plan.kseg : (int)(a.vs / kBK), lds);
}

// Second step for the tail tiles: kTailParts workgroups share tail tile b (16 rows each) -- they sum its
// segments in order, then apply the same running-sum / final-store rules as the tile kernel's own epilogue.
constexpr int kTailParts = 16;
template <class T>
__global__ __launch_bounds__(256) void dx_tail_kernel(const BwdArgs a) {
  typedef typename elem_of<T>::type E;
  const int64_t rows = packed_rows(a.n_rows, a.N);
  const int tiles_p = (int)(a.Hp / kTile), tiles_q = (int)((rows + kTile - 1) / kTile);
  const DxPlan plan = dx_plan(a, tiles_p * tiles_q);
  const int b = (int)blockIdx.x / kTailParts, piece = (int)blockIdx.x % kTailParts;
  if (b >= plan.tail_tiles) return;
  int tp, tq;
  tile_coords(plan.full + b, plan.tiles, tiles_p, tiles_q, 8, 8, tp, tq);
  const bool packed = rows != a.N || a.perm_always != 0, copy = packed && a.dxc != nullptr;
  void* out = copy ? a.dxc : a.dx;
  const int64_t ldo = copy ? a.lddxc : a.lddx;
  const int* perm = packed && !copy ? a.perm : nullptr;
  const float coef = final_factor_of(a);
  const float* part = a.dx_part + (int64_t)b * plan.nseg * kTile * kTile;
  constexpr int kQuads = kTile * kTile / 4 / kTailParts;  // quads of this workgroup: 16 rows of the tile
  for (int i = piece * kQuads + threadIdx.x; i < (piece + 1) * kQuads; i += 256) {
    const int row = i / (kTile / 4), hl = (i - row * (kTile / 4)) * 4;
    const int64_t tok = (int64_t)tq * kTile + row, h = (int64_t)tp * kTile + hl;
    if (tok >= rows || h >= a.H) continue;
    f32x4_t v = *reinterpret_cast<const f32x4_t*>(part + row * kTile + hl);
#pragma unroll 4
    for (int s = 1; s < plan.nseg; ++s)
      v += *reinterpret_cast<const f32x4_t*>(part + (int64_t)s * kTile * kTile + row * kTile + hl);
    const int64_t o = tok * a.Hp + h;
    if (!a.first) v += *reinterpret_cast<const f32x4_t*>(a.dx_acc + o);
    if (!a.last) {
      *reinterpret_cast<f32x4_t*>(a.dx_acc + o) = v;
    } else {
      const int64_t dst_row = perm != nullptr ? packed_token(perm, tok, a.N) : tok;
      if (a.dx_dtype == DT_F32) {
        *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(out) + dst_row * ldo + h) = v * coef;
      } else {
        u32x2_t b;
        b[0] = pack2<T>(v[0] * coef, v[1] * coef);
        b[1] = pack2<T>(v[2] * coef, v[3] * coef);
        *reinterpret_cast<u32x2_t*>(reinterpret_cast<E*>(out) + dst_row * ldo + h) = b;
      }
    }
  }
}

template <class T, bool KMASK, bool WVH, int MODE> hipError_t launch_tiles(const BwdArgs& a, hipStream_t s) {
  auto kern = bwd_dx_persistent_kernel<T, KMASK, WVH, MODE>;
  static LdsOptIn optin;
  hipError_t e = optin.ensure(reinterpret_cast<const void*>(kern), kMainloopLds);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3(a.dx_grid), dim3(kThreads), kMainloopLds, s, a);
  return hipGetLastError();
}

template <class T, bool KMASK, bool WVH> hipError_t launch_layout(const BwdArgs& a, bool tails, hipStream_t s) {
  // (a small problem whose tiles are all split along K has no whole tile to launch; known here when rows are not packed)
  const bool none_whole = tails && a.n_rows == nullptr &&
                          all_tiles_are_tails((a.Np / kTile) * (a.Hp / kTile), a.dx_grid, a.vs / kBK);
  hipError_t e = none_whole ? hipSuccess
               : a.first ? (a.last ? launch_tiles<T, KMASK, WVH, kDxOnly>(a, s) : launch_tiles<T, KMASK, WVH, kDxFirst>(a, s))
                         : (a.last ? launch_tiles<T, KMASK, WVH, kDxLast>(a, s) : launch_tiles<T, KMASK, WVH, kDxMiddle>(a, s));
  if (e == hipSuccess && tails) e = launch_tiles<T, KMASK, WVH, kDxTails>(a, s);
  return e;
}

template <class T> hipError_t launch_persistent(const BwdArgs& a, hipStream_t s) {
  // A last round of tiles may be split along K.  Without packed rows the tile count is known here; with them
  // it is decided on the device, and a launch without items returns at once.
  const bool tails = a.dx_part != nullptr && dx_tail_blocks(a.Np, a.Hp, a.vs) != 0 &&
                     (a.n_rows != nullptr || has_split_tail((a.Np / kTile) * (a.Hp / kTile), a.dx_grid));
  // the K mask is only needed when the K tiles of a work item can run past the columns that exist
  const bool exact_k = a.vw == a.vs && dx_segments_exact(a.vs);
  hipError_t e = a.w_vh ? (exact_k ? launch_layout<T, false, true>(a, tails, s) : launch_layout<T, true, true>(a, tails, s))
                        : (exact_k ? launch_layout<T, false, false>(a, tails, s) : launch_layout<T, true, false>(a, tails, s));
  if (e != hipSuccess || !tails) return e;
  // at most dx_grid / 2 tail tiles can be split (two segments each)
  const unsigned tail_most = (unsigned)(a.dx_grid / 2 > 0 ? a.dx_grid / 2 : 1);
  hipLaunchKernelGGL(dx_tail_kernel<T>, dim3(tail_most * kTailParts), dim3(256), 0, s, a);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_bwd_dx(const BwdArgs& a, hipStream_t s) {
  // (an fp32 weight arrives here as a 16-bit slab copy; x_dtype is the compute type by now)
  if (a.x_dtype == DT_BF16 && a.w_dtype == DT_BF16) return launch_persistent<BF16>(a, s);
  if (a.x_dtype == DT_F16 && a.w_dtype == DT_F16) return launch_persistent<F16>(a, s);
  return hipErrorInvalidValue;
}

}  // namespace lce
