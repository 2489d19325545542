// C ABI of liblce_gfx950.so (declared in include/lce.h): argument checking,
// scratch planning and the launch sequences.  The host side does what
// LinearXentImplementation.forward does around its Triton launches
// (linear_cross_entropy/ops.py:681-802) -- minus every allocation, which is the
// caller's -- and what its backward does (ops.py:804-810).
#include <hip/hip_runtime.h>
#include <atomic>
#include <stdio.h>
#include <string.h>

#include "../../include/lce.h"
#include "lce_internal.h"

namespace {

thread_local char g_hip_error[256] = "";

int hip_fail(hipError_t e, const char* what) {
  snprintf(g_hip_error, sizeof(g_hip_error), "%s: %s", what, hipGetErrorString(e));
  return LCE_EHIP;
}

size_t align_up(size_t v) { return (v + 255) & ~(size_t)255; }

bool is16(int d) { return d == LCE_BF16 || d == LCE_F16; }

int check(const lce_problem* p, bool backward) {
  if (!p) return LCE_EINVAL_ARG;
  if (p->N <= 0 || p->H <= 0 || p->V <= 0 || p->n_chunk <= 0) return LCE_EINVAL_SHAPE;
  // Any N, H, V; only the row strides are constrained (below).
  if (p->N > (int64_t)1 << 30 || p->V > (int64_t)1 << 30 || p->H > (int64_t)1 << 20) return LCE_EINVAL_SHAPE;
  // bf16 pairs: bwd_dz reaches the three parts of its stage through 32-bit byte offsets (two parts of at least
  // Np * 256 * 2 bytes each)
  if (p->x_dtype == LCE_F32 && p->N > (int64_t)1 << 20) return LCE_EINVAL_SHAPE;
  const int xd = p->x_dtype, wd = p->w_dtype;
  const bool ok = (is16(xd) && (wd == xd || wd == LCE_F32)) || (xd == LCE_F32 && wd == LCE_F32);
  if (!ok) return LCE_EINVAL_DTYPE;
  if (!(p->logit_scale > 0.f) || !(p->z_reg >= 0.f)) return LCE_EINVAL_ARG;
  if (p->pack_rows != LCE_PACK_AUTO && p->pack_rows != LCE_PACK_ALWAYS && p->pack_rows != LCE_PACK_NEVER) return LCE_EINVAL_ARG;
  if (p->max_workgroups < 0) return LCE_EINVAL_ARG;
  if (p->w_layout != LCE_W_HV && p->w_layout != LCE_W_VH) return LCE_EINVAL_ARG;
  if ((p->route & ~LCE_ROUTE_EXACT_SUMS) != LCE_ROUTE_AUTO && (p->route & ~LCE_ROUTE_EXACT_SUMS) != LCE_ROUTE_ONE_PASS &&
      (p->route & ~LCE_ROUTE_EXACT_SUMS) != LCE_ROUTE_TWO_PASS)
    return LCE_EINVAL_ARG;
  const bool vh = p->w_layout == LCE_W_VH;
  // (V, H) weight: both operands of the logit contraction run along H in memory, so no 16-byte piece may
  // straddle the end of a row (H a multiple of 8), and there is no bf16-pair form of it
  if (vh && xd == LCE_F32) return LCE_EINVAL_DTYPE;
  if (vh && p->H % 8) return LCE_EINVAL_ARG;
  const int64_t w_cols = vh ? p->H : p->V;  // row length of w and dw as stored
  const int64_t xa = xd == LCE_F32 ? 4 : 8, wa = wd == LCE_F32 ? 4 : 8;  // 16-byte rows
  if (p->ldx < p->H || p->ldx % xa || p->ldw < w_cols || p->ldw % wa) return LCE_EINVAL_ARG;
  // The kernels address a 256-row tile of x, of a 16-bit W and of dx with 32-bit byte offsets: 256 rows must
  // stay below 2 GiB.  (An fp32 W is only read by the slab conversion, which uses 64-bit addresses.)
  const int64_t tile_limit = ((int64_t)1 << 31) / 256;
  if (p->ldx * (xd == LCE_F32 ? 4 : 2) > tile_limit) return LCE_EINVAL_ARG;
  if (is16(wd) && p->ldw * 2 > tile_limit) return LCE_EINVAL_ARG;
  // tile and work-item counts are 32-bit
  if (lce::padded_tokens(p->N) / 256 * (lce::padded_vocab(p->V) / 256) > (int64_t)1 << 28) return LCE_EINVAL_SHAPE;
  if (backward) {
    if (p->dx_dtype != xd && p->dx_dtype != LCE_F32) return LCE_EINVAL_DTYPE;
    if (p->dw_dtype != wd && p->dw_dtype != LCE_F32) return LCE_EINVAL_DTYPE;
    // dx is stored in 8-byte (16-bit types) or 16-byte pieces, dW in 16-byte pieces
    if (p->lddx < p->H || p->lddx % 4 || p->lddw < w_cols || p->lddw % (p->dw_dtype == LCE_F32 ? 4 : 8)) return LCE_EINVAL_ARG;
    if (p->lddx * (p->dx_dtype == LCE_F32 ? 4 : 2) > tile_limit) return LCE_EINVAL_ARG;
  }
  return LCE_OK;
}

// Buffers of the packing pre-pass (tokens with an ignored label dropped), relative to `base`.
struct PackPlan {
  size_t cnt, n_rows, perm, yc, xc, xk, end;
  int64_t ldxc;  // row stride of the packed copy of x, elements: rows of whole 16-byte pieces
  int64_t ldxk;  // fp32 activations, backward: row stride of the copy stacked along the tokens (lce_compact.hip)
  size_t xes;    // element size of the packed copy: that of x, or 2 for fp32 activations (stored as bf16 pairs)
};

// fp32 activations (and with them an fp32 weight) are computed as bf16 pairs, hi + lo (lce_gemm.h).
bool splits(const lce_problem* p) { return p->x_dtype == LCE_F32; }

// Whether the tokens with an ignored label are packed away before the tile kernels run (lce.h).
bool packs_rows(const lce_problem* p) {
  if (p->pack_rows == LCE_PACK_ALWAYS) return true;
  if (p->pack_rows == LCE_PACK_NEVER) return false;
  return 8.0 * (double)p->N * (double)p->H * (double)p->V >= 2199023255552.0;  // 2^41
}

PackPlan plan_pack(const lce_problem* p, size_t base, bool backward) {
  PackPlan k;
  const size_t N = (size_t)p->N, es = 2;
  k.xes = es;
  k.ldxc = lce::pad_to(splits(p) ? 3 * p->H : p->H, (int64_t)(16 / es));
  k.ldxk = lce::pad_to(p->H, (int64_t)(16 / es));
  size_t o = base;
  k.cnt = o; o += align_up((size_t)lce::compact_segments(p->N) * 4);
  k.n_rows = o; o += 256;
  k.perm = o; o += align_up(N * 4);
  k.yc = o; o += align_up(N * 8);
  k.xc = o; o += align_up(N * (size_t)k.ldxc * es);
  k.xk = o;
  if (splits(p) && backward) o += align_up(3 * (size_t)lce::padded_tokens(p->N) * (size_t)k.ldxk * es);
  k.end = o;
  return k;
}

struct FwdPlan {
  size_t part_lse, part_max, part_pz, part_sq, tgt, blk, w16, total;
  // When monitoring is off (the monitoring values are taken over all rows), and for fp32 activations, which
  // reach the tile kernels through the packed copy (rounded to bf16 there).
  PackPlan pack;
  int64_t vs;  // columns per forward launch: all of V, or the width of the 16-bit slab copy of an fp32 weight
  int64_t nc;  // token rows per forward launch (a multiple of 256): the width of the partial-sum buffers
};

// The forward works through the tokens in chunks, so that its partial sums (V/32 bytes per token of a chunk)
// do not grow with the number of tokens: chunks of n_chunk rows, but at least 16384 -- shorter chunks only
// add launches -- and at least 65536 under an fp32 weight, whose 16-bit slab copies are made once per chunk.
int64_t fwd_chunk_rows(const lce_problem* p) {
  const int64_t Np = lce::padded_tokens(p->N);
  int64_t nc = lce::pad_to(p->n_chunk, 256);
  const int64_t least = p->w_dtype == LCE_F32 ? 65536 : 16384;
  if (nc < least) nc = least;
  return nc < Np ? nc : Np;
}

// 16-bit type the kernels compute in: that of the activations (bf16 for fp32 activations).
int compute_dtype(const lce_problem* p) { return p->x_dtype == LCE_F16 ? LCE_F16 : LCE_BF16; }

FwdPlan plan_fwd(const lce_problem* p) {
  FwdPlan f;
  const size_t Np = (size_t)lce::padded_tokens(p->N), Vp = (size_t)lce::padded_vocab(p->V);
  f.nc = fwd_chunk_rows(p);
  const size_t part = align_up(Vp / lce::kChunkV * (size_t)f.nc * 4);
  size_t o = 0;
  f.part_lse = o; o += part;
  f.part_max = o; if (p->monitoring) o += part;
  f.part_pz = o; if (p->monitoring) o += part;
  f.part_sq = o; if (p->monitoring) o += part;
  f.tgt = o; o += align_up(Np * 4);
  f.blk = o; o += align_up(Np / lce::kMergeRows * 8 * sizeof(double));
  f.w16 = o;
  f.vs = (int64_t)Vp;
  // A chunk of activations that does not fit the 256 MB Infinity Cache (more than 128 MiB of it) is streamed from
  // memory by all eight XCDs; over a long launch they drift apart and stop sharing what they fetch.  Launches
  // of 32768 columns bring them back in step (measured at N = 16384, H = 8192, V = 131072: 24.6 ms against 27.3
  // in one launch; no difference at H = 2048, where x stays in the cache).
  // (fp32 activations reach the tile kernels as bf16 pairs, three times as wide)
  if ((size_t)f.nc * (size_t)(splits(p) ? 3 * p->H : p->H) * 2 > ((size_t)128 << 20) && f.vs > 32768) f.vs = 32768;
  if (p->w_dtype == LCE_F32) {
    // slab copies of at most 256 MiB (at least one tile column)
    const int64_t hw = splits(p) ? 3 * p->H : p->H;  // rows of the copy
    int64_t cols = ((int64_t)256 << 20) / (hw * 2) / 256 * 256;
    if (cols < 256) cols = 256;
    if (cols < f.vs) f.vs = cols;
    o += align_up((size_t)hw * (size_t)f.vs * 2);
  }
  if ((!p->monitoring && packs_rows(p)) || p->x_dtype == LCE_F32) {
    f.pack = plan_pack(p, o, false);
    o = f.pack.end;
  }
  f.total = o;
  return f;
}

struct BwdPlan {
  int64_t slabs, vs;
  double cost;  // modelled time of the plan's tile kernels (kernel_cost units)
  PackPlan pack;
  size_t lse_c, dxc;  // lse of the packed rows; packed dx before it is moved to its place (only for a dx of >= 2 GiB)
  bool stage_dx;
  bool pack_on;   // tokens with an ignored label are packed away in this backward
  bool parts_on;  // tail tiles of dx / dW may be split along K (partial-sum blocks exist)
  int64_t lddxc;
  size_t dz, dx_acc, dx_part, dw_part, w16, total;
};

// Bytes of the split-K partial sums of dx for slabs of `vs` columns (0 when dx is not split).
size_t dx_part_bytes(size_t Np, size_t Hp, int64_t vs, int64_t last_vs) {
  const int64_t b0 = lce::dx_tail_blocks((int64_t)Np, (int64_t)Hp, vs), b1 = lce::dx_tail_blocks((int64_t)Np, (int64_t)Hp, last_vs);
  return (size_t)(b0 > b1 ? b0 : b1) * 256 * 256 * 4;
}

// The same for dW.
size_t dw_part_bytes(size_t Np, size_t Hp, int64_t vs, int64_t last_vs) {
  const int64_t b0 = lce::dw_tail_blocks((int64_t)Np, (int64_t)Hp, vs), b1 = lce::dw_tail_blocks((int64_t)Np, (int64_t)Hp, last_vs);
  return (size_t)(b0 > b1 ? b0 : b1) * 256 * 256 * 4;
}

// Modelled time of a tile kernel with T output tiles of L K tiles each, in units of one 64-deep K tile of a 256 x 256
// output tile on a full chip.  A kernel runs its tiles in rounds of kPlanCUs; a last round that fills a
// fraction f of the compute units runs 1 + 0.9 (1 - f) times faster per compute unit (the part is limited by
// power: measured 1.14 / 1.30 / 1.46 / 1.54 at f = 0.81 / 0.69 / 0.47 / 0.34), and is cut along K when the
// partial-sum blocks exist (`parts`; a small kernel then adds the segments: 12 units).  `e`: the epilogue of a
// tile; a launch costs about 10.
constexpr double kPlanCUs = 256.0;
double kernel_cost(double T, double L, double e, bool parts) {
  const double full = (double)(int64_t)(T / kPlanCUs), r = T - full * kPlanCUs;
  double cost = full * (L + e) + 10.0;
  if (r > 0) {
    double seg = 1;
    if (parts) while (r * seg * 2 <= kPlanCUs && L / (seg * 2) >= 16) seg *= 2;
    const double f = r * seg / kPlanCUs;
    cost += (L / seg + e) / (1.0 + 0.9 * (1.0 - f)) + (seg > 1 ? 12.0 : 0.0);
  }
  return cost;
}

// Vocabulary slabs (of a width that is a multiple of 256 columns; the last one may be narrower) whose staging
// fits the scratch bound: the fewest that fit, or somewhat more of them when a model of the three kernels'
// rounds of workgroups says that those run faster (slab_cost below).  The dz stage itself is additionally
// capped at 1 GiB: wider slabs are not faster, so a generous N_chunk_size does not translate into a larger
// footprint.
//
// The bound is n_chunk * V * 4 bytes, what the reference spends on its logits
// chunk (ops.py:700).  Everything counts towards it: the dz stage, the fp32 running dx, the packed rows and
// the partial sums of split tail tiles.  The two optional items are given up when the plan without them is
// the faster one by the same model -- `lean`: tokens with an ignored label are then not packed away in the
// backward and tail tiles are not split, which buys wider slabs under a tight bound.
// Shapes with a small vocabulary and many tokens cannot meet the bound at all (the fp32 running dx alone is
// larger, and a split into very narrow slabs leaves the GPU idle); for those the bound is widened by
// N * H * 4 bytes, the fp32 x_grad buffer the reference allocates next to its logits chunk (ops.py:693) and
// this library does not -- and by the split-K partial sums.  If even that fails, the narrowest split is used:
// the bound is a target, the operator never refuses a shape.
int plan_bwd(const lce_problem* p, BwdPlan* b) {
  const size_t strict = (size_t)p->n_chunk * (size_t)p->V * 4;
  const size_t dz_cap = (size_t)1 << 30;
  const size_t Np = (size_t)lce::padded_tokens(p->N), Hp = (size_t)lce::padded_hidden(p->H);
  const int64_t Vp = lce::padded_vocab(p->V);
  const int64_t cols = Vp / 256;
  const bool split = splits(p);
  const size_t dxes = p->dx_dtype == LCE_F32 ? 4 : 2;
  b->pack = plan_pack(p, 0, true);
  b->lddxc = lce::pad_to(p->H, 8);
  b->lse_c = b->pack.end;
  b->dxc = b->lse_c + align_up((size_t)p->N * 4);

  // Modelled time of the three kernels over one slab of `w` columns (kernel_cost above).  Per tile, the epilogues
  // cost about 6 (dz), 21 (dx adding into the fp32 running sum: 512 KiB of traffic at a compute unit's share of the
  // memory bandwidth; 5 when it is written once) and 5 (dW) units.  The model ranks the slab
  // widths measured at N = 16384, H = 2048, V = 32768 and 65536 (2 ... 18 slabs) in their measured order.
  // bands of W tiles that bwd_dz keeps in flight (tile_coords in lce_gemm.h), and the slab width that is a whole group of them
  const int live = lce::live_bands(lce::padded_k(split ? 3 * p->H : p->H) * 2);
  const int64_t gran = live < 8 ? (int64_t)256 * 8 * live : 256;
  auto slab_cost = [&](int64_t w, bool parts, bool sums) -> double {
    const double tq = (double)(Np / 256), th = (double)(Hp / 256), tv = (double)(w / 256), k3 = split ? 3.0 : 1.0;
    // (bwd_dz runs about 4 % slower on a slab that is not whole groups of the bands it keeps in flight when K is long)
    const double dz_order = live < 8 && (w / 256) % (8 * live) != 0 ? 1.04 : 1.0;
    return dz_order * kernel_cost(tq * tv, k3 * (double)((p->H + 63) / 64), 6.0, false) +
           k3 * kernel_cost(tq * th, (double)(w / 64), sums ? 21.0 : 5.0, parts) +
           kernel_cost(tv * th, k3 * (double)(Np / 64), 5.0, parts);
  };

  // mode 0: everything; mode 1: lean (at the strict bound only); mode 2: everything, widened bound.
  // Tries a split into `s` slabs of equal width (the last one may be narrower); cost: its modelled time.
  auto fits = [&](int mode, int64_t s, bool whole_groups, BwdPlan* out, double* cost) -> bool {
    const bool lean = mode == 1;
    const bool pack = packs_rows(p) && !(lean && p->pack_rows == LCE_PACK_AUTO);
    // The dx kernels store packed rows straight to their tokens' places through 32-bit offsets into dx; a dx
    // that large offsets cannot span is staged packed and moved afterwards.
    const bool stage_dx = pack && (size_t)p->N * (size_t)p->lddx * dxes >= ((size_t)1 << 31);
    size_t fixed = 0;  // buffers of the packed rows come first (fp32 activations need the copies of x even when rows are not packed)
    if (pack) fixed = b->dxc + (stage_dx ? align_up((size_t)p->N * (size_t)b->lddxc * dxes) : 0);
    else if (split) fixed = b->pack.end;
    const size_t budget = strict + (mode == 2 ? (size_t)p->N * (size_t)p->H * 4 : 0);
    int64_t vs = (cols + s - 1) / s * 256;
    if (whole_groups) vs = (vs + gran - 1) / gran * gran;  // the next width that is whole groups of bands
    const int64_t slabs = (Vp + vs - 1) / vs;
    // (bf16 pairs: three blocks of dz, and dx is summed over three passes per slab, so it always needs the running sum)
    const size_t dz = align_up(Np * (size_t)vs * 2 * (split ? 3 : 1));
    const size_t acc = slabs > 1 || split ? align_up(Np * Hp * 4) : 0;
    const int64_t last_vs = Vp - (slabs - 1) * vs;  // padded width of the last slab
    const size_t dxp = lean ? 0 : dx_part_bytes(Np, Hp, vs, last_vs);  // at most 64 MiB
    const size_t dwp = lean ? 0 : dw_part_bytes(split ? 3 * Np : Np, Hp, vs, last_vs);
    const size_t part = dxp > dwp ? dxp : dwp;  // one buffer: the dx kernels are done with it before the dW kernels start
    const size_t w16 = p->w_dtype == LCE_F32 ? align_up((size_t)p->H * (size_t)vs * 2 * (split ? 3 : 1)) : 0;  // 16-bit copy of the slab of W
    // the widened bound is for the staging proper; the split-K partial sums (at most 64 MiB, shared by dx
    // and dW) and the packed rows come on top of it there
    // (reserve: what the caller holds besides the workspace between forward and backward -- lse and a few scalars)
    const size_t reserve = align_up((size_t)p->N * 4) + 4096;
    const size_t counted = dz + acc + w16 + (mode != 2 ? fixed + part + reserve : 0);
    if (!((counted <= budget && (dz <= dz_cap || vs == 256)) || (mode == 2 && vs == 256))) return false;
    out->slabs = slabs;
    out->vs = vs;
    out->pack_on = pack;
    out->parts_on = !lean;
    out->stage_dx = stage_dx;
    out->dz = fixed;
    out->dx_acc = fixed + dz;
    out->dx_part = fixed + dz + acc;
    out->dw_part = out->dx_part;
    out->w16 = fixed + dz + acc + part;
    out->total = fixed + dz + acc + part + w16;
    // (a lean plan computes the tokens with an ignored label too; how many there are is not known here)
    *cost = ((double)(slabs - 1) * slab_cost(vs, !lean, acc != 0) + slab_cost(last_vs, !lean, acc != 0)) *
            (lean && packs_rows(p) ? 1.02 : 1.0);
    return true;
  };
  // The fewest slabs that fit, or a few more of them when the model says that their tiles fill the rounds of
  // workgroups better (four slabs of 8192 columns against three of 11008 at H = 2048, say).
  auto choose = [&](int mode, BwdPlan* out, double* cost) -> bool {
    int64_t first = 0;
    BwdPlan cand = *out;
    double c = 0;
    for (int64_t s = 1; s <= cols; ++s) {
      if (s > 1 && (cols + s - 2) / (s - 1) == (cols + s - 1) / s) continue;  // same width as with one slab fewer
      if (first != 0 && (mode == 2 || s > 4 * first + 8)) break;
      for (int whole = 0; whole < (gran > 256 ? 2 : 1); ++whole) {
        if (!fits(mode, s, whole != 0, &cand, &c)) continue;
        if (first == 0 || c < *cost) { *out = cand; *cost = c; }
        if (first == 0) first = s;
      }
    }
    return first != 0;
  };
  BwdPlan full = *b, lean = *b;
  double cost_full = 0, cost_lean = 0;
  const bool ok_full = choose(0, &full, &cost_full), ok_lean = choose(1, &lean, &cost_lean);
  if (ok_full && (!ok_lean || cost_full <= cost_lean)) { *b = full; b->cost = cost_full; return LCE_OK; }
  if (ok_lean) { *b = lean; b->cost = cost_lean; return LCE_OK; }
  double wide = 0;
  if (choose(2, b, &wide)) { b->cost = wide; return LCE_OK; }
  return LCE_EWORKSPACE;
}

// lce_forward_backward: the logits are computed once.  The tokens go through in chunks of `nc` rows against the
// whole vocabulary: logit kernel (partials of the loss, and e = exp(z - slice max) into the stage), row merge
// (lse), the pass that turns e into dz, then dx of the chunk (complete: K = the vocabulary) and the chunk's
// term of dW, which is summed over the chunks in fp32 (the reference's fp32 At_grad, ops.py:692): in the caller's
// buffer if dW is fp32, else as 16-bit halves -- the upper ones in the caller's dW, the lower ones in a plane here.
// Everything counts towards the bound n_chunk * V * 4 (the reference's logits chunk, ops.py:700): the chunk is
// the longest that fits.  Problems outside the set below -- and those whose plane alone does not fit -- take the
// two-pass route (forward, then a backward that recomputes the logits).
struct FusedPlan {
  bool ok;
  bool pack;
  int64_t nc;
  int chunks;
  PackPlan k;
  size_t chunk_rows, lse_rows, tgt, blk, w16, xc, part_lse, part_max, part_pz, part_sq, stage, plane, plane_hi, part, total;
  int64_t ld16;    // row stride of the 16-bit copy of an fp32 weight
  bool parts_on;
  bool dw_direct;  // fp32 dW: the chunks' terms are added in the caller's buffer, there is no plane
  bool lo8;        // the lower halves of a 16-bit dW's sums are cut to a byte (lce_bwd_dw.hip)
  double cost;     // modelled time of the plan (kernel_cost units)
};

bool plan_fused_with(const lce_problem* p, bool want_dx, bool want_dw, bool lo8, FusedPlan* f);

// The lower halves of the fp32 sums of a 16-bit dW at 16 bits (the sums are then exact fp32) or at 8 (sums of 24
// bits): the latter where the former does not fit the bound, or leaves so little of it to the chunks that the model
// puts the plan with bytes at least 3 % ahead of the exact alternatives (the plan with halves, two passes) -- measured
// on one box: 5.9 % at config 3, 7-10 % at the output layers of Llama-3-8B / Llama-2-7B, 11-20 % at config 4's
// N_chunk_size = 2048 points, 0.7 % at the headline shape (which keeps the halves).  Never with LCE_ROUTE_EXACT_SUMS.
constexpr double kBytesMargin = 0.97;
bool plan_fused(const lce_problem* p, bool want_dx, bool want_dw, FusedPlan* f) {
  const bool halves = plan_fused_with(p, want_dx, want_dw, false, f);
  if ((p->route & LCE_ROUTE_EXACT_SUMS) || !want_dw || p->dw_dtype == LCE_F32) return halves;
  FusedPlan b;
  if (plan_fused_with(p, want_dx, want_dw, true, &b) && (!halves || b.cost < kBytesMargin * f->cost)) {
    *f = b;
    return true;
  }
  return halves;
}

bool plan_fused_with(const lce_problem* p, bool want_dx, bool want_dw, bool lo8, FusedPlan* f) {
  memset(f, 0, sizeof(*f));
  f->lo8 = lo8;
  const bool x16 = p->x_dtype == LCE_BF16 || p->x_dtype == LCE_F16;
  if (!x16 || (p->w_dtype != p->x_dtype && p->w_dtype != LCE_F32) || (p->route & ~LCE_ROUTE_EXACT_SUMS) == LCE_ROUTE_TWO_PASS) return false;
  const size_t Np = (size_t)lce::padded_tokens(p->N), Vp = (size_t)lce::padded_vocab(p->V), Hp = (size_t)lce::padded_hidden(p->H);
  const size_t dxes = p->dx_dtype == LCE_F32 ? 4 : 2;
  // (packed rows of dx go to their tokens through 32-bit offsets into dx)
  // (the monitoring values are taken over all rows: the dropped tokens then follow the kept ones, the logit kernel
  // and the row merge run over all of a chunk's rows, the gradient kernels over its kept ones)
  f->pack = packs_rows(p) && (size_t)p->N * (size_t)p->lddx * dxes < ((size_t)1 << 31);
  f->dw_direct = p->dw_dtype == LCE_F32;
  // (a 16-bit dW summed over chunks keeps the upper halves of its sums in dW itself, addressed through 32-bit
  // offsets that span the 256 rows of a tile: lce_bwd_dw.hip)
  const bool halves_ok = (size_t)p->lddw * 2 * 256 < ((size_t)1 << 31);
  f->k = plan_pack(p, 0, false);
  size_t o = f->k.xc;  // the labels are always counted; the packed copy of x is made chunk by chunk (below)
  f->chunk_rows = o; o += align_up(2048 * 8);
  f->lse_rows = o; o += align_up(Np * 4);
  f->tgt = o; o += align_up(Np * 4);
  f->blk = o; o += align_up(Np / lce::kMergeRows * 8 * sizeof(double));
  // an fp32 master weight is rounded to the compute type once per call, all of it
  const bool vh = p->w_layout == LCE_W_VH;
  f->ld16 = vh ? p->H : (int64_t)Vp;
  f->w16 = o;
  if (p->w_dtype == LCE_F32) o += align_up((vh ? (size_t)p->V : (size_t)p->H) * (size_t)f->ld16 * 2);
  const size_t fixed = o;
  const size_t bound = (size_t)p->n_chunk * (size_t)p->V * 4;
  const size_t reserve = align_up((size_t)p->N * 4) + 4096;  // what the caller holds besides the workspace: lse and a few scalars
  auto total_for = [&](int64_t nc, int chunks, FusedPlan* out) -> size_t {
    size_t t = fixed;
    out->xc = t;
    if (f->pack) t += align_up((size_t)nc * (size_t)f->k.ldxc * 2);
    const size_t part = align_up(Vp / lce::kChunkV * (size_t)nc * 4);
    out->part_lse = t; t += part;
    out->part_max = t; t += part;
    out->part_pz = t; if (p->monitoring) t += part;
    out->part_sq = t; if (p->monitoring) t += part;
    out->stage = t; t += align_up((size_t)nc * Vp * 2);
    // split-K partial sums of dx (and, with a single chunk, of dW): one buffer
    size_t pb = want_dx ? dx_part_bytes((size_t)nc, Hp, (int64_t)Vp, (int64_t)Vp) : 0;
    if (chunks == 1 && want_dw) {
      const size_t w = dw_part_bytes((size_t)nc, Hp, (int64_t)Vp, (int64_t)Vp);
      if (w > pb) pb = w;
    }
    out->part = t; t += pb;
    out->parts_on = pb != 0;
    out->plane = t;
    if (chunks > 1 && want_dw && !f->dw_direct) t += align_up(Hp * Vp * (lo8 ? 1 : 2));
    // (upper halves of the tiles that the edge of dW cuts: the last tile row over h, the last over v)
    out->plane_hi = t;
    if (chunks > 1 && want_dw && !f->dw_direct)
      t += align_up(((Hp != (size_t)p->H ? Vp / 256 : 0) + (Vp != (size_t)p->V ? Hp / 256 : 0)) * (size_t)(256 * 256 * 2));
    out->total = t;
    return t;
  };
  // Chunks of equal length (whole token tiles): of the lengths that fit, the one for which a model of the three tile
  // kernels' rounds of workgroups gives the shortest time -- not always the longest: at the headline shape 13
  // token tiles fit, whose 104 tiles of dx fill 208 of 256 compute units when each is cut in two along K, while
  // chunks of 8 token tiles (64 tiles of dx, cut in four) fill them all -- but the part is limited by power, the
  // partly filled rounds run at a higher clock, and the longer chunk wins: measured 22.07 ms a step with 13 token
  // tiles, 22.60 with 8, 22.85 with 11, 23.87 with 7, 26.1 with 4, the order the model gives.
  const int64_t tiles = (int64_t)(Np / 256);
  const double th = (double)(Hp / 256), tv = (double)(Vp / 256);
  double best = 0;
  int64_t first = 0;  // chunks of the longest chunk that fits
  for (int64_t t = tiles; t >= 1; --t) {
    const int64_t chunks = (tiles + t - 1) / t;
    if (chunks > 1024 || (first != 0 && chunks > 4 * first + 8)) break;
    if (t < tiles && (tiles + t) / (t + 1) == chunks) continue;  // a longer chunk gives the same number of chunks
    if (chunks > 1 && want_dw && !f->dw_direct && !halves_ok) continue;
    const int64_t t_even = (tiles + chunks - 1) / chunks;  // equal lengths
    FusedPlan cand = *f;
    if (total_for(t_even * 256, (int)chunks, &cand) + reserve > bound) continue;
    const int64_t t_last = tiles - (chunks - 1) * t_even;
    auto chunk_cost = [&](double tt) -> double {
      return kernel_cost(tt * tv, (double)(lce::padded_k(p->H) / 64), 8.0, false) +
             (want_dx ? kernel_cost(tt * th, (double)(Vp / 64), 5.0, true) : 0.0) +
             (want_dw ? kernel_cost(tv * th, tt * 4.0, chunks > 1 ? (f->dw_direct ? 16.0 : lo8 ? 10.0 : 12.0) : 5.0, chunks == 1) : 0.0);
    };
    // (per chunk, besides the tile kernels: the row merge, the kernel that adds dx's K segments, launch gaps -- about 25 units)
    const double cost = (double)(chunks - 1) * chunk_cost((double)t_even) + chunk_cost((double)t_last) + 25.0 * (double)chunks;
    if (first == 0) first = chunks;
    // (what the chunks do not change: the pass over the stage at 4 bytes per logit -- about 8 MB of memory traffic
    // per unit)
    if (!f->ok || cost < best) {
      best = cost;
      *f = cand;
      f->nc = t_even * 256;
      f->chunks = (int)chunks;
      f->ok = true;
    }
  }
  if (!f->ok) return false;
  // The two-pass route by the same model: the forward over all tokens, then the backward's plan.  It wins where the
  // scratch bound leaves only short chunks (every chunk adds a round trip of all the fp32 sums of dW).
  BwdPlan b;
  const double scale_pass = (double)Np * (double)Vp * 4.0 / 8.0e6;
  f->cost = best + scale_pass;
  if ((p->route & ~LCE_ROUTE_EXACT_SUMS) == LCE_ROUTE_AUTO && plan_bwd(p, &b) == LCE_OK) {
    const double two = kernel_cost((double)tiles * tv, (double)(lce::padded_k(p->H) / 64), 4.0, false) + b.cost;
    // (sums of 24 bits have to be ahead of two passes, which are exact, by the margin as well)
    if (best + scale_pass > two * (lo8 ? kBytesMargin : 1.0)) {
      f->ok = false;  // (f->chunks stays: a plan fitted)
      return false;
    }
  }
  return true;
}

bool misaligned(const void* p) { return ((uintptr_t)p & 15) != 0; }

// Scratch of lce_forward_static: a fixed array in device memory, one copy per GPU the library runs on,
// held until the process ends.  On the host `scratch` is only a handle for hipGetSymbolAddress; the
// device address is looked up once per device and kept in g_scratch_ptr.
constexpr size_t kStaticScratchBytes = LCE_STATIC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
std::atomic<void*> g_scratch_ptr[kMaxDevices];

// Device address of `scratch` on the current device (looked up on the first call per device).
int static_scratch(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
  if (dev < 0 || dev >= kMaxDevices) return LCE_EINVAL_ARG;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) return hip_fail(e, "hipGetSymbolAddress(scratch)");
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // every thread finds the same address
  }
  *out = ptr;
  return LCE_OK;
}

// Compute units of the current device (grid size of the persistent kernels), capped by `cap` when that is positive.
int current_num_cus(int* out, int cap) {
  int dev = 0, n = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e == hipSuccess) e = hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return hip_fail(e, "device query");
  *out = n > 0 ? n : 1;
  if (cap > 0 && cap < *out) *out = cap;
  return LCE_OK;
}

// Body of lce_forward; `ws` is the caller's workspace or the library's static scratch.
int forward_impl(const lce_problem* p, const void* x, const void* w, const int64_t* y, float* lse, float* out5,
                 int64_t* n_valid, void* ws, size_t ws_bytes, void* stream) {
  int rc = check(p, false);
  if (rc != LCE_OK) return rc;
  if (!x || !w || !y || !lse || !out5 || !n_valid) return LCE_EINVAL_ARG;
  if (misaligned(x) || misaligned(w)) return LCE_EINVAL_ARG;
  const FwdPlan f = plan_fwd(p);
  if (!ws || ws_bytes < f.total || misaligned(ws)) return LCE_EWORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  char* base = (char*)ws;

  lce::FwdArgs a;
  memset(&a, 0, sizeof(a));
  a.x = x; a.w = w; a.y = y;
  a.N = p->N; a.H = p->H; a.V = p->V; a.ldx = p->ldx; a.ldw = p->ldw;
  a.Np = lce::padded_tokens(p->N); a.Vp = lce::padded_vocab(p->V);
  a.x_dtype = p->x_dtype; a.w_dtype = p->w_dtype;
  a.w_vh = p->w_layout == LCE_W_VH;
  a.ignore_index = p->ignore_index;
  a.scale = p->logit_scale; a.z_reg = p->z_reg; a.monitoring = p->monitoring ? 1 : 0;
  a.lse = lse; a.out5 = out5; a.n_valid = n_valid;
  a.part_lse = (float*)(base + f.part_lse);
  a.part_max = (float*)(base + f.part_max);
  a.part_pz = (float*)(base + f.part_pz);
  a.part_sq = (float*)(base + f.part_sq);
  a.tgt = (float*)(base + f.tgt);
  a.blk = (float*)(base + f.blk);
  rc = current_num_cus(&a.num_cus, p->max_workgroups);
  if (rc != LCE_OK) return rc;
  a.live = lce::live_bands(lce::padded_k(splits(p) ? 3 * p->H : p->H) * 2);

  const int ph = p->phases ? p->phases : ~0;
  hipError_t e;
  const bool pack = !p->monitoring && packs_rows(p), x32 = p->x_dtype == LCE_F32;
  if (pack || x32) {
    const PackPlan& k = f.pack;
    if (pack) {
      // Tokens with an ignored label add nothing to the loss: the tile kernel runs on the others only.
      a.n_rows = (const int64_t*)(base + k.n_rows);
      a.perm = (const int*)(base + k.perm);
      a.y0 = y;
      a.y = (const int64_t*)(base + k.yc);
    }
    a.xc = base + k.xc;
    a.ldxc = k.ldxc;
    if (ph & LCE_PHASE_PACK) {
      if (pack) {
        e = lce::launch_compact_labels(y, p->N, p->ignore_index, (int*)(base + k.cnt), (int64_t*)(base + k.n_rows),
                                       (int*)(base + k.perm), (int64_t*)(base + k.yc), s);
        if (e != hipSuccess) return hip_fail(e, "compact_labels");
      }
      e = x32 ? lce::launch_gather_rows_split((const float*)x, p->ldx, p->H, a.perm, a.n_rows, p->N, base + k.xc,
                                              k.ldxc, nullptr, 0, nullptr, nullptr, a.num_cus, s)
              : lce::launch_gather_rows(x, p->ldx * 2, p->H * 2, a.perm, a.n_rows, p->N, base + k.xc, k.ldxc * 2, nullptr, nullptr,
                                        a.num_cus, s);
      if (e != hipSuccess) return hip_fail(e, "gather_rows");
    }
    if (x32) {  // the tile kernels read the copy in bf16 pairs ([hi | hi | lo], K = 3 H), whether or not rows were dropped
      a.x = a.xc;
      a.ldx = a.ldxc;
      a.x_dtype = lce::DT_BF16;
      a.H = 3 * p->H;
    }
  }
  // The tokens go through in chunks of f.nc rows (one chunk at the benchmark shapes): tile kernels, then the row
  // merge of that chunk, on partial-sum buffers that are one chunk wide.
  a.nc = f.nc;
  for (a.row0 = 0; a.row0 < a.Np; a.row0 += f.nc) {
    if (ph & LCE_PHASE_FWD_TILES) {
      // One launch over the whole vocabulary, or -- fp32 weight -- one per slab, each on a
      // 16-bit copy of its columns made just before it (same stream, one buffer).
      for (int64_t v0 = 0; v0 < p->V; v0 += f.vs) {
        lce::FwdArgs t = a;
        t.v0 = v0;
        t.vw = p->V - v0 < f.vs ? p->V - v0 : f.vs;
        if (p->w_dtype == LCE_F32) {
          const int64_t ld16 = a.w_vh ? p->H : lce::pad_to(t.vw, 256);
          e = a.w_vh ? lce::launch_convert_w_rows((const float*)w, p->ldw, p->H, v0, t.vw, base + f.w16, ld16,
                                                  compute_dtype(p), s)
                     : lce::launch_convert_w_slab((const float*)w, p->ldw, p->H, v0, t.vw, base + f.w16, ld16,
                                                  compute_dtype(p), splits(p), s);
          if (e != hipSuccess) return hip_fail(e, "convert_w");
          t.w = base + f.w16; t.ldw = ld16; t.w_dtype = compute_dtype(p); t.wv0 = v0; t.Vw = t.vw;
        } else {
          t.wv0 = 0; t.Vw = p->V;
        }
        e = lce::launch_fwd_tiles(t, s);
        if (e != hipSuccess) return hip_fail(e, "fwd_tiles");
      }
    }
    if (ph & LCE_PHASE_FWD_REDUCE) {
      e = lce::launch_fwd_rows(a, s);
      if (e != hipSuccess) return hip_fail(e, "fwd_rows");
    }
  }
  if (ph & LCE_PHASE_FWD_REDUCE) {
    e = lce::launch_fwd_final(a, s);
    if (e != hipSuccess) return hip_fail(e, "fwd_final");
  }
  return LCE_OK;
}

// Body of lce_forward_backward for a problem that plan_fused accepts.
int fused_impl(const lce_problem* p, const FusedPlan& f, const void* x, const void* w, const int64_t* y,
               const float* grad_out, float* lse, float* out5, int64_t* n_valid, void* dx, void* dw, void* ws,
               void* stream) {
  hipStream_t s = (hipStream_t)stream;
  char* base = (char*)ws;
  const PackPlan& k = f.k;
  const int64_t Np = lce::padded_tokens(p->N), Vp = lce::padded_vocab(p->V);
  const int64_t dxes = p->dx_dtype == LCE_F32 ? 4 : 2;
  int num_cus = 0;
  int rc = current_num_cus(&num_cus, p->max_workgroups);
  if (rc != LCE_OK) return rc;
  int64_t* n_rows = (int64_t*)(base + k.n_rows);
  int* perm = (int*)(base + k.perm);
  int64_t* yc = (int64_t*)(base + k.yc);
  int64_t* chunk_rows = (int64_t*)(base + f.chunk_rows);

  // row merge and final sums: the forward's own kernels
  lce::FwdArgs fa;
  memset(&fa, 0, sizeof(fa));
  fa.x = x; fa.w = w; fa.y = y;
  fa.N = p->N; fa.H = p->H; fa.V = p->V; fa.ldx = p->ldx; fa.ldw = p->ldw;
  fa.Np = Np; fa.Vp = Vp;
  fa.x_dtype = p->x_dtype; fa.w_dtype = p->w_dtype;
  fa.ignore_index = p->ignore_index;
  fa.scale = p->logit_scale; fa.z_reg = p->z_reg; fa.monitoring = p->monitoring ? 1 : 0;
  fa.lse = lse; fa.out5 = out5; fa.n_valid = n_valid;
  fa.part_lse = (float*)(base + f.part_lse);
  fa.part_max = (float*)(base + f.part_max);
  fa.part_pz = (float*)(base + f.part_pz);
  fa.part_sq = (float*)(base + f.part_sq);
  fa.tgt = (float*)(base + f.tgt);
  fa.blk = (float*)(base + f.blk);
  fa.lse_rows = (float*)(base + f.lse_rows);
  fa.num_cus = num_cus;
  fa.nc = f.nc;
  const bool all_rows = f.pack && p->monitoring;  // every row is computed, the kept ones first
  if (f.pack) {
    fa.n_rows = all_rows ? nullptr : n_rows; fa.perm = perm; fa.y0 = y; fa.y = yc;
  }

  // (a call restricted to some kernels works on what a full call left in the workspace)
  const int ph = p->phases ? p->phases : ~0;
  // the count of valid labels comes first (the gradients' factor needs it), with it the packing
  hipError_t e = hipSuccess;
  if (ph & LCE_PHASE_PACK) {
    e = lce::launch_compact_labels(y, p->N, p->ignore_index, (int*)(base + k.cnt), n_rows, perm, yc, s);
    if (e != hipSuccess) return hip_fail(e, "compact_labels");
  }
  if (f.pack && (ph & LCE_PHASE_PACK)) {
    e = lce::launch_chunk_rows(n_rows, p->N, f.nc, f.chunks, chunk_rows, s);
    if (e != hipSuccess) return hip_fail(e, "chunk_rows");
  }
  // an fp32 master weight: one 16-bit copy of all of it, which the three tile kernels of every chunk read
  const void* wk = w;
  int64_t ldwk = p->ldw;
  int wk_dtype = p->w_dtype;
  if (p->w_dtype == LCE_F32) {
    wk = base + f.w16;
    ldwk = f.ld16;
    wk_dtype = compute_dtype(p);
    if (ph & LCE_PHASE_PACK) {
      e = p->w_layout == LCE_W_VH
              ? lce::launch_convert_w_rows((const float*)w, p->ldw, p->H, 0, p->V, base + f.w16, f.ld16, compute_dtype(p), s)
              : lce::launch_convert_w_slab((const float*)w, p->ldw, p->H, 0, p->V, base + f.w16, f.ld16, compute_dtype(p), false, s);
      if (e != hipSuccess) return hip_fail(e, "convert_w");
    }
  }

  lce::BwdArgs b;
  memset(&b, 0, sizeof(b));
  b.w = wk; b.n_valid = n_rows; b.grad_out = grad_out;
  b.H = p->H; b.V = p->V; b.Hp = lce::padded_hidden(p->H);
  b.ldw = ldwk; b.lddx = p->lddx; b.lddw = p->lddw;
  b.x_dtype = p->x_dtype; b.w_dtype = wk_dtype; b.dx_dtype = p->dx_dtype; b.dw_dtype = p->dw_dtype;
  b.w_vh = p->w_layout == LCE_W_VH;
  b.ignore_index = p->ignore_index;
  b.scale = p->logit_scale; b.z_reg = p->z_reg;
  b.dw = dw;
  b.dz_shift = p->x_dtype == LCE_F16 && p->z_reg <= 0.03125f ? 10 : 0;  // (as in lce_backward)
  b.dz = base + f.stage;
  b.v0 = 0; b.vw = p->V; b.vs = Vp; b.wv0 = 0; b.Vw = p->V;
  b.first = 1; b.last = 1;
  b.num_cus = num_cus; b.dx_grid = num_cus; b.dw_grid = num_cus;
  b.live = lce::live_bands(lce::padded_k(p->H) * 2);
  b.part_lse = (float*)(base + f.part_lse);
  b.part_max = (float*)(base + f.part_max);
  b.part_pz = p->monitoring ? (float*)(base + f.part_pz) : nullptr;
  b.part_sq = p->monitoring ? (float*)(base + f.part_sq) : nullptr;
  b.nc = f.nc;
  b.dx_part = f.parts_on && dx ? (float*)(base + f.part) : nullptr;
  b.dw_part = f.parts_on && dw && f.chunks == 1 ? (float*)(base + f.part) : nullptr;
  b.dw_plane = f.chunks > 1 && !f.dw_direct ? (void*)(base + f.plane) : nullptr;
  b.dw_plane_hi = f.chunks > 1 && !f.dw_direct && f.total != f.plane_hi ? (void*)(base + f.plane_hi) : nullptr;

  for (int c = 0; c < f.chunks; ++c) {
    const int64_t row0 = (int64_t)c * f.nc;
    lce::BwdArgs a = b;
    a.Np = Np - row0 < f.nc ? Np - row0 : f.nc;
    a.dz_rows = a.Np;
    a.lse = (const float*)(base + f.lse_rows) + row0;
    a.tgt = (float*)(base + f.tgt) + row0;
    if (f.pack) {
      a.N = p->N;
      a.n_rows = chunk_rows + c;
      a.perm = perm + row0;
      a.perm_always = 1;
      a.x = a.xc = base + f.xc;  // the chunk's kept rows, gathered just below
      a.ldx = a.ldxc = k.ldxc;
      a.y = yc + row0;
      a.dx = dx;
    } else {
      a.N = p->N - row0 < f.nc ? p->N - row0 : f.nc;
      a.x = a.xc = (const char*)x + (size_t)row0 * (size_t)p->ldx * 2;
      a.ldx = a.ldxc = p->ldx;
      a.y = y + row0;
      a.dx = dx ? (char*)dx + (size_t)row0 * (size_t)p->lddx * dxes : nullptr;
    }
    // dW over the chunks: as halves (1: store, 2: add, 5: add and store dW; 6, 7, 8 with the lower halves cut to a byte), or
    // -- fp32 dW -- in the caller's buffer itself (3: store, 4: add)
    const bool last = c == f.chunks - 1;
    a.dw_acc = f.chunks == 1 ? 0 : f.dw_direct ? (c == 0 ? 3 : 4) : f.lo8 ? (c == 0 ? 6 : last ? 8 : 7) : (c == 0 ? 1 : last ? 5 : 2);
    if (f.pack && (ph & (LCE_PHASE_PACK | LCE_PHASE_FWD_TILES | LCE_PHASE_BWD_DW))) {
      e = lce::launch_gather_rows(x, p->ldx * 2, p->H * 2, perm + row0, chunk_rows + (all_rows ? 1024 : 0) + c, p->N,
                                  base + f.xc, k.ldxc * 2, nullptr, nullptr, num_cus, s, true);
      if (e != hipSuccess) return hip_fail(e, "gather_rows");
    }
    if (ph & LCE_PHASE_FWD_TILES) {
      lce::BwdArgs af = a;
      if (all_rows) af.n_rows = chunk_rows + 1024 + c;
      e = lce::launch_fwd_stage(af, s);
      if (e != hipSuccess) return hip_fail(e, "fwd_stage");
    }
    if (ph & LCE_PHASE_FWD_REDUCE) {
      lce::FwdArgs r = fa;
      r.row0 = row0;
      e = lce::launch_fwd_rows(r, s);
      if (e != hipSuccess) return hip_fail(e, "fwd_rows");
    }
    if ((dx || dw) && (ph & LCE_PHASE_BWD_DZ)) {
      e = lce::launch_stage_scale(a, s);
      if (e != hipSuccess) return hip_fail(e, "stage_scale");
    }
    if (dx && (ph & LCE_PHASE_BWD_DX)) {
      e = lce::launch_bwd_dx(a, s);
      if (e != hipSuccess) return hip_fail(e, "bwd_dx");
    }
    if (dw && (ph & LCE_PHASE_BWD_DW)) {
      e = lce::launch_bwd_dw(a, s);
      if (e != hipSuccess) return hip_fail(e, "bwd_dw");
    }
  }
  if (ph & LCE_PHASE_FWD_REDUCE) {
    e = lce::launch_fwd_final(fa, s);
    if (e != hipSuccess) return hip_fail(e, "fwd_final");
  }
  if (f.pack && dx && (ph & LCE_PHASE_BWD_DX)) {
    // tokens that were dropped get exact zeros (nothing to do if none was)
    e = lce::launch_scatter_rows(nullptr, 0, perm, n_rows, p->N, y, p->ignore_index, dx, p->lddx * dxes, p->H * dxes,
                                 num_cus, s);
    if (e != hipSuccess) return hip_fail(e, "scatter_rows");
  }
  return LCE_OK;
}

}  // namespace

extern "C" {

int lce_version(void) { return 500; }  // 0.5.0: lce_problem.route, lce_forward_backward, lce_scale

const char* lce_strerror(int status) {
  switch (status) {
    case LCE_OK: return "ok";
    case LCE_EINVAL_SHAPE:
      return "shape outside the supported set (need N, H, V, N_chunk_size >= 1; N <= 2^30 (2^20 for fp32 activations), "
             "V <= 2^30, H <= 2^20; "
             "ceil(N/256) * ceil(V/256) <= 2^28)";
    case LCE_EINVAL_DTYPE:
      return "unsupported dtype combination (x: bf16/f16/f32; w: x dtype or f32; grads: same dtype or f32)";
    case LCE_EINVAL_ARG:
      return "invalid argument (null or misaligned pointer; row strides must be >= the row length and multiples of 8 "
             "elements for 16-bit data, 4 for fp32, and at most 8 MiB for x, a 16-bit w and dx; logit_scale <= 0 or "
             "z_reg < 0)";
    case LCE_EWORKSPACE: return "workspace missing or too small for this problem and N_chunk_size";
    case LCE_EHIP: return "HIP error";
    case LCE_ESTATIC:
      return "problem needs more forward scratch than the library's static buffer (LCE_STATIC_SCRATCH_BYTES = 64 MiB); "
             "call lce_forward with a workspace instead";
    default: return "unknown status";
  }
}

const char* lce_last_hip_error(void) { return g_hip_error; }

int lce_check_problem(const lce_problem* p) { return check(p, true); }

int lce_workspace_bytes(const lce_problem* p, size_t* fwd_bytes, size_t* bwd_bytes) {
  int rc = check(p, false);
  if (rc != LCE_OK) return rc;
  if (fwd_bytes) *fwd_bytes = plan_fwd(p).total;
  if (bwd_bytes) {
    BwdPlan b;
    rc = plan_bwd(p, &b);
    if (rc != LCE_OK) return rc;
    *bwd_bytes = b.total;
  }
  return LCE_OK;
}

int lce_backward_plan(const lce_problem* p, int64_t* slabs, int64_t* slab_width) {
  int rc = check(p, false);
  if (rc != LCE_OK) return rc;
  BwdPlan b;
  rc = plan_bwd(p, &b);
  if (rc != LCE_OK) return rc;
  if (slabs) *slabs = b.slabs;
  if (slab_width) *slab_width = b.vs;
  return LCE_OK;
}

int lce_forward(const lce_problem* p, const void* x, const void* w, const int64_t* y, float* lse,
                float* out5, int64_t* n_valid, void* ws, size_t ws_bytes, void* stream) {
  return forward_impl(p, x, w, y, lse, out5, n_valid, ws, ws_bytes, stream);
}

int lce_forward_static(const lce_problem* p, const void* x, const void* w, const int64_t* y, float* lse,
                       float* out5, int64_t* n_valid, void* stream) {
  int rc = check(p, false);
  if (rc != LCE_OK) return rc;
  if (plan_fwd(p).total > kStaticScratchBytes) return LCE_ESTATIC;  // before any device call
  void* ptr = nullptr;
  rc = static_scratch(&ptr);
  if (rc != LCE_OK) return rc;
  // Nothing in the forward scratch has to start at zero: every cell a kernel reads was written by an
  // earlier kernel of the same call, so the contents the previous call left behind are never looked at.
  return forward_impl(p, x, w, y, lse, out5, n_valid, ptr, kStaticScratchBytes, stream);
}

int lce_backward(const lce_problem* p, const void* x, const void* w, const int64_t* y,
                 const float* lse, const int64_t* n_valid, const float* grad_out, void* dx,
                 void* dw, void* ws, size_t ws_bytes, void* stream) {
  int rc = check(p, true);
  if (rc != LCE_OK) return rc;
  if (!x || !w || !y || !lse || !n_valid || !grad_out) return LCE_EINVAL_ARG;
  if (misaligned(x) || misaligned(w) || misaligned(dx) || misaligned(dw)) return LCE_EINVAL_ARG;
  if (!dx && !dw) return LCE_OK;
  BwdPlan b;
  rc = plan_bwd(p, &b);
  if (rc != LCE_OK) return rc;
  if (!ws || ws_bytes < b.total || misaligned(ws)) return LCE_EWORKSPACE;
  hipStream_t s = (hipStream_t)stream;
  char* base = (char*)ws;

  lce::BwdArgs a;
  memset(&a, 0, sizeof(a));
  a.x = x; a.w = w; a.y = y; a.lse = lse; a.n_valid = n_valid; a.grad_out = grad_out;
  a.N = p->N; a.H = p->H; a.V = p->V;
  a.Np = lce::padded_tokens(p->N); a.Hp = lce::padded_hidden(p->H);
  a.ldx = p->ldx; a.ldw = p->ldw; a.lddx = p->lddx; a.lddw = p->lddw;
  a.x_dtype = p->x_dtype; a.w_dtype = p->w_dtype; a.dx_dtype = p->dx_dtype; a.dw_dtype = p->dw_dtype;
  a.w_vh = p->w_layout == LCE_W_VH;
  a.ignore_index = p->ignore_index;
  a.scale = p->logit_scale; a.z_reg = p->z_reg;
  a.dx = dx; a.dw = dw;
  // fp16 staging of dz: times 2^10, unless z_reg is so large that the factor 1 + 2 * z_reg * lse on top of it would
  // leave fp16's range for ordinary logits (with the factor 2^10 in place bwd_dz clamps that factor to +-63, which
  // |lse| < 992 never reaches at z_reg <= 1/32)
  a.dz_shift = p->x_dtype == LCE_F16 && p->z_reg <= 0.03125f ? 10 : 0;
  a.dz = base + b.dz;
  a.dx_acc = b.slabs > 1 || splits(p) ? (float*)(base + b.dx_acc) : nullptr;
  a.dx_part = b.parts_on ? (float*)(base + b.dx_part) : nullptr;
  a.dw_part = b.parts_on ? (float*)(base + b.dw_part) : nullptr;
  rc = current_num_cus(&a.num_cus, p->max_workgroups);
  if (rc != LCE_OK) return rc;
  a.live = lce::live_bands(lce::padded_k(splits(p) ? 3 * p->H : p->H) * 2);
  const int ph = p->phases ? p->phases : ~0;

  // Tokens with an ignored label have dz == 0: the kernels run on the other rows only, packed to the front.
  const PackPlan& k = b.pack;
  const bool pack = b.pack_on, x32 = p->x_dtype == LCE_F32;
  const int64_t dxes = p->dx_dtype == LCE_F32 ? 4 : 2;
  a.xc = base + k.xc;
  a.ldxc = k.ldxc;
  if (pack) {
    a.n_rows = (const int64_t*)(base + k.n_rows);
    a.perm = (const int*)(base + k.perm);
    a.dxc = b.stage_dx ? base + b.dxc : nullptr;
    a.lddxc = b.lddxc;
    a.y = (const int64_t*)(base + k.yc);
    a.lse = (const float*)(base + b.lse_c);
  }
  if ((pack || x32) && (ph & LCE_PHASE_PACK)) {
    const int* perm = pack ? (const int*)(base + k.perm) : nullptr;
    hipError_t e;
    if (pack) {
      e = lce::launch_compact_labels(y, p->N, p->ignore_index, (int*)(base + k.cnt), (int64_t*)(base + k.n_rows),
                                     (int*)(base + k.perm), (int64_t*)(base + k.yc), s);
      if (e != hipSuccess) return hip_fail(e, "compact_labels");
    }
    float* lse_c = pack ? (float*)(base + b.lse_c) : nullptr;
    e = x32 ? lce::launch_gather_rows_split((const float*)x, p->ldx, p->H, perm, a.n_rows, p->N, base + k.xc, k.ldxc,
                                            base + k.xk, k.ldxk, pack ? lse : nullptr, lse_c, a.num_cus, s)
            : lce::launch_gather_rows(x, p->ldx * 2, p->H * 2, perm, a.n_rows, p->N, base + k.xc, k.ldxc * 2, lse, lse_c,
                                      a.num_cus, s);
    if (e != hipSuccess) return hip_fail(e, "gather_rows");
  }
  if (x32) {  // fp32 activations reach the tile kernels as copies in bf16 pairs, whether or not rows were dropped
    a.x = a.xc;
    a.ldx = a.ldxc;
    a.x_dtype = lce::DT_BF16;
  }
  const bool split = splits(p);
  a.dz_rows = split ? 3 * a.Np : a.Np;  // rows of the dz stage (BwdArgs::dz)

  for (int64_t i = 0; i < b.slabs; ++i) {
    a.v0 = i * b.vs;
    a.vw = p->V - a.v0 < b.vs ? p->V - a.v0 : b.vs;   // columns of this slab that exist
    a.vs = lce::pad_to(a.vw, 256);                    // its padded width: dz row stride and K extent of dx
    a.dx_grid = a.num_cus;
    a.dw_grid = a.num_cus;
    hipError_t e;
    if (p->w_dtype == LCE_F32) {
      // dz and dx of this slab read a 16-bit copy of its columns of the fp32 weight
      if ((ph & LCE_PHASE_BWD_DZ) || (dx && (ph & LCE_PHASE_BWD_DX))) {
        e = a.w_vh ? lce::launch_convert_w_rows((const float*)w, p->ldw, p->H, a.v0, a.vw, base + b.w16, p->H,
                                                compute_dtype(p), s)
                   : lce::launch_convert_w_slab((const float*)w, p->ldw, p->H, a.v0, a.vw, base + b.w16, a.vs,
                                                compute_dtype(p), split, s);
        if (e != hipSuccess) return hip_fail(e, "convert_w");
      }
      a.w = base + b.w16; a.ldw = a.w_vh ? p->H : a.vs; a.w_dtype = compute_dtype(p); a.wv0 = a.v0; a.Vw = a.vw;
    } else {
      a.wv0 = 0; a.Vw = p->V;
    }
    a.first = i == 0;
    a.last = i == b.slabs - 1;
    if (!split) {
      if (ph & LCE_PHASE_BWD_DZ) {
        e = lce::launch_bwd_dz(a, s);
        if (e != hipSuccess) return hip_fail(e, "bwd_dz");
      }
      if (dx && (ph & LCE_PHASE_BWD_DX)) {
        e = lce::launch_bwd_dx(a, s);
        if (e != hipSuccess) return hip_fail(e, "bwd_dx");
      }
      if (dw && (ph & LCE_PHASE_BWD_DW)) {
        e = lce::launch_bwd_dw(a, s);
        if (e != hipSuccess) return hip_fail(e, "bwd_dw");
      }
      continue;
    }
    // fp32 tensors as bf16 pairs (lce_gemm.h): x = [hi | hi | lo] against W = [hi ; lo ; hi] along a K axis of
    // 3 H for the logits; dz comes back as three parts [hi ; lo ; hi] of Np rows.
    char* dz0 = (char*)a.dz;
    const int64_t blk = a.Np * a.vs * 2;  // bytes from the first row of a part to that of the next
    if (ph & LCE_PHASE_BWD_DZ) {
      lce::BwdArgs z = a;
      z.H = 3 * p->H;
      z.split = 1;
      e = lce::launch_bwd_dz(z, s);
      if (e != hipSuccess) return hip_fail(e, "bwd_dz");
    }
    if (dx && (ph & LCE_PHASE_BWD_DX)) {
      // dx += dz_hi W_hi^T + dz_lo W_hi^T + dz_hi W_lo^T: three passes over the running fp32 sum
      const char* w_hi = (const char*)a.w;
      const char* w_lo = w_hi + p->H * a.ldw * 2;
      for (int pass = 0; pass < 3; ++pass) {
        lce::BwdArgs d = a;
        d.dz = dz0 + (pass == 1 ? blk : 0);
        d.w = pass == 2 ? w_lo : w_hi;
        d.first = a.first && pass == 0;
        d.last = a.last && pass == 2;
        e = lce::launch_bwd_dx(d, s);
        if (e != hipSuccess) return hip_fail(e, "bwd_dx");
      }
    }
    if (dw && (ph & LCE_PHASE_BWD_DW)) {
      // dW = x_hi^T dz_hi + x_hi^T dz_lo + x_lo^T dz_hi: one contraction over 3 Np token rows, the copy of x
      // stacked [hi ; hi ; lo] against the three blocks of dz (rows past the last kept token are zeros in both)
      lce::BwdArgs g = a;
      g.x = base + k.xk;
      g.ldx = k.ldxk;
      g.n_rows = nullptr;
      g.N = 3 * a.Np;
      g.Np = 3 * a.Np;
      e = lce::launch_bwd_dw(g, s);
      if (e != hipSuccess) return hip_fail(e, "bwd_dw");
    }
  }
  if (pack && dx && (ph & LCE_PHASE_BWD_DX)) {
    // dropped tokens get exact zeros, staged packed rows go to their tokens (nothing to do if none was dropped)
    hipError_t e = lce::launch_scatter_rows(a.dxc, b.lddxc * dxes, (const int*)(base + k.perm), a.n_rows, p->N, y,
                                            p->ignore_index, dx, p->lddx * dxes, p->H * dxes, a.num_cus, s);
    if (e != hipSuccess) return hip_fail(e, "scatter_rows");
  }
  return LCE_OK;
}

int lce_scale(void* t, int dtype, int64_t rows, int64_t cols, int64_t ld, const float* factor, void* stream) {
  if (dtype != LCE_BF16 && dtype != LCE_F16 && dtype != LCE_F32) return LCE_EINVAL_DTYPE;
  if (rows < 0 || cols < 0 || ld < cols || ld % (dtype == LCE_F32 ? 4 : 8) || !factor) return LCE_EINVAL_ARG;
  if (rows == 0 || cols == 0) return LCE_OK;
  if (!t || misaligned(t)) return LCE_EINVAL_ARG;
  int num_cus = 0;
  int rc = current_num_cus(&num_cus, 0);
  if (rc != LCE_OK) return rc;
  hipError_t e = lce::launch_scale_rows(t, dtype, rows, cols, ld, factor, num_cus, (hipStream_t)stream);
  if (e != hipSuccess) return hip_fail(e, "scale_rows");
  return LCE_OK;
}

int lce_forward_backward_workspace_bytes(const lce_problem* p, size_t* bytes) {
  int rc = check(p, true);
  if (rc != LCE_OK) return rc;
  if (!bytes) return LCE_EINVAL_ARG;
  FusedPlan f;
  if (plan_fused(p, true, true, &f)) { *bytes = f.total; return LCE_OK; }
  size_t fw = 0, bw = 0;
  rc = lce_workspace_bytes(p, &fw, &bw);
  if (rc != LCE_OK) return rc;
  *bytes = fw > bw ? fw : bw;
  return LCE_OK;
}

int lce_forward_backward_plan(const lce_problem* p, int64_t* chunks, int64_t* chunk_rows) {
  int rc = check(p, true);
  if (rc != LCE_OK) return rc;
  FusedPlan f;
  const bool ok = plan_fused(p, true, true, &f);
  if (chunks) *chunks = ok ? f.chunks : 0;
  if (chunk_rows) *chunk_rows = ok ? f.nc : 0;
  return LCE_OK;
}

int lce_forward_backward(const lce_problem* p, const void* x, const void* w, const int64_t* y,
                         const float* grad_out, float* lse, float* out5, int64_t* n_valid, void* dx,
                         void* dw, void* ws, size_t ws_bytes, void* stream) {
  int rc = check(p, true);
  if (rc != LCE_OK) return rc;
  if (!x || !w || !y || !grad_out || !lse || !out5 || !n_valid) return LCE_EINVAL_ARG;
  if (misaligned(x) || misaligned(w) || misaligned(dx) || misaligned(dw)) return LCE_EINVAL_ARG;
  FusedPlan f;
  if ((dx || dw) && plan_fused(p, true, true, &f)) {
    if (!ws || ws_bytes < f.total || misaligned(ws)) return LCE_EWORKSPACE;
    return fused_impl(p, f, x, w, y, grad_out, lse, out5, n_valid, dx, dw, ws, stream);
  }
  // two passes over the logits, on the same workspace one after the other
  rc = forward_impl(p, x, w, y, lse, out5, n_valid, ws, ws_bytes, stream);
  if (rc != LCE_OK || (!dx && !dw)) return rc;
  return lce_backward(p, x, w, y, lse, n_valid, grad_out, dx, dw, ws, ws_bytes, stream);
}

}  // extern "C"
