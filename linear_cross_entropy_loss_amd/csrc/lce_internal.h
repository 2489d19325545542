// Internal launch interface between the C ABI (lce_api.hip) and the kernel
// translation units.  Not installed; the public surface is include/lce.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>

namespace lce {

enum { DT_BF16 = 0, DT_F16 = 1, DT_F32 = 2 };

// The tile kernels use more dynamic LDS than a kernel gets by default and have to opt in
// (hipFuncAttributeMaxDynamicSharedMemorySize): once per kernel and device, not before every launch.  One object
// per kernel (a function-local static of its launcher); thread-safe.
struct LdsOptIn {
  std::atomic<uint64_t> done{0};  // bit d: set on device d (devices from 64 on are set every time)
  hipError_t ensure(const void* kernel, int bytes) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return e;
    if (dev >= 0 && dev < 64 && ((done.load(std::memory_order_acquire) >> dev) & 1)) return hipSuccess;
    e = hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess && dev >= 0 && dev < 64) done.fetch_or((uint64_t)1 << dev, std::memory_order_release);
    return e;
  }
};

// Columns of logits covered by one forward partial (one wave's slice of a tile).
constexpr int kChunkV = 128;
// Rows handled by one workgroup of the row-merge kernel.
constexpr int kMergeRows = 64;

// Shapes need not be multiples of the tile sizes: the kernels work on the padded
// extents below, operand loads past the real extents return zero (buffer range
// checks and a K mask), and the epilogues neither use logits of columns >= V nor
// store anything for rows >= N, columns >= V or hidden indices >= H.
constexpr int64_t pad_to(int64_t v, int64_t m) { return (v + m - 1) / m * m; }
constexpr int64_t padded_tokens(int64_t N) { return pad_to(N, 256); }   // token tiles; K tiles of the dW contraction
constexpr int64_t padded_vocab(int64_t V) { return pad_to(V, 256); }    // vocabulary tiles
constexpr int64_t padded_hidden(int64_t H) { return pad_to(H, 256); }   // hidden tiles of dx and dW
// K extent of the logit contraction: an even number of 64-wide K tiles, at least four
constexpr int64_t padded_k(int64_t H) { return pad_to(H, 128) < 256 ? 256 : pad_to(H, 128); }

struct FwdArgs {
  const void* x;
  const void* w;
  const int64_t* y;
  int64_t N, H, V, ldx, ldw;
  int64_t Np, Vp;  // padded_tokens(N), padded_vocab(V)
  // Token rows [row0, row0 + nc) covered by this launch (both multiples of 256): the forward works through the
  // rows in chunks of nc, so that the per-slice partials below are nc rows wide however many tokens there are.
  int64_t row0, nc;
  // Vocabulary columns [v0, v0 + vw) covered by this launch (v0 a multiple of 256), and the
  // window of W that the buffer `w` holds: columns [wv0, wv0 + Vw) of the weight, row stride ldw.
  // (`w` is the caller's matrix, wv0 = 0, Vw = V -- or a 16-bit copy of one slab of an fp32 weight.)
  int64_t v0, vw, wv0, Vw;
  // w_vh != 0: the weight is stored with the vocabulary as its row index, w[v * ldw + h] (the buffer `w` then
  // holds ROWS [wv0, wv0 + Vw)); otherwise w[h * ldw + v].
  int w_vh;
  int x_dtype, w_dtype;  // compute type = x_dtype (bf16 / f16)
  int64_t ignore_index;
  float scale, z_reg;
  int monitoring;
  // Packed rows (tokens with an ignored label dropped; null / unused when the call works on all rows):
  // *n_rows (device) rows are worked on; when *n_rows != N they are the rows of xc (row stride ldxc) and
  // `y` holds their labels; perm[j] is the token that packed row j came from, y0 the labels of all tokens.
  const int64_t* n_rows;
  const void* xc;
  int64_t ldxc;
  const int* perm;
  const int64_t* y0;
  int num_cus;  // compute units of the device: grid size of the persistent kernels
  int live;     // bands of W that the XCDs keep in flight together (lce_gemm.h, tile_coords)
  // outputs / scratch
  float* lse;        // [N]
  float* out5;       // [5]
  int64_t* n_valid;  // [1]
  float* part_lse;   // [Vp/128][nc]  per-slice logsumexp (-inf for a slice with no valid column), rows of the current chunk
  float* part_max;   // [Vp/128][nc]  per-slice max            (monitoring)
  float* part_pz;    // [Vp/128][nc]  per-slice sum softmax*z  (monitoring)
  float* part_sq;    // [Vp/128][nc]  per-slice sum z^2        (monitoring)
  float* tgt;        // [Np]          target logit (written for tokens whose label is a column of W)
  float* blk;        // [Np/64][8]    per-merge-block partial sums
  float* lse_rows;   // [Np] or null  lse of every row in the order the tile kernels see them (packed rows), whatever its label
};

struct BwdArgs {
  const void* x;
  const void* w;
  const int64_t* y;
  const float* lse;
  const int64_t* n_valid;
  const float* grad_out;
  int64_t N, H, V, ldx, ldw, lddx, lddw;
  int64_t Np, Hp;  // padded_tokens(N), padded_hidden(H)
  int x_dtype, w_dtype, dx_dtype, dw_dtype;
  int64_t ignore_index;
  float scale, z_reg;
  void* dx;
  void* dw;
  // slab being processed
  int64_t v0, vs;   // first column and padded width (multiple of 256) of the vocabulary slab
  int64_t vw;       // columns of the slab that exist: min(vs, V - v0)
  int64_t wv0, Vw;  // `w` holds columns [wv0, wv0 + Vw) of the weight (the whole matrix, or a 16-bit copy of this slab)
  // w_vh != 0: weight and dW are stored with the vocabulary as their row index, w[v * ldw + h], dw[v * lddw + h]
  // (and the buffer `w` holds ROWS [wv0, wv0 + Vw)); otherwise w[h * ldw + v], dw[h * lddw + v].
  int w_vh;
  // Staged dz in the compute type (exact zeros outside N x vw), stored in blocks of 256 rows x 64 columns,
  // [rows / 256][vs / 64][256][64] (dz_block_offset below): the 64-deep K tiles of the dx contraction (K = v) are
  // consecutive 32 KiB blocks, the K tiles of the dW contraction (K = tokens) quarters of four neighbouring blocks,
  // and a token's 64 columns of a group are one 128-byte line.  dz_rows = Np rows, or 3 Np when dz is carried as
  // bf16 pairs (`split` below).
  void* dz;
  int64_t dz_rows;
  float* dx_acc;    // [Np][Hp] fp32 running dx (null when there is a single slab)
  // dx: tiles of a last, mostly idle round of workgroups are cut along K instead (planned on the device,
  // see lce_bwd_dx.hip); the segments' partial sums meet in dx_part, dx_tail_blocks() blocks of 256 x 256
  // floats, and a small kernel adds them in a fixed order.  dx_grid = workgroups of the tile kernel.
  int dx_grid;
  float* dx_part;
  // The same for dW (K = tokens): dw_part holds dw_tail_blocks() blocks, dw_grid = workgroups of the tile kernel.
  int dw_grid;
  float* dw_part;
  // The staged dz = softmax * gain - onehot is multiplied by 2^dz_shift before it is rounded to the 16-bit compute
  // type, and the dx / dW kernels fold 2^-dz_shift into their final factor.  bf16 has fp32's exponent range and
  // needs none (0); in fp16 the softmax probabilities of a large vocabulary (of order 1/V) would fall below the
  // normal range (6.1e-5) and lose precision bit by bit -- with 10 they stay normal down to 6e-8, while
  // |dz| * 2^10 stays below fp16's maximum for any gain = 1 + 2 * z_reg * lse below 63: bwd_dz clamps the gain to
  // +-63 when the factor is in place, and the host takes 0 instead when z_reg > 1/32, where logits of ordinary size
  // (|lse| < 992 at 1/32) would already reach that.
  int dz_shift;
  int first, last;  // slab position
  int num_cus;      // compute units of the device: grid size of the persistent kernels
  int live;         // bwd_dz: bands of W that the XCDs keep in flight together (lce_gemm.h, tile_coords)
  // fp32 tensors carried as bf16 pairs (lce_gemm.h): the stage holds three parts of Np rows each, [hi ; lo ; hi];
  // only bwd_dz looks at this flag (the dx and dW launches get plain 16-bit problems over these parts: dx with `dz`
  // pointing at the first row of a part, dW with 3 Np token rows).
  int split;
  // Packed rows (tokens with an ignored label dropped; n_rows == null: the call works on all rows).
  // *n_rows (device) rows are worked on.  When *n_rows != N they are the rows of xc (row stride ldxc) and
  // row j of dx belongs to token perm[j]: the dx kernels store it there themselves, or -- dxc != null, a dx
  // of 2 GiB or more -- into dxc (row stride lddxc), from where it is moved afterwards.  In either case `y`
  // and `lse` hold the labels / lse of the packed rows.
  const int64_t* n_rows;
  const int* perm;
  const void* xc;
  int64_t ldxc;
  void* dxc;
  int64_t lddxc;
  // One pass over the logits (lce_forward_backward): the problem is a chunk of token rows against the whole
  // vocabulary, and the logit kernel (launch_fwd_stage) leaves, instead of dz,
  //     e[token][v] = 2^dz_shift * exp(z[token][v] - m[token][v / 128])
  // in the stage, m = the largest logit of the token in that slice of 128 columns, together with the forward's
  // per-slice partials of the chunk: part_lse, part_max = m ([Vp/128][nc], as in FwdArgs) and the target logits
  // tgt (first row of the chunk).  Once the rows' lse are known, launch_stage_scale turns e into dz in place.
  float* part_lse;
  float* part_max;
  float* part_pz;  // both null, or the monitoring partials of FwdArgs as well
  float* part_sq;
  float* tgt;
  int64_t nc;
  // rows of dx always go to the tokens perm[] names (the rows of a chunk can be all there and still not be the
  // tokens of the same numbers)
  int perm_always;
  // 16-bit dW summed over chunks of token rows: the fp32 sums are kept as 16-bit halves, the upper ones in dw
  // itself, the lower ones in dw_plane (one block of 256 x 256 halves per tile of dW); dw_plane_hi takes the upper
  // halves of the tiles that the edge of the matrix cuts (null if there is none) -- see lce_bwd_dw.hip.
  // dw_acc: 0 = no sums over chunks (dW is stored as it comes), 1 = the sums are stored (first chunk), 2 = added
  // to, 5 = added to, and the result scaled and stored as dW (last chunk); 6, 7, 8 = the same three with only the
  // upper byte of each lower half kept (dw_plane: 256 x 256 bytes per tile; the sums are rounded at 24 bits).
  // fp32 dW: 3 = the sums times the final factor are stored to dw itself (first chunk), 4 = added to it.
  void* dw_plane;
  void* dw_plane_hi;
  int dw_acc;
  int vtail_all;  // the logit kernel for the tile column that straddles the end of the vocabulary takes every column
};

// Element offset of block (row tile, column group) of a dz stage that is `vs` columns wide.
constexpr int kDzBlockElems = 256 * 64;
__host__ __device__ inline int64_t dz_block_offset(int64_t row_tile, int64_t group, int64_t vs) {
  return (row_tile * (vs / 64) + group) * kDzBlockElems;
}

// Factor applied to dx and dW after their fp32 accumulation: grad_out * logit_scale / n_valid
// (linear_cross_entropy/ops.py:332, 443-447, 810), times the power of two that undoes the scaling of the staged
// dz.  With no valid label at all every dz is zero and the factor is taken as 0, so both
// gradients are exact zeros (what F.cross_entropy's backward gives for such a batch; the loss itself is NaN).
__device__ __forceinline__ float final_factor_of(const BwdArgs& a) {
  const int64_t n = a.n_valid[0];
  const float unscale = __builtin_bit_cast(float, (127 - a.dz_shift) << 23);  // 2^-dz_shift
  return n > 0 ? a.grad_out[0] * a.scale / (float)n * unscale : 0.f;
}

hipError_t launch_fwd_tiles(const FwdArgs& a, hipStream_t s);
// Row merge of the current chunk (lse, per-block sums), and -- once, after the last chunk -- the final reduction.
hipError_t launch_fwd_rows(const FwdArgs& a, hipStream_t s);
hipError_t launch_fwd_final(const FwdArgs& a, hipStream_t s);
hipError_t launch_bwd_dz(const BwdArgs& a, hipStream_t s);
// The logit kernel of lce_forward_backward and the pass that follows the row merge (see BwdArgs).
hipError_t launch_fwd_stage(const BwdArgs& a, hipStream_t s);
hipError_t launch_stage_scale(const BwdArgs& a, hipStream_t s);
// t[r][c] *= g[0] (device scalar), in fp32; nothing is touched when g[0] == 1.  Rows on 16-byte boundaries.
hipError_t launch_scale_rows(void* t, int dtype, int64_t rows, int64_t cols, int64_t ld, const float* g, int num_cus,
                             hipStream_t s);
// out[c] = rows of chunk c (of `nc` rows each) among the *n_rows packed rows: min(max(*n_rows - c * nc, 0), nc);
// out[1024 + c] = the same among all N rows (out holds 2048 entries).
hipError_t launch_chunk_rows(const int64_t* n_rows, int64_t N, int64_t nc, int chunks, int64_t* out, hipStream_t s);
hipError_t launch_bwd_dx(const BwdArgs& a, hipStream_t s);
hipError_t launch_bwd_dw(const BwdArgs& a, hipStream_t s);
// dst[h][c] = 16-bit rounding of src[h * ld + v0 + c] for c < vw, 0 for vw <= c < dst_ld; h < H.
// compute_dtype: DT_BF16 or DT_F16.  split: dst has 3 H rows, [bf16 hi ; bf16 lo ; bf16 hi] of the fp32 values.
hipError_t launch_convert_w_slab(const float* src, int64_t ld, int64_t H, int64_t v0, int64_t vw, void* dst,
                                 int64_t dst_ld, int compute_dtype, bool split, hipStream_t s);
// The same for a weight stored (V, H) row-major (H a multiple of 8): rows [v0, v0 + vw) go to dst[vw][dst_ld].
hipError_t launch_convert_w_rows(const float* src, int64_t ld, int64_t H, int64_t v0, int64_t vw, void* dst,
                                 int64_t dst_ld, int compute_dtype, hipStream_t s);

// Row count / row -> token map of the packed rows as the kernels read them from device memory, forced
// into range: a call restricted to some phases on a workspace whose packing pre-pass did not run must
// give wrong numbers, not wild addresses.
__device__ __forceinline__ int64_t packed_rows(const int64_t* n_rows, int64_t N) {
  if (n_rows == nullptr) return N;  // this call works on all rows
  const int64_t r = n_rows[0];
  return r < 0 ? 0 : (r > N ? N : r);
}
__device__ __forceinline__ int64_t packed_token(const int* perm, int64_t j, int64_t N) {
  const int64_t t = perm[j];
  return t < 0 ? 0 : (t >= N ? N - 1 : t);
}

// Packing of the tokens whose label is not ignore_index (lce_compact.hip).  `cnt` holds one int per
// compact_segments(N); perm and yc hold N entries each: the kept tokens first (*n_rows of them), then the dropped ones.
int64_t compact_segments(int64_t N);
hipError_t launch_compact_labels(const int64_t* y, int64_t N, int64_t ignore_index, int* cnt, int64_t* n_rows,
                                 int* perm, int64_t* yc, hipStream_t s);
// xc[j] = x[perm[j]] for j < *n_rows, in 16-byte pieces of rows ldxc_bytes long (skipped when *n_rows == N);
// row_bytes = bytes of a row that hold elements (nothing past them is read of the last row of x);
// lse_c[j] = lse[perm[j]] when lse is not null (always).  `always`: the rows are copied also when *n_rows == N.
hipError_t launch_gather_rows(const void* x, int64_t ldx_bytes, int64_t row_bytes, const int* perm,
                              const int64_t* n_rows, int64_t N, void* xc, int64_t ldxc_bytes, const float* lse,
                              float* lse_c, int num_cus, hipStream_t s, bool always = false);
// fp32 activations: xc[j] = [hi | hi | lo] of x[perm[j]] as bf16 (3 H elements per row, row stride ldxc), and
// -- xk not null -- the same three parts stacked along the tokens, xk[b * Np + j] (row stride ldxk, rows from
// *n_rows to Np of each block zeroed).  Always made, also when no token is dropped; perm / n_rows may be null
// (all N rows in their order).  Strides in elements.
hipError_t launch_gather_rows_split(const float* x, int64_t ldx, int64_t H, const int* perm, const int64_t* n_rows,
                                    int64_t N, void* xc, int64_t ldxc, void* xk, int64_t ldxk, const float* lse,
                                    float* lse_c, int num_cus, hipStream_t s);
// dx[perm[j]] = dxc[j] for j < *n_rows (skipped when dxc is null) and dx[i] = 0 for every token i with
// y[i] == ignore_index, in 8-byte pieces covering row_bytes; nothing when *n_rows == N.
hipError_t launch_scatter_rows(const void* dxc, int64_t lddxc_bytes, const int* perm, const int64_t* n_rows,
                               int64_t N, const int64_t* y, int64_t ignore_index, void* dx, int64_t lddx_bytes,
                               int64_t row_bytes, int num_cus, hipStream_t s);

// Bands to keep in flight (tile_coords in lce_gemm.h) for P bands of 8 tiles of 256 rows and `k_bytes` bytes per row:
// as many of 8, 4, 2, 1 as stay within a quarter of the Infinity Cache together (measured at H = 8192, where a band is
// 32 MiB: bwd_dz 27.5 / 26.4 / 25.0 / 25.2 ms with 8 / 4 / 2 / 1 bands in flight; no difference at H = 4096; 8 best at H = 2048).
inline int live_bands(int64_t k_bytes) {
  const int64_t band_bytes = 8 * 256 * k_bytes;
  int live = 8;
  while (live > 1 && live * band_bytes > ((int64_t)64 << 20)) live /= 2;
  return live;
}

// dx of one slab: at most (Np/256) x (Hp/256) tiles, K = vs columns.  Upper bound on the 256 x 256 fp32
// blocks of partial sums that the device-side plan of the dx kernel can ask for (0: it never splits).
constexpr int kTailBlocks = 256;
// most segments per tile: a power of two that leaves at least 16 K tiles per segment
inline int64_t max_k_segments(int64_t kt) {
  int64_t s = 1;
  while (kt / (s * 2) >= 16 && s * 2 <= kTailBlocks) s *= 2;
  return s;
}
inline int64_t dx_tail_blocks(int64_t Np, int64_t Hp, int64_t vs) {
  const int64_t s = max_k_segments(vs / 64);
  if (s == 1) return 0;
  const int64_t most = (Np / 256) * (Hp / 256) * s;
  return most < kTailBlocks ? most : kTailBlocks;
}
// Whether T output tiles on G workgroups end in a last round that the kernels cut along K (at most half full).
inline bool has_split_tail(int64_t T, int64_t G) {
  const int64_t r = T % G, cap = G < kTailBlocks ? G : kTailBlocks;
  return r > 0 && r * 2 <= cap;
}
// Whether every one of T output tiles with `kt` K tiles each is a tail tile of the device-side plans (dx_plan,
// dw_plan): fewer tiles than workgroups, few enough to split, and a K extent long enough for two segments.
inline bool all_tiles_are_tails(int64_t T, int64_t G, int64_t kt) {
  return T < G && has_split_tail(T, G) && kt / 2 >= 16;
}
// true if every split the dx kernel may choose cuts the K tiles of a slab into equal, even segments
inline bool dx_segments_exact(int64_t vs) { return (vs / 64) % (2 * max_k_segments(vs / 64)) == 0; }
// dW of one slab: (vs/256) x (Hp/256) tiles, K = at most Np tokens.  The same bound for the dW kernel, whose
// segments need not divide the K tiles evenly.
inline int64_t dw_tail_blocks(int64_t Np, int64_t Hp, int64_t vs) {
  const int64_t s = max_k_segments(Np / 64);
  if (s == 1) return 0;
  const int64_t most = (vs / 256) * (Hp / 256) * s;
  return most < kTailBlocks ? most : kTailBlocks;
}

}  // namespace lce
