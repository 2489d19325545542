/*
 * lce.h -- C ABI of liblce_gfx950.so: fused linear + cross-entropy loss for
 * AMD MI355X (gfx950), forward and backward.
 *
 * The library replaces the device side of the reference operator
 * (JonasGeiping/linear_cross_entropy_loss).  Citations below are to files of
 * that repository.
 *
 * Conventions
 *   - All pointers except `lce_problem*` are DEVICE pointers; all work is
 *     enqueued on `stream` (a hipStream_t passed as void*) and nothing is
 *     synchronised.  No entry point allocates or frees device memory and the
 *     library keeps no state between calls: scratch comes in through `ws`.
 *   - x is (N, H) row-major with row stride ldx; w is the TRANSPOSED weight
 *     (H, V) row-major with row stride ldw (linear_cross_entropy/ops.py:913);
 *     y is N contiguous int64 labels (ops.py:210), each ignore_index or in
 *     [0, V); any other value makes the returned loss NaN.
 *   - Shapes: any N, H, V, n_chunk >= 1 (N <= 2^30 -- 2^20 for fp32
 *     activations --, V <= 2^30, H <= 2^20).  The
 *     reference's divisibility rules (N % 512, H % 256, V % 4096,
 *     ops.py:689-691, 905-907) are lifted; shapes that obey them run at full
 *     speed, others pay for partly empty tiles.
 *     256 rows of x, of a 16-bit w and of dx must span less than 2 GiB (row
 *     stride in bytes <= 8 MiB, i.e. 4 Mi elements of 16-bit data), and
 *     ceil(N/256) * ceil(V/256) <= 2^28; beyond that the calls return
 *     LCE_EINVAL_ARG / LCE_EINVAL_SHAPE.
 *   - Row strides keep every row 16-byte aligned: ldx, ldw (and lddw for a
 *     16-bit dW) are multiples of 8 elements for 16-bit data, 4 for fp32; lddx
 *     is a multiple of 4.  A stride larger than the row length is fine.  When
 *     the row length is not such a multiple, the elements between the end of a
 *     row and the next multiple ("stride padding") are read, must be finite,
 *     and never influence a result; the same positions of dx / dW rows may be
 *     written.  Of the LAST row of x and w nothing is read past the 4-byte
 *     word that holds its last element, so a matrix may end with that row's
 *     elements (an allocation of (rows - 1) * ld + cols elements, rounded up to
 *     4 bytes; with an odd row length the other half of that last word counts
 *     as stride padding and must be finite).  dx and dw are written in pieces of up to 16 bytes and need
 *     all rows * ld elements.
 *   - Every function returns LCE_OK (0) or a negative lce_status; nothing
 *     throws or aborts.
 */
#ifndef LCE_H_
#define LCE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum lce_dtype {
  LCE_BF16 = 0,
  LCE_F16 = 1,
  LCE_F32 = 2
} lce_dtype;

typedef enum lce_status {
  LCE_OK = 0,
  LCE_EINVAL_SHAPE = -1, /* non-positive or oversized N, H, V, n_chunk (ops.py:43-44)  */
  LCE_EINVAL_DTYPE = -2, /* unsupported dtype combination                            */
  LCE_EINVAL_ARG = -3,   /* null pointer, bad stride, bad scalar                     */
  LCE_EWORKSPACE = -4,   /* workspace missing or smaller than lce_workspace_bytes    */
  LCE_EHIP = -5,         /* a HIP launch failed; see lce_last_hip_error              */
  LCE_ESTATIC = -6       /* lce_forward_static: problem needs more than LCE_STATIC_SCRATCH_BYTES */
} lce_status;

/*
 * One problem instance.  Mirrors the argument list of
 * LinearXentImplementation.forward (ops.py:669-679) plus the strides and
 * dtypes the Triton launches took from the tensors (ops.py:731-734).
 */
typedef struct lce_problem {
  int64_t N;            /* tokens (x flattened to (N, H), ops.py:681)         */
  int64_t H;            /* in_features                                         */
  int64_t V;            /* out_features (vocabulary)                           */
  int64_t ldx;          /* row stride of x, elements                           */
  int64_t ldw;          /* row stride of w, elements (see w_layout)            */
  int64_t lddx;         /* row stride of dx, elements (backward only)          */
  int64_t lddw;         /* row stride of dw, elements (backward only; see w_layout) */
  int32_t x_dtype;      /* LCE_BF16 | LCE_F16 | LCE_F32 (see "Arithmetic" below)  */
  int32_t w_dtype;      /* same as x_dtype, or LCE_F32 (master weight, rounded slab by slab in ws) */
  int32_t dx_dtype;     /* x_dtype or LCE_F32                                  */
  int32_t dw_dtype;     /* w_dtype or LCE_F32                                  */
  int64_t ignore_index; /* any int64 (ops.py:674)                              */
  float logit_scale;    /* > 0 (ops.py:908)                                    */
  float z_reg;          /* >= 0 (ops.py:909)                                   */
  int64_t n_chunk;      /* N_chunk_size: scratch bound n_chunk*V*4 bytes (ops.py:677) */
  int32_t monitoring;   /* 0/1: also produce max / entropy / norm (ops.py:678) */
  int32_t phases;       /* 0 = everything; otherwise a mask of LCE_PHASE_* (profiling aid) */
  int32_t pack_rows;    /* LCE_PACK_AUTO | LCE_PACK_ALWAYS | LCE_PACK_NEVER: see below        */
  int32_t max_workgroups; /* profiling aid: cap on the persistent workgroups of the tile kernels (0 = one per compute unit) */
  int32_t w_layout;     /* LCE_W_HV (0) | LCE_W_VH: how w and dw are stored, see below */
  int32_t route;        /* lce_forward_backward only: LCE_ROUTE_AUTO (0) | LCE_ROUTE_ONE_PASS | LCE_ROUTE_TWO_PASS, [+ LCE_ROUTE_EXACT_SUMS], see there */
} lce_problem;

/*
 * Layout of the weight and of its gradient.  The reference takes At of shape
 * (H, V) with whatever strides the tensor has (ops.py:733-734 pass
 * At.stride(0), At.stride(1) to the kernels, and At_grad = zeros_like(At) keeps
 * them, ops.py:693), so a tied embedding matrix stored (V, H) can be handed
 * over as its transposed view without a copy.  Here the two dense cases are:
 *   LCE_W_HV  w[h * ldw + v],  ldw  >= V   -- At stored row-major (H, V)
 *   LCE_W_VH  w[v * ldw + h],  ldw  >= H   -- At is the transposed view of a
 *             row-major (V, H) matrix (an nn.Embedding / nn.Linear(H, V) weight)
 * dw has the layout of w with row stride lddw.  LCE_W_VH needs 16-bit x, and
 * H a multiple of 8 (both operands of the logit contraction then run along
 * H in memory, and no 16-byte piece may straddle the end of a row).
 */
enum {
  LCE_W_HV = 0,
  LCE_W_VH = 1
};

/*
 * Arithmetic.  16-bit x: products of 16-bit operands (an fp32 master weight is
 * rounded to the type of x), fp32 accumulation (one exception, described at
 * lce_forward_backward: a 16-bit dW's sums over chunks of token rows at 24
 * bits where the scratch bound has no room for 32); dz is rounded once to the
 * type of x before the two gradient contractions, as the reference casts it
 * (ops.py:314, 422).  fp32 x (with an fp32 w): every operand of every
 * contraction, dz included, is carried as a PAIR of bf16 numbers hi + lo
 * (16 bits of mantissa) and each product as hi*hi + hi*lo + lo*hi with fp32
 * accumulation -- more accurate than the tf32 products the reference's tl.dot
 * uses for fp32 tensors (ops.py:195), at three times the matrix work of the
 * 16-bit path.  Observed against an fp64 evaluation: loss within 1e-6
 * relative, gradients within 1e-5 of their largest entry.
 */

/*
 * Tokens whose label equals ignore_index add nothing to the loss or to either
 * gradient (ops.py:213, 314, 422).  With packing the kept rows are gathered to
 * the front on the device and the tile kernels run on them only, so time
 * scales with the number of labelled tokens; the pre-pass costs a few small
 * launches (about 0.04 ms per forward + backward), which a small problem does
 * not earn back.  LCE_PACK_AUTO packs when 8*N*H*V >= 2^41 FLOPs; results are
 * the same either way up to the summation order of dW and the loss.  Use the same value in lce_workspace_bytes,
 * lce_forward and lce_backward of one problem.
 */
enum {
  LCE_PACK_AUTO = 0,
  LCE_PACK_ALWAYS = 1,
  LCE_PACK_NEVER = 2
};

/*
 * Profiling aid: a non-zero lce_problem.phases restricts a call to the named
 * kernels so that each can be bracketed by events.  Results of a restricted
 * call are only meaningful if the skipped phases ran before on the same
 * buffers and the same workspace (that of the same entry point).
 */
enum {
  LCE_PHASE_FWD_TILES = 1,  /* lce_forward: the MFMA tile kernel            */
  LCE_PHASE_FWD_REDUCE = 2, /* lce_forward: row merge + final reduction     */
  LCE_PHASE_BWD_DZ = 4,     /* lce_backward: recompute + dz staging         */
  LCE_PHASE_BWD_DX = 8,     /* lce_backward: dx contraction                 */
  LCE_PHASE_BWD_DW = 16,    /* lce_backward: dW contraction                 */
  LCE_PHASE_PACK = 32       /* either call: packing of the tokens whose label is not ignore_index */
};

/* Library version: major*10000 + minor*100 + patch. */
int lce_version(void);

/* Static description of a status code. */
const char* lce_strerror(int status);

/* Text of the last HIP error seen by this thread ("" if none). */
const char* lce_last_hip_error(void);

/*
 * Validates `p` exactly as lce_forward / lce_backward would (no device work).
 * Replaces the asserts of ops.py:685-691 and the ValueError of ops.py:43-44.
 */
int lce_check_problem(const lce_problem* p);

/*
 * Scratch sizes in bytes for lce_forward and lce_backward on problem `p`.
 * The forward works through the tokens in chunks of max(n_chunk, 16384) rows
 * (65536 under an fp32 weight): V/32 bytes of partial sums per token of one
 * chunk (four times that with monitoring), plus a 16-bit copy of at most
 * 256 MiB of an fp32 weight, plus 12 bytes per token, plus -- when tokens are
 * packed or x is fp32 -- a packed copy of x.
 * The backward size stays within n_chunk * V * 4 bytes -- the memory bound the
 * reference documents for N_chunk_size (ops.py:677, 700, 860) -- whenever the
 * narrowest split (256-column slabs plus an fp32 running dx) fits in it; for
 * the remaining shapes (a small vocabulary with many tokens) that narrowest
 * split is used and its size reported: the bound is a target, not a reason
 * to refuse a shape the reference runs.
 */
int lce_workspace_bytes(const lce_problem* p, size_t* fwd_bytes, size_t* bwd_bytes);

/*
 * How lce_backward will split problem `p`: it stages dz for all tokens of one
 * vocabulary slab at a time (`slab_width` columns, a multiple of 256; `slabs`
 * passes, the last one over whatever columns remain).  The counterpart of the reference's loop over N_chunk_size-row
 * groups (ops.py:721), which exists for the same purpose: bounding scratch.
 */
int lce_backward_plan(const lce_problem* p, int64_t* slabs, int64_t* slab_width);

/*
 * Forward.  Replaces the launch of linear_xent_fwd_prep_bwd_kernel_matmul_t
 * (ops.py:722-752) and the torch reductions around it (ops.py:705, 753-761,
 * 793-794, 802), without ever writing logits to memory.
 *
 *   lse     out, N floats: logsumexp of the scaled logits of every row whose
 *           label is not ignore_index; 0 for the other rows, whether rows are
 *           packed (such rows are then not computed at all) or not
 *   out5    out, 5 floats: loss, z_reg, logit_max, logit_entropy, logit_norm
 *           (the 5-tuple of ops.py:802 with the meanings of ops.py:9-17; the
 *           last three are 0 when monitoring == 0)
 *   n_valid out, 1 int64: number of labels != ignore_index (ops.py:705)
 */
int lce_forward(const lce_problem* p, const void* x, const void* w, const int64_t* y,
                float* lse, float* out5, int64_t* n_valid,
                void* ws, size_t ws_bytes, void* stream);

/*
 * Forward without a workspace argument, for callers that cannot allocate
 * device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  No counterpart in the reference (every buffer there
 * is a torch allocation, ops.py:693-703).  Same inputs, outputs and results
 * (bit for bit) as lce_forward; the scratch is a fixed array of
 * LCE_STATIC_SCRATCH_BYTES in device memory that every GPU the library runs on
 * holds until the process ends.  The call allocates and frees nothing.
 *
 *   - A problem whose lce_workspace_bytes forward size exceeds
 *     LCE_STATIC_SCRATCH_BYTES is refused with LCE_ESTATIC: use lce_forward.
 *     At V = 131072, H = 2048: N = 4096 rows need 32.1 MiB with monitoring
 *     == 0 and fit; with monitoring != 0 they need 64.02 MiB (four partial
 *     buffers of 16 MiB plus the per-token items) and do not, N = 2048 does;
 *     N = 16384 does not fit either way.
 *   - The array is part of the library's code object: every process holds
 *     LCE_STATIC_SCRATCH_BYTES of device memory on every GPU it runs the
 *     library on, whether or not this entry point is ever called, outside any
 *     allocator's statistics.
 *   - All calls on one GPU share that GPU's array: calls that overlap in time
 *     on one GPU (two streams, two threads) race.  Calls on one stream, or
 *     otherwise ordered, are fine; nothing is carried from one call to the next.
 *   - The first call on a device looks the array's address up
 *     (hipGetSymbolAddress, which may load the code object): make one call
 *     outside any graph capture before capturing.
 */
#define LCE_STATIC_SCRATCH_BYTES ((size_t)64 << 20)
int lce_forward_static(const lce_problem* p, const void* x, const void* w, const int64_t* y,
                       float* lse, float* out5, int64_t* n_valid, void* stream);

/*
 * Backward.  Replaces linear_xent_bwd_dispatcher and its dx / dA programs
 * (ops.py:239-337, 340-456, 544-658, launch at ops.py:763-791) and the
 * rescaling in LinearXentImplementation.backward (ops.py:804-810).
 *
 *   lse, n_valid   as produced by lce_forward on the same inputs
 *   grad_out       device pointer to 1 float: upstream gradient of the loss
 *   dx             out, (N, H) in dx_dtype, or NULL to skip
 *   dw             out, (H, V) in dw_dtype, or NULL to skip
 *
 * Gradients are accumulated in fp32 and scaled by grad_out*logit_scale/n_valid
 * after accumulation (ops.py:332, 443-447).  Rows whose label equals
 * ignore_index get dx == 0 exactly and contribute exact zeros to dw
 * (ops.py:314, 422).
 */
int lce_backward(const lce_problem* p, const void* x, const void* w, const int64_t* y,
                 const float* lse, const int64_t* n_valid, const float* grad_out,
                 void* dx, void* dw, void* ws, size_t ws_bytes, void* stream);

enum {
  LCE_ROUTE_AUTO = 0,
  LCE_ROUTE_ONE_PASS = 1,
  LCE_ROUTE_TWO_PASS = 2,
  /* a flag, to be or-ed to one of the above: a 16-bit dW's sums over chunks are never kept at fewer than 32 bits */
  LCE_ROUTE_EXACT_SUMS = 4
};

/*
 * Forward and backward in one call, from ONE evaluation of the logits.
 * Replaces LinearXentImplementation.forward as the reference runs it when a
 * gradient is wanted (ops.py:687-802): there the loop over N_chunk_size-row
 * groups computes the logits of a group once, keeps them in memory (ops.py:700)
 * and launches the dx / dA programs on them before the next group
 * (ops.py:721-791).  Same inputs and outputs as lce_forward followed by
 * lce_backward; the gradients differ from theirs by rounding only (the staged
 * dz is rounded to the 16-bit compute type twice instead of once, see below).
 *
 * The tokens go through in chunks of `chunk_rows` rows (lce_forward_backward_plan)
 * against the whole vocabulary.  Per chunk: the logit kernel writes the forward's
 * per-slice partials and, in the 16-bit compute type, e = exp(z - slice max)
 * for every logit (chunk_rows * V * 2 bytes); the row merge gives lse; one pass
 * over the stage turns e into dz; dx of the chunk is complete after one
 * contraction; dW is summed over the chunks in fp32 (the reference's fp32
 * At_grad, ops.py:692): an fp32 dW in the caller's buffer itself; a 16-bit dW
 * as two 16-bit halves per sum, the upper halves in the caller's dw -- which
 * holds no meaningful values until the call is done --, the lower halves in
 * H * V * 2 bytes of the workspace (nothing of this with a single chunk).
 * Where the bound has no room for those (H near 2 * n_chunk and above), or
 * where they leave so little room for the chunks that the library's model of
 * its kernels finds the alternative at least 3 % faster (typically H near
 * n_chunk and above), one byte of each lower half is kept instead (H * V
 * bytes): the sums are then rounded to nearest at 24 bits, 16 of mantissa,
 * each time they go back to memory -- with C chunks a relative error of at
 * most C * 2^-17 before the final rounding to the 16-bit dW (2^-9 in bf16,
 * 2^-12 in fp16).  LCE_ROUTE_EXACT_SUMS in lce_problem.route rules that out:
 * the sums are then fp32 between chunks or the problem takes two passes.
 * The chunks are as long as n_chunk * V * 4 bytes allow, or shorter where the
 * library's model of its kernels finds that faster.  8*N*H*V FLOPs become
 * 6*N*H*V.
 *
 * lce_problem.route: LCE_ROUTE_AUTO takes this route when a model of the tile
 * kernels' rounds of workgroups says it is the faster one (short chunks are
 * not: every chunk costs a round trip of dW's fp32 sums, so small problems
 * and tight bounds take two passes); LCE_ROUTE_ONE_PASS takes it whenever it
 * fits the bound; LCE_ROUTE_TWO_PASS never.
 *
 * Problems this route does not cover take the two calls above, one after the
 * other on the same workspace, inside this entry point: fp32 activations, a
 * weight that is neither of x's dtype nor fp32, and shapes whose sums of dW leave no
 * room for a chunk within the bound (a 16-bit dW with H near 4 * n_chunk or
 * above; lce_forward_backward_plan then reports 0 chunks).  `phases` selects kernels of either route; on the one-pass
 * route LCE_PHASE_FWD_TILES is the logit kernel and LCE_PHASE_BWD_DZ the pass
 * that turns e into dz.
 *
 *   grad_out   device pointer to 1 float: upstream gradient of the loss
 *              (the reference multiplies it in afterwards, ops.py:810).  A
 *              caller that learns it later passes a stand-in and rescales
 *              with lce_scale: 1 for bf16 / fp32 gradients; for fp16
 *              gradients a power of two near the number of valid labels,
 *              since entries of order 1/n_valid would leave fp16's normal
 *              range before a loss scale could be applied
 *   dx, dw     as for lce_backward; with both NULL this is lce_forward
 *   ws         lce_forward_backward_workspace_bytes(p) bytes
 */
int lce_forward_backward_workspace_bytes(const lce_problem* p, size_t* bytes);
int lce_forward_backward_plan(const lce_problem* p, int64_t* chunks, int64_t* chunk_rows);
int lce_forward_backward(const lce_problem* p, const void* x, const void* w, const int64_t* y,
                         const float* grad_out, float* lse, float* out5, int64_t* n_valid,
                         void* dx, void* dw, void* ws, size_t ws_bytes, void* stream);

/*
 * t[r][c] *= *factor for r < rows, c < cols, in place, the product formed in
 * fp32; `factor` is a device pointer to 1 float, and when it holds 1 the call
 * reads and writes nothing else.  Replaces the x_grad.mul_(grad_output) /
 * At_grad.mul_(grad_output) of LinearXentImplementation.backward (ops.py:810)
 * for gradients that lce_forward_backward produced with a grad_out of 1
 * (a caller that only learns the upstream gradient later, as autograd does).
 * Row stride `ld` in elements: a multiple of 8 (16-bit) or 4 (fp32), rows on
 * 16-byte boundaries.
 */
int lce_scale(void* t, int dtype, int64_t rows, int64_t cols, int64_t ld, const float* factor, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LCE_H_ */
