// Backward, step 2: dx[token][h] (+)= sum_v dz[token][v] * W[h][v] over one
// vocabulary slab (the contraction of linear_cross_entropy/ops.py:317).  Both
// operands are K-contiguous (K = v).  The running sum over slabs is kept in
// fp32; the factor grad_out * logit_scale / n_valid is applied once, after the
// last slab, as the reference does after its accumulation (ops.py:332, 810).
#include "lce_gemm3.h"
#include "lce_internal.h"

namespace lce {

namespace {

// The running sum lives in a padded [Np][Hp] fp32 buffer and needs no bounds.
// The final result goes out through range-checked buffer stores: the descriptor
// ends at the last element of dx, so rows past N are dropped by the hardware,
// and quads of hidden indices that start at or past H are given an
// out-of-range offset (a quad that H cuts through is written whole: the row
// stride is a multiple of 4, so it stays inside its row).  No branches: a branch
// around accumulator reads makes the compiler read all of them up front.
// `out` / `ldo` / `rows`: dx itself, or the packed copy when tokens were dropped (see BwdArgs).
template <class T>
LCE_DEV void dx_epilogue(const BwdArgs& a, int64_t rows, void* out, int64_t ldo, f32x16_t (&acc)[kNB][kNB], int tp,
                         int tq) {
  typedef typename elem_of<T>::type E;
  const int64_t h0 = (int64_t)tp * kTile, t0 = (int64_t)tq * kTile;
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  const float coef = a.grad_out[0] * a.scale / (float)a.n_valid[0];
  const int es = a.dx_dtype == DT_F32 ? 4 : 2;
  // descriptor over the rows of this tile: base = first row, range = bytes to the end of dx
  const char* tile_base = reinterpret_cast<const char*>(out) + t0 * ldo * es;
  // whole dwords: with 16-bit data and an odd H the last row ends one element into its stride padding
  const int64_t hcols = es == 2 ? (a.H + 1) & ~(int64_t)1 : a.H;
  const int64_t left = (reinterpret_cast<const char*>(out) + ((rows - 1) * ldo + hcols) * es) - tile_base;
  const unsigned range = left <= 0 ? 0u : (left > 0x7fffffff ? 0x7fffffffu : (unsigned)left);
  const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(tile_base), 0, (int)range, 0x00020000);
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    const int row = wq * kWaveTile + qb * kBlk + (lane & 31);  // row inside the tile
    const int64_t tok = t0 + row;
    const unsigned row_off = (unsigned)(row * ldo * es);
#pragma unroll
    for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int64_t hrun = h0 + wp * kWaveTile + pb * kBlk + 8 * rq;
        const int64_t h = hrun + 4 * (lane >> 5);
        f32x4_t v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = acc[pb][qb][rq * 4 + j];
        if (!a.first) v += *reinterpret_cast<const f32x4_t*>(a.dx_acc + tok * a.Hp + h);
        if (!a.last) {
          *reinterpret_cast<f32x4_t*>(a.dx_acc + tok * a.Hp + h) = v;
        } else {
          const unsigned off = h < a.H ? row_off + (unsigned)(h * es) : 0x80000000u;
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

// Split mode: the raw fp32 partial sum of K segment `seg` goes to dx_part[seg][Np][Hp].
LCE_DEV void dx_partial_epilogue(const BwdArgs& a, f32x16_t (&acc)[kNB][kNB], int tp, int tq, int seg) {
  const int64_t h0 = (int64_t)tp * kTile, t0 = (int64_t)tq * kTile;
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  float* part = a.dx_part + (int64_t)seg * a.Np * a.Hp;
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    const int64_t tok = t0 + wq * kWaveTile + qb * kBlk + (lane & 31);
#pragma unroll
    for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int64_t h = h0 + wp * kWaveTile + pb * kBlk + 8 * rq + 4 * (lane >> 5);
        f32x4_t v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = acc[pb][qb][rq * 4 + j];
        *reinterpret_cast<f32x4_t*>(part + tok * a.Hp + h) = v;
      }
  }
}

// Work item = (output tile, K segment); segment fastest, so that with a
// power-of-two split the workgroups of one XCD work on the same segment and
// share its W rows and dz columns in their L2.
template <class T, class WSrc, bool SPLIT, bool KMASK> struct DxProblem {
  static constexpr bool kKMask = KMASK;
  typedef typename elem_of<T>::type E;
  const BwdArgs& a;
  int64_t rows;  // token rows: all, or the packed ones (see BwdArgs)
  int tiles_p, tiles_q, split, kseg;
  LCE_DEV DxProblem(const BwdArgs& a_)
      : a(a_), rows(packed_rows(a_.n_rows, a_.N)), tiles_p((int)(a_.Hp / kTile)), split(SPLIT ? a_.dx_split : 1), kseg(a_.dx_kseg) {
    tiles_q = (int)((rows + kTile - 1) / kTile);
  }
  LCE_DEV int num_tiles() const { return tiles_p * tiles_q * split; }
  LCE_DEV void decode(int item, int& tp, int& tq, int& seg) const {
    seg = SPLIT ? item % split : 0;
    tile_coords(SPLIT ? item / split : item, tiles_p * tiles_q, tiles_p, tiles_q, 8, tp, tq);
  }
  LCE_DEV void origins(int item, const void*& p, const void*& q) const {
    int tp, tq, seg;
    decode(item, tp, tq, seg);
    const int64_t k0 = (int64_t)seg * kseg * kBK;
    p = reinterpret_cast<const WSrc*>(a.w) + (int64_t)tp * kTile * a.ldw + (a.v0 - a.wv0) + k0;
    q = reinterpret_cast<const E*>(a.dz) + (int64_t)tq * kTile * a.vs + k0;
  }
  LCE_DEV const void* p_end() const { return matrix_end<WSrc>(a.w, a.H, a.ldw, a.Vw); }
  LCE_DEV const void* q_end() const { return reinterpret_cast<const E*>(a.dz) + (int64_t)tiles_q * kTile * a.vs; }
  LCE_DEV int k_valid(int item) const {
    const int seg = SPLIT ? item % split : 0;
    const int64_t left = a.vw - (int64_t)seg * kseg * kBK;
    return (int)(left < 0 ? 0 : left);
  }
  LCE_DEV void epilogue(int item, f32x16_t (&acc)[kNB][kNB], char*) const {
    int tp, tq, seg;
    decode(item, tp, tq, seg);
    if (SPLIT) {
      dx_partial_epilogue(a, acc, tp, tq, seg);
    } else {
      const bool packed = rows != a.N;
      dx_epilogue<T>(a, rows, packed ? a.dxc : a.dx, packed ? a.lddxc : a.lddx, acc, tp, tq);
    }
  }
};

template <class T, class WSrc, bool SPLIT, bool KMASK>
__global__ __launch_bounds__(kThreads) void bwd_dx_persistent_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  typedef typename elem_of<T>::type E;
  DxProblem<T, WSrc, SPLIT, KMASK> prob(a);
  Pipe3<T, WSrc, true, E, true, DxProblem<T, WSrc, SPLIT, KMASK>> pipe(prob);
  pipe.run(a.ldw, a.vs, SPLIT ? a.dx_kseg : (int)(a.vs / kBK), lds);
}

// Split mode, second step: dx (+)= sum over segments, in segment order; same
// running-sum / final-store rules as the tile kernel's own epilogue.
template <class T>
__global__ __launch_bounds__(256) void dx_reduce_kernel(const BwdArgs a) {
  typedef typename elem_of<T>::type E;
  const int64_t quads_per_row = a.Hp / 4;
  const int64_t rows = packed_rows(a.n_rows, a.N);
  const int64_t total = rows * quads_per_row;
  const bool packed = rows != a.N;
  void* out = packed ? a.dxc : a.dx;
  const int64_t ldo = packed ? a.lddxc : a.lddx;
  const float coef = a.grad_out[0] * a.scale / (float)a.n_valid[0];
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t tok = i / quads_per_row, h = (i - tok * quads_per_row) * 4;
    if (h >= a.H) continue;
    const int64_t o = tok * a.Hp + h;
    f32x4_t v = *reinterpret_cast<const f32x4_t*>(a.dx_part + o);
    for (int s = 1; s < a.dx_split; ++s) v += *reinterpret_cast<const f32x4_t*>(a.dx_part + (int64_t)s * a.Np * a.Hp + o);
    if (!a.first) v += *reinterpret_cast<const f32x4_t*>(a.dx_acc + o);
    if (!a.last) {
      *reinterpret_cast<f32x4_t*>(a.dx_acc + o) = v;
    } else if (a.dx_dtype == DT_F32) {
      *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(out) + tok * ldo + h) = v * coef;
    } else {
      u32x2_t b;
      b[0] = pack2<T>(v[0] * coef, v[1] * coef);
      b[1] = pack2<T>(v[2] * coef, v[3] * coef);
      *reinterpret_cast<u32x2_t*>(reinterpret_cast<E*>(out) + tok * ldo + h) = b;
    }
  }
}

template <class T, class WSrc, bool SPLIT, bool KMASK> hipError_t launch_tiles(const BwdArgs& a, hipStream_t s) {
  auto kern = bwd_dx_persistent_kernel<T, WSrc, SPLIT, KMASK>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kMainloopLds);
  if (e != hipSuccess) return e;
  const int64_t items = (a.Hp / kTile) * (a.Np / kTile) * (SPLIT ? a.dx_split : 1);
  const int grid = (int)(items < a.num_cus ? items : a.num_cus);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), kMainloopLds, s, a);
  return hipGetLastError();
}

template <class T, class WSrc> hipError_t launch_persistent(const BwdArgs& a, hipStream_t s) {
  // the K mask is only needed when the K tiles of a work item run past the columns that exist
  if (a.dx_split <= 1) return a.vw == a.vs ? launch_tiles<T, WSrc, false, false>(a, s) : launch_tiles<T, WSrc, false, true>(a, s);
  const bool exact_k = a.vw == a.vs && (int64_t)a.dx_split * a.dx_kseg * kBK == a.vs;
  hipError_t e = exact_k ? launch_tiles<T, WSrc, true, false>(a, s) : launch_tiles<T, WSrc, true, true>(a, s);
  if (e != hipSuccess) return e;
  const int64_t quads = a.N * (a.Hp / 4);
  int64_t blocks = (quads + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  hipLaunchKernelGGL(dx_reduce_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, s, a);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_bwd_dx(const BwdArgs& a, hipStream_t s) {
  typedef elem_of<BF16>::type bf;
  typedef elem_of<F16>::type hf;
  const bool bf_compute = a.x_dtype == DT_BF16 || a.x_dtype == DT_F32;
  // an fp32 weight arrives here as a 16-bit slab copy
  if (bf_compute && a.w_dtype == DT_BF16) return launch_persistent<BF16, bf>(a, s);
  if (a.x_dtype == DT_F16 && a.w_dtype == DT_F16) return launch_persistent<F16, hf>(a, s);
  return hipErrorInvalidValue;
}

}  // namespace lce
