// Backward, step 3: dW[h][v] = coef * sum_token x[token][h] * dz[token][v] for
// the columns of one vocabulary slab (the contraction of
// linear_cross_entropy/ops.py:424).  K = token, so both operands are read
// through the LDS transpose path.  Each workgroup owns its dW tile over ALL
// tokens: the fp32 accumulator never leaves registers, no cross-workgroup
// reduction exists, and the result is written once in the output dtype after
// scaling by grad_out * logit_scale / n_valid (ops.py:443-447, 810).
#include "lce_gemm3.h"
#include "lce_internal.h"

namespace lce {

namespace {

template <class T>
LCE_DEV void dw_epilogue(const BwdArgs& a, f32x16_t (&acc)[kNB][kNB], int tp, int tq) {
  typedef typename elem_of<T>::type E;
  const int64_t vl0 = (int64_t)tp * kTile, h0 = (int64_t)tq * kTile;
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  const float coef = a.grad_out[0] * a.scale / (float)a.n_valid[0];
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
      if (a.dw_dtype == DT_F32) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          if (vb + 8 * rq + 4 * half >= a.V || !row_exists) continue;
          f32x4_t o;
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = acc[pb][qb][rq * 4 + j] * coef;
          *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(a.dw) + h * a.lddw + vb + 8 * rq + 4 * half) = o;
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

// Split mode: the raw fp32 partial sum of K segment `seg` goes to dw_part[seg][Hp][vs].
LCE_DEV void dw_partial_epilogue(const BwdArgs& a, f32x16_t (&acc)[kNB][kNB], int tp, int tq, int seg) {
  const int64_t vl0 = (int64_t)tp * kTile, h0 = (int64_t)tq * kTile;
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  float* part = a.dw_part + (int64_t)seg * a.Hp * a.vs;
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    const int64_t h = h0 + wq * kWaveTile + qb * kBlk + (lane & 31);
#pragma unroll
    for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int64_t vl = vl0 + wp * kWaveTile + pb * kBlk + 8 * rq + 4 * (lane >> 5);
        f32x4_t v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = acc[pb][qb][rq * 4 + j];
        *reinterpret_cast<f32x4_t*>(part + h * a.vs + vl) = v;
      }
  }
}

// Work item = (output tile, K segment), segment fastest (see the dx kernel).
template <class T, bool SPLIT> struct DwProblem {
  static constexpr bool kVarK = false;
  static constexpr bool kKMask = false;  // both operands have K as their slow index: nothing to mask
  typedef typename elem_of<T>::type E;
  const BwdArgs& a;
  int64_t rows, ldx;  // token rows (the K extent): all of x, or the packed rows (see BwdArgs)
  const E* x;
  int tiles_p, tiles_q, split, kseg;
  LCE_DEV DwProblem(const BwdArgs& a_)
      : a(a_), tiles_p((int)(a_.vs / kTile)), tiles_q((int)(a_.Hp / kTile)), split(SPLIT ? a_.dw_split : 1),
        kseg(a_.dw_kseg) {
    rows = packed_rows(a.n_rows, a.N);
    const bool packed = rows != a.N;
    x = reinterpret_cast<const E*>(packed ? a.xc : a.x);
    ldx = packed ? a.ldxc : a.ldx;
  }
  // K tiles of an unsplit contraction: an even number, at least four, covering the rows
  LCE_DEV int ktiles() const {
    const int64_t kt = (rows + 2 * kBK - 1) / (2 * kBK) * 2;
    return (int)(kt < 4 ? 4 : kt);
  }
  LCE_DEV int num_tiles() const { return tiles_p * tiles_q * split; }
  LCE_DEV void decode(int item, int& tp, int& tq, int& seg) const {
    seg = SPLIT ? item % split : 0;
    tile_coords(SPLIT ? item / split : item, tiles_p * tiles_q, tiles_p, tiles_q, 4, tp, tq);
  }
  LCE_DEV void origins(int item, const void*& p, const void*& q) const {
    int tp, tq, seg;
    decode(item, tp, tq, seg);
    const int64_t k0 = (int64_t)seg * kseg * kBK;  // first token of the segment
    p = reinterpret_cast<const E*>(a.dz) + k0 * a.vs + (int64_t)tp * kTile;
    q = x + k0 * ldx + (int64_t)tq * kTile;
  }
  // rows past the end of either operand (a last segment running past the tokens) read as zeros
  // dz is written for whole token tiles; x rows past the last one read as zeros
  LCE_DEV const void* p_end() const {
    return reinterpret_cast<const E*>(a.dz) + (rows + kTile - 1) / kTile * kTile * a.vs;
  }
  LCE_DEV const void* q_end() const { return matrix_end<E>(x, rows, ldx, a.H); }
  LCE_DEV int k_valid(int) const { return (int)a.Np; }
  LCE_DEV void epilogue(int item, f32x16_t (&acc)[kNB][kNB], char*) const {
    int tp, tq, seg;
    decode(item, tp, tq, seg);
    if (SPLIT) {
      dw_partial_epilogue(a, acc, tp, tq, seg);
    } else {
      dw_epilogue<T>(a, acc, tp, tq);
    }
  }
};

template <class T, bool SPLIT>
__global__ __launch_bounds__(kThreads) void bwd_dw_persistent_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  typedef typename elem_of<T>::type E;
  DwProblem<T, SPLIT> prob(a);
  Pipe3<T, E, false, E, false, DwProblem<T, SPLIT>> pipe(prob);
  pipe.run(a.vs, prob.ldx, SPLIT ? a.dw_kseg : prob.ktiles(), lds);
}

// Split mode, second step: dW[:, slab] = coef * sum over segments, in segment order.
template <class T>
__global__ __launch_bounds__(256) void dw_reduce_kernel(const BwdArgs a) {
  typedef typename elem_of<T>::type E;
  const int64_t quads_per_row = a.vs / 4;
  const int64_t total = a.H * quads_per_row;
  const float coef = a.grad_out[0] * a.scale / (float)a.n_valid[0];
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t h = i / quads_per_row, vl = (i - h * quads_per_row) * 4;
    const int64_t v = a.v0 + vl;
    if (v >= a.V) continue;  // a quad that V cuts through is written whole, into the stride padding of its row
    const int64_t o = h * a.vs + vl;
    f32x4_t acc = *reinterpret_cast<const f32x4_t*>(a.dw_part + o);
    for (int s = 1; s < a.dw_split; ++s) acc += *reinterpret_cast<const f32x4_t*>(a.dw_part + (int64_t)s * a.Hp * a.vs + o);
    if (a.dw_dtype == DT_F32) {
      *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(a.dw) + h * a.lddw + v) = acc * coef;
    } else {
      u32x2_t b;
      b[0] = pack2<T>(acc[0] * coef, acc[1] * coef);
      b[1] = pack2<T>(acc[2] * coef, acc[3] * coef);
      *reinterpret_cast<u32x2_t*>(reinterpret_cast<E*>(a.dw) + h * a.lddw + v) = b;
    }
  }
}

template <class T, bool SPLIT> hipError_t launch_tiles(const BwdArgs& a, hipStream_t s) {
  auto kern = bwd_dw_persistent_kernel<T, SPLIT>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kMainloopLds);
  if (e != hipSuccess) return e;
  const int64_t items = (a.vs / kTile) * (a.Hp / kTile) * (SPLIT ? a.dw_split : 1);
  const int grid = (int)(items < a.num_cus ? items : a.num_cus);
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), kMainloopLds, s, a);
  return hipGetLastError();
}

template <class T> hipError_t launch_persistent(const BwdArgs& a, hipStream_t s) {
  if (a.dw_split <= 1) return launch_tiles<T, false>(a, s);
  hipError_t e = launch_tiles<T, true>(a, s);
  if (e != hipSuccess) return e;
  const int64_t quads = a.H * (a.vs / 4);
  int64_t blocks = (quads + 255) / 256;
  if (blocks > 2048) blocks = 2048;
  hipLaunchKernelGGL(dw_reduce_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, s, a);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_bwd_dw(const BwdArgs& a, hipStream_t s) {
  if (a.x_dtype == DT_BF16) return launch_persistent<BF16>(a, s);
  if (a.x_dtype == DT_F16) return launch_persistent<F16>(a, s);
  return hipErrorInvalidValue;
}

}  // namespace lce
