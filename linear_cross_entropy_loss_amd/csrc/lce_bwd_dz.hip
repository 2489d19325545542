// Backward, step 1: recompute a 256(v) x 256(token) logit tile with the same
// MFMA main loop as the forward (so the logits are bit-identical to the ones
// the saved lse was built from) and turn it, in registers, into
//     dz = softmax * (1 + 2*z_reg*lse) - onehot(y),   0 for ignored tokens
// (linear_cross_entropy/ops.py:309-314 and 415-422), rounded once to the
// 16-bit compute type exactly where the reference casts dz before its dot
// products (ops.py:314, 422).  The tile is transposed through LDS and written
// to the row-major staging buffer dz[N][vs] of the current vocabulary slab
// with 16-byte stores.
#include "lce_gemm2.h"
#include "lce_internal.h"

namespace lce {

namespace {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kDzRowBytes = kTile * 2 + 16;          // padded LDS row of the dz tile
constexpr int kDzLds = kTile * kDzRowBytes;          // 135168 bytes
static_assert(kDzLds >= kMainloopLds, "dz tile reuses the main-loop LDS");

template <class T, class XSrc, class WSrc>
__global__ __launch_bounds__(kThreads) void bwd_dz_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  const int tiles_p = (int)(a.vs / kTile), tiles_q = (int)(a.N / kTile);
  int tp, tq;
  tile_coords(blockIdx.x, gridDim.x, tiles_p, tiles_q, 4, tp, tq);
  const int64_t v0 = a.v0 + (int64_t)tp * kTile, t0 = (int64_t)tq * kTile;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  const int64_t slice_v0 = v0 + wp * kWaveTile;

  int ycol[kNB];
  float nlse[kNB], gain[kNB];
  bool valid[kNB];
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    const int64_t tok = t0 + wq * kWaveTile + qb * kBlk + (lane & 31);
    const int64_t yy = a.y[tok];
    const int64_t rel = yy - slice_v0;
    valid[qb] = yy != a.ignore_index;
    ycol[qb] = (valid[qb] && rel >= 0 && rel < kWaveTile) ? (int)rel : -1;
    const float l = a.lse[tok];
    nlse[qb] = -l * kLog2e;
    gain[qb] = 1.f + 2.f * a.z_reg * l;
  }

  f32x16_t acc[kNB][kNB];
  gemm_tile<T, WSrc, false, XSrc, true>(
      acc, reinterpret_cast<const WSrc*>(a.w) + v0, a.ldw,
      reinterpret_cast<const XSrc*>(a.x) + t0 * a.ldx, a.ldx, (int)(a.H / kBK), lds);

  const float c1 = a.scale * kLog2e;
#pragma unroll
  for (int qb = 0; qb < kNB; ++qb) {
    const int row = wq * kWaveTile + qb * kBlk + (lane & 31);
#pragma unroll
    for (int pb = 0; pb < kNB; ++pb)
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        const int col = pb * kBlk + 8 * rq + 4 * (lane >> 5);  // inside the wave's slice
        float d[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float p = __builtin_amdgcn_exp2f(fmaf(acc[pb][qb][rq * 4 + j], c1, nlse[qb])) * gain[qb];
          if (col + j == ycol[qb]) p -= 1.f;
          d[j] = valid[qb] ? p : 0.f;
        }
        u32x2_t v;
        v[0] = pack2<T>(d[0], d[1]);
        v[1] = pack2<T>(d[2], d[3]);
        *reinterpret_cast<u32x2_t*>(lds + row * kDzRowBytes + (wp * kWaveTile + col) * 2) = v;
      }
  }
  __syncthreads();
  typedef typename elem_of<T>::type E;
  E* out = reinterpret_cast<E*>(a.dz) + t0 * a.vs + (int64_t)tp * kTile;
#pragma unroll 4
  for (int i = 0; i < kTile * 32 / kThreads; ++i) {
    const int idx = i * kThreads + threadIdx.x;
    const int row = idx >> 5, u = idx & 31;
    const u32x4_t v = *reinterpret_cast<const u32x4_t*>(lds + row * kDzRowBytes + u * 16);
    *reinterpret_cast<u32x4_t*>(out + (int64_t)row * a.vs + u * 8) = v;
  }
}

template <class T, class XSrc, class WSrc> hipError_t launch(const BwdArgs& a, hipStream_t s) {
  auto kern = bwd_dz_kernel<T, XSrc, WSrc>;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, kDzLds);
  if (e != hipSuccess) return e;
  const int grid = (int)((a.vs / kTile) * (a.N / kTile));
  hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), kDzLds, s, a);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_bwd_dz(const BwdArgs& a, hipStream_t s) {
  typedef elem_of<BF16>::type bf;
  typedef elem_of<F16>::type hf;
  if (a.x_dtype == DT_BF16 && a.w_dtype == DT_BF16) return launch<BF16, bf, bf>(a, s);
  if (a.x_dtype == DT_BF16 && a.w_dtype == DT_F32) return launch<BF16, bf, float>(a, s);
  if (a.x_dtype == DT_F16 && a.w_dtype == DT_F16) return launch<F16, hf, hf>(a, s);
  if (a.x_dtype == DT_F16 && a.w_dtype == DT_F32) return launch<F16, hf, float>(a, s);
  if (a.x_dtype == DT_F32 && a.w_dtype == DT_F32) return launch<BF16, float, float>(a, s);
  return hipErrorInvalidValue;
}

}  // namespace lce
