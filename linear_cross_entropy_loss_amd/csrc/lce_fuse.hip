// The pass between the logit kernel and the two gradient contractions when the logits are computed once
// (lce_forward_backward; the reference computes its gradients in the forward pass too,
// linear_cross_entropy/ops.py:721-799, from the logits chunk it keeps in memory).
//
// The logit kernel (launch_fwd_stage, lce_bwd_dz.hip) left e = 2^shift * exp(z - m) in the stage, m = the
// largest logit of the token within a slice of 128 columns, because a token's lse is only known once all its
// slices are done.  Here, with lse at hand,
//     dz[token][v] = e[token][v] * exp(m[token][v / 128] - lse[token]) * (1 + 2 * z_reg * lse[token])
//                  = 2^shift * softmax * gain                                       (ops.py:309-314, 415-422)
// in place, exact zeros for tokens with an ignored label and rows past the last one, and the target column
// gets the rounding of the fp32 value 2^shift * (softmax * gain - 1), formed from the target logit the logit
// kernel wrote, as in the kernel that recomputes the logits (lce_bwd_dz.hip).  The pass is bound by memory
// traffic: 2 bytes read and 2 written per logit.
#include "lce_gemm.h"
#include "lce_internal.h"

namespace lce {

namespace {

constexpr float kLog2e = 1.4426950408889634f;

template <class T> LCE_DEV float from_bits(unsigned short b);
template <> LCE_DEV float from_bits<BF16>(unsigned short b) { return __builtin_bit_cast(float, (unsigned)b << 16); }
template <> LCE_DEV float from_bits<F16>(unsigned short b) { return (float)__builtin_bit_cast(_Float16, b); }

// One workgroup per block of the stage (256 token rows x 64 columns, 32 KiB, BwdArgs::dz): blockIdx.x = column
// group, blockIdx.y = token tile.  Thread t first works out the factor of row t, then the block is
// rewritten in 16-byte pieces, consecutive lanes on consecutive pieces.
template <class T>
__global__ __launch_bounds__(256) void stage_scale_kernel(const BwdArgs a) {
  __shared__ float sh_f[kTile];
  __shared__ int sh_col[kTile];             // target column inside the block, or -1
  __shared__ unsigned short sh_tv[kTile];   // what goes there
  const int64_t rows = packed_rows(a.n_rows, a.N);
  const int64_t t0 = (int64_t)blockIdx.y * kTile;
  if (t0 >= rows) return;  // (token tiles without a row were not written and are not read)
  const int g = blockIdx.x;
  {
    const int64_t tok = t0 + threadIdx.x;
    const bool exists = tok < rows;
    const int64_t yy = exists ? a.y[tok] : a.ignore_index;
    const bool valid = yy != a.ignore_index;
    float f = 0.f;
    int col = -1;
    unsigned short tv = 0;
    if (valid) {
      const float lse = a.lse[tok];
      const float m = a.part_max[(a.v0 + (int64_t)g * 64) / kChunkV * a.nc + tok];
      float gain = 1.f + 2.f * a.z_reg * lse;
      if (a.dz_shift != 0) gain = fminf(fmaxf(gain, -63.f), 63.f);  // (as in lce_bwd_dz.hip)
      f = __builtin_amdgcn_exp2f((m - lse) * kLog2e) * gain;
      const int64_t rel = yy - (a.v0 + (int64_t)g * 64);
      if (rel >= 0 && rel < 64) {
        col = (int)rel;
        const float p = __builtin_amdgcn_exp2f(fmaf(a.tgt[tok] - lse, kLog2e, (float)a.dz_shift)) * gain;
        tv = to_bits<T>(p - __builtin_bit_cast(float, (127 + a.dz_shift) << 23));
      }
    }
    sh_f[threadIdx.x] = f;
    sh_col[threadIdx.x] = col;
    sh_tv[threadIdx.x] = tv;
  }
  __syncthreads();
  typedef typename elem_of<T>::type E;
  u32x4_t* blk = reinterpret_cast<u32x4_t*>(reinterpret_cast<E*>(a.dz) + dz_block_offset(blockIdx.y, g, a.vs));
  u32x4_t v[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) v[i] = blk[i * 256 + threadIdx.x];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int piece = i * 256 + threadIdx.x, r = piece >> 3, c0 = (piece & 7) * 8;
    const float f = sh_f[r];
    const int hit = sh_col[r] - c0;  // 0..7: the target is element `hit` of this piece
    u32x4_t o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float lo = from_bits<T>((unsigned short)(v[i][j] & 0xffffu)) * f;
      const float hi = from_bits<T>((unsigned short)(v[i][j] >> 16)) * f;
      unsigned w = pack2<T>(lo, hi);
      if (hit == 2 * j) w = (w & 0xffff0000u) | sh_tv[r];
      if (hit == 2 * j + 1) w = (w & 0x0000ffffu) | ((unsigned)sh_tv[r] << 16);
      o[j] = w;
    }
    blk[piece] = o;
  }
}

__global__ void chunk_rows_kernel(const int64_t* n_rows, int64_t N, int64_t nc, int chunks, int64_t* out) {
  const int c = threadIdx.x;
  if (c >= chunks) return;
  const int64_t left = packed_rows(n_rows, N) - (int64_t)c * nc;
  out[c] = left < 0 ? 0 : (left > nc ? nc : left);
  const int64_t all = N - (int64_t)c * nc;  // the chunk's rows when the dropped tokens follow the kept ones
  out[1024 + c] = all < 0 ? 0 : (all > nc ? nc : all);
}

// t[r][c] *= g[0] for r < rows, c < cols (row stride ld, rows on 16-byte boundaries), the product formed in fp32;
// nothing is read or written when g[0] is 1.  Pieces of 16 bytes, the last piece of a row element by element.
// v * f rounded to fp32 before anything else happens to it (the compiler may otherwise fold the product into
// a conversion that rounds the exact product once: another result on ties, and not the same in every code path).
LCE_DEV float scaled(float v, float f) {
  float p = v * f;
  asm volatile("" : "+v"(p));
  return p;
}

template <class E, int PER>
__global__ __launch_bounds__(256) void scale_rows_kernel(E* t, int64_t rows, int64_t cols, int64_t ld, const float* g) {
  const float f = g[0];
  if (f == 1.f) return;
  const int64_t pieces = (cols + PER - 1) / PER;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < rows * pieces; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / pieces, c0 = (i - r * pieces) * PER;
    E* at = t + r * ld + c0;
    if (c0 + PER <= cols) {
      u32x4_t v = *reinterpret_cast<const u32x4_t*>(at);
      E e[PER];
      __builtin_memcpy(e, &v, 16);
#pragma unroll
      for (int j = 0; j < PER; ++j) e[j] = (E)scaled((float)e[j], f);
      __builtin_memcpy(&v, e, 16);
      *reinterpret_cast<u32x4_t*>(at) = v;
    } else {
      for (int64_t c = c0; c < cols; ++c) t[r * ld + c] = (E)scaled((float)t[r * ld + c], f);
    }
  }
}

}  // namespace

hipError_t launch_scale_rows(void* t, int dtype, int64_t rows, int64_t cols, int64_t ld, const float* g, int num_cus,
                             hipStream_t s) {
  if (rows <= 0 || cols <= 0) return hipSuccess;
  const int per = dtype == DT_F32 ? 4 : 8;
  const int64_t work = rows * ((cols + per - 1) / per);
  int64_t grid = (work + 255) / 256;
  if (grid > (int64_t)num_cus * 16) grid = (int64_t)num_cus * 16;
  if (dtype == DT_BF16)
    hipLaunchKernelGGL((scale_rows_kernel<__bf16, 8>), dim3((unsigned)grid), dim3(256), 0, s, (__bf16*)t, rows, cols, ld, g);
  else if (dtype == DT_F16)
    hipLaunchKernelGGL((scale_rows_kernel<_Float16, 8>), dim3((unsigned)grid), dim3(256), 0, s, (_Float16*)t, rows, cols, ld, g);
  else if (dtype == DT_F32)
    hipLaunchKernelGGL((scale_rows_kernel<float, 4>), dim3((unsigned)grid), dim3(256), 0, s, (float*)t, rows, cols, ld, g);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_stage_scale(const BwdArgs& a, hipStream_t s) {
  if (a.split || a.part_max == nullptr || a.tgt == nullptr || a.lse == nullptr) return hipErrorInvalidValue;
  const dim3 grid((unsigned)(a.vs / 64), (unsigned)(a.Np / kTile));
  if (a.x_dtype == DT_BF16) hipLaunchKernelGGL(stage_scale_kernel<BF16>, grid, dim3(256), 0, s, a);
  else if (a.x_dtype == DT_F16) hipLaunchKernelGGL(stage_scale_kernel<F16>, grid, dim3(256), 0, s, a);
  else return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_chunk_rows(const int64_t* n_rows, int64_t N, int64_t nc, int chunks, int64_t* out, hipStream_t s) {
  if (chunks < 1 || chunks > 1024) return hipErrorInvalidValue;
  hipLaunchKernelGGL(chunk_rows_kernel, dim3(1), dim3(1024), 0, s, n_rows, N, nc, chunks, out);
  return hipGetLastError();
}

}  // namespace lce
