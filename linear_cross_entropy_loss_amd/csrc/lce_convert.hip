// An fp32 (master) weight is rounded to the 16-bit compute type one vocabulary
// slab at a time, into a workspace buffer that the tile kernels of that slab
// then read like a 16-bit weight.  The reference converts the whole weight to
// fp16 on entry (custom_fwd(cast_inputs=torch.float16), linear_cross_entropy/ops.py:665-667);
// here the copy is one slab wide, is made in the compute type that the
// activations have, and costs one read of the slab.  The rounding (nearest
// even) is the same one the kernels apply to fp32 activations.
#include "lce_gemm.h"
#include "lce_internal.h"

namespace lce {

namespace {

// One thread converts 8 consecutive columns of one row (two 16-byte loads, one 16-byte store).
// SPLIT (fp32 activations as well as weight): the copy has 3 H rows -- bf16(w), then bf16(w - bf16(w)),
// then bf16(w) again -- the [hi | lo | hi] operand of the three-term product described in lce_gemm.h.
template <class T, bool SPLIT>
__global__ __launch_bounds__(256) void convert_w_slab_kernel(const float* src, int64_t ld, int64_t H, int64_t v0,
                                                               int64_t vw, unsigned short* dst, int64_t dst_ld) {
  const int64_t runs_per_row = dst_ld / 8;
  const int64_t total = H * runs_per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t h = i / runs_per_row, c = (i - h * runs_per_row) * 8;
    const float* s = src + h * ld + v0 + c;
    float v[8];
    if (c + 8 <= vw) {
      const f32x4_t a = *reinterpret_cast<const f32x4_t*>(s), b = *reinterpret_cast<const f32x4_t*>(s + 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[j] = a[j];
        v[4 + j] = b[j];
      }
    } else {
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = c + j < vw ? s[j] : 0.f;
    }
    u32x4_t o;
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = pack2<T>(v[2 * j], v[2 * j + 1]);
    *reinterpret_cast<u32x4_t*>(dst + h * dst_ld + c) = o;
    if (SPLIT) {
      *reinterpret_cast<u32x4_t*>(dst + (2 * H + h) * dst_ld + c) = o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = pack2<T>(bf16_lo(v[2 * j]), bf16_lo(v[2 * j + 1]));
      *reinterpret_cast<u32x4_t*>(dst + (H + h) * dst_ld + c) = o;
    }
  }
}

// The same for a weight stored (V, H) row-major: rows [v0, v0 + vw) of it, H columns (a multiple of 8).
template <class T>
__global__ __launch_bounds__(256) void convert_w_rows_kernel(const float* src, int64_t ld, int64_t H, int64_t v0,
                                                               int64_t vw, unsigned short* dst, int64_t dst_ld) {
  const int64_t runs_per_row = H / 8;
  const int64_t total = vw * runs_per_row;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / runs_per_row, c = (i - r * runs_per_row) * 8;
    const float* s = src + (v0 + r) * ld + c;
    const f32x4_t a = *reinterpret_cast<const f32x4_t*>(s), b = *reinterpret_cast<const f32x4_t*>(s + 4);
    u32x4_t o;
    o[0] = pack2<T>(a[0], a[1]);
    o[1] = pack2<T>(a[2], a[3]);
    o[2] = pack2<T>(b[0], b[1]);
    o[3] = pack2<T>(b[2], b[3]);
    *reinterpret_cast<u32x4_t*>(dst + r * dst_ld + c) = o;
  }
}

}  // namespace

hipError_t launch_convert_w_rows(const float* src, int64_t ld, int64_t H, int64_t v0, int64_t vw, void* dst,
                                 int64_t dst_ld, int compute_dtype, hipStream_t s) {
  if (H % 8 != 0 || dst_ld % 8 != 0) return hipErrorInvalidValue;
  const int64_t total = vw * (H / 8);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  if (blocks < 1) return hipSuccess;
  unsigned short* d = reinterpret_cast<unsigned short*>(dst);
  if (compute_dtype == DT_F16) {
    hipLaunchKernelGGL((convert_w_rows_kernel<F16>), dim3((unsigned)blocks), dim3(256), 0, s, src, ld, H, v0, vw, d, dst_ld);
  } else {
    hipLaunchKernelGGL((convert_w_rows_kernel<BF16>), dim3((unsigned)blocks), dim3(256), 0, s, src, ld, H, v0, vw, d, dst_ld);
  }
  return hipGetLastError();
}

hipError_t launch_convert_w_slab(const float* src, int64_t ld, int64_t H, int64_t v0, int64_t vw, void* dst,
                                 int64_t dst_ld, int compute_dtype, bool split, hipStream_t s) {
  const int64_t total = H * (dst_ld / 8);
  int64_t blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  if (blocks < 1) return hipSuccess;
  unsigned short* d = reinterpret_cast<unsigned short*>(dst);
  if (split) {
    hipLaunchKernelGGL((convert_w_slab_kernel<BF16, true>), dim3((unsigned)blocks), dim3(256), 0, s, src, ld, H, v0, vw, d, dst_ld);
  } else if (compute_dtype == DT_F16) {
    hipLaunchKernelGGL((convert_w_slab_kernel<F16, false>), dim3((unsigned)blocks), dim3(256), 0, s, src, ld, H, v0, vw, d, dst_ld);
  } else {
    hipLaunchKernelGGL((convert_w_slab_kernel<BF16, false>), dim3((unsigned)blocks), dim3(256), 0, s, src, ld, H, v0, vw, d, dst_ld);
  }
  return hipGetLastError();
}

}  // namespace lce
