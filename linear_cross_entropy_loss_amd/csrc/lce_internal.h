// Internal launch interface between the C ABI (lce_api.hip) and the kernel
// translation units.  Not installed; the public surface is include/lce.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace lce {

enum { DT_BF16 = 0, DT_F16 = 1, DT_F32 = 2 };

// Columns of logits covered by one forward partial (one wave's slice of a tile).
constexpr int kChunkV = 128;
// Rows handled by one workgroup of the row-merge kernel.
constexpr int kMergeRows = 64;

struct FwdArgs {
  const void* x;
  const void* w;
  const int64_t* y;
  int64_t N, H, V, ldx, ldw;
  int x_dtype, w_dtype;  // compute type = x_dtype (bf16 / f16)
  int64_t ignore_index;
  float scale, z_reg;
  int monitoring;
  int num_cus;  // compute units of the device: grid size of the persistent kernels
  // outputs / scratch
  float* lse;        // [N]
  float* out5;       // [5]
  int64_t* n_valid;  // [1]
  float* part_lse;   // [V/128][N]  per-slice logsumexp
  float* part_max;   // [V/128][N]  per-slice max            (monitoring)
  float* part_pz;    // [V/128][N]  per-slice sum softmax*z  (monitoring)
  float* part_sq;    // [V/128][N]  per-slice sum z^2        (monitoring)
  float* tgt;        // [N]         target logit, pre-zeroed
  float* blk;        // [N/64][8]   per-merge-block partial sums
};

struct BwdArgs {
  const void* x;
  const void* w;
  const int64_t* y;
  const float* lse;
  const int64_t* n_valid;
  const float* grad_out;
  int64_t N, H, V, ldx, ldw, lddx, lddw;
  int x_dtype, w_dtype, dx_dtype, dw_dtype;
  int64_t ignore_index;
  float scale, z_reg;
  void* dx;
  void* dw;
  // slab being processed
  int64_t v0, vs;   // first column and width of the vocabulary slab
  void* dz;         // [N][vs] staged dz in the compute type
  float* dx_acc;    // [N][H] fp32 running dx (null when there is a single slab)
  int first, last;  // slab position
  int num_cus;      // compute units of the device: grid size of the persistent kernels
};

hipError_t launch_fwd_tiles(const FwdArgs& a, hipStream_t s);
hipError_t launch_fwd_reduce(const FwdArgs& a, hipStream_t s);
hipError_t launch_fill_f32(float* p, int64_t n, float v, hipStream_t s);
hipError_t launch_bwd_dz(const BwdArgs& a, hipStream_t s);
hipError_t launch_bwd_dx(const BwdArgs& a, hipStream_t s);
hipError_t launch_bwd_dw(const BwdArgs& a, hipStream_t s);

}  // namespace lce
