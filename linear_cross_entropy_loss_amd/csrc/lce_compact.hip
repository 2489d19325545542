// Tokens whose label equals ignore_index contribute nothing to the loss or to
// either gradient (linear_cross_entropy/ops.py:213, 314, 422), so the tile
// kernels never look at them: the kept tokens are packed to the front, in
// their original order, and the kernels run on the packed rows only.  The
// number of kept tokens stays on the device (the kernels read it), so nothing
// here synchronises with the host.  (The reference computes the ignored rows
// and multiplies them away.)
//
//   compact_labels  perm[j] = original index of the j-th kept token, yc[j] its label, n_rows = how many; the dropped
//                   tokens follow in perm from n_rows on, in their order (yc = ignore_index), for a caller that
//                   wants all rows with the kept ones first
//   gather_rows     xc[j] = x[perm[j]], lse_c[j] = lse[perm[j]]  (fp32 activations: as bf16 pairs, see gather_rows_split_kernel)
//   scatter_rows    rows of dropped tokens of dx = 0 (and dx[perm[j]] = dxc[j] where dx was staged packed)
//
// When no token is dropped (n_rows == N) the row copies are skipped and the
// tile kernels read x and write dx in place.
#include "lce_gemm.h"
#include "lce_internal.h"

namespace lce {

namespace {

constexpr int kSegTokens = 2048;  // tokens per workgroup of the counting / packing kernels
constexpr int kPerThread = kSegTokens / 256;

// Sum of `v` over the 256 threads of the workgroup; exclusive prefix of this thread in `excl`.
LCE_DEV int block_scan(int v, int& excl, int* sh /* [4] */) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = v;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int up = __shfl_up(incl, d);
    if (lane >= d) incl += up;
  }
  if (lane == 63) sh[wave] = incl;
  __syncthreads();
  int before = 0, total = 0;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    if (w < wave) before += sh[w];
    total += sh[w];
  }
  __syncthreads();  // sh may be reused by the caller
  excl = before + incl - v;
  return total;
}

__global__ __launch_bounds__(256) void count_kept_kernel(const int64_t* y, int64_t N, int64_t ignore_index, int* cnt) {
  __shared__ int sh[4];
  const int64_t base = (int64_t)blockIdx.x * kSegTokens + (int64_t)threadIdx.x * kPerThread;
  int c = 0;
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) c += (base + k < N && y[base + k] != ignore_index) ? 1 : 0;
  int excl;
  const int total = block_scan(c, excl, sh);
  if (threadIdx.x == 0) cnt[blockIdx.x] = total;
}

// One workgroup: cnt[] becomes its own exclusive prefix sum, n_rows the total.
__global__ __launch_bounds__(256) void scan_counts_kernel(int* cnt, int64_t nseg, int64_t* n_rows) {
  __shared__ int sh[4];
  int64_t running = 0;
  for (int64_t base = 0; base < nseg; base += 256) {
    const int64_t i = base + threadIdx.x;
    const int v = i < nseg ? cnt[i] : 0;
    int excl;
    const int total = block_scan(v, excl, sh);
    if (i < nseg) cnt[i] = (int)(running + excl);
    running += total;
  }
  if (threadIdx.x == 0) n_rows[0] = running;
}

__global__ __launch_bounds__(256) void pack_kept_kernel(const int64_t* y, int64_t N, int64_t ignore_index,
                                                        const int* offs, const int64_t* n_rows, int* perm, int64_t* yc) {
  __shared__ int sh[4];
  const int64_t base = (int64_t)blockIdx.x * kSegTokens + (int64_t)threadIdx.x * kPerThread;
  int64_t lab[kPerThread];
  int c = 0;
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    lab[k] = base + k < N ? y[base + k] : ignore_index;
    c += lab[k] != ignore_index ? 1 : 0;
  }
  int excl;
  block_scan(c, excl, sh);
  int64_t j = (int64_t)offs[blockIdx.x] + excl;
  const int64_t kept = n_rows[0];
#pragma unroll
  for (int k = 0; k < kPerThread; ++k) {
    if (base + k >= N) break;
    // j kept tokens come before token base + k: a dropped one is number base + k - j among the dropped
    const int64_t at = lab[k] != ignore_index ? j++ : kept + (base + k - j);
    perm[at] = (int)(base + k);
    yc[at] = lab[k];
  }
}

// One workgroup per packed row (grid-stride).  Rows are moved in 16-byte pieces; `chunks` pieces per row.
// The last row of x may end with its last element (a caller's matrix need not own the stride padding of its
// last row): of that row only the whole pieces are moved as such, the rest 16 bits at a time, zero-filled.
__global__ __launch_bounds__(256) void gather_rows_kernel(const char* x, int64_t ldx_bytes, const int* perm,
                                                          const int64_t* n_rows, int64_t N, char* xc,
                                                          int64_t ldxc_bytes, int chunks, int64_t row_bytes,
                                                          const float* lse, float* lse_c, int always) {
  const int64_t rows = packed_rows(n_rows, N);
  const bool copy_x = rows != N || always != 0;
  for (int64_t j = blockIdx.x; j < rows; j += gridDim.x) {
    const int64_t src = packed_token(perm, j, N);
    if (lse != nullptr && threadIdx.x == 0) lse_c[j] = lse[src];
    if (copy_x) {
      const u32x4_t* s = reinterpret_cast<const u32x4_t*>(x + src * ldx_bytes);
      u32x4_t* d = reinterpret_cast<u32x4_t*>(xc + j * ldxc_bytes);
      const int whole = src == N - 1 ? (int)(row_bytes / 16) : chunks;
      for (int c = threadIdx.x; c < whole; c += 256) d[c] = s[c];
      if (whole < chunks && threadIdx.x < 8) {  // the piece that the end of the last row cuts through
        const int64_t b = (int64_t)whole * 16 + threadIdx.x * 2;
        const unsigned short v = b < row_bytes ? *reinterpret_cast<const unsigned short*>(x + src * ldx_bytes + b) : 0;
        *reinterpret_cast<unsigned short*>(xc + j * ldxc_bytes + b) = v;
      }
    }
  }
}

// fp32 activations reach the tile kernels as bf16 pairs, x = hi + lo (lce_gemm.h), in two copies that are made
// even when no token is dropped (`perm` / `n_rows` may be null: all rows, in their order):
//   xc  [rows][3 H]       row j = [hi | hi | lo] of x[perm[j]]: the K axis of the logit contraction, three
//                         times as long, against a weight copy laid out [hi ; lo ; hi]
//   xk  [3][Np][H]        hi, hi, lo again, stacked along the TOKEN axis, which is the K axis of
//                         dW = x^T dz (against dz staged as [hi ; lo ; hi]); rows from `rows` to Np of each
//                         block are zeros, since K runs through them.  Null in the forward.
// One workgroup per packed row (grid-stride); elements go out as single 16-bit stores, consecutive lanes to
// consecutive addresses (H need not be a multiple of anything, so the three parts of a row of xc do not
// start on 16-byte boundaries).
__global__ __launch_bounds__(256) void gather_rows_split_kernel(const float* x, int64_t ldx, int64_t H, const int* perm,
                                                                const int64_t* n_rows, int64_t N, int64_t Np,
                                                                unsigned short* xc, int64_t ldxc, unsigned short* xk,
                                                                int64_t ldxk, const float* lse, float* lse_c) {
  const int64_t rows = n_rows != nullptr ? packed_rows(n_rows, N) : N;
  const int64_t jend = xk != nullptr ? Np : rows;
  for (int64_t j = blockIdx.x; j < jend; j += gridDim.x) {
    if (j >= rows) {  // K padding of the dW contraction
      for (int64_t k = threadIdx.x; k < ldxk; k += 256)
        xk[j * ldxk + k] = xk[(Np + j) * ldxk + k] = xk[(2 * Np + j) * ldxk + k] = 0;
      continue;
    }
    const int64_t src = perm != nullptr ? packed_token(perm, j, N) : j;
    if (lse != nullptr && threadIdx.x == 0) lse_c[j] = lse[src];
    const float* s = x + src * ldx;
    unsigned short* c = xc + j * ldxc;
    for (int64_t k = threadIdx.x; k < H; k += 256) {
      const float v = s[k];
      const unsigned short hi = to_bits<BF16>(v), lo = to_bits<BF16>(bf16_lo(v));
      c[k] = hi;
      c[H + k] = hi;
      c[2 * H + k] = lo;
      if (xk != nullptr) {
        xk[j * ldxk + k] = hi;
        xk[(Np + j) * ldxk + k] = hi;
        xk[(2 * Np + j) * ldxk + k] = lo;
      }
    }
    // stride padding is read by the tile kernels and must be finite
    for (int64_t k = 3 * H + threadIdx.x; k < ldxc; k += 256) c[k] = 0;
    if (xk != nullptr)
      for (int64_t k = H + threadIdx.x; k < ldxk; k += 256)
        xk[j * ldxk + k] = xk[(Np + j) * ldxk + k] = xk[(2 * Np + j) * ldxk + k] = 0;
  }
}

// One workgroup per token (grid-stride): token i moves packed row i to its place (if there is a packed
// row i) and clears its own row of dx if it was dropped.  8-byte pieces, `chunks` per row.
__global__ __launch_bounds__(256) void scatter_rows_kernel(const char* dxc, int64_t lddxc_bytes, const int* perm,
                                                           const int64_t* n_rows, int64_t N, const int64_t* y,
                                                           int64_t ignore_index, char* dx, int64_t lddx_bytes,
                                                           int chunks) {
  const int64_t rows = packed_rows(n_rows, N);
  if (rows == N) return;  // nothing was dropped: the tile kernel wrote dx itself
  for (int64_t i = blockIdx.x; i < N; i += gridDim.x) {
    if (dxc != nullptr && i < rows) {
      const u32x2_t* s = reinterpret_cast<const u32x2_t*>(dxc + i * lddxc_bytes);
      u32x2_t* d = reinterpret_cast<u32x2_t*>(dx + packed_token(perm, i, N) * lddx_bytes);
      for (int c = threadIdx.x; c < chunks; c += 256) d[c] = s[c];
    }
    if (y[i] == ignore_index) {
      u32x2_t* d = reinterpret_cast<u32x2_t*>(dx + i * lddx_bytes);
      u32x2_t z;
      z[0] = 0u;
      z[1] = 0u;
      for (int c = threadIdx.x; c < chunks; c += 256) d[c] = z;
    }
  }
}

unsigned row_grid(int64_t N, int num_cus) {
  int64_t g = (int64_t)num_cus * 8;
  if (g > N) g = N;
  return (unsigned)(g < 1 ? 1 : g);
}

}  // namespace

int64_t compact_segments(int64_t N) { return (N + kSegTokens - 1) / kSegTokens; }

hipError_t launch_compact_labels(const int64_t* y, int64_t N, int64_t ignore_index, int* cnt, int64_t* n_rows,
                                 int* perm, int64_t* yc, hipStream_t s) {
  const int64_t nseg = compact_segments(N);
  hipLaunchKernelGGL(count_kept_kernel, dim3((unsigned)nseg), dim3(256), 0, s, y, N, ignore_index, cnt);
  hipLaunchKernelGGL(scan_counts_kernel, dim3(1), dim3(256), 0, s, cnt, nseg, n_rows);
  hipLaunchKernelGGL(pack_kept_kernel, dim3((unsigned)nseg), dim3(256), 0, s, y, N, ignore_index, cnt, n_rows, perm, yc);
  return hipGetLastError();
}

hipError_t launch_gather_rows_split(const float* x, int64_t ldx, int64_t H, const int* perm, const int64_t* n_rows,
                                    int64_t N, void* xc, int64_t ldxc, void* xk, int64_t ldxk, const float* lse,
                                    float* lse_c, int num_cus, hipStream_t s) {
  const int64_t Np = padded_tokens(N);
  hipLaunchKernelGGL(gather_rows_split_kernel, dim3(row_grid(Np, num_cus)), dim3(256), 0, s, x, ldx, H, perm, n_rows, N,
                     Np, reinterpret_cast<unsigned short*>(xc), ldxc, reinterpret_cast<unsigned short*>(xk), ldxk, lse,
                     lse_c);
  return hipGetLastError();
}

hipError_t launch_gather_rows(const void* x, int64_t ldx_bytes, int64_t row_bytes, const int* perm,
                              const int64_t* n_rows, int64_t N, void* xc, int64_t ldxc_bytes, const float* lse,
                              float* lse_c, int num_cus, hipStream_t s, bool always) {
  hipLaunchKernelGGL(gather_rows_kernel, dim3(row_grid(N, num_cus)), dim3(256), 0, s,
                     reinterpret_cast<const char*>(x), ldx_bytes, perm, n_rows, N, reinterpret_cast<char*>(xc),
                     ldxc_bytes, (int)(ldxc_bytes / 16), row_bytes, lse, lse_c, always ? 1 : 0);
  return hipGetLastError();
}

hipError_t launch_scatter_rows(const void* dxc, int64_t lddxc_bytes, const int* perm, const int64_t* n_rows,
                               int64_t N, const int64_t* y, int64_t ignore_index, void* dx, int64_t lddx_bytes,
                               int64_t row_bytes, int num_cus, hipStream_t s) {
  hipLaunchKernelGGL(scatter_rows_kernel, dim3(row_grid(N, num_cus)), dim3(256), 0, s,
                     reinterpret_cast<const char*>(dxc), lddxc_bytes, perm, n_rows, N, y, ignore_index,
                     reinterpret_cast<char*>(dx), lddx_bytes, (int)((row_bytes + 7) / 8));
  return hipGetLastError();
}

}  // namespace lce
