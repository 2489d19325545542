// Measurement probes (liblce_probe_gfx950.so; not part of the operator: built on demand by
// `python -m linear_cross_entropy_loss_amd.build --probes` and loaded only by `bench.py --probe`).
//
//   lce_probe_mfma    what the matrix pipes of this part sustain with no data movement at all: every wave
//                     keeps 4 A and 4 B fragments in registers and issues v_mfma_f32_32x32x16_bf16 over a
//                     4 x 4 grid of accumulator blocks (the 128 x 128 wave tile of the operator's kernels),
//                     on constant or on random operands.  The ceiling the tile kernels are measured against.
//                     Two further patterns add the LDS traffic of the tile kernels and nothing else (no global
//                     loads, no barriers, no epilogue): every k step's 8 fragments are re-read from LDS, and
//                     4 x 16 bytes per lane are written to it.
//   lce_probe_mfma_loads  the same loop with the tile kernels' operand fetch added as well: 4 x 16 bytes per lane
//                     and k step are fetched with buffer loads (64 KiB per workgroup and 64-deep K tile, the window
//                     shared by all workgroups so that it is served by the L2s) and are what the LDS writes store;
//                     optionally with the one workgroup barrier per K tile that the tile kernels need.
//   lce_probe_overlap how much of an epilogue's vector ALU work (fma, exp2, add per logit) hides behind matrix
//                     instructions of the same wave: the register-only loop with k such triples behind every
//                     MFMA, against the MFMAs alone and the triples alone.
//   lce_probe_flush   what adding 256 x 256 fp32 blocks of partial sums into a matrix in memory costs, with
//                     atomics or as plain read-modify-write: the traffic a backward that fed dz straight into
//                     the dx and dW contractions would generate once per dz tile (its H-wide accumulators do
//                     not fit a compute unit, so each dz tile's contribution would have to be flushed).
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) short s16x8_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;

__device__ __forceinline__ unsigned hash32(unsigned x) {
  x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
  return x;
}

// A bf16 with random sign and mantissa and an exponent in [2^-2, 2^1): every operand bit toggles from one
// fragment to the next, as with real activations and weights.
__device__ __forceinline__ short random_bf16(unsigned seed) {
  const unsigned h = hash32(seed);
  const unsigned exp = 125u + (h >> 8 & 3u);
  return (short)((h & 0x8000u) | (exp << 7) | (h & 0x7fu));
}

// pattern 0: all operands 1.0 (no bit toggles between consecutive instructions); 1: random operands, a different
// (A, B) fragment pair in each of the 16 MFMAs of a step -- what the operator's kernels issue between LDS reads.
__global__ __launch_bounds__(256) void mfma_loop_kernel(int pattern, int iters, float* out) {
  s16x8_t a[4], b[4];
  const unsigned tid = blockIdx.x * 256u + threadIdx.x;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      a[i][e] = pattern == 0 ? (short)0x3f80 : random_bf16(tid * 64u + i * 8u + e);
      b[i][e] = pattern == 0 ? (short)0x3f80 : random_bf16(tid * 64u + 32u + i * 8u + e);
    }
  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[i]),
                                                            __builtin_bit_cast(bf16x8_t, b[j]), acc[i][j], 0, 0, 0);
    asm volatile("" ::: "memory");
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  out[tid] = s;
}

// pattern 2: random operands, the 4 + 4 fragments of every k step read from LDS (8 ds_read_b128 per 16 MFMAs, the
// rate of the operator's tile kernels), one k step ahead; pattern 3: additionally 4 ds_write_b128 per 16 MFMAs (the
// rate at which those kernels refill their LDS stages).  Reads and writes are interleaved with the MFMAs one by one.
// LOADS (lce_probe_mfma_loads): the 4 pieces written per k step come from memory, loaded three k steps earlier
// (the tile kernels give a load one K tile = four k steps) with buffer loads, one after every fourth MFMA: `src`
// holds `src_bytes` (a power of two) bytes, and all workgroups walk the same window of it, 16 KiB per k step.
// BARRIER: a workgroup barrier after every fourth k step (one per 64-deep K tile).
// `grouped`: instead of one window for all, every four workgroups of an XCD (workgroup b runs on XCD b % 8) walk a
// window of their own, `src_bytes` long, 64 windows in all: three of four requests hit in L2, as for the tile kernels'
// operand bands, and the rest comes over the fabric.
template <bool WRITES, bool LOADS, bool BARRIER>
__global__ __launch_bounds__(256) void mfma_lds_loop_kernel(int iters, float* out, const char* src, unsigned src_bytes,
                                                            int grouped) {
  if (LOADS && grouped) src += (size_t)((blockIdx.x & 7) * 8 + ((blockIdx.x >> 3) / 4 & 7)) * src_bytes;
  __shared__ __attribute__((aligned(16))) short lds[65536];  // 128 KiB, the two stages of a tile kernel
  const unsigned tid = blockIdx.x * 256u + threadIdx.x;
  for (int i = threadIdx.x; i < 65536; i += 256) lds[i] = random_bf16(blockIdx.x * 65536u + i);
  __syncthreads();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  s16x8_t fa[8], fb[8];
  const s16x8_t* rd = reinterpret_cast<const s16x8_t*>(lds);  // 8192 pieces of 16 bytes
  s16x8_t* wr = reinterpret_cast<s16x8_t*>(lds);
#pragma unroll
  for (int f = 0; f < 8; ++f) fa[f] = rd[(wave * 2048 + f * 64 + lane) & 8191];
  u32x4_t g[4][4];  // LOADS: four sets of pieces in flight
  // (raw 32-bit data format, as in the tile kernels; the scalar offset selects the piece, the vector offset the lane)
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(src), 0, LOADS ? (int)src_bytes : 0, 0x00020000);
  const unsigned voff = threadIdx.x * 16u;
  auto load = [&](int it, int f) -> u32x4_t {
    const unsigned o = ((unsigned)(it * 16384 + f * 4096)) & (src_bytes - 1);
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff, (int)o, 0);
  };
  if (LOADS) {
#pragma unroll
    for (int u = 1; u < 4; ++u)
#pragma unroll
      for (int f = 0; f < 4; ++f) g[u][f] = load(u, f);
  }
  auto step = [&](s16x8_t (&cur)[8], s16x8_t (&nxt)[8], u32x4_t (&fill)[4], u32x4_t (&drain)[4], int it) {
    const int o = (it + 1) * 512 + wave * 2048;
#pragma unroll
    for (int f = 0; f < 8; ++f) nxt[f] = rd[(o + f * 64 + lane) & 8191];
    if (WRITES) {
#pragma unroll
      for (int f = 0; f < 4; ++f)
        wr[(o + 4096 + f * 64 + lane) & 8191] = LOADS ? __builtin_bit_cast(s16x8_t, drain[f]) : cur[f];
    }
    if (LOADS) {
#pragma unroll
      for (int f = 0; f < 4; ++f) fill[f] = load(it + 4, f);
    }
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      const int i = s >> 2, j = (i & 1) ? 3 - (s & 3) : (s & 3);
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, cur[i]),
                                                          __builtin_bit_cast(bf16x8_t, cur[4 + j]), acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                       // one MFMA
      if (s < 8) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                            // one LDS read
      if (WRITES && s >= 8 && (s & 1) == 0) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // one LDS write
      if (LOADS && (s & 3) == 1) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);            // one buffer load
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  // (the fragment sets and the sets of loaded pieces change roles: no register moves; a set written to LDS in one k
  // step is refilled in the same step, after the writes)
  for (int it = 0; it < iters; it += 4) {
    step(fa, fb, g[0], g[1], it);
    step(fb, fa, g[1], g[2], it + 1);
    step(fa, fb, g[2], g[3], it + 2);
    step(fb, fa, g[3], g[0], it + 3);
    if (BARRIER) __syncthreads();
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) s += acc[i][j][r];
  out[tid] = s;
}

// Each workgroup adds `tiles` blocks of 256 x 256 floats into dst[rows][ld]: it walks down the row tiles of
// column tile b / 4, then of the next one, so that (as in a tile order that shares operand bands between
// neighbouring workgroups) four workgroups add into the same block at about the same time -- the pattern
// of four token tiles of one vocabulary tile flushing their contributions to dW.
template <bool ATOMIC>
__global__ __launch_bounds__(256) void flush_kernel(float* dst, int64_t rows, int64_t ld, int tiles) {
  const int col_tiles = (int)(ld / 256), row_tiles = (int)(rows / 256);
  const int lane_col = (threadIdx.x & 63) * 4, row0 = threadIdx.x >> 6;
  for (int k = 0; k < tiles; ++k) {
    const int ct = ((int)blockIdx.x / 4 + k / row_tiles) % col_tiles, rt = k % row_tiles;
    float* base = dst + (int64_t)rt * 256 * ld + (int64_t)ct * 256;
    for (int r = row0; r < 256; r += 4) {
      float* p = base + (int64_t)r * ld + lane_col;
      if (ATOMIC) {
#pragma unroll
        for (int e = 0; e < 4; ++e) atomicAdd(p + e, 1.0f);
      } else {
        f32x4_t v = *reinterpret_cast<f32x4_t*>(p);
        v += 1.0f;
        *reinterpret_cast<f32x4_t*>(p) = v;
      }
    }
  }
}

// mode 0: 16 MFMAs per iteration (random operands in registers); 1: KV (fma, exp2, add) triples per iteration and no
// MFMA; 2: both, KV / 16 triples behind each MFMA.  One wave per SIMD, as in the tile kernels.
template <int MODE, int KV>
__global__ __launch_bounds__(256) void overlap_kernel(int iters, float* out) {
  s16x8_t a[4], b[4];
  const unsigned tid = blockIdx.x * 256u + threadIdx.x;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      a[i][e] = random_bf16(tid * 64u + i * 8u + e);
      b[i][e] = random_bf16(tid * 64u + 32u + i * 8u + e);
    }
  f32x16_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  float v[16], s[16];
#pragma unroll
  for (int q = 0; q < 16; ++q) {
    v[q] = -1.f - 0.001f * (tid & 63) - q;
    s[q] = 0.f;
  }
  const float c = 0.999f + 1e-6f * (tid & 3);
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        if (MODE != 1)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[i]),
                                                              __builtin_bit_cast(bf16x8_t, b[j]), acc[i][j], 0, 0, 0);
        if (MODE != 0) {
#pragma unroll
          for (int u = 0; u < KV / 16; ++u) {
            const int q = (i * 4 + j + u * 5) & 15;
            s[q] += __builtin_amdgcn_exp2f(fmaf(v[q], c, -0.5f));
            v[q] = v[q] * 0.99999f;  // (keeps the inputs changing)
          }
        }
        if (MODE == 2) {
          __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
          __builtin_amdgcn_sched_group_barrier(0x402, 4 * (KV / 16), 0);
        }
      }
    asm volatile("" ::: "memory");
  }
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) t += acc[i][j][r];
#pragma unroll
  for (int q = 0; q < 16; ++q) t += s[q] + v[q];
  out[tid] = t;
}

}  // namespace

extern "C" {

// Launches `wgs` workgroups of 4 waves, each wave issuing iters * 16 MFMAs (32 x 32 x 16, bf16); iters a multiple of 4.
// pattern 0 constant / 1 random operands in registers; 2 random operands re-read from LDS; 3 plus LDS writes.
// out: wgs * 256 floats.  FLOPs = wgs * 4 * iters * 16 * 32768.
int lce_probe_mfma(int pattern, int wgs, int iters, float* out, void* stream) {
  if (pattern < 0 || pattern > 3 || wgs <= 0 || iters <= 0 || (iters & 3) || !out) return -3;
  const dim3 grid((unsigned)wgs), block(256);
  hipStream_t s = (hipStream_t)stream;
  if (pattern == 2) hipLaunchKernelGGL((mfma_lds_loop_kernel<false, false, false>), grid, block, 0, s, iters, out, nullptr, 1u, 0);
  else if (pattern == 3) hipLaunchKernelGGL((mfma_lds_loop_kernel<true, false, false>), grid, block, 0, s, iters, out, nullptr, 1u, 0);
  else hipLaunchKernelGGL(mfma_loop_kernel, grid, block, 0, s, pattern, iters, out);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

// Pattern 3 of lce_probe_mfma with the pieces written to LDS loaded from `src` (device memory): 16 KiB per workgroup
// and k step out of a window of `window_bytes` (a power of two from 64 KiB to 1 GiB).  windows == 1: every workgroup
// walks the same window; windows == 64: every four workgroups of an XCD walk their own (src holds 64 * window_bytes).
// barrier != 0: with a workgroup barrier after every fourth k step.
int lce_probe_mfma_loads(int wgs, int iters, const void* src, uint64_t window_bytes, int windows, int barrier, float* out,
                         void* stream) {
  if (wgs <= 0 || iters <= 0 || (iters & 3) || !out || !src || (windows != 1 && windows != 64)) return -3;
  if (window_bytes < 65536 || (window_bytes & (window_bytes - 1)) || window_bytes > (1ull << 30)) return -3;
  const dim3 grid((unsigned)wgs), block(256);
  hipStream_t s = (hipStream_t)stream;
  const char* p = reinterpret_cast<const char*>(src);
  const unsigned wb = (unsigned)window_bytes;
  const int grouped = windows == 64;
  if (barrier) hipLaunchKernelGGL((mfma_lds_loop_kernel<true, true, true>), grid, block, 0, s, iters, out, p, wb, grouped);
  else hipLaunchKernelGGL((mfma_lds_loop_kernel<true, true, false>), grid, block, 0, s, iters, out, p, wb, grouped);
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

// Launches `wgs` workgroups, each adding `tiles` blocks of 256 x 256 floats into dst[rows][ld] (rows and ld
// multiples of 256).  atomic != 0: one fp32 atomic add per element; else 16-byte loads and stores.
// Payload = wgs * tiles * 256 KiB.
int lce_probe_flush(int atomic, float* dst, int64_t rows, int64_t ld, int tiles, int wgs, void* stream) {
  if (!dst || rows < 256 || ld < 256 || rows % 256 || ld % 256 || tiles <= 0 || wgs <= 0) return -3;
  if (atomic) {
    hipLaunchKernelGGL(flush_kernel<true>, dim3((unsigned)wgs), dim3(256), 0, (hipStream_t)stream, dst, rows, ld, tiles);
  } else {
    hipLaunchKernelGGL(flush_kernel<false>, dim3((unsigned)wgs), dim3(256), 0, (hipStream_t)stream, dst, rows, ld, tiles);
  }
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

// Launches `wgs` workgroups of 4 waves running `iters` iterations of: mode 0, 16 MFMAs; mode 1, 16 * per_mfma
// (fma, exp2, add) triples; mode 2, both, per_mfma triples behind each MFMA.  per_mfma: 1, 2 or 4.  out: wgs * 256 floats.
int lce_probe_overlap(int mode, int per_mfma, int wgs, int iters, float* out, void* stream) {
  if (mode < 0 || mode > 2 || wgs <= 0 || iters <= 0 || !out) return -3;
  const dim3 grid((unsigned)wgs), block(256);
  hipStream_t s = (hipStream_t)stream;
#define LCE_OVL(M, K) hipLaunchKernelGGL((overlap_kernel<M, K>), grid, block, 0, s, iters, out)
  if (mode == 0) LCE_OVL(0, 16);
  else if (per_mfma == 1) { if (mode == 1) LCE_OVL(1, 16); else LCE_OVL(2, 16); }
  else if (per_mfma == 2) { if (mode == 1) LCE_OVL(1, 32); else LCE_OVL(2, 32); }
  else if (per_mfma == 4) { if (mode == 1) LCE_OVL(1, 64); else LCE_OVL(2, 64); }
  else return -3;
#undef LCE_OVL
  return hipGetLastError() == hipSuccess ? 0 : -5;
}

}  // extern "C"
