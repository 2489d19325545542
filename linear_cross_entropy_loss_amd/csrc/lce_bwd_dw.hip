// Backward, step 3: dW[h][v] = coef * sum_token x[token][h] * dz[token][v] for
// the columns of one vocabulary slab (the contraction of
// linear_cross_entropy/ops.py:424).  K = token, so both operands are read
// through the LDS transpose path.  A workgroup owns its dW tile over ALL tokens
// (the rows that are left after tokens with an ignored label were packed away):
// the fp32 accumulator never leaves registers and the result is written once
// in the output dtype after scaling by grad_out * logit_scale / n_valid
// (ops.py:443-447, 810).  Only the tiles of a mostly idle last round of
// workgroups are cut along K instead and summed by a second kernel (DwPlan).
//
// x is the P operand of the tile loop and dz the Q operand, for either layout of dW: bands of tiles that
// span all of H then walk along the vocabulary, so that dz streams through once while the small x is re-read
// (measured 5-7 % faster than the other way round).  What changes with the layout is which operand goes
// to which side of the matrix instruction, i.e. which index runs along the accumulator registers:
//   dW stored (H, V) row-major: dz feeds the A side, v runs along registers, a lane stores runs of 8 v for its h;
//   dW stored (V, H) row-major (WVH): x feeds the A side, h runs along registers, a lane stores runs of 8 h for its v.
#include <type_traits>

#include "lce_gemm3.h"
#include "lce_internal.h"

namespace lce {

namespace {

// First row / column of tile (tp = h tile, tq = v tile of the slab) in the stored matrix, and the matrix' limits.
template <bool WVH> struct DwTileGeom {
  int64_t row0, col0, row_limit, col_limit;
  LCE_DEV DwTileGeom(const BwdArgs& a, int tp, int tq) {
    if (WVH) {
      row0 = a.v0 + (int64_t)tq * kTile; row_limit = a.V;
      col0 = (int64_t)tp * kTile;        col_limit = a.H;
    } else {
      row0 = (int64_t)tp * kTile;        row_limit = a.H;
      col0 = a.v0 + (int64_t)tq * kTile; col_limit = a.V;
    }
  }
};

// dW stored (H, V) row-major: its rows are V elements apart (256 KiB for 16-bit data at V = 131072), and the
// 32-byte pieces that the lanes of a wave hold for 32 different rows make poor use of the memory channels
// (measured: the tile kernel 5-7 % slower than with the 4 KiB rows of the (V, H) layout).  So a wave stages its
// own 128 (h) x 128 (v) sub-tile through a private 16 KiB slice of `scratch` (main-loop stage 1, idle during an
// epilogue) in passes of 128 bytes per row -- two of 64 columns for 16-bit dW, four of 32 columns for fp32 dW --
// and reads each pass back as whole 128-byte rows: dW leaves the compute unit as full lines.  Staging rows have
// their 16-byte piece index XOR-ed by (row & 7) ^ ((row >> 3) & 1), as in the dz staging of lce_bwd_dz.hip; no
// other wave is involved until the barrier at the end.
constexpr int kDwSliceBytes = kWaveTile * 128;
static_assert(4 * kDwSliceBytes <= kMainloopLds - kStageBytes, "four wave slices must fit beside one stage");

template <class T, bool F32OUT>
LCE_DEV void dw_store_rows_hv(const BwdArgs& a, f32x16_t (&acc)[kNB][kNB], int tp, int tq, char* scratch) {
  typedef typename elem_of<T>::type E;
  typedef typename std::conditional<F32OUT, float, E>::type O;
  constexpr int kPasses = F32OUT ? 4 : 2, kPassCols = kWaveTile / kPasses, kPieceCols = 16 / (int)sizeof(O);
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;  // rows h come from the P half, columns v from the Q half
  const int half = lane >> 5;
  const float coef = final_factor_of(a);
  char* mine = scratch + wave * kDwSliceBytes;
  const int64_t h0 = (int64_t)tp * kTile + wp * kWaveTile;             // first row of this wave's sub-tile
  const int64_t v0 = a.v0 + (int64_t)tq * kTile + wq * kWaveTile;      // its first column
  O* out = reinterpret_cast<O*>(a.dw) + h0 * a.lddw + v0;
#pragma unroll
  for (int ph = 0; ph < kPasses; ++ph) {
#pragma unroll
    for (int rb = 0; rb < kNB; ++rb) {
      const int row = rb * kBlk + (lane & 31);
      char* lrow = mine + row * 128;
      const int sw = (row & 7) ^ ((row >> 3) & 1);
      if (F32OUT) {
        // one 32-column block per pass; a register quad is a 16-byte piece as it stands
        const f32x16_t& blk = acc[rb][ph];
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          f32x4_t o;
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = blk[rq * 4 + j] * coef;
          *reinterpret_cast<f32x4_t*>(lrow + (((2 * rq + half) ^ sw) << 4)) = o;
        }
      } else {
#pragma unroll
        for (int pp = 0; pp < 2; ++pp) {
          const f32x16_t& blk = acc[rb][2 * ph + pp];
#pragma unroll
          for (int gq = 0; gq < 4; gq += 2) {
            // lanes l and l+32 hold the two halves of every run of 8 columns: one lane-half swap per pair of
            // register quads gives each lane a whole run (16 bytes)
            float d[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) d[i] = blk[gq * 4 + i] * coef;
            const unsigned x0 = pack2<T>(d[0], d[1]), x1 = pack2<T>(d[2], d[3]);
            const unsigned y0 = pack2<T>(d[4], d[5]), y1 = pack2<T>(d[6], d[7]);
            const auto s0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
            const auto s1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
            u32x4_t o;
            o[0] = s0[0];
            o[1] = s1[0];
            o[2] = s0[1];
            o[3] = s1[1];
            const int chunk = pp * 4 + gq + half;  // 16-byte piece of the 64-column pass
            *reinterpret_cast<u32x4_t*>(lrow + ((chunk ^ sw) << 4)) = o;
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);  // (keeps the register footprint small: an operand tile is in flight)
    }
    // read the pass back as 128-byte rows and send it out: 8 rows per instruction, 8 lanes each; the upper 32
    // lanes take their four rows in the order 5, 4, 7, 6 so that lanes l and l+32 sit in rows of opposite parity
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int row = i * 8 + (lane >> 3) + ((lane >> 5) ? 1 - 2 * ((lane >> 3) & 1) : 0), chunk = lane & 7;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(mine + row * 128 + ((chunk ^ (row & 7) ^ ((row >> 3) & 1)) << 4));
      // Pieces (8 columns of 16-bit data, 4 of fp32) that start at or past V are not stored; one that V cuts
      // through is written whole, into the stride padding of its row.  (Streaming store: nothing reads dW back.)
      const int64_t col = ph * kPassCols + chunk * kPieceCols;
      if (h0 + row < a.H && v0 + col < a.V)
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>(out + (int64_t)row * a.lddw + col));
      if ((i & 3) == 3) __builtin_amdgcn_sched_barrier(0);  // at most 4 rows in registers at a time
    }
  }
  __syncthreads();  // scratch is handed back to the main loop
}

// acc[pb][qb] is the block of P block pb (h) and Q block qb (v).  The index fed to the B side of the matrix
// instruction runs along lanes and is the row of the stored matrix; the other runs along registers (runs of 8
// per lane pair) and is the column: WVH rows = v (Q), columns = h (P); otherwise rows = h (P), columns = v (Q).
// `part` != null: this is a K segment of a tail tile (see DwPlan); its raw fp32 sum goes to that
// 256 (rows) x 256 (columns) block, through the statements of the fp32 output path (another destination, row
// stride and factor, no bounds) -- a separate code path behind a branch would read the accumulator twice.
template <class T, bool WVH>
LCE_DEV void dw_epilogue(const BwdArgs& a, float* part, f32x16_t (&acc)[kNB][kNB], int tp, int tq) {
  typedef typename elem_of<T>::type E;
  const DwTileGeom<WVH> g(a, tp, tq);
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;          // this wave's half of the P and of the Q extent
  const int w_row = WVH ? wq : wp, w_col = WVH ? wp : wq;
  const bool tail = part != nullptr;
  const float coef = tail ? 1.f : final_factor_of(a);
  // fp32 destination addressed as [row][col] of the whole stored matrix
  float* f32dst = tail ? part - (g.row0 * kTile + g.col0) : reinterpret_cast<float*>(a.dw);
  const int64_t f32ld = tail ? kTile : a.lddw;
  const int half = lane >> 5;
#pragma unroll
  for (int rb = 0; rb < kNB; ++rb) {
    const int64_t row = g.row0 + w_row * kWaveTile + rb * kBlk + (lane & 31);
    const bool row_exists = row < g.row_limit;
#pragma unroll
    for (int cbk = 0; cbk < kNB; ++cbk) {
      const f32x16_t& blk = WVH ? acc[cbk][rb] : acc[rb][cbk];
      const int64_t cb = g.col0 + w_col * kWaveTile + cbk * kBlk;
      // Pieces (4 columns in fp32, 8 in the 16-bit types) that start at or past the last column are not
      // stored; one that it cuts through is written whole, into the stride padding of its row.
      if (a.dw_dtype == DT_F32 || tail) {
#pragma unroll
        for (int rq = 0; rq < 4; ++rq) {
          if (!tail && (cb + 8 * rq + 4 * half >= g.col_limit || !row_exists)) continue;
          f32x4_t o;
#pragma unroll
          for (int j = 0; j < 4; ++j) o[j] = blk[rq * 4 + j] * coef;
          *reinterpret_cast<f32x4_t*>(f32dst + row * f32ld + cb + 8 * rq + 4 * half) = o;
        }
      } else {
        // Lanes l and l+32 hold the two halves of every run of 8 columns; one
        // lane-half swap per pair of register quads gives each lane a whole run,
        // so a store writes 32 contiguous bytes (a full sector) per row of dW.
#pragma unroll
        for (int gq = 0; gq < 4; gq += 2) {
          float d[8];
#pragma unroll
          for (int i = 0; i < 8; ++i) d[i] = blk[gq * 4 + i] * coef;
          const unsigned x0 = pack2<T>(d[0], d[1]), x1 = pack2<T>(d[2], d[3]);
          const unsigned y0 = pack2<T>(d[4], d[5]), y1 = pack2<T>(d[6], d[7]);
          const auto s0 = __builtin_amdgcn_permlane32_swap(x0, y0, false, false);
          const auto s1 = __builtin_amdgcn_permlane32_swap(x1, y1, false, false);
          u32x4_t o;
          o[0] = s0[0];
          o[1] = s1[0];
          o[2] = s0[1];
          o[3] = s1[1];
          if (cb + 8 * (gq + half) < g.col_limit && row_exists)
            *reinterpret_cast<u32x4_t*>(reinterpret_cast<E*>(a.dw) + row * a.lddw + cb + 8 * (gq + half)) = o;
        }
      }
    }
  }
}

// dW summed over chunks of token rows when dW is 16-bit (BwdArgs::dw_plane): the fp32 sums of a tile are kept as two
// 16-bit halves.  The upper halves lie in the caller's dW itself, in the 256 rows x 512 bytes that the tile's
// results will take -- nothing else needs that memory before the last chunk is done --, the lower halves in a
// 128 KiB block of the plane; a tile that the matrix' edge cuts has no whole region of dW, and its upper halves
// go to a block of BwdArgs::dw_plane_hi.  Both halves together are the fp32 sum, bit for bit.
//   Two register quads of a thread (the pair p: quads 2p and 2p+1, eight sums) give 16 bytes of upper and 16 of
// lower halves.  Lower halves: pair p of thread t at byte p * 4096 + t * 16 of the block.  Upper halves: each
// wave keeps to the 128 rows x 256 bytes of its own quarter of the tile's results, and within those the eight
// pairs of one block row of results (32 rows) to the 32 rows x 256 bytes that these results will take: pair
// j = 2 * column block + rq / 2 of a block row is 4 rows, a lane's 16 bytes at row 4 j + lane / 16, byte
// (lane % 16) * 16.  So the last chunk can turn the sums into dW in place, 32 rows at a time (dw_plane_split_final).
// (Hardware fp32 atomic adds into an fp32 plane instead of load - add - store were measured at the headline
// shape: the 268 M atomics of a chunk take longer than the chunk's matrix work, 30.6 ms a step against 22.3.)
//   LO8 (BwdArgs::dw_acc 6 to 8), for problems whose scratch bound has no room for H * V * 2 bytes of lower halves: only
// the upper byte of each lower half is kept (H * V bytes; pair p of thread t at byte p * 2048 + t * 8 of a 64 KiB
// block), and a sum is rounded to nearest at those 24 bits -- 16 of mantissa -- every time it goes back to memory:
// with C chunks a relative error of at most C * 2^-17 before the final rounding to the 16-bit dW.
constexpr unsigned kSelLow = 0x05040100u, kSelHigh = 0x07060302u;  // v_perm selectors: the lower / upper halves of (S0, S1)

// Sum number e (0..7) of a pair from the dword of upper halves that holds its upper half and the lower parts.
template <bool LO8, class L> LCE_DEV float dw_sum_of(const u32x4_t& h, const L& l, int e) {
  if constexpr (LO8) {
    // bytes (0, lower part e % 4 of dword e / 4, the two bytes of upper half e % 2 of dword e / 2)
    const unsigned sel = ((5u + 2u * (e & 1)) << 24) | ((4u + 2u * (e & 1)) << 16) | ((unsigned)(e & 3) << 8) | 0x0cu;
    return __builtin_bit_cast(float, __builtin_amdgcn_perm(h[e >> 1], l[e >> 2], sel));
  } else {
    return __builtin_bit_cast(float, __builtin_amdgcn_perm(h[e >> 1], l[e >> 1], (e & 1) ? kSelHigh : kSelLow));
  }
}

// Where the upper halves of tile (tp, tq) lie, and the distance of their rows in bytes.
template <bool WVH>
LCE_DEV char* dw_hi_block(const BwdArgs& a, int tp, int tq, int& stride) {
  const DwTileGeom<WVH> g(a, tp, tq);
  if (g.row0 + kTile <= g.row_limit && g.col0 + kTile <= g.col_limit) {
    stride = (int)a.lddw * 2;
    return reinterpret_cast<char*>(a.dw) + (g.row0 * a.lddw + g.col0) * 2;
  }
  // tiles cut by the edge, numbered: those of the last tile row over h first (if H cuts it), then the last over v
  const int tiles_p = (int)(a.Hp / kTile), tiles_q = (int)(a.vs / kTile);
  const bool cut_p = a.Hp != a.H;
  const int e = cut_p && tp == tiles_p - 1 ? tq : (cut_p ? tiles_q : 0) + tp;
  stride = 512;
  return reinterpret_cast<char*>(a.dw_plane_hi) + (int64_t)e * (kTile * kTile * 2);
}

template <bool LOAD, bool WVH, bool LO8>
LCE_DEV void dw_plane_split_io(char* hi, int hi_stride, char* lo, f32x16_t (&acc)[kNB][kNB]) {
  typedef typename std::conditional<LO8, u32x2_t, u32x4_t>::type L;
  constexpr int kLoBytes = LO8 ? 8 : 16;  // of a pair and thread
  // one descriptor per block, the thread's place as the vector offset, the pair as a scalar offset: no 64-bit
  // address per pair
  const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(hi, 0, 255 * hi_stride + 512, 0x00020000);
  const __amdgpu_buffer_rsrc_t rl = __builtin_amdgcn_make_buffer_rsrc(lo, 0, 32 * kThreads * kLoBytes, 0x00020000);
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  const int w_row = WVH ? wq : wp, w_col = WVH ? wp : wq;
  const int vh = (w_row * kWaveTile + (lane >> 4)) * hi_stride + w_col * 256 + (lane & 15) * 16;
  const int vl = tid * kLoBytes;
  // kBatch pairs are fetched together before any is used: their loads are in flight together (2, 8 and 16 pairs
  // measured the same)
  constexpr int kBatch = 8;
#pragma unroll
  for (int p0 = 0; p0 < 32; p0 += kBatch) {
    u32x4_t oh[kBatch];
    L ol[kBatch];
    if (LOAD) {
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        const int p = p0 + u, i = p >> 3, k = (p >> 1) & 3, rb = WVH ? k : i, cb = WVH ? i : k;
        oh[u] = __builtin_amdgcn_raw_buffer_load_b128(rh, vh, (rb * kBlk + (cb * 2 + (p & 1)) * 4) * hi_stride, 0);
        if constexpr (LO8) ol[u] = __builtin_amdgcn_raw_buffer_load_b64(rl, vl, p * (kThreads * kLoBytes), 0);
        else ol[u] = __builtin_amdgcn_raw_buffer_load_b128(rl, vl, p * (kThreads * kLoBytes), 0);
      }
    }
#pragma unroll
    for (int u = 0; u < kBatch; ++u) {
      const int p = p0 + u, i = p >> 3, k = (p >> 1) & 3, rb = WVH ? k : i, cb = WVH ? i : k;
      unsigned r[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // (a volatile read: the compiler would otherwise read all 256 accumulator registers before the first load)
        float f;
        asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(f) : "a"(acc[i][k][(p & 1) * 8 + j]));
        if (LOAD) f += dw_sum_of<LO8>(oh[u], ol[u], j);
        r[j] = __builtin_bit_cast(unsigned, f);
        if constexpr (LO8) r[j] += 0x7fu + ((r[j] >> 8) & 1u);  // to nearest (even) at 24 bits; the last byte is dropped below
      }
      u32x4_t nh;
#pragma unroll
      for (int d = 0; d < 4; ++d) nh[d] = __builtin_amdgcn_perm(r[2 * d + 1], r[2 * d], kSelHigh);
      __builtin_amdgcn_raw_buffer_store_b128(nh, rh, vh, (rb * kBlk + (cb * 2 + (p & 1)) * 4) * hi_stride, 0);
      if constexpr (LO8) {
        u32x2_t nl;
#pragma unroll
        for (int w = 0; w < 2; ++w)  // byte 1 of four sums
          nl[w] = __builtin_amdgcn_perm(r[4 * w + 1], r[4 * w], 0x0c0c0501u) | __builtin_amdgcn_perm(r[4 * w + 3], r[4 * w + 2], 0x05010c0cu);
        __builtin_amdgcn_raw_buffer_store_b64(nl, rl, vl, p * (kThreads * kLoBytes), 0);
      } else {
        u32x4_t nl;
#pragma unroll
        for (int d = 0; d < 4; ++d) nl[d] = __builtin_amdgcn_perm(r[2 * d + 1], r[2 * d], kSelLow);
        __builtin_amdgcn_raw_buffer_store_b128(nl, rl, vl, p * (kThreads * kLoBytes), 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);  // (one batch in registers at a time: an operand tile is in flight)
  }
}

// The last chunk of a 16-bit dW summed over chunks: the tile's sums are added to those of the earlier chunks and leave
// as dW at once -- scaled, rounded, as whole 256-byte rows -- instead of going back to the halves.  A wave takes the
// 32 rows of one block row of its results at a time: the 8 KiB of upper halves come from exactly the 32 rows x 256
// bytes of dW that these results will take (dw_plane_split_io), so all of them are loaded before the first row is
// stored; the values pass through the wave's slice of `scratch` (main-loop stage 1, idle during an epilogue; rows of
// the slice are 272 bytes apart: 16-byte pieces stay aligned; the 8-byte writes of 32 lanes to 32 rows meet two-way
// bank conflicts, a few microseconds per launch).
template <class T, bool WVH, bool LO8>
LCE_DEV void dw_plane_split_final(const BwdArgs& a, const char* hi, int hi_stride, const char* lo, f32x16_t (&acc)[kNB][kNB],
                                  int tp, int tq, char* scratch) {
  typedef typename elem_of<T>::type E;
  typedef typename std::conditional<LO8, u32x2_t, u32x4_t>::type L;
  constexpr int kLoBytes = LO8 ? 8 : 16;
  constexpr int kRowBytes = 256 + 16;
  static_assert(kBlk * kRowBytes <= kDwSliceBytes, "a block row of results fits a wave's slice");
  const DwTileGeom<WVH> g(a, tp, tq);
  const float coef = final_factor_of(a);
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1, half = lane >> 5;
  const int w_row = WVH ? wq : wp, w_col = WVH ? wp : wq;
  const __amdgpu_buffer_rsrc_t rh = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(hi), 0, 255 * hi_stride + 512, 0x00020000);
  const __amdgpu_buffer_rsrc_t rl = __builtin_amdgcn_make_buffer_rsrc(const_cast<char*>(lo), 0, 32 * kThreads * kLoBytes, 0x00020000);
  const int vh = (w_row * kWaveTile + (lane >> 4)) * hi_stride + w_col * 256 + (lane & 15) * 16;
  const int vl = tid * kLoBytes;
  char* my = scratch + wave * kDwSliceBytes;
  E* out = reinterpret_cast<E*>(a.dw);
#pragma unroll
  for (int rb = 0; rb < kNB; ++rb) {
    u32x4_t h[8];
    L l[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int cb = j >> 1, i = WVH ? cb : rb, k = WVH ? rb : cb;  // the pair is of block acc[i][k]
      h[j] = __builtin_amdgcn_raw_buffer_load_b128(rh, vh, (rb * kBlk + j * 4) * hi_stride, 0);
      if constexpr (LO8) l[j] = __builtin_amdgcn_raw_buffer_load_b64(rl, vl, ((i * 4 + k) * 2 + (j & 1)) * (kThreads * kLoBytes), 0);
      else l[j] = __builtin_amdgcn_raw_buffer_load_b128(rl, vl, ((i * 4 + k) * 2 + (j & 1)) * (kThreads * kLoBytes), 0);
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int cb = j >> 1, i = WVH ? cb : rb, k = WVH ? rb : cb;
#pragma unroll
      for (int qq = 0; qq < 2; ++qq) {
        float v[4];
#pragma unroll
        for (int d = 0; d < 2; ++d) {
          float a0, a1;
          // (volatile reads: the compiler would otherwise read all 256 accumulator registers before the first load)
          asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(a0) : "a"(acc[i][k][(j & 1) * 8 + qq * 4 + 2 * d]));
          asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(a1) : "a"(acc[i][k][(j & 1) * 8 + qq * 4 + 2 * d + 1]));
          v[2 * d] = (a0 + dw_sum_of<LO8>(h[j], l[j], qq * 4 + 2 * d)) * coef;
          v[2 * d + 1] = (a1 + dw_sum_of<LO8>(h[j], l[j], qq * 4 + 2 * d + 1)) * coef;
        }
        const int rq = (j & 1) * 2 + qq;
        u32x2_t o;
        o[0] = pack2<T>(v[0], v[1]);
        o[1] = pack2<T>(v[2], v[3]);
        *reinterpret_cast<u32x2_t*>(my + (lane & 31) * kRowBytes + (cb * kBlk + 8 * rq + 4 * half) * 2) = o;
      }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      const int r = it * 4 + (lane >> 4), piece = lane & 15;
      const u32x4_t v = *reinterpret_cast<const u32x4_t*>(my + r * kRowBytes + piece * 16);
      const int64_t row = g.row0 + w_row * kWaveTile + rb * kBlk + r;
      const int64_t col = g.col0 + w_col * kWaveTile + piece * 8;
      // pieces that start at or past the last column are not stored; one that it cuts through is written whole,
      // into the stride padding of its row
      if (row < g.row_limit && col < g.col_limit)
        __builtin_nontemporal_store(v, reinterpret_cast<u32x4_t*>(out + row * a.lddw + col));
    }
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_sched_barrier(0);  // (one block row in registers at a time: an operand tile is in flight)
  }
  __syncthreads();  // scratch is handed back to the main loop
}

// fp32 dW summed over chunks of token rows in the caller's buffer itself (BwdArgs::dw_acc 3 / 4): the tile's sum times
// the final factor is stored (first chunk) or added to what is there (ADD), in the 16-byte quads a lane holds -- rows
// of the stored matrix along the lanes, as in dw_epilogue; the four quads of an accumulator block are fetched
// together before any is used.
template <bool WVH, bool ADD>
LCE_DEV void dw_epilogue_f32_sum(const BwdArgs& a, f32x16_t (&acc)[kNB][kNB], int tp, int tq) {
  const DwTileGeom<WVH> g(a, tp, tq);
  const int tid = opaque_tid();
  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave & 1, wq = wave >> 1;
  const int w_row = WVH ? wq : wp, w_col = WVH ? wp : wq;
  const int half = lane >> 5;
  const float coef = final_factor_of(a);
#pragma unroll
  for (int rb = 0; rb < kNB; ++rb) {
    const int64_t row = g.row0 + w_row * kWaveTile + rb * kBlk + (lane & 31);
    const bool row_exists = row < g.row_limit;
    const int64_t c0 = g.col0 + w_col * kWaveTile + 4 * half;  // this lane's first column
    float* prow = reinterpret_cast<float*>(a.dw) + row * a.lddw + c0;
#pragma unroll
    for (int cbk = 0; cbk < kNB; ++cbk) {
      f32x4_t old[4];
      bool ok[4];
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        // quads that start at or past the last column are left alone; one that it cuts through is written whole,
        // into the stride padding of its row
        ok[rq] = row_exists && c0 + cbk * kBlk + 8 * rq < g.col_limit;
        if (ADD) {
          const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
          old[rq] = ok[rq] ? *reinterpret_cast<const f32x4_t*>(prow + cbk * kBlk + 8 * rq) : zero;
        }
      }
#pragma unroll
      for (int rq = 0; rq < 4; ++rq) {
        f32x4_t v;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          // (a volatile read: the compiler would otherwise read all 256 accumulator registers before the first load)
          float t;
          if (WVH) asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t) : "a"(acc[cbk][rb][rq * 4 + j]));
          else asm volatile("v_accvgpr_read_b32 %0, %1" : "=v"(t) : "a"(acc[rb][cbk][rq * 4 + j]));
          v[j] = t * coef;
        }
        if (ADD) v += old[rq];
        if (ok[rq]) *reinterpret_cast<f32x4_t*>(prow + cbk * kBlk + 8 * rq) = v;
      }
      __builtin_amdgcn_sched_barrier(0);  // (one block in registers at a time: an operand tile is in flight)
    }
  }
}

// How one launch divides its work: as for dx (lce_bwd_dx.hip).  The T = (vs/256) x (Hp/256) output tiles
// go to G persistent workgroups in rounds; a last round with r <= G/2 tiles is cut along K = tokens into
// `nseg` segments of `kseg` K tiles (r * nseg <= G, at least 16 K tiles each), whose fp32 sums meet in
// 256 x 256 blocks of dw_part and are added, in segment order, by dw_tail_kernel.  With few tiles in all
// (a small vocabulary slab times a small hidden size) every tile is a tail tile.  The K extent comes from
// the row count on the device, so the plan is made there; the segments cover the K tiles exactly.
struct DwPlan {
  int tiles, full, tail_tiles, nseg, kseg, kt;
};
LCE_DEV DwPlan dw_plan(const BwdArgs& a, int64_t rows) {
  DwPlan p;
  const int G = a.dw_grid;
  const int64_t kt2 = (rows + 2 * kBK - 1) / (2 * kBK) * 2;  // K tiles: an even number, at least four, covering the rows
  p.kt = (int)(kt2 < 4 ? 4 : kt2);
  p.tiles = (int)(a.vs / kTile) * (int)(a.Hp / kTile);
  p.full = p.tiles / G * G;
  const int r = p.tiles - p.full, cap = G < kTailBlocks ? G : kTailBlocks;
  int s = 1;
  if (r > 0 && a.dw_part != nullptr)  // (no blocks for partial sums: nothing is split)
    while (r * s * 2 <= cap && p.kt / (s * 2) >= 16) s *= 2;
  if (s == 1) {
    p.full = p.tiles;
    p.tail_tiles = 0;
    p.nseg = 1;
    p.kseg = p.kt;
  } else {
    // s segments that cover the K tiles exactly: an even number each, the last one takes what is left over
    // (fewer than 2 s K tiles more than the others)
    p.tail_tiles = r;
    p.kseg = (p.kt / s) & ~1;
    p.nseg = s;
  }
  return p;
}

// Which work items of the plan a launch covers, and how whole tiles leave the registers.  A kernel holds one
// epilogue only: two of them behind a run-time branch make the compiler read all 256 accumulator registers for
// both arms at once.
//   kDwAll       every item, direct stores (dW stored (V, H))
//   kDwStaged    whole tiles only, stored as full lines through LDS (16-bit dW stored (H, V))
//   kDwStaged32  the same for fp32 dW
//   kDwTails     the K segments of the tail tiles only (their launch follows that of the whole tiles)
enum { kDwAll = 0, kDwStaged = 1, kDwTails = 2, kDwStaged32 = 3 };

// ACC: what the plane of sums over chunks of token rows has to do with a tile (BwdArgs::dw_acc; whole tiles only).
template <class T, bool WVH, int MODE, int ACC = 0> struct DwProblem {
  static constexpr bool kSwapAB = !WVH;  // (H, V) output: dz, the Q operand, feeds the A side (v along registers)
  static constexpr bool kVarK = true;    // whole tiles and segment items have different K extents
  static constexpr bool kKMask = false;  // both operands have K as their slow index: nothing to mask
  static constexpr bool kQBlocked = true;  // dz is staged in blocks of 256 rows x 64 columns (BwdArgs::dz)
  static constexpr bool kColumnEpilogue = false;
  typedef typename elem_of<T>::type E;
  const BwdArgs& a;
  int64_t rows, ldx;  // token rows (the K extent): all of x, or the packed rows (see BwdArgs)
  const E* x;
  int tiles_p, tiles_q;  // P = x: tiles over h; Q = dz: tiles over the columns of the slab
  DwPlan plan;
  int first, count;      // this launch's items of the plan: [first, first + count)
  LCE_DEV DwProblem(const BwdArgs& a_) : a(a_), tiles_p((int)(a_.Hp / kTile)), tiles_q((int)(a_.vs / kTile)) {
    rows = packed_rows(a.n_rows, a.N);
    const bool packed = rows != a.N;
    x = reinterpret_cast<const E*>(packed ? a.xc : a.x);
    ldx = packed ? a.ldxc : a.ldx;
    plan = dw_plan(a, rows);
    const int tails = plan.tail_tiles * plan.nseg;
    first = MODE == kDwTails ? plan.full : 0;
    count = MODE == kDwAll ? plan.full + tails : (MODE == kDwTails ? tails : plan.full);
  }
  LCE_DEV int num_tiles() const { return count; }
  // `local` counts this launch's items; seg < 0: a whole tile
  LCE_DEV void decode(int local, int& item, int& tp, int& tq, int& seg) const {
    item = first + local;
    int tile = item;
    seg = -1;
    if (item >= plan.full) {
      const int j = item - plan.full;
      tile = plan.full + j / plan.nseg;
      seg = j % plan.nseg;
    }
    tile_coords(tile, plan.tiles, tiles_p, tiles_q, 8, 8, tp, tq);
  }
  LCE_DEV int item_ktiles(int local) const {
    const int item = first + local;
    if (item < plan.full) return plan.kt;
    const int seg = (item - plan.full) % plan.nseg;
    return seg == plan.nseg - 1 ? plan.kt - seg * plan.kseg : plan.kseg;
  }
  LCE_DEV void origins(int local, const void*& p, const void*& q) const {
    int item, tp, tq, seg;
    decode(local, item, tp, tq, seg);
    const int64_t k0 = seg < 0 ? 0 : (int64_t)seg * plan.kseg * kBK;  // first token of the segment
    p = x + k0 * ldx + (int64_t)tp * kTile;
    q = reinterpret_cast<const E*>(a.dz) + dz_block_offset(k0 / kTile, (int64_t)tq * (kTile / kBK), a.vs) + (k0 % kTile) * kBK;
  }
  // (segments start at even numbers of K tiles: in the first or the third quarter of a row of blocks)
  LCE_DEV int q_phase(int local) const {
    int item, tp, tq, seg;
    decode(local, item, tp, tq, seg);
    return seg < 0 ? 0 : (seg * plan.kseg) & 3;
  }
  // x rows past the last one read as zeros.  dz is written for whole token tiles of 256 rows, and the K tiles of
  // the plan end with the pair of K tiles that holds the last row (dw_plan), so none of them reaches past
  // the rows that were written -- except when there is no row at all: then dz reads as zeros too.
  LCE_DEV const void* p_end() const { return matrix_end<E>(x, rows, ldx, a.H); }
  LCE_DEV const void* q_end() const {
    return reinterpret_cast<const E*>(a.dz) + (rows > 0 ? a.dz_rows * a.vs : 0);
  }
  LCE_DEV int k_valid(int) const { return (int)a.Np; }
  LCE_DEV void prefetch(int) {}
  LCE_DEV void epilogue(int local, f32x16_t (&acc)[kNB][kNB], char* scratch) const {
    int item, tp, tq, seg;
    decode(local, item, tp, tq, seg);
    if constexpr (ACC == 3 || ACC == 4) {
      dw_epilogue_f32_sum<WVH, ACC == 4>(a, acc, tp, tq);
      return;
    } else if constexpr (ACC != 0) {
      int stride;
      char* hi = dw_hi_block<WVH>(a, tp, tq, stride);
      constexpr bool kLo8 = ACC >= 6;
      char* lo = reinterpret_cast<char*>(a.dw_plane) + ((int64_t)tq * tiles_p + tp) * (kTile * kTile * (kLo8 ? 1 : 2));
      if constexpr (ACC == 5 || ACC == 8) dw_plane_split_final<T, WVH, kLo8>(a, hi, stride, lo, acc, tp, tq, scratch);
      else dw_plane_split_io<ACC == 2 || ACC == 7, WVH, kLo8>(hi, stride, lo, acc);
      return;
    }
    if (MODE == kDwStaged || MODE == kDwStaged32) {
      dw_store_rows_hv<T, MODE == kDwStaged32>(a, acc, tp, tq, scratch);
    } else {
      float* part = seg >= 0 ? a.dw_part + (int64_t)(item - plan.full) * kTile * kTile : nullptr;
      dw_epilogue<T, WVH>(a, part, acc, tp, tq);
    }
  }
};

template <class T, bool WVH, int MODE, int ACC>
__global__ __launch_bounds__(kThreads) void bwd_dw_persistent_kernel(const BwdArgs a) {
  extern __shared__ __attribute__((aligned(16))) char lds[];
  typedef typename elem_of<T>::type E;
  DwProblem<T, WVH, MODE, ACC> prob(a);
  // (a chunk without a kept row adds nothing to the sums of the earlier chunks)
  if ((ACC == 2 || ACC == 4 || ACC == 7) && prob.rows == 0) return;
  Pipe3<T, E, false, E, false, DwProblem<T, WVH, MODE, ACC>> pipe(prob);
  pipe.run(prob.ldx, a.vs / kBK, prob.plan.kt, lds);
}

// Second step for the tail tiles: kTailParts workgroups share tail tile b (16 of its rows each) -- they sum
// its segments in order, scale, and store the tile of dW in the output dtype.
constexpr int kTailParts = 16;
template <class T, bool WVH>
__global__ __launch_bounds__(256) void dw_tail_kernel(const BwdArgs a) {
  typedef typename elem_of<T>::type E;
  const DwPlan plan = dw_plan(a, packed_rows(a.n_rows, a.N));
  const int b = (int)blockIdx.x / kTailParts, piece = (int)blockIdx.x % kTailParts;
  if (b >= plan.tail_tiles) return;
  int tp, tq;
  tile_coords(plan.full + b, plan.tiles, (int)(a.Hp / kTile), (int)(a.vs / kTile), 8, 8, tp, tq);
  const DwTileGeom<WVH> g(a, tp, tq);
  const float coef = final_factor_of(a);
  const float* part = a.dw_part + (int64_t)b * plan.nseg * kTile * kTile;
  constexpr int kQuads = kTile * kTile / 4 / kTailParts;
  for (int i = piece * kQuads + threadIdx.x; i < (piece + 1) * kQuads; i += 256) {
    const int r = i / (kTile / 4), c = (i - r * (kTile / 4)) * 4;
    const int64_t row = g.row0 + r, col = g.col0 + c;
    if (row >= g.row_limit || col >= g.col_limit) continue;  // a quad that the last column cuts through is written whole, into the stride padding of its row
    f32x4_t acc = *reinterpret_cast<const f32x4_t*>(part + r * kTile + c);
#pragma unroll 4
    for (int s = 1; s < plan.nseg; ++s)
      acc += *reinterpret_cast<const f32x4_t*>(part + (int64_t)s * kTile * kTile + r * kTile + c);
    if (a.dw_dtype == DT_F32) {
      *reinterpret_cast<f32x4_t*>(reinterpret_cast<float*>(a.dw) + row * a.lddw + col) = acc * coef;
    } else {
      u32x2_t o;
      o[0] = pack2<T>(acc[0] * coef, acc[1] * coef);
      o[1] = pack2<T>(acc[2] * coef, acc[3] * coef);
      *reinterpret_cast<u32x2_t*>(reinterpret_cast<E*>(a.dw) + row * a.lddw + col) = o;
    }
  }
}

template <class T, bool WVH, int MODE, int ACC = 0> hipError_t launch_tiles(const BwdArgs& a, hipStream_t s) {
  auto kern = bwd_dw_persistent_kernel<T, WVH, MODE, ACC>;
  static LdsOptIn optin;
  hipError_t e = optin.ensure(reinterpret_cast<const void*>(kern), kMainloopLds);
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(kern, dim3(a.dw_grid), dim3(kThreads), kMainloopLds, s, a);
  return hipGetLastError();
}

// Whole tiles that meet the plane of sums over chunks of token rows (nothing is split along K then).
template <class T, bool WVH, int MODE> hipError_t launch_plane(const BwdArgs& a, hipStream_t s) {
  switch (a.dw_acc) {
    case 1: return launch_tiles<T, WVH, MODE, 1>(a, s);
    case 2: return launch_tiles<T, WVH, MODE, 2>(a, s);
    case 5: return launch_tiles<T, WVH, MODE, 5>(a, s);  // the last chunk: the sums leave as dW at once
    case 6: return launch_tiles<T, WVH, MODE, 6>(a, s);  // the same three with the lower halves cut to a byte
    case 7: return launch_tiles<T, WVH, MODE, 7>(a, s);
    case 8: return launch_tiles<T, WVH, MODE, 8>(a, s);
    default: return hipErrorInvalidValue;
  }
}

template <class T, bool WVH> hipError_t launch_persistent(const BwdArgs& a, hipStream_t s) {
  if (a.dw_acc == 3 || a.dw_acc == 4) {  // fp32 dW summed in the caller's buffer: whole tiles only
    if (a.dw_dtype != DT_F32 || a.dw_part != nullptr) return hipErrorInvalidValue;
    return a.dw_acc == 3 ? launch_tiles<T, WVH, kDwAll, 3>(a, s) : launch_tiles<T, WVH, kDwAll, 4>(a, s);
  }
  if (a.dw_acc != 0) {
    // (16-bit dW only, and a place for the upper halves of the tiles that the edge of the matrix cuts)
    const bool cut = a.Hp != a.H || a.v0 + a.vs != a.V;
    if (a.dw_plane == nullptr || a.dw_part != nullptr || a.dw_dtype == DT_F32 || (cut && a.dw_plane_hi == nullptr))
      return hipErrorInvalidValue;
    return launch_plane<T, WVH, kDwAll>(a, s);
  }
  // a last round of tiles may be split along K (the tile count does not depend on the rows; whether its K
  // extent is long enough to split is decided on the device, and a launch without items returns at once)
  const bool tails = a.dw_part != nullptr && dw_tail_blocks(a.Np, a.Hp, a.vs) != 0 &&
                     has_split_tail((a.vs / kTile) * (a.Hp / kTile), a.dw_grid);
  hipError_t e = hipSuccess;
  if constexpr (WVH) {
    e = launch_tiles<T, true, kDwAll>(a, s);
  } else {
    // (a small problem whose tiles are all split along K has no whole tile to launch; known here when rows are not packed)
    const int64_t kt2 = (a.N + 2 * kBK - 1) / (2 * kBK) * 2;
    const bool none_whole = tails && a.n_rows == nullptr &&
                            all_tiles_are_tails((a.vs / kTile) * (a.Hp / kTile), a.dw_grid, kt2 < 4 ? 4 : kt2);
    if (!none_whole)
      e = a.dw_dtype == DT_F32 ? launch_tiles<T, false, kDwStaged32>(a, s) : launch_tiles<T, false, kDwStaged>(a, s);
    if (e == hipSuccess && tails) e = launch_tiles<T, false, kDwTails>(a, s);
  }
  if (e != hipSuccess || !tails) return e;
  // at most dw_grid / 2 tail tiles can be split (two segments each)
  const unsigned tail_most = (unsigned)(a.dw_grid / 2 > 0 ? a.dw_grid / 2 : 1);
  hipLaunchKernelGGL((dw_tail_kernel<T, WVH>), dim3(tail_most * kTailParts), dim3(256), 0, s, a);
  return hipGetLastError();
}

}  // namespace

hipError_t launch_bwd_dw(const BwdArgs& a, hipStream_t s) {
  if (a.x_dtype == DT_BF16) return a.w_vh ? launch_persistent<BF16, true>(a, s) : launch_persistent<BF16, false>(a, s);
  if (a.x_dtype == DT_F16) return a.w_vh ? launch_persistent<F16, true>(a, s) : launch_persistent<F16, false>(a, s);
  return hipErrorInvalidValue;
}

}  // namespace lce
