// Rank-r ("skinny") products of the LoRA branch for gfx950.  All are HBM-bandwidth bound:
// each streams one [M, K] or [M, N] operand once and does a few MFMA 16x16x32 per 16 rows.
//
//   xa      : S  = drop(X) A^T                       (replaces seeded_dropout + cuBLAS X~ A^T,
//             lorafusion/ops/lora_v1.py:111-119, and fused_dropout_matmul.py:152-277)
//   dys_dyb : dS = scale dY B ; dB = scale dY^T S    (fused_lora_dys_dyb.py:71-179,
//             fused_multi_lora_dys_dyb.py:61-185; fp32 atomics there, two-stage sums here)
//   da      : dA = dS^T X~                           (the cuBLAS call at lora_v1.py:153,
//             multi_lora.py:576-581; X~ is rebuilt from X and the keep-mask, never stored)
//
// Every kernel works on 128-row token blocks (= the routing block of the multi-LoRA batch
// info) and writes fp32 partial sums; the small reduce kernels add the partials in a fixed
// order, apply scale / 1/(1-p), zero padded rows and rank columns, and cast.  Results are
// therefore run-to-run deterministic.
//
// Streaming: the big operand moves as 128-row x 64-column tiles.  Global loads are coalesced
// (8 consecutive lanes read one 128-byte row segment) and the tile sits in LDS with the same XOR
// swizzle as the GEMM (granule g of row r at slot g ^ ((r>>1)&7)), from where both MFMA access
// patterns are bank-conflict free: row fragments (ds_read_b128) and transposed fragments
// (ds_read_b64_tr_b16).  Loading MFMA fragments straight from global memory would put every
// lane on a different row (one cache line per lane) and runs at a quarter of the coalesced rate.
// Two transports: through registers (load, keep-mask applied on the way, LDS store; xa, and
// dys_dyb / da above rank 64), or as buffer loads that write LDS themselves, several tiles
// ahead through a ring of stages (dys_dyb / da up to rank 64; second half of this file).
//
// MFMA 16x16x32 operand layout (64 lanes): lane l holds row/col (l & 15) and the 8
// contraction elements of chunk (l >> 4).  Where the contraction index is the slow memory
// dimension, tiles are staged in LDS and read with ds_read_b64_tr_b16 (16 lanes read a
// 4-row x 16-column patch; lane 4j+c addresses row j, columns 4c..4c+3; each lane receives
// its column's 4 rows).
#include "lf_common.h"
#include "act_math.h"
#include "philox.h"
#include <type_traits>

namespace {

constexpr int ROWS = 128;  // rows per workgroup = one routing block

template <typename T> struct Mfma16;
template <> struct Mfma16<__bf16> {
  static __device__ __forceinline__ lf_f32x4 run(lf_u32x4 a, lf_u32x4 b, lf_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lf_bf16x8, a), __builtin_bit_cast(lf_bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint16_t cvt(float f) { return __builtin_bit_cast(uint16_t, (__bf16)f); }
};
template <> struct Mfma16<_Float16> {
  static __device__ __forceinline__ lf_f32x4 run(lf_u32x4 a, lf_u32x4 b, lf_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(lf_f16x8, a), __builtin_bit_cast(lf_f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint16_t cvt(float f) { return __builtin_bit_cast(uint16_t, (_Float16)f); }
};

struct BlockInfo {
  int rank, valid, seg;
  float scale, p;
};

// Routing of the 128-row block `blk` (wave-uniform).
__device__ __forceinline__ BlockInfo block_info(const LfSegTable& seg, int blk, int M) {
  BlockInfo b;
  if (seg.table == nullptr) {
    b.rank = seg.rank[0];
    b.valid = min(ROWS, M - blk * ROWS);
    b.seg = 0;
    b.scale = seg.scale;
    b.p = seg.p;
  } else {
    b.rank = seg.table[3 * blk + 0];
    b.valid = seg.table[3 * blk + 1];
    const int fb = seg.table[3 * blk + 2];
    int s = 0;
    for (int i = 1; i < seg.n_seg; i++) s = (seg.first_block[i] == fb) ? i : s;
    b.seg = s;
    b.scale = seg.block_scale ? seg.block_scale[blk] : 1.f;
    b.p = seg.block_p ? seg.block_p[blk] : 0.f;
  }
  return b;
}

// keep ? x : 0 on 8 packed 16-bit elements given their 8 mask bytes.
__device__ __forceinline__ lf_u32x4 apply_mask8(lf_u32x4 x, lf_u32x2 m) {
  lf_u32x4 r;
#pragma unroll
  for (int d = 0; d < 4; d++) {
    const uint32_t mw = d < 2 ? m[0] : m[1];
    const uint32_t two = (mw >> (16 * (d & 1))) & 0xffffu;           // bytes (2d, 2d+1)
    const uint32_t sel = ((two & 0xffu) ? 0x0000ffffu : 0u) | ((two & 0xff00u) ? 0xffff0000u : 0u);
    r[d] = x[d] & sel;
  }
  return r;
}

// Bit-packed keep-masks: element k of a row = bit k & 7 of byte k >> 3 of the row (K / 8 bytes per row).
// The eight keep bytes (0/1 each, `lo` = the first four) as eight bits, and back: one multiply gathers / spreads four
// single bits (no two partial products meet in one bit position, so nothing carries).
__device__ __forceinline__ uint32_t pack_keep8(uint32_t lo, uint32_t hi) {
  return ((lo * 0x01020408u) >> 24) | (((hi * 0x01020408u) >> 24) << 4);
}
__device__ __forceinline__ lf_u32x2 expand_keep8(uint32_t b) {
  return lf_u32x2{((b & 0xfu) * 0x00204081u) & 0x01010101u, (((b >> 4) & 0xfu) * 0x00204081u) & 0x01010101u};
}

__device__ __forceinline__ lf_u32x4 tr_read8(const char* p, int pitch) {
  // 8 contraction elements (rows r..r+3 and r+4..r+7) of this lane's column
  lf_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(p));
  lf_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(p + 4 * pitch));
  lf_u32x2 a = __builtin_bit_cast(lf_u32x2, lo), b = __builtin_bit_cast(lf_u32x2, hi);
  return lf_u32x4{a[0], a[1], b[0], b[1]};
}


constexpr int TILE_BYTES = ROWS * 128;  // 128 rows x 64 columns of 16-bit

// Swizzle key of a tile row: granule g of row r sits at slot g ^ tile_key(r).  LDS serves a 16-byte read 16 lanes at
// a time and an 8-byte (transposed) read 32 lanes at a time, in both cases 256 bytes = all 64 banks.  Row fragments:
// 16 consecutive rows, one granule each -- the 8 rows of one parity need 8 different keys.  Transposed fragments:
// rows j, 8+j (j = 0..3), two neighbouring granules each -- the 4 rows of one parity (r>>1 = 0, 1, 4, 5 mod 8) need 4
// different key>>1.  The three bits of r>>1 rotated by one do both (with the bits in place, 0/1 and 4/5 share key>>1:
// every transposed read took two passes).
__device__ __forceinline__ int tile_key(int row) {
  const int x = (row >> 1) & 7;
  return ((x & 1) << 2) | (x >> 1);
}

// One thread's share of a 128x64 tile: 4 granules of 8 elements (+ their 8 mask bytes each).
struct TileRegs {
  lf_u32x4 x[4];
  lf_u32x2 m[4];
};

// Coalesced load of the tile whose first element is src[row0*ld + col0]; rows are clamped to max_row-1.
template <typename T>
__device__ __forceinline__ void tile_load(TileRegs& r, const T* __restrict__ src, const uint8_t* __restrict__ mask,
                                          int64_t ld, int row0, int max_row, int col0, int tid, bool use_mask, bool mask_bits) {
  const int srcg = (tid & 7) ^ tile_key(tid >> 3);   // rows i*32 + (tid>>3) share their key
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int row = min(row0 + i * 32 + (tid >> 3), max_row - 1);
    const int64_t off = (int64_t)row * ld + col0 + srcg * 8;
    r.x[i] = *((const lf_u32x4*)(src + off));
    // (bit format: the byte is only requested here; tile_store spreads it into eight bytes)
    if (use_mask) {
      if (mask_bits) r.m[i][0] = mask[off >> 3];
      else r.m[i] = *((const lf_u32x2*)(mask + off));
    }
  }
}

__device__ __forceinline__ void tile_store(const TileRegs& r, char* tile, int tid, bool use_mask, bool mask_bits = false) {
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const lf_u32x2 m = (use_mask && mask_bits) ? expand_keep8(r.m[i][0]) : r.m[i];
    *(lf_u32x4*)(tile + (i * 256 + tid) * 16) = use_mask ? apply_mask8(r.x[i], m) : r.x[i];
  }
}

// Row fragment: 8 consecutive columns (granule g) of `row`.
__device__ __forceinline__ lf_u32x4 tile_row_frag(const char* tile, int row, int g) {
  return *(const lf_u32x4*)(tile + row * 128 + ((g ^ tile_key(row)) << 4));
}

// Transposed fragment: rows row..row+3 and row+4..row+7 of the lane's column; `col` is the first
// of the 4 columns this lane addresses (multiple of 4).
__device__ __forceinline__ lf_u32x4 tile_tr_frag(const char* tile, int row, int col) {
  const int g = col >> 3, within = (col & 7) * 2;
  const char* p0 = tile + row * 128 + ((g ^ tile_key(row)) << 4) + within;
  const char* p1 = tile + (row + 4) * 128 + ((g ^ tile_key(row + 4)) << 4) + within;
  lf_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(p0));
  lf_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(p1));
  lf_u32x2 a = __builtin_bit_cast(lf_u32x2, lo), b = __builtin_bit_cast(lf_u32x2, hi);
  return lf_u32x4{a[0], a[1], b[0], b[1]};
}

// ------------------------------------------------------------------------------------ xa
// One workgroup of 8 waves (2 above rank 64) per 16 rows (64 at ranks 48-64, 32 above); no partial sums leave the workgroup.  The K range is dealt
// to the waves in 64-column steps (step s goes to wave s % waves), each wave streams its steps of the
// 16 rows with coalesced 16-byte loads (8 lanes cover one 128-byte line), all loads of a batch
// of steps in flight at once, applies the keep-mask in registers and turns the row-major
// granules into MFMA row fragments through a 2 KB LDS patch of its own (same-wave LDS traffic is
// ordered: no barrier).  The adapter matrix A (L2 resident) takes the same route: fragment-shaped
// loads would put the four lanes of every quad on four different rows, a quarter of the
// coalesced rate in the texture addresser.  The eight partial [16, R] accumulators are added in a fixed order through LDS,
// scaled by 1/(1-p), zeroed in padded rows and beyond the adapter's rank, and stored as S.
// Rows per workgroup: every workgroup reads the whole adapter matrix (from L2), which at rank 64 is four times the
// bytes of 16 rows of X: with 32 rows per workgroup the pass ran at the L2's rate, not HBM's (268 workgroups x 1 MB of
// A next to 140 MB of X at 8576 x 8192).  Ranks 48-64 take 64 rows (four row blocks share one set of A fragments)
// and eight waves: 0.50 -> 0.40 ms over the four linears of the rank-64 layer.  At rank 16 two row blocks per
// workgroup measured slower (0.27 -> 0.34 ms at the 8B layer: the registers of the second block cost loads in flight).
// (with the activation prologue the up-half registers of four row blocks do not fit next to the rest at ranks 48-64: two)
constexpr int xa_nb(int rt, bool act = false) { return rt == 4 ? (act ? 2 : 4) : rt > 4 ? 2 : 1; }
constexpr int xa_rows(int rt, bool act = false) { return 16 * xa_nb(rt, act); }
// waves per workgroup and steps in flight per wave, by rank tiles (LDS: 2 KB * (1+RT) per wave; registers: 8 * RT per step)
constexpr int xa_waves(int rt) { return rt <= 4 ? 8 : 2; }
constexpr int xa_unroll(int rt) { return rt <= 1 ? 4 : rt <= 2 ? 2 : 1; }

// GEN: the keep-mask is not read but drawn here (Philox, the definition of the standalone mask
// kernel) from (seed, element index) and written to `mask_out` for the backward pass: the integer
// work hides behind the X stream, and one launch and one 1-byte-per-element read disappear.
// ACT: the rows of X do not exist yet: X = round16(round16(silu(G)) * U) is computed here from the gate and up halves of a
// SwiGLU MLP (`X` = G, `U`, rows `ldx` elements apart: the two halves of one merged projection output, or two
// tensors), written once to `act_out` [rows, K] (every element of X is loaded by exactly one lane of the grid) for the
// base GEMM and the backward, and fed to the rank-r product from registers: the activation pass and this pass's own
// read of X disappear.
template <typename T, int RT, bool GEN, bool ACT>
__global__ void __launch_bounds__(xa_waves(RT) * 64)
lora_xa_kernel(const T* __restrict__ X, const T* __restrict__ U, int64_t ldx, T* __restrict__ act_out,
               const uint8_t* __restrict__ mask, uint8_t* __restrict__ mask_out, int mask_bits,
               uint32_t seed_lo, uint32_t seed_hi, T* __restrict__ S, int M, int K, int R, const LfSegTable seg) {
  constexpr int XA_WAVES = xa_waves(RT), XA_U = xa_unroll(RT), NB = xa_nb(RT, ACT), XA_ROWS = xa_rows(RT, ACT);
  // the partial accumulators of the final sum reuse the patches (a barrier separates the two uses): at
  // rank 64 the separate 16 KB pushed the workgroup over 40 KB, and a CU then holds two workgroups, not four
  constexpr int PATCH_BYTES = XA_WAVES * 2048 * (NB + RT), RED_BYTES = XA_WAVES * XA_ROWS * RT * 16 * 4;
  __shared__ __attribute__((aligned(16))) char patch_all[PATCH_BYTES > RED_BYTES ? PATCH_BYTES : RED_BYTES];
  float (*red)[XA_ROWS][RT * 16] = (float (*)[XA_ROWS][RT * 16])patch_all;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, qq = lane >> 4;
  const int row0 = blockIdx.x * XA_ROWS;
  const int blk = row0 / ROWS;
  const BlockInfo bi = block_info(seg, blk, M);
  const T* __restrict__ A = (const T*)seg.ptr[bi.seg];
  const bool use_mask = GEN ? true : (mask != nullptr && bi.p > 0.f);
  const uint32_t thr = lf_keep_threshold(bi.p);
  const int Mrows = seg.table ? seg.n_blocks * ROWS : M;
  const int nsteps = K / 64;
  char* patch = patch_all + wave * 2048 * (NB + RT);  // one X patch per 16-row block, then one patch per 16 rank rows of A

  // loader mapping: lane -> (row lane>>3 (+8), granule lane&7); fragment mapping: (row li, granule 4h+qq)
  const int lrow = lane >> 3, lg = lane & 7;
  const T* xrow[2 * NB];
  const uint8_t* mrow[2 * NB];
  int64_t erow[2 * NB];    // GEN, ACT: element index of this lane's first column in each of its rows (two per 16-row block)
  bool row_real[2 * NB];   // GEN, ACT: the row exists (is not a clamped duplicate): its mask bytes / activations are written
#pragma unroll
  for (int i = 0; i < 2 * NB; i++) {
    const int r = min(row0 + i * 8 + lrow, Mrows - 1);
    xrow[i] = X + (int64_t)r * ldx + lg * 8;
    mrow[i] = mask_bits ? mask + (((int64_t)r * K + lg * 8) >> 3) : mask + (int64_t)r * K + lg * 8;
    erow[i] = (int64_t)r * K + lg * 8;
    row_real[i] = row0 + i * 8 + lrow < Mrows;
  }
  // ACT: the up half lies at one distance from the gate half for every row (a scalar, not a second set of row pointers)
  const int64_t u_off = ACT ? (int64_t)((uintptr_t)U - (uintptr_t)X) : 0;
  const int wr_off[2] = {lrow * 128 + ((lg ^ ((lrow >> 1) & 7)) << 4), (8 + lrow) * 128 + ((lg ^ (((8 + lrow) >> 1) & 7)) << 4)};
  const int rd_row = li * 128, rd_key = (li >> 1) & 7;

  lf_f32x4 acc[NB][RT];
#pragma unroll
  for (int nb = 0; nb < NB; nb++)
#pragma unroll
    for (int c = 0; c < RT; c++) acc[nb][c] = lf_f32x4{0.f, 0.f, 0.f, 0.f};

  // Two register sets of one step each at ranks up to 32, one set above: the loads of one set are requested before
  // the other set is used, so a wave's memory time and its integer / LDS / MFMA time overlap.  All waves of a launch
  // start together and would otherwise sit in the same phase -- everyone waiting for memory, then everyone
  // computing.  Measured at 16512 x 4096, rank 16, mask drawn in the kernel: one set of four steps 44.5 us, two sets
  // of two steps 45.4 (126 registers: half the waves per SIMD), two sets of one step 42.2.
  constexpr int NSET = XA_U >= 2 ? 2 : 1, UB = 1;
  lf_u32x4 xv[NSET][UB][2 * NB], av[NSET][UB][RT][2];
  lf_u32x4 uv[NSET][UB][ACT ? 2 * NB : 1];
  lf_u32x2 mv[NSET][UB][2 * NB];
  auto load_batch = [&](auto B, int s0) {
    constexpr int b = B.value;
#pragma unroll
    for (int u = 0; u < UB; u++) {
      const int s = s0 + u * XA_WAVES;
      if (s < nsteps) {
#pragma unroll
        for (int i = 0; i < 2 * NB; i++) {
          if constexpr (ACT) {
            // gate and up are read once, here: loads that do not allocate in the caches
            xv[b][u][i] = __builtin_nontemporal_load((const lf_u32x4*)(xrow[i] + s * 64));
            uv[b][u][i] = __builtin_nontemporal_load((const lf_u32x4*)((const char*)(xrow[i] + s * 64) + u_off));
          } else {
            xv[b][u][i] = *((const lf_u32x4*)(xrow[i] + s * 64));
          }
          if constexpr (!GEN) {
            // (bit format: the byte is only requested here and spread into eight bytes where it is used, so that no
            // wait for it separates the loads of a batch)
            if (use_mask) {
              if (mask_bits) mv[b][u][i][0] = mrow[i][s * 8];
              else mv[b][u][i] = *((const lf_u32x2*)(mrow[i] + s * 64));
            }
          }
        }
#pragma unroll
        for (int i = 0; i < 2; i++) {
#pragma unroll
          for (int c = 0; c < RT; c++) {
            const int ar = c * 16 + i * 8 + lrow;
            av[b][u][c][i] = lf_u32x4{0, 0, 0, 0};
            if (ar < bi.rank) av[b][u][c][i] = *(const lf_u32x4*)(A + (int64_t)ar * K + s * 64 + lg * 8);
          }
        }
      }
    }
  };
  auto use_batch = [&](auto B, int s0) {
    constexpr int b = B.value;
#pragma unroll
    for (int u = 0; u < UB; u++) {
      const int s = s0 + u * XA_WAVES;
      if (s < nsteps) {
#pragma unroll
        for (int i = 0; i < 2 * NB; i++) {
          if constexpr (ACT) {
            xv[b][u][i] = silu_mul8<T>(xv[b][u][i], uv[b][u][i]);
            if (row_real[i]) __builtin_nontemporal_store(xv[b][u][i], (lf_u32x4*)(act_out + erow[i] + s * 64));
          }
          if constexpr (GEN) {
            uint32_t klo, khi;
            lf_keep8((uint64_t)(erow[i] + s * 64) >> 3, thr, seed_lo, seed_hi, klo, khi);
            mv[b][u][i] = lf_u32x2{klo, khi};
            if (mask_bits) {
              // this lane's eight bits are byte lg of the row's eight bytes of the step: the four lanes of a quad join
              // theirs (two cross-lane moves) and one of them stores the dword
              uint32_t w = pack_keep8(klo, khi) << (8 * (lg & 3));
              w |= (uint32_t)__builtin_amdgcn_mov_dpp((int)w, 0xB1, 0xf, 0xf, true);   // lanes 1 0 3 2
              w |= (uint32_t)__builtin_amdgcn_mov_dpp((int)w, 0x4E, 0xf, 0xf, true);   // lanes 2 3 0 1
              if (row_real[i] && (lg & 3) == 0) *(uint32_t*)(mask_out + ((erow[i] + s * 64) >> 3)) = w;
            } else {
              if (row_real[i]) *(lf_u32x2*)(mask_out + erow[i] + s * 64) = mv[b][u][i];
            }
          }
          if constexpr (!GEN) {
            if (use_mask && mask_bits) mv[b][u][i] = expand_keep8(mv[b][u][i][0]);
          }
          *(lf_u32x4*)(patch + (i >> 1) * 2048 + wr_off[i & 1]) = use_mask ? apply_mask8(xv[b][u][i], mv[b][u][i]) : xv[b][u][i];
        }
#pragma unroll
        for (int i = 0; i < 2; i++)
#pragma unroll
          for (int c = 0; c < RT; c++) *(lf_u32x4*)(patch + (NB + c) * 2048 + wr_off[i]) = av[b][u][c][i];
#pragma unroll
        for (int h = 0; h < 2; h++) {
          const int fo = rd_row + (((h * 4 + qq) ^ rd_key) << 4);
          lf_u32x4 af[RT];
#pragma unroll
          for (int c = 0; c < RT; c++) af[c] = *(const lf_u32x4*)(patch + (NB + c) * 2048 + fo);
#pragma unroll
          for (int nb = 0; nb < NB; nb++) {
            const lf_u32x4 xf = *(const lf_u32x4*)(patch + nb * 2048 + fo);
#pragma unroll
            for (int c = 0; c < RT; c++) acc[nb][c] = Mfma16<T>::run(xf, af[c], acc[nb][c]);
          }
        }
      }
    }
  };
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, NSET - 1>;
  constexpr int STRIDE = XA_WAVES * UB;   // steps between a wave's consecutive batches
  if constexpr (NSET == 1) {
    for (int s0 = wave; s0 < nsteps; s0 += STRIDE) {
      load_batch(Set0{}, s0);
      use_batch(Set0{}, s0);
    }
  } else {
    load_batch(Set0{}, wave);
    for (int s0 = wave; s0 < nsteps; s0 += 2 * STRIDE) {
      load_batch(Set1{}, s0 + STRIDE);      // (steps beyond the row's end are skipped inside)
      use_batch(Set0{}, s0);
      load_batch(Set0{}, s0 + 2 * STRIDE);
      use_batch(Set1{}, s0 + STRIDE);
    }
  }
  __syncthreads();  // every wave is done with its patches
  // C layout: lane holds column (lane & 15), rows 4*(lane >> 4) + e
#pragma unroll
  for (int nb = 0; nb < NB; nb++)
#pragma unroll
    for (int c = 0; c < RT; c++)
#pragma unroll
      for (int e = 0; e < 4; e++) red[wave][nb * 16 + qq * 4 + e][c * 16 + li] = acc[nb][c][e];
  __syncthreads();
  const float mult = (use_mask && bi.p > 0.f) ? 1.f / (1.f - bi.p) : 1.f;  // no mask given: no dropout, whatever p says
  for (int o = tid; o < XA_ROWS * RT * 16; o += XA_WAVES * 64) {
    const int r = o / (RT * 16), c = o % (RT * 16);
    const int row = row0 + r;
    if (row < Mrows && c < R) {
      float v = 0.f;
      if (row - blk * ROWS < bi.valid && c < bi.rank) {
#pragma unroll
        for (int w = 0; w < XA_WAVES; w++) v += red[w][r][c];
        v *= mult;
      }
      ((uint16_t*)S)[(int64_t)row * R + c] = Mfma16<T>::cvt(v);
    }
  }
}

// S[row][col] = cast( mult * sum_p part[p][row][col] ), zero for padded rows / rank columns.
// Sum of `n` fp32x4 partials `stride` floats apart, in index order (deterministic).
__device__ __forceinline__ lf_f32x4 sum_parts(const float* __restrict__ p, int64_t stride, int n) {
  // Up to sixteen partials are requested before the first is added: these second stages are short launches whose
  // time is the chain of memory round trips of one thread, and with four loads in flight a sum of sixteen was four
  // round trips long (5 us for a few hundred KB).  The order of the additions is the index order either way.
  lf_f32x4 v = {0.f, 0.f, 0.f, 0.f};
  int i = 0;
  for (; i + 16 <= n; i += 16) {
    lf_f32x4 t[16];
#pragma unroll
    for (int k = 0; k < 16; k++) t[k] = *(const lf_f32x4*)(p + (int64_t)(i + k) * stride);
#pragma unroll
    for (int k = 0; k < 16; k++) v += t[k];
  }
  if (i < n) {
    lf_f32x4 t[16];
#pragma unroll
    for (int k = 0; k < 16; k++) t[k] = (i + k < n) ? *(const lf_f32x4*)(p + (int64_t)(i + k) * stride) : lf_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 16; k++) v += t[k];   // (adding the zeros beyond n changes nothing: x + 0 = x, and -0 cannot arise from a sum that started at +0)
  }
  return v;
}
template <typename T>
__device__ __forceinline__ lf_u32x2 pack4(lf_f32x4 v) {
  return lf_u32x2{(uint32_t)Mfma16<T>::cvt(v[0]) | ((uint32_t)Mfma16<T>::cvt(v[1]) << 16),
                  (uint32_t)Mfma16<T>::cvt(v[2]) | ((uint32_t)Mfma16<T>::cvt(v[3]) << 16)};
}

template <typename T>
__device__ __forceinline__ void reduce_rows_body(int bx, const float* __restrict__ part, T* __restrict__ out, int nparts, int M, int R,
                   int mode /*0: times 1/(1-p); 1: times scale*/, const LfSegTable seg) {
  // four consecutive columns per thread (R and every rank are multiples of 8): 16-byte loads
  const int Mrows = seg.table ? seg.n_blocks * ROWS : M;
  const int64_t idx = ((int64_t)bx * 256 + threadIdx.x) * 4;
  if (idx >= (int64_t)Mrows * R) return;
  const int row = (int)(idx / R), col = (int)(idx % R);
  const int blk = row / ROWS;
  const BlockInfo bi = block_info(seg, blk, M);
  lf_f32x4 v = {0.f, 0.f, 0.f, 0.f};
  if (row - blk * ROWS < bi.valid && col < bi.rank) {
    v = sum_parts(part + idx, (int64_t)Mrows * R, nparts);
    v *= (mode == 0) ? (bi.p > 0.f ? 1.f / (1.f - bi.p) : 1.f) : bi.scale;
  }
  *(lf_u32x2*)((uint16_t*)out + idx) = pack4<T>(v);
}

// Blocks [b0, b1) of segment s.
__device__ __forceinline__ void segment_blocks(const LfSegTable& seg, int s, int M, int& b0, int& b1) {
  if (seg.table == nullptr) {
    b0 = 0;
    b1 = (M + ROWS - 1) / ROWS;
  } else {
    b0 = seg.first_block[s];
    b1 = (s + 1 < seg.n_seg) ? seg.first_block[s + 1] : seg.n_blocks;
  }
}

// Chunk ch of the blocks [b0, b1) when they are cut into ceil((b1 - b0) / group) chunks of nearly equal size (empty
// beyond the last chunk).
__device__ __forceinline__ void chunk_blocks(int b0, int b1, int group, int ch, int& bb0, int& bb1) {
  const int n = b1 - b0, nch = (n + group - 1) / group;
  if (n <= 0 || ch >= nch) { bb0 = bb1 = b1; return; }
  const int base = n / nch, rem = n % nch;
  bb0 = b0 + ch * base + min(ch, rem);
  bb1 = bb0 + base + (ch < rem ? 1 : 0);
}

// ------------------------------------------------------------------------------- dys_dyb
// grid (n_seg * max_chunks, nsplit).  Workgroup (s, ch, ns) owns the `group` consecutive 128-row blocks ch*group.. of
// segment s and the N slice ns (tiles_per_wg <= TPW tiles of 64 columns); it walks its blocks, and per block the
// tiles of the slice:
//   dS partial  [128 rows, R]  += dY_tile * B_tile      (per block, over the slice; written once per block)
//   dB partial  [64 cols, R]   += dY_tile^T * S_block    (per tile of the slice, kept in registers over ALL blocks of the
//                                                         chunk; written once per workgroup)
// so dB leaves the chip once per chunk of blocks, not once per block: at rank 64 and N = 28672 the per-block slabs
// were as large as dY itself.  TPW bounds the registers of the dB accumulators (TPW * RT * 4).
// LDS: two dY tiles, the S block [128][R] and two B tiles [64][R] (pitch 2R+32 bytes keeps the 4-row transpose reads on
// distinct banks).  The S block is single-buffered: at a block switch one extra barrier separates its last readers
// from the store of the next block's S (prefetched in registers one tile earlier).
template <typename T, int RT, int TPW>
__global__ void __launch_bounds__(256, RT == 1 ? 3 : RT <= 4 ? 2 : 1)   // waves per SIMD: the register budget follows the LDS footprint
lora_dys_dyb_kernel(const T* __restrict__ dY, const T* __restrict__ S, float* __restrict__ ds_part,
                    float* __restrict__ db_part, int M, int N, int R, int tiles_per_wg, int group, int max_chunks,
                    const LfSegTable seg) {
  constexpr int RP = RT * 32 + 32;
  constexpr int NBR = (64 * RT * 2 + 255) / 256;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* ys = lds;
  char* ss = lds + 2 * TILE_BYTES;
  char* bs = ss + ROWS * RP;

  const int s = blockIdx.x / max_chunks, ch = blockIdx.x % max_chunks, ns = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, qq = lane >> 4, j4 = li >> 2, c4 = li & 3;
  int b0, b1;
  segment_blocks(seg, s, M, b0, b1);
  const int bb0 = b0 + ch * group, bb1 = min(bb0 + group, b1);
  if (bb0 >= b1) return;  // this segment has fewer chunks (uniform for the whole workgroup)
  const int rank = seg.rank[s];
  const T* __restrict__ Bl = (const T*)seg.ptr[s];
  const int Mrows = seg.table ? seg.n_blocks * ROWS : M;
  const int n_begin = ns * tiles_per_wg * 64;
  const int ntiles = min(tiles_per_wg, N / 64 - ns * tiles_per_wg);  // the last slice may be shorter
  const int total = (bb1 - bb0) * ntiles;                             // (block, tile) pairs, block-major

  auto valid_rows = [&](int b) { return seg.table ? seg.table[3 * b + 1] : min(ROWS, M - b * ROWS); };
  auto load_b = [&](lf_u32x4 (&br)[NBR], int n0) {
#pragma unroll
    for (int i = 0; i < NBR; i++) {
      const int g = i * 256 + tid;
      const int row = g / (RT * 2), gc = g % (RT * 2);
      lf_u32x4 v = {0, 0, 0, 0};
      if (g < 64 * RT * 2 && gc * 8 < rank) v = *(const lf_u32x4*)(Bl + (int64_t)(n0 + row) * rank + gc * 8);
      br[i] = v;
    }
  };
  auto store_b = [&](const lf_u32x4 (&br)[NBR], char* dst) {
#pragma unroll
    for (int i = 0; i < NBR; i++) {
      const int g = i * 256 + tid;
      if (g < 64 * RT * 2) *(lf_u32x4*)(dst + (g / (RT * 2)) * RP + (g % (RT * 2)) * 16) = br[i];
    }
  };
  // S block of row block b (rows beyond its valid count as zeros, so they add nothing to dB).  S has R columns; R may
  // be smaller than the RT * 16 columns of the register tiling (R = 48, 80, 96, 112)
  auto load_s = [&](lf_u32x4 (&sr)[RT], int b) {
    const int valid = valid_rows(b);
#pragma unroll
    for (int i = 0; i < RT; i++) {
      const int g = i * 256 + tid;
      const int row = g / (RT * 2), gc = g % (RT * 2);
      lf_u32x4 v = {0, 0, 0, 0};
      if (row < valid && gc * 8 < R) v = *(const lf_u32x4*)(S + (int64_t)(b * ROWS + row) * R + gc * 8);
      sr[i] = v;
    }
  };
  auto store_s = [&](const lf_u32x4 (&sr)[RT]) {
#pragma unroll
    for (int i = 0; i < RT; i++) {
      const int g = i * 256 + tid;
      *(lf_u32x4*)(ss + (g / (RT * 2)) * RP + (g % (RT * 2)) * 16) = sr[i];
    }
  };
  // coordinates of pair q
  auto blk_of = [&](int q) { return bb0 + q / ntiles; };
  auto col_of = [&](int q) { return n_begin + (q % ntiles) * 64; };

  TileRegs tr;
  lf_u32x4 br[NBR], sr[RT];
  tile_load(tr, dY, (const uint8_t*)nullptr, N, bb0 * ROWS, Mrows, n_begin, tid, false, false);
  load_b(br, n_begin);
  load_s(sr, bb0);
  store_s(sr);
  tile_store(tr, ys, tid, false);
  store_b(br, bs);
  if (total > 1) {
    tile_load(tr, dY, (const uint8_t*)nullptr, N, blk_of(1) * ROWS, Mrows, col_of(1), tid, false, false);
    load_b(br, col_of(1));
    if (ntiles == 1) load_s(sr, blk_of(1));
  }
  __syncthreads();

  lf_f32x4 acc_db[TPW][RT];
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int c = 0; c < RT; c++) acc_db[t][c] = lf_f32x4{0.f, 0.f, 0.f, 0.f};

  int q = 0;
  for (int b = bb0; b < bb1; b++) {
    lf_f32x4 acc_ds[2][RT];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int c = 0; c < RT; c++) acc_ds[a][c] = lf_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < TPW; t++) {
      if (t < ntiles) {
        const char* ycur = ys + (q & 1) * TILE_BYTES;
        const char* bcur = bs + (q & 1) * 64 * RP;
        // dS += dY_tile * B_tile : a = dY row fragment, b = B^T through the transpose read
#pragma unroll
        for (int step = 0; step < 2; step++) {
          lf_u32x4 yf[2];
#pragma unroll
          for (int rt = 0; rt < 2; rt++) yf[rt] = tile_row_frag(ycur, wave * 32 + rt * 16 + li, step * 4 + qq);
#pragma unroll
          for (int c = 0; c < RT; c++) {
            const lf_u32x4 bf = tr_read8(bcur + (step * 32 + qq * 8 + j4) * RP + (c * 16 + 4 * c4) * 2, RP);
#pragma unroll
            for (int rt = 0; rt < 2; rt++) acc_ds[rt][c] = Mfma16<T>::run(yf[rt], bf, acc_ds[rt][c]);
          }
        }
        // dB tile: D[n][r] += sum_m dY[m][n] S[m][r]; wave w owns columns 16w..16w+15 of the tile
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
          const int mrow = kk * 32 + qq * 8 + j4;
          const lf_u32x4 yt = tile_tr_frag(ycur, mrow, wave * 16 + 4 * c4);
#pragma unroll
          for (int c = 0; c < RT; c++) {
            const lf_u32x4 sf = tr_read8(ss + mrow * RP + (c * 16 + 4 * c4) * 2, RP);
            acc_db[t][c] = Mfma16<T>::run(yt, sf, acc_db[t][c]);
          }
        }
        if (q + 1 < total) {
          if (t + 1 == ntiles) {  // the next pair opens a new block: everyone is done with this block's S
            __syncthreads();
            store_s(sr);
          }
          tile_store(tr, ys + ((q + 1) & 1) * TILE_BYTES, tid, false);
          store_b(br, bs + ((q + 1) & 1) * 64 * RP);
          if (q + 2 < total) {
            tile_load(tr, dY, (const uint8_t*)nullptr, N, blk_of(q + 2) * ROWS, Mrows, col_of(q + 2), tid, false, false);
            load_b(br, col_of(q + 2));
            if ((q + 2) % ntiles == 0) load_s(sr, blk_of(q + 2));
          }
        }
        __syncthreads();
        q++;
      }
    }
    float* dso = ds_part + (int64_t)ns * Mrows * R;
#pragma unroll
    for (int rt = 0; rt < 2; rt++)
#pragma unroll
      for (int c = 0; c < RT; c++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int row = b * ROWS + wave * 32 + rt * 16 + qq * 4 + e;
          if (row < Mrows && c * 16 < R) dso[(int64_t)row * R + c * 16 + li] = acc_ds[rt][c][e];
        }
  }
  // C layout: column (r) = lane & 15, rows (n) = 4*(lane >> 4) + e
  float* dbo = db_part + (((int64_t)s * max_chunks + ch) * N + n_begin) * R;
#pragma unroll
  for (int t = 0; t < TPW; t++)
    if (t < ntiles) {
#pragma unroll
      for (int c = 0; c < RT; c++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (c * 16 < R) dbo[(int64_t)(t * 64 + wave * 16 + qq * 4 + e) * R + c * 16 + li] = acc_db[t][c][e];
    }
}

// out_s = cast( mult * sum over parts of part[...] ) for segment s = blockIdx.y.
//   transposed == 0 (dB): parts are the segment's chunks, part[(s*max_chunks + ch)][n][R] -> out [rows, rank]
//   transposed == 1 (dA): parts are the segment's chunks, part[(s*max_chunks + ch)][R][rows] -> out [rank, rows]
//   mult_mode 0: segment scale ; 1: 1/(1-p) of the segment ; 2: none (no keep-mask was given: no dropout).
template <typename T>
__device__ __forceinline__ void reduce_segments_body(int bx, int s, const float* __restrict__ part, int rows, int R, int transposed, int mult_mode, int M,
                       int group, int max_chunks, const LfSegTable seg) {
  const int rank = seg.rank[s];
  const int64_t idx = ((int64_t)bx * 256 + threadIdx.x) * 4;  // four consecutive outputs of [rows, rank] or [rank, rows]
  if (idx >= (int64_t)rows * rank) return;
  int b0, b1;
  segment_blocks(seg, s, M, b0, b1);
  float mult;
  if (mult_mode == 2) {
    mult = 1.f;
  } else if (seg.table == nullptr) {
    mult = mult_mode == 0 ? seg.scale : (seg.p > 0.f ? 1.f / (1.f - seg.p) : 1.f);
  } else {
    mult = mult_mode == 0 ? (seg.block_scale ? seg.block_scale[b0] : 1.f)
                          : ((seg.block_p && seg.block_p[b0] > 0.f) ? 1.f / (1.f - seg.block_p[b0]) : 1.f);
  }
  lf_f32x4 v;
  const int nch = (b1 - b0 + group - 1) / group;
  if (!transposed) {
    const int n = (int)(idx / rank), r = (int)(idx % rank);
    v = sum_parts(part + (int64_t)s * max_chunks * rows * R + (int64_t)n * R + r, (int64_t)rows * R, nch);
  } else {
    const int r = (int)(idx / rows), k = (int)(idx % rows);
    v = sum_parts(part + (int64_t)s * max_chunks * R * rows + (int64_t)r * rows + k, (int64_t)R * rows, nch);
  }
  *(lf_u32x2*)((uint16_t*)seg.out[s] + idx) = pack4<T>(v * mult);
}

template <typename T>
__global__ void __launch_bounds__(256)
reduce_segments_kernel(const float* __restrict__ part, int rows, int R, int transposed, int mult_mode, int M,
                       int group, int max_chunks, const LfSegTable seg) {
  reduce_segments_body<T>((int)blockIdx.x, (int)blockIdx.y, part, rows, R, transposed, mult_mode, M, group, max_chunks, seg);
}

// Second stage of dys_dyb in one launch: blocks [0, nb_rows) reduce the dS partials, the rest the
// dB partials (nb_seg blocks per segment).
template <typename T>
__global__ void __launch_bounds__(256)
reduce_ds_db_kernel(const float* __restrict__ ds_part, T* __restrict__ dS, int nparts, int M, int R, int nb_rows,
                    const float* __restrict__ db_part, int N, int nb_seg, int group, int max_chunks, const LfSegTable seg) {
  const int b = blockIdx.x;
  if (b < nb_rows) {
    reduce_rows_body<T>(b, ds_part, dS, nparts, M, R, 1, seg);
  } else {
    const int c = b - nb_rows;
    reduce_segments_body<T>(c % nb_seg, c / nb_seg, db_part, N, R, 0, 0, M, group, max_chunks, seg);
  }
}

// ------------------------------------------------------------------------------------ da
// grid (K/64, max_chunks, n_seg).  Workgroup (kt, ch, s) owns the 64 columns kt*64.. of dA_s and
// the `group` consecutive 128-row blocks ch*group.. of segment s; it accumulates
//   D[r][k] = sum_m dS[m][r] * mask*X[m][k]     (1/(1-p) is applied by the reduce)
// over its blocks and writes one fp32 partial [R][64].  Both operands are read from LDS through
// the transpose path since the contraction index m is the slow dimension of both.
template <typename T, int RT>
__global__ void __launch_bounds__(256)
lora_da_kernel(const T* __restrict__ X, const uint8_t* __restrict__ mask, int mask_bits, const T* __restrict__ dS,
               float* __restrict__ part, int M, int K, int R, int group, int max_chunks, const LfSegTable seg) {
  constexpr int RP = RT * 32 + 32;
  extern __shared__ __attribute__((aligned(16))) char lds[];
  char* xs = lds;
  char* dss = lds + 2 * TILE_BYTES;
  const int kt = blockIdx.x, ch = blockIdx.y, s = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, qq = lane >> 4, j4 = li >> 2, c4 = li & 3;
  int b0, b1;
  segment_blocks(seg, s, M, b0, b1);
  const int bb0 = b0 + ch * group, bb1 = min(bb0 + group, b1);
  if (bb0 >= b1) return;  // this segment has fewer chunks (uniform for the whole workgroup)
  const float p = seg.table ? (seg.block_p ? seg.block_p[b0] : 0.f) : seg.p;
  const bool use_mask = mask != nullptr && p > 0.f;
  const int Mrows = seg.table ? seg.n_blocks * ROWS : M;

  auto valid_rows = [&](int b) { return seg.table ? seg.table[3 * b + 1] : min(ROWS, M - b * ROWS); };
  auto load_ds = [&](lf_u32x4 (&dr)[RT], int b) {
    const int valid = valid_rows(b);
#pragma unroll
    for (int i = 0; i < RT; i++) {
      const int g = i * 256 + tid;
      const int row = g / (RT * 2), gc = g % (RT * 2);
      lf_u32x4 v = {0, 0, 0, 0};
      if (row < valid && gc * 8 < R) v = *(const lf_u32x4*)(dS + (int64_t)(b * ROWS + row) * R + gc * 8);
      dr[i] = v;
    }
  };
  auto store_ds = [&](const lf_u32x4 (&dr)[RT], char* dst) {
#pragma unroll
    for (int i = 0; i < RT; i++) {
      const int g = i * 256 + tid;
      *(lf_u32x4*)(dst + (g / (RT * 2)) * RP + (g % (RT * 2)) * 16) = dr[i];
    }
  };

  TileRegs tr;
  lf_u32x4 dr[RT];
  tile_load(tr, X, mask, K, bb0 * ROWS, Mrows, kt * 64, tid, use_mask, mask_bits != 0);
  load_ds(dr, bb0);
  tile_store(tr, xs, tid, use_mask, mask_bits != 0);
  store_ds(dr, dss);
  if (bb0 + 1 < bb1) {
    tile_load(tr, X, mask, K, (bb0 + 1) * ROWS, Mrows, kt * 64, tid, use_mask, mask_bits != 0);
    load_ds(dr, bb0 + 1);
  }
  __syncthreads();

  lf_f32x4 acc[RT];
#pragma unroll
  for (int c = 0; c < RT; c++) acc[c] = lf_f32x4{0.f, 0.f, 0.f, 0.f};

  for (int b = bb0; b < bb1; b++) {
    const int t = b - bb0;
    const char* xcur = xs + (t & 1) * TILE_BYTES;
    const char* dcur = dss + (t & 1) * ROWS * RP;
#pragma unroll
    for (int kk = 0; kk < 4; kk++) {
      const int mrow = kk * 32 + qq * 8 + j4;
      const lf_u32x4 xt = tile_tr_frag(xcur, mrow, wave * 16 + 4 * c4);
#pragma unroll
      for (int c = 0; c < RT; c++) {
        const lf_u32x4 df = tr_read8(dcur + mrow * RP + (c * 16 + 4 * c4) * 2, RP);
        acc[c] = Mfma16<T>::run(df, xt, acc[c]);
      }
    }
    if (b + 1 < bb1) {
      tile_store(tr, xs + ((t + 1) & 1) * TILE_BYTES, tid, use_mask, mask_bits != 0);
      store_ds(dr, dss + ((t + 1) & 1) * ROWS * RP);
      if (b + 2 < bb1) {
        tile_load(tr, X, mask, K, (b + 2) * ROWS, Mrows, kt * 64, tid, use_mask, mask_bits != 0);
        load_ds(dr, b + 2);
      }
    }
    __syncthreads();
  }
  // C layout: column (k) = lane & 15, rows (r) = 4*(lane >> 4) + e
  float* po = part + ((int64_t)s * max_chunks + ch) * R * K;
#pragma unroll
  for (int c = 0; c < RT; c++)
#pragma unroll
    for (int e = 0; e < 4; e++)
      if (c * 16 < R) po[(int64_t)(c * 16 + qq * 4 + e) * K + kt * 64 + wave * 16 + li] = acc[c][e];  // the partial has R rows
}

// ------------------------------------------------------------------ streaming through a ring of direct-to-LDS loads
// The passes above keep one tile per workgroup in flight (it waits in registers between its load and its LDS store);
// the LDS footprint allows two or three workgroups per CU, so a CU has 32-48 KB on order -- half of what the HBM
// latency asks for, less at rank 64.  The kernels below (ranks up to 64) order their tiles as buffer loads that
// write LDS themselves (no registers, no store instructions), NS - 1 tiles ahead of the one being consumed.
//
// A load group is waited for by count: vector memory operations complete in issue order, so "at most n younger
// operations outstanding" means the group has landed.  The loop therefore contains no other vector memory
// instruction (the compiler would count only its own and wait for everything), issues a group of the same size
// every iteration (past the end: the last tile again, unconsumed), and drains the ring before the workgroup ends.
// Rows past the end of a matrix are not clamped: every tile gets a buffer descriptor that ends where the matrix
// ends, and lanes beyond it read zeros, which add nothing to a sum over rows.
__device__ __forceinline__ uint32_t to_sgpr(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

__device__ __forceinline__ lf_u32x4 window_rsrc(const void* base, int64_t bytes) {
  const uint64_t a = (uint64_t)(uintptr_t)base;
  const int64_t n = bytes > 0xffffffffll ? 0xffffffffll : bytes;   // (never negative: a window starts inside its matrix)
  return lf_u32x4{to_sgpr((uint32_t)a), to_sgpr((uint32_t)(a >> 32)) & 0xffffu, to_sgpr((uint32_t)n), 0x00020000u};
}
// one wave instruction: lane l fetches 16 bytes at window offset `voff` into LDS byte lds_addr + 16 l
__device__ __forceinline__ void dma16(const lf_u32x4& rsrc, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" ::"s"(lds_addr), "v"(voff), "s"(rsrc) : "memory");
}
// one wave instruction: lane l fetches 4 bytes at window offset `voff` into LDS byte lds_addr + 4 l
__device__ __forceinline__ void dma4(const lf_u32x4& rsrc, uint32_t voff, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds" ::"s"(lds_addr), "v"(voff), "s"(rsrc) : "memory");
}
constexpr int da_mask_tile_bytes(int fmt) { return fmt == 1 ? ROWS * 64 : fmt == 2 ? ROWS * 8 : 0; }
template <int N>
__device__ __forceinline__ void wait_vm() { asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory"); }
// at most `groups` groups of G operations each may still be outstanding
template <int G>
__device__ __forceinline__ void wait_groups(int groups) {
  switch (groups) {
    case 0: wait_vm<0>(); break;
    case 1: wait_vm<G>(); break;
    case 2: wait_vm<2 * G>(); break;
    case 3: wait_vm<3 * G>(); break;
    default: wait_vm<4 * G>(); break;
  }
}
__device__ __forceinline__ void ring_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// Per-thread window offsets of a 128-row x 64-column tile of a 16-bit matrix with `ld` elements per row, in the LDS
// layout the fragment readers expect (position p = i*256 + tid: row p>>3, slot p&7 holds granule slot ^ tile_key(row)).
__device__ __forceinline__ void tile_voffs(uint32_t (&v)[4], int64_t ld, int tid) {
  const int srcg = (tid & 7) ^ tile_key(tid >> 3);
#pragma unroll
  for (int i = 0; i < 4; i++) v[i] = (uint32_t)((int64_t)(i * 32 + (tid >> 3)) * ld * 2 + srcg * 16);
}
__device__ __forceinline__ void tile_dma(const lf_u32x4& rsrc, const uint32_t (&v)[4], uint32_t lds_tile, int wave) {
#pragma unroll
  for (int i = 0; i < 4; i++) dma16(rsrc, v[i], lds_tile + i * 4096 + wave * 1024);
}
// keep-mask bytes of the same tile: 128 rows of 64 bytes, row-major (position p = i*256 + tid: row p>>2, 16-byte chunk p&3)
__device__ __forceinline__ void mask_voffs(uint32_t (&v)[2], int64_t ld, int tid) {
#pragma unroll
  for (int i = 0; i < 2; i++) v[i] = (uint32_t)((int64_t)(i * 64 + (tid >> 2)) * ld + (tid & 3) * 16);
}
__device__ __forceinline__ void mask_dma(const lf_u32x4& rsrc, const uint32_t (&v)[2], uint32_t lds_mask, int wave) {
#pragma unroll
  for (int i = 0; i < 2; i++) dma16(rsrc, v[i], lds_mask + i * 4096 + wave * 1024);
}
// keep-mask applied in place to a landed tile (any thread mapping; here each thread takes the positions p = i*256 + tid)
// (BITS: the mask tile holds 8 bytes per row, one bit per element)
template <bool BITS>
__device__ __forceinline__ void tile_apply_mask(char* tile, const char* mtile, int tid) {
  lf_u32x4 x[4];
  lf_u32x2 m[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {   // all reads first: behind a store the compiler would not start the next read
    const int p = i * 256 + tid, row = p >> 3, g = (p & 7) ^ tile_key(row);
    x[i] = *(const lf_u32x4*)(tile + p * 16);
    if constexpr (BITS) m[i] = expand_keep8(*(const uint8_t*)(mtile + row * 8 + g));
    else m[i] = *(const lf_u32x2*)(mtile + row * 64 + g * 8);
  }
#pragma unroll
  for (int i = 0; i < 4; i++) *(lf_u32x4*)(tile + (i * 256 + tid) * 16) = apply_mask8(x[i], m[i]);
}

// A [rows x RT*16] side operand (S or dS block: 128 rows; B tile: 64 rows) in LDS: rows of RT*32 bytes; granule g of
// source row r at slot g ^ side_key(r) of LDS row side_row(r).  A transposed read is served 32 lanes at a time: rows
// j, 8+j (j = 0..3), 32 bytes of each, which must land on eight different 32-byte groups of the 64 banks.  At 128-byte
// rows the key separates (r>>3)&1 and (r>>1)&1 (the row's parity picks the half of the banks); at 64-byte rows
// (r>>3)&1; at 32-byte rows no key can (a row is one group): rows 8..15 of every 16 swap their halves instead.
template <int RT>
__device__ __forceinline__ int side_key(int row) {
  return RT >= 4 ? ((((row >> 3) & 1) << 1) | (((row >> 1) & 1) << 2)) : RT == 2 ? ((row >> 3) & 1) << 1 : 0;
}
template <int RT>
__device__ __forceinline__ int side_row(int row) { return RT == 1 ? row ^ (((row >> 3) & 1) << 2) : row; }
// window offsets of the granules this thread fetches: position p = i*256 + tid -> row p / (2 RT), slot p % (2 RT); a
// granule beyond `cols` columns does not exist in memory: the first one is fetched instead (its products land in
// rank columns that the reduce discards)
template <int RT, int NI>
__device__ __forceinline__ void side_voffs(uint32_t (&v)[NI], int pitch_elems, int cols, int tid) {
#pragma unroll
  for (int i = 0; i < NI; i++) {
    const int p = i * 256 + tid, row = side_row<RT>(p / (RT * 2)), g = (p % (RT * 2)) ^ side_key<RT>(row);   // side_row is its own inverse
    v[i] = (uint32_t)(row * pitch_elems * 2 + (g * 8 < cols ? g : 0) * 16);
  }
}
template <int NI>
__device__ __forceinline__ void side_dma(const lf_u32x4& rsrc, const uint32_t (&v)[NI], uint32_t lds_side, int wave) {
#pragma unroll
  for (int i = 0; i < NI; i++) dma16(rsrc, v[i], lds_side + i * 4096 + wave * 1024);
}
// transposed fragment: rows row..row+3 and row+4..row+7 (row % 8 < 4) of the lane's column among columns c*16 + 4*c4 ..
template <int RT>
__device__ __forceinline__ lf_u32x4 side_tr8(const char* blk, int row, int c, int c4) {
  const int g = c * 2 + (c4 >> 1), within = (c4 & 1) * 8;
  const char* p0 = blk + side_row<RT>(row) * (RT * 32) + ((g ^ side_key<RT>(row)) << 4) + within;
  const char* p1 = blk + side_row<RT>(row + 4) * (RT * 32) + ((g ^ side_key<RT>(row + 4)) << 4) + within;
  lf_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(p0));
  lf_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(p1));
  lf_u32x2 a = __builtin_bit_cast(lf_u32x2, lo), b = __builtin_bit_cast(lf_u32x2, hi);
  return lf_u32x4{a[0], a[1], b[0], b[1]};
}

// ---- da.  grid (n_slices, max_chunks, n_seg).  Workgroup (ks, ch, s): the k-tiles of slice ks (at most TPW, at least
// two: slices are balanced) and the `group` row blocks ch*group.. of segment s; pairs (block, tile) in block-major
// order, the dS block of a row block is fetched once, with the block's first tile, into one of two buffers (a slice
// of nt tiles keeps at most min(NS, nt + 1) stages of the ring busy, so a third block is never on order).
//   D_j[r][k] += sum_m dS[m][r] * keep*X[m][k]   per tile j of the slice, in registers over all blocks of the chunk.
// With a keep-mask the tile is masked in place one iteration before it is consumed.
template <typename T, int RT, int TPW, int NS, int MASK>
__global__ void __launch_bounds__(256, 2)
lora_da_ring_kernel(const T* __restrict__ X, const uint8_t* __restrict__ mask, const T* __restrict__ dS, float* __restrict__ part,
                    int M, int K, int R, int n_slices, int group, int max_chunks, const LfSegTable seg) {
  // MASK: 0 no keep-mask; 1 one byte per element (8 KB per tile, two loads per thread); 2 one bit per element (1 KB per
  // tile, one 4-byte load per thread)
  constexpr int STAGE = TILE_BYTES + da_mask_tile_bytes(MASK);
  constexpr int SIDE = ROWS * RT * 32;
  constexpr int G = 4 + (MASK == 1 ? 2 : MASK == 2 ? 1 : 0);   // operations per load group and thread, not counting a dS block
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  char* ring = lds;
  char* side = lds + NS * STAGE;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const int ks = blockIdx.x, ch = blockIdx.y, s = blockIdx.z;
  const int tid = threadIdx.x, lane = tid & 63, wave = to_sgpr(tid >> 6);
  const int li = lane & 15, qq = lane >> 4, j4 = li >> 2, c4 = li & 3;
  int b0, b1, bb0, bb1;
  segment_blocks(seg, s, M, b0, b1);
  chunk_blocks(b0, b1, group, ch, bb0, bb1);
  if (bb0 >= bb1) return;  // this segment has fewer chunks (uniform for the whole workgroup)
  const float p = seg.table ? (seg.block_p ? seg.block_p[b0] : 0.f) : seg.p;
  const bool use_mask = MASK && mask != nullptr && p > 0.f;
  const int64_t Mrows = seg.table ? (int64_t)seg.n_blocks * ROWS : M;
  const int T64 = K / 64;
  const int kt0 = ks * (T64 / n_slices) + min(ks, T64 % n_slices);
  const int nt = T64 / n_slices + (ks < T64 % n_slices ? 1 : 0);
  const int ns = min(NS, nt + 1);   // stages in use

  uint32_t xv[4], mv[2], dv[RT];
  tile_voffs(xv, K, tid);
  if constexpr (MASK == 2) mv[0] = mv[1] = (uint32_t)((tid >> 1) * (K >> 3) + (tid & 1) * 4);   // row tid>>1, half tid&1 of its 8 bytes
  else mask_voffs(mv, K, tid);
  side_voffs<RT, RT>(dv, R, R, tid);

  // Load group of the next pair into stage `ist`; behind the last pair the last tile is ordered again.  The windows
  // move with the pair (byte pointers and bytes left up to the end of the matrix): a few scalar additions per group.
  int ib = bb0, ij = 0, ist = 0;
  const char* xb = (const char*)(X + (int64_t)bb0 * ROWS * K + (int64_t)kt0 * 64);
  int64_t xleft = (((int64_t)Mrows - (int64_t)bb0 * ROWS) * K - (int64_t)kt0 * 64) * 2;
  const char* sb = (const char*)(dS + (int64_t)bb0 * ROWS * R);
  int64_t sleft = ((int64_t)Mrows - (int64_t)bb0 * ROWS) * R * 2;
  const int64_t xnext = (int64_t)ROWS * K * 2 - (int64_t)nt * 128;   // from behind a block's last tile to the next block's first
  auto issue = [&]() {
    tile_dma(window_rsrc(xb, xleft), xv, lds0 + ist * STAGE, wave);
    if constexpr (MASK == 1) {
      // the mask has one byte where X has two: same element offsets, half the byte offsets
      const int64_t eoff = (xb - (const char*)X) >> 1;
      mask_dma(window_rsrc(mask != nullptr ? (const char*)mask + eoff : (const char*)X, mask != nullptr ? (xleft >> 1) : 0), mv,
               lds0 + ist * STAGE + TILE_BYTES, wave);
    }
    if constexpr (MASK == 2) {
      // one bit where X has sixteen: the tile's 128 rows x 8 bytes land row-major (wave w: rows 32w .. 32w+31)
      const int64_t boff = (xb - (const char*)X) >> 4;
      dma4(window_rsrc(mask != nullptr ? (const char*)mask + boff : (const char*)X, mask != nullptr ? (xleft >> 4) : 0), mv[0],
           lds0 + ist * STAGE + TILE_BYTES + wave * 256);
    }
    if (ij == 0 && ib < bb1) side_dma<RT>(window_rsrc(sb, sleft), dv, lds0 + NS * STAGE + ((ib - bb0) & 1) * SIDE, wave);
    ist = ist + 1 == ns ? 0 : ist + 1;
    if (ib < bb1) {
      if (++ij < nt) {
        xb += 128, xleft -= 128;
      } else if (ib + 1 < bb1) {
        ij = 0, ib++;
        xb += 128 + xnext, xleft -= 128 + xnext;
        sb += ROWS * R * 2, sleft -= ROWS * R * 2;
      } else {
        ib = bb1;   // the cursor stays on the last tile
      }
    }
  };
#pragma unroll 1
  for (int i = 0; i < ns - 1; i++) issue();

  lf_f32x4 acc[TPW][RT];
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int c = 0; c < RT; c++) acc[t][c] = lf_f32x4{0.f, 0.f, 0.f, 0.f};

  int cst = 0;   // stage of the pair being consumed
  if constexpr (MASK) {
    wait_groups<G>(ns - 2);
    ring_barrier();
    if (use_mask) tile_apply_mask<MASK == 2>(ring, ring + TILE_BYTES, tid);
  }
  for (int b = bb0; b < bb1; b++) {
    const char* dcur = side + ((b - bb0) & 1) * SIDE;
    lf_u32x4 df[4][RT];
#pragma unroll
    for (int t = 0; t < TPW; t++) {
      if (t < nt) {
        // MASK: the next pair's group has landed (it is masked during this iteration); else this pair's
        wait_groups<G>(MASK ? ns - 3 : ns - 2);
        ring_barrier();   // ... for every thread; and everyone is done with the previous pair's stage
        issue();
        if constexpr (MASK) {
          const int nst = cst + 1 == ns ? 0 : cst + 1;
          if (use_mask) tile_apply_mask<MASK == 2>(ring + nst * STAGE, ring + nst * STAGE + TILE_BYTES, tid);
        }
        const char* xcur = ring + cst * STAGE;
        // all fragments of the tile first, then the MFMAs: with one or two waves per SIMD nothing else hides the LDS
        // latency, and read-wait-multiply in turns costs a latency per MFMA
        lf_u32x4 xt[4];
        if (t == 0) {   // the dS fragments serve every tile of the block
#pragma unroll
          for (int kk = 0; kk < 4; kk++)
#pragma unroll
            for (int c = 0; c < RT; c++) df[kk][c] = side_tr8<RT>(dcur, kk * 32 + qq * 8 + j4, c, c4);
        }
#pragma unroll
        for (int kk = 0; kk < 4; kk++) xt[kk] = tile_tr_frag(xcur, kk * 32 + qq * 8 + j4, wave * 16 + 4 * c4);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int kk = 0; kk < 4; kk++)
#pragma unroll
          for (int c = 0; c < RT; c++) acc[t][c] = Mfma16<T>::run(df[kk][c], xt[kk], acc[t][c]);
        __builtin_amdgcn_sched_barrier(0);
        cst = cst + 1 == ns ? 0 : cst + 1;
      }
    }
  }
  wait_vm<0>();   // the unconsumed loads behind the last pair must not land in another workgroup's LDS
  // C layout: column (k) = lane & 15, rows (r) = 4*(lane >> 4) + e
  float* po = part + ((int64_t)s * max_chunks + ch) * R * K;
#pragma unroll
  for (int t = 0; t < TPW; t++)
    if (t < nt) {
#pragma unroll
      for (int c = 0; c < RT; c++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (c * 16 < R) po[(int64_t)(c * 16 + qq * 4 + e) * K + (kt0 + t) * 64 + wave * 16 + li] = acc[t][c][e];
    }
}

// ---- dys_dyb.  grid (n_seg * max_chunks, n_slices).  Workgroup (s, ch, ns): the tiles of N slice ns (balanced, 2 .. TPW
// tiles) and chunk ch of segment s (chunks are balanced too); pairs (block, tile) in block-major order.  A load group
// is the dY tile and its B tile [64, rank]; the S block of a row block comes with the block's first tile, into one of
// two buffers.  Per pair:
//   dS partial [128, R] += dY_tile * B_tile      (registers over the slice; stored when the block ends)
//   dB partial [64, R]  += dY_tile^T * S_block    (registers over ALL blocks of the chunk; stored at the end)
// The stores of a block's dS partial are vector memory operations like the loads: the group counts that follow them
// wait for more than they must (the ring runs empty once per block), never for less.
template <typename T, int RT, int TPW, int NS>
__global__ void __launch_bounds__(256, RT >= 4 ? 1 : 2)
lora_dys_dyb_ring_kernel(const T* __restrict__ dY, const T* __restrict__ S, float* __restrict__ ds_part, float* __restrict__ db_part,
                         int M, int N, int R, int n_slices, int group, int max_chunks, const LfSegTable seg) {
  constexpr int NIB = RT >= 2 ? RT / 2 : 1;         // B tile: 64 rows of RT*32 bytes (a 4 KB region at rank 16: all threads fetch)
  constexpr int BT = NIB * 4096;
  constexpr int STAGE = TILE_BYTES + BT;
  constexpr int SIDE = ROWS * RT * 32;
  constexpr int G = 4 + NIB;
  extern __shared__ __attribute__((aligned(1024))) char lds[];
  char* ring = lds;
  char* side = lds + NS * STAGE;
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)lds;
  const int s = blockIdx.x / max_chunks, ch = blockIdx.x % max_chunks, sl = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = to_sgpr(tid >> 6);
  const int li = lane & 15, qq = lane >> 4, j4 = li >> 2, c4 = li & 3;
  int b0, b1, bb0, bb1;
  segment_blocks(seg, s, M, b0, b1);
  chunk_blocks(b0, b1, group, ch, bb0, bb1);
  if (bb0 >= bb1) return;  // this segment has fewer chunks (uniform for the whole workgroup)
  const int rank = seg.rank[s];
  const T* __restrict__ Bl = (const T*)seg.ptr[s];
  const int64_t Mrows = seg.table ? (int64_t)seg.n_blocks * ROWS : M;
  const int T64 = N / 64;
  const int t0 = sl * (T64 / n_slices) + min(sl, T64 % n_slices);
  const int nt = T64 / n_slices + (sl < T64 % n_slices ? 1 : 0);
  const int ns = min(NS, nt + 1);   // stages in use

  uint32_t yv[4], bv[NIB], sv[RT];
  tile_voffs(yv, N, tid);
  side_voffs<RT, NIB>(bv, rank, rank, tid);
  side_voffs<RT, RT>(sv, R, R, tid);

  // Load group of the next pair into stage `ist`; behind the last pair the last tile is ordered again.  The windows
  // move with the pair (byte pointers and bytes left up to the end of the matrix): a few scalar additions per group.
  int ib = bb0, ij = 0, ist = 0;
  const char* yb = (const char*)(dY + (int64_t)bb0 * ROWS * N + (int64_t)t0 * 64);
  int64_t yleft = (((int64_t)Mrows - (int64_t)bb0 * ROWS) * N - (int64_t)t0 * 64) * 2;
  const char* bp = (const char*)(Bl + (int64_t)t0 * 64 * rank);
  int64_t bleft = ((int64_t)N - (int64_t)t0 * 64) * rank * 2;
  const char* sb = (const char*)(S + (int64_t)bb0 * ROWS * R);
  int64_t sleft = ((int64_t)Mrows - (int64_t)bb0 * ROWS) * R * 2;
  const int64_t ynext = (int64_t)ROWS * N * 2 - (int64_t)nt * 128;   // from behind a block's last tile to the next block's first
  const int64_t bstep = (int64_t)64 * rank * 2;
  auto issue = [&]() {
    tile_dma(window_rsrc(yb, yleft), yv, lds0 + ist * STAGE, wave);
    side_dma<NIB>(window_rsrc(bp, bleft), bv, lds0 + ist * STAGE + TILE_BYTES, wave);
    if (ij == 0 && ib < bb1) side_dma<RT>(window_rsrc(sb, sleft), sv, lds0 + NS * STAGE + ((ib - bb0) & 1) * SIDE, wave);
    ist = ist + 1 == ns ? 0 : ist + 1;
    if (ib < bb1) {
      if (++ij < nt) {
        yb += 128, yleft -= 128;
        bp += bstep, bleft -= bstep;
      } else if (ib + 1 < bb1) {
        ij = 0, ib++;
        yb += 128 + ynext, yleft -= 128 + ynext;
        bp -= (nt - 1) * bstep, bleft += (nt - 1) * bstep;
        sb += ROWS * R * 2, sleft -= ROWS * R * 2;
      } else {
        ib = bb1;   // the cursor stays on the last tile
      }
    }
  };
#pragma unroll 1
  for (int i = 0; i < ns - 1; i++) issue();

  lf_f32x4 acc_db[TPW][RT];
#pragma unroll
  for (int t = 0; t < TPW; t++)
#pragma unroll
    for (int c = 0; c < RT; c++) acc_db[t][c] = lf_f32x4{0.f, 0.f, 0.f, 0.f};

  int cst = 0;
  for (int b = bb0; b < bb1; b++) {
    const char* scur = side + ((b - bb0) & 1) * SIDE;
    lf_f32x4 acc_ds[2][RT];
    lf_u32x4 sf[4][RT];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int c = 0; c < RT; c++) acc_ds[a][c] = lf_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int t = 0; t < TPW; t++) {
      if (t < nt) {
        wait_groups<G>(ns - 2);
        ring_barrier();
        issue();
        const char* ycur = ring + cst * STAGE;
        const char* bcur = ycur + TILE_BYTES;
        // All fragments of the tile first, then the MFMAs (one wave per SIMD at rank 64: nothing else hides the LDS
        // latency).  dS += dY_tile * B_tile: a = dY row fragment, b = B^T through the transpose read; dB tile:
        // D[n][r] += sum_m dY[m][n] S[m][r], wave w owns columns 16w..16w+15 of the tile
        lf_u32x4 yf[2][2], bf[2][RT], yt[4];
        if (t == 0) {   // the S fragments serve every tile of the block
#pragma unroll
          for (int kk = 0; kk < 4; kk++)
#pragma unroll
            for (int c = 0; c < RT; c++) sf[kk][c] = side_tr8<RT>(scur, kk * 32 + qq * 8 + j4, c, c4);
        }
#pragma unroll
        for (int step = 0; step < 2; step++) {
#pragma unroll
          for (int rt = 0; rt < 2; rt++) yf[step][rt] = tile_row_frag(ycur, wave * 32 + rt * 16 + li, step * 4 + qq);
#pragma unroll
          for (int c = 0; c < RT; c++) bf[step][c] = side_tr8<RT>(bcur, step * 32 + qq * 8 + j4, c, c4);
        }
#pragma unroll
        for (int kk = 0; kk < 4; kk++) {
          const int mrow = kk * 32 + qq * 8 + j4;
          yt[kk] = tile_tr_frag(ycur, mrow, wave * 16 + 4 * c4);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int step = 0; step < 2; step++)
#pragma unroll
          for (int c = 0; c < RT; c++)
#pragma unroll
            for (int rt = 0; rt < 2; rt++) acc_ds[rt][c] = Mfma16<T>::run(yf[step][rt], bf[step][c], acc_ds[rt][c]);
#pragma unroll
        for (int kk = 0; kk < 4; kk++)
#pragma unroll
          for (int c = 0; c < RT; c++) acc_db[t][c] = Mfma16<T>::run(yt[kk], sf[kk][c], acc_db[t][c]);
        __builtin_amdgcn_sched_barrier(0);
        cst = cst + 1 == ns ? 0 : cst + 1;
      }
    }
    float* dso = ds_part + (int64_t)sl * Mrows * R;
#pragma unroll
    for (int rt = 0; rt < 2; rt++)
#pragma unroll
      for (int c = 0; c < RT; c++)
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int64_t row = (int64_t)b * ROWS + wave * 32 + rt * 16 + qq * 4 + e;
          if (row < Mrows && c * 16 < R) dso[row * R + c * 16 + li] = acc_ds[rt][c][e];
        }
  }
  wait_vm<0>();   // the unconsumed loads behind the last pair must not land in another workgroup's LDS
  // C layout: column (r) = lane & 15, rows (n) = 4*(lane >> 4) + e
  float* dbo = db_part + (((int64_t)s * max_chunks + ch) * N + (int64_t)t0 * 64) * R;
#pragma unroll
  for (int t = 0; t < TPW; t++)
    if (t < nt) {
#pragma unroll
      for (int c = 0; c < RT; c++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          if (c * 16 < R) dbo[(int64_t)(t * 64 + wave * 16 + qq * 4 + e) * R + c * 16 + li] = acc_db[t][c][e];
    }
}

int rt_of(int R) { return R <= 16 ? 1 : R <= 32 ? 2 : R <= 64 ? 4 : 8; }

}  // namespace

static int n_row_blocks(int M, const LfSegTable& seg) { return seg.table ? seg.n_blocks : (M + ROWS - 1) / ROWS; }

// Split of a length-`len` axis into slices (multiples of 64) so that blocks * split fills the
// chip; `min_split` bounds the slice length from above.
// Work split of the streaming passes.  A launch runs in rounds of resident workgroups (LDS-limited
// slots per CU x 256 CUs); a workgroup walks `t` tiles in sequence, so the pass takes about
// rounds * t tile times, plus a little per extra partial sum that the second stage must add.
// Picks the t that minimises that (ties: larger t, fewer partials).  count(t) = workgroups at t.
template <typename Count>
static int pick_tiles_per_wg(int max_t, int slots, Count count) {
  int best = 1;
  double best_cost = 1e30;
  for (int t = 1; t <= max_t; t++) {
    const long wgs = count(t);
    const double cost = (double)((wgs + slots - 1) / slots) * t + 0.15 * (double)wgs / (double)count(max_t);
    if (cost <= best_cost) { best_cost = cost; best = t; }
  }
  return best;
}
static int lds_slots(int smem_bytes) {
  const int per_cu = (160 * 1024) / smem_bytes;
  return 256 * (per_cu > 0 ? per_cu : 1);
}
static int dys_smem(int rt) { return 2 * TILE_BYTES + ROWS * (rt * 32 + 32) + 2 * 64 * (rt * 32 + 32); }
// Shape of a dys_dyb launch: tiles per workgroup (<= the kernel's TPW), row blocks per chunk, chunks of the longest
// segment.  Chosen by bytes moved: the dY stream counted in whole rounds of resident workgroups (a partly filled
// round streams as long as a full one) plus the fp32 partial sums, written by the first stage and read by the second:
// dS partials grow with the number of N slices, dB partials with the number of chunks.
constexpr int dys_tpw(int rt) { return rt <= 2 ? 16 : rt == 4 ? 6 : 4; }   // dB accumulators: TPW * RT * 4 registers, next to 8 * RT of dS
struct DysPlan { int tiles_per_wg, group, max_chunks, nsplit; };
static DysPlan dys_plan(int M, int N, int R, const LfSegTable& seg) {
  const int rt = rt_of(R), T = N / 64, nseg = seg.table ? seg.n_seg : 1;
  const int nblk = n_row_blocks(M, seg);
  const int64_t rows = seg.table ? (int64_t)nblk * ROWS : M;
  int blocks[LF_MAX_SEG];
  for (int s = 0; s < nseg; s++) {
    const int b0 = seg.table ? seg.first_block[s] : 0;
    const int b1 = seg.table ? ((s + 1 < nseg) ? seg.first_block[s + 1] : seg.n_blocks) : nblk;
    blocks[s] = b1 - b0;
  }
  // two workgroups per CU from rank 32 on (registers), else what the LDS footprint allows
  const int slots = rt >= 8 ? 256 : rt >= 2 ? 512 : lds_slots(dys_smem(rt));
  DysPlan best{1, 1, 1, T};
  double best_cost = 1e300;
  for (int t = 1; t <= dys_tpw(rt) && t <= T; t++) {
    const int nsplit = (T + t - 1) / t;
    for (int g = 1; g <= 32; g *= 2) {
      long chunks = 0;
      int max_chunks = 1;
      for (int s = 0; s < nseg; s++) {
        const int c = (blocks[s] + g - 1) / g;
        chunks += c;
        max_chunks = c > max_chunks ? c : max_chunks;
      }
      const long wgs = chunks * nsplit;
      const double rounds = (double)((wgs + slots - 1) / slots);
      const double stream = rounds * slots * g * t * (double)TILE_BYTES;
      const double partial = 2.0 * 4.0 * R * ((double)nsplit * rows + (double)nseg * max_chunks * N);
      const double cost = stream + partial;
      if (cost < best_cost) { best_cost = cost; best = DysPlan{t, g, max_chunks, nsplit}; }
    }
  }
  return best;
}

// ---- work split of the ring kernels.  Workgroups (slice x chunk) of w tiles each run on `slots` resident slots; the
// pass lasts about as long as its busiest slot.  Two upper bounds of that (in tiles): whole rounds of the largest
// workgroup, and the list-scheduling bound sum / slots + largest; the smaller one is the estimate.
struct RingSplit { long wgs; long chunks; int max_chunks; double span; };
static RingSplit ring_split(const int* blocks, int nseg, int g, int T, int nsl, int slots) {
  RingSplit r{0, 0, 1, 0.0};
  const int t_max = (T + nsl - 1) / nsl;
  long total = 0;
  int big = 0;
  for (int s = 0; s < nseg; s++) {
    const int c = (blocks[s] + g - 1) / g;
    if (c <= 0) continue;
    r.chunks += c;
    r.max_chunks = c > r.max_chunks ? c : r.max_chunks;
    const int sz = (blocks[s] + c - 1) / c;
    big = sz > big ? sz : big;
    total += blocks[s];
  }
  r.wgs = r.chunks * nsl;
  const double sum = (double)total * T / slots, largest = (double)big * t_max;
  const double by_rounds = (double)((r.wgs + slots - 1) / slots) * largest, by_list = sum + largest;
  r.span = by_rounds < by_list ? by_rounds : by_list;
  if (r.span < sum) r.span = sum;
  return r;
}
static void seg_block_counts(int M, const LfSegTable& seg, int* blocks, int& nseg) {
  nseg = seg.table ? seg.n_seg : 1;
  for (int s = 0; s < nseg; s++) {
    const int b0 = seg.table ? seg.first_block[s] : 0;
    const int b1 = seg.table ? ((s + 1 < nseg) ? seg.first_block[s + 1] : seg.n_blocks) : (M + ROWS - 1) / ROWS;
    blocks[s] = b1 - b0;
  }
}
static const int kGroups[] = {1, 2, 3, 4, 6, 8, 12, 16, 24, 32, 64};

constexpr int dysr_tpw(int rt) { return rt >= 2 ? 12 : 16; }
constexpr int dysr_ns(int rt) { return rt >= 4 ? 5 : 3; }
static int dysr_smem(int rt) { return dysr_ns(rt) * (TILE_BYTES + (rt >= 2 ? rt / 2 : 1) * 4096) + 2 * ROWS * rt * 32; }
struct DysRingPlan { int n_slices, group, max_chunks; };
// By bytes: the dY (+ B tile) stream over the busiest slot, the S blocks every workgroup fetches (from L2: half weight),
// and the fp32 partials written here and read by the reduce (dS: one [rows, R] slab per slice; dB: one [N, R] slab per
// chunk).
static DysRingPlan dysr_plan(int M, int N, int R, const LfSegTable& seg) {
  const int rt = rt_of(R), T = N / 64;
  int blocks[LF_MAX_SEG], nseg;
  seg_block_counts(M, seg, blocks, nseg);
  const int64_t rows = seg.table ? (int64_t)seg.n_blocks * ROWS : M;
  const int slots = lds_slots(dysr_smem(rt));
  const double tile_bytes = TILE_BYTES + 64.0 * R * 2;
  DysRingPlan best{1, 1, 1};
  if (T < 2) return best;   // fewer than two column tiles: nothing to split (and no division by a zero slice count)
  double best_cost = 1e300;
  for (int t = dysr_tpw(rt); t >= 2; t--) {   // tiles of the longest slice -> fewest slices that reach it
    const int nsl = (T + t - 1) / t;
    if (nsl > T / 2 || (T + nsl - 1) / nsl != t) continue;
    for (int g : kGroups) {
      const RingSplit sp = ring_split(blocks, nseg, g, T, nsl, slots);
      const double cost = sp.span * slots * tile_bytes + 0.5 * (double)sp.wgs * g * ROWS * R * 2 +
                          2.0 * 4.0 * R * ((double)nsl * rows + (double)sp.chunks * N);
      if (cost < best_cost) { best_cost = cost; best = DysRingPlan{nsl, g, sp.max_chunks}; }
    }
  }
  return best;
}

size_t lf_xa_workspace(int, int, int, const LfSegTable&) { return 0; }

template <typename T, int RT>
static int xa_launch(const void* X, const void* U, int64_t ldx, void* act_out, const uint8_t* mask, uint8_t* mask_out, int mask_bits,
                     uint64_t seed, void* S, int M, int K, int R, int64_t rows, const LfSegTable& seg, hipStream_t st) {
  const bool gen = mask_out != nullptr, act = U != nullptr;
  const int wg_rows = xa_rows(RT, act);
  const unsigned grid = (unsigned)((rows + wg_rows - 1) / wg_rows);
  const uint32_t lo = gen ? (uint32_t)seed : 0u, hi = gen ? (uint32_t)(seed >> 32) : 0u;
#define LF_XA(GEN, ACT)                                                                                              \
  return lf_launch((lora_xa_kernel<T, RT, GEN, ACT>), dim3(grid), dim3(xa_waves(RT) * 64), 0, st, (const T*)X,       \
                   (const T*)U, ldx, (T*)act_out, mask, mask_out, mask_bits, lo, hi, (T*)S, M, K, R, seg)
  if (gen && act) LF_XA(true, true);
  if (gen) LF_XA(true, false);
  if (act) LF_XA(false, true);
  LF_XA(false, false);
#undef LF_XA
}

template <typename T>
static int xa_impl(const void* X, const void* U, int64_t ldx, void* act_out, const uint8_t* mask, uint8_t* mask_out, int mask_bits,
                   uint64_t seed, void* S, int M, int K, int R, const LfSegTable& seg, hipStream_t st) {
  const int nblk = n_row_blocks(M, seg);
  const int64_t rows = seg.table ? (int64_t)nblk * ROWS : M;
  switch (rt_of(R)) {
    case 1: return xa_launch<T, 1>(X, U, ldx, act_out, mask, mask_out, mask_bits, seed, S, M, K, R, rows, seg, st);
    case 2: return xa_launch<T, 2>(X, U, ldx, act_out, mask, mask_out, mask_bits, seed, S, M, K, R, rows, seg, st);
    case 4: return xa_launch<T, 4>(X, U, ldx, act_out, mask, mask_out, mask_bits, seed, S, M, K, R, rows, seg, st);
    default: return xa_launch<T, 8>(X, U, ldx, act_out, mask, mask_out, mask_bits, seed, S, M, K, R, rows, seg, st);
  }
}

// mask_out != nullptr: draw the keep-mask from `seed` (written to mask_out [rows, K]) instead of reading `mask`.
// U != nullptr: X and U are the gate and up halves (rows ldx elements apart) and the pass's input
// round16(round16(silu(X)) * U) is written to act_out [rows, K]; otherwise X [rows, K] is dense.
int lf_launch_xa(const void* X, const void* U, int64_t ldx, void* act_out, const uint8_t* mask, uint8_t* mask_out, int mask_bits,
                 uint64_t seed, void* S, int M, int K, int R, const LfSegTable& seg, int dtype, hipStream_t st) {
  if (!X || !S || M <= 0 || K <= 0) return LF_EINVAL;
  if (K % 128 != 0 || R % 16 != 0 || R <= 0 || R > LF_MAX_RANK) return LF_ESHAPE;
  if (seg.table && seg.block_size_m != ROWS) return LF_ESHAPE;
  if (mask_out != nullptr && ((uintptr_t)mask_out & (mask_bits ? 3 : 7)) != 0) return LF_ESHAPE;
  if (U != nullptr) {
    if (!act_out) return LF_EINVAL;
    if (ldx < K || ldx % 8 != 0 || (((uintptr_t)X | (uintptr_t)U | (uintptr_t)act_out) & 15) != 0) return LF_ESHAPE;
  } else {
    ldx = K;
  }
  if (dtype == LF_BF16) return xa_impl<__bf16>(X, U, ldx, act_out, mask, mask_out, mask_bits, seed, S, M, K, R, seg, st);
  if (dtype == LF_F16) return xa_impl<_Float16>(X, U, ldx, act_out, mask, mask_out, mask_bits, seed, S, M, K, R, seg, st);
  return LF_EINVAL;
}

size_t lf_dys_dyb_workspace(int M, int N, int R, const LfSegTable& seg) {
  const int nblk = n_row_blocks(M, seg);
  const int64_t rows = seg.table ? (int64_t)nblk * ROWS : M;
  const int nseg = seg.table ? seg.n_seg : 1;
  if (rt_of(R) <= 4) {
    const DysRingPlan pl = dysr_plan(M, N, R, seg);
    return ((size_t)pl.n_slices * rows * R + (size_t)nseg * pl.max_chunks * N * R) * sizeof(float);
  }
  const DysPlan pl = dys_plan(M, N, R, seg);
  return ((size_t)pl.nsplit * rows * R + (size_t)nseg * pl.max_chunks * N * R) * sizeof(float);
}

template <typename T, int RT>
static int dysr_launch(const void* dY, const void* S, float* ds_part, float* db_part, int M, int N, int R, const DysRingPlan& pl,
                       int nseg, const LfSegTable& seg, hipStream_t st) {
  auto kern = lora_dys_dyb_ring_kernel<T, RT, dysr_tpw(RT), dysr_ns(RT)>;
  const int smem = dysr_smem(RT);
  static LfLdsFlags lds_ok;
  if (!lf_allow_lds(kern, smem, lds_ok)) return LF_ELAUNCH;
  return lf_launch(kern, dim3(nseg * pl.max_chunks, pl.n_slices), dim3(256), smem, st, (const T*)dY, (const T*)S, ds_part, db_part, M, N, R,
                   pl.n_slices, pl.group, pl.max_chunks, seg);
}

template <typename T, int RT>
static int dys_launch(const void* dY, const void* S, float* ds_part, float* db_part, int M, int N, int R, const DysPlan& pl,
                      dim3 grid, const LfSegTable& seg, hipStream_t st) {
  auto kern = lora_dys_dyb_kernel<T, RT, dys_tpw(RT)>;
  const int smem = dys_smem(RT);
  static LfLdsFlags lds_ok;
  if (!lf_allow_lds(kern, smem, lds_ok)) return LF_ELAUNCH;
  return lf_launch(kern, grid, dim3(256), smem, st, (const T*)dY, (const T*)S, ds_part, db_part, M, N, R, pl.tiles_per_wg,
                   pl.group, pl.max_chunks, seg);
}

template <typename T>
static int dys_dyb_impl(const void* dY, const void* S, void* dS, void* ws, int M, int N, int R, const LfSegTable& seg, hipStream_t st) {
  const int nblk = n_row_blocks(M, seg);
  const int64_t rows = seg.table ? (int64_t)nblk * ROWS : M;
  const int nseg = seg.table ? seg.n_seg : 1;
  float* ds_part = (float*)ws;   // [slices][rows][R], then the dB partials [nseg * max_chunks][N][R]
  float* db_part;
  int rc, nparts, group, max_chunks;
  if (rt_of(R) <= 4) {
    const DysRingPlan pl = dysr_plan(M, N, R, seg);
    db_part = ds_part + (int64_t)pl.n_slices * rows * R;
    nparts = pl.n_slices, group = pl.group, max_chunks = pl.max_chunks;
    switch (rt_of(R)) {
      case 1: rc = dysr_launch<T, 1>(dY, S, ds_part, db_part, M, N, R, pl, nseg, seg, st); break;
      case 2: rc = dysr_launch<T, 2>(dY, S, ds_part, db_part, M, N, R, pl, nseg, seg, st); break;
      default: rc = dysr_launch<T, 4>(dY, S, ds_part, db_part, M, N, R, pl, nseg, seg, st); break;
    }
  } else {
    const DysPlan pl = dys_plan(M, N, R, seg);
    db_part = ds_part + (int64_t)pl.nsplit * rows * R;
    nparts = pl.nsplit, group = pl.group, max_chunks = pl.max_chunks;
    rc = dys_launch<T, 8>(dY, S, ds_part, db_part, M, N, R, pl, dim3(nseg * pl.max_chunks, pl.nsplit), seg, st);
  }
  if (rc != LF_OK) return rc;
  const int64_t n = rows * R;
  int maxrank = 0;
  for (int s = 0; s < nseg; s++) maxrank = seg.rank[s] > maxrank ? seg.rank[s] : maxrank;
  const int64_t nout = (int64_t)N * maxrank;
  const int nb_rows = (int)((n + 1023) / 1024), nb_seg = (int)((nout + 1023) / 1024);  // four outputs per thread
  return lf_launch((reduce_ds_db_kernel<T>), dim3((unsigned)(nb_rows + nb_seg * nseg)), dim3(256), 0, st, (const float*)ds_part,
                     (T*)dS, nparts, M, R, nb_rows, (const float*)db_part, N, nb_seg, group, max_chunks, seg);
}

int lf_launch_dys_dyb(const void* dY, const void* S, void* dS, void* ws, size_t ws_bytes, int M, int N, int R,
                      const LfSegTable& seg, int dtype, hipStream_t st) {
  if (!dY || !S || !dS || M <= 0 || N <= 0) return LF_EINVAL;
  if (N % 128 != 0 || R % 16 != 0 || R <= 0 || R > LF_MAX_RANK) return LF_ESHAPE;
  if (seg.table && seg.block_size_m != ROWS) return LF_ESHAPE;
  const int nseg = seg.table ? seg.n_seg : 1;
  for (int s = 0; s < nseg; s++) if (!seg.out[s] || !seg.ptr[s] || seg.rank[s] % 8 != 0 || seg.rank[s] > R) return LF_EINVAL;
  for (int s = 0; s < nseg; s++) if (((uintptr_t)seg.out[s] & 7) != 0) return LF_ESHAPE;  // 8-byte stores of dB
  if (((uintptr_t)dS & 7) != 0) return LF_ESHAPE;
  if (!ws || ws_bytes < lf_dys_dyb_workspace(M, N, R, seg)) return LF_EWORKSPACE;
  if (dtype == LF_BF16) return dys_dyb_impl<__bf16>(dY, S, dS, ws, M, N, R, seg, st);
  if (dtype == LF_F16) return dys_dyb_impl<_Float16>(dY, S, dS, ws, M, N, R, seg, st);
  return LF_EINVAL;
}

// dA chunking: `group` consecutive 128-row blocks of a segment per workgroup, chosen by the same
// round model as the other passes (a segment of b blocks gives ceil(b / group) chunks per K tile).
static int da_smem(int rt) { return 2 * TILE_BYTES + 2 * ROWS * (rt * 32 + 32); }
static void da_shape(int M, int K, int R, const LfSegTable& seg, int& group, int& max_chunks) {
  const int nseg = seg.table ? seg.n_seg : 1;
  int blocks[LF_MAX_SEG];
  int max_blocks = 0;
  for (int s = 0; s < nseg; s++) {
    int b0 = seg.table ? seg.first_block[s] : 0;
    int b1 = seg.table ? ((s + 1 < nseg) ? seg.first_block[s + 1] : seg.n_blocks) : (M + ROWS - 1) / ROWS;
    blocks[s] = b1 - b0;
    max_blocks = blocks[s] > max_blocks ? blocks[s] : max_blocks;
  }
  if (max_blocks < 1) max_blocks = 1;
  group = pick_tiles_per_wg(max_blocks < 16 ? max_blocks : 16, lds_slots(da_smem(rt_of(R))), [&](int g) {
    long chunks = 0;
    for (int s = 0; s < nseg; s++) chunks += (blocks[s] + g - 1) / g;
    return (long)(K / 64) * chunks;
  });
  max_chunks = (max_blocks + group - 1) / group;
  if (max_chunks < 1) max_chunks = 1;
}

// Ring kernel shapes by rank tiles: tiles per slice (registers: TPW * RT * 4 accumulators) and ring depth (LDS: NS
// stages of 16 KB, 24 KB with a keep-mask, plus two dS blocks of RT * 4 KB; two workgroups per CU where that fits).
constexpr int da_tpw(int rt) { return rt >= 4 ? 8 : 16; }
constexpr int da_ns(int rt, int maskfmt) { return maskfmt ? (rt == 1 ? 3 : 5) : (rt == 4 ? 3 : 4); }
static int da_ring_smem(int rt, int maskfmt) { return da_ns(rt, maskfmt) * (TILE_BYTES + da_mask_tile_bytes(maskfmt)) + 2 * ROWS * rt * 32; }
struct DaPlan { int n_slices, group, max_chunks; };
// Slices of the K axis (balanced, 2 .. TPW tiles each) x chunks of `group` row blocks per segment, by bytes moved: the
// X stream in whole rounds of resident workgroups, the dS blocks every workgroup fetches, and the fp32 partials
// (one [R, K] slab per chunk, written here and read by the reduce).
static DaPlan da_plan(int M, int K, int R, int maskfmt, const LfSegTable& seg) {
  const int rt = rt_of(R), T = K / 64;
  int blocks[LF_MAX_SEG], nseg;
  seg_block_counts(M, seg, blocks, nseg);
  const int slots = lds_slots(da_ring_smem(rt, maskfmt));
  const double tile_bytes = TILE_BYTES + da_mask_tile_bytes(maskfmt);
  DaPlan best{1, 1, 1};
  if (T < 2) return best;   // as in dysr_plan
  double best_cost = 1e300;
  for (int t = da_tpw(rt); t >= 2; t--) {   // tiles of the longest slice -> fewest slices that reach it
    const int nsl = (T + t - 1) / t;
    if (nsl > T / 2 || (T + nsl - 1) / nsl != t) continue;
    for (int g : kGroups) {
      const RingSplit sp = ring_split(blocks, nseg, g, T, nsl, slots);
      const double cost = sp.span * slots * tile_bytes + 0.5 * (double)sp.wgs * g * ROWS * R * 2 + 2.0 * 4.0 * R * K * (double)sp.chunks;
      if (cost < best_cost) { best_cost = cost; best = DaPlan{nsl, g, sp.max_chunks}; }
    }
  }
  return best;
}

size_t lf_da_workspace(int M, int K, int R, const LfSegTable& seg) {
  const int nseg = seg.table ? seg.n_seg : 1;
  int max_chunks;
  if (rt_of(R) <= 4) {
    // the launch plans with or without a keep-mask (one byte or one bit per element): room for any
    const int a = da_plan(M, K, R, 1, seg).max_chunks, b = da_plan(M, K, R, 0, seg).max_chunks, c = da_plan(M, K, R, 2, seg).max_chunks;
    max_chunks = a > b ? a : b;
    max_chunks = c > max_chunks ? c : max_chunks;
  } else {
    int group;
    da_shape(M, K, R, seg, group, max_chunks);
  }
  return (size_t)nseg * max_chunks * R * K * sizeof(float);
}

template <typename T, int RT>
static int da_launch(const void* X, const uint8_t* mask, int mask_bits, const void* dS, float* part, int M, int K, int R, int group,
                     int max_chunks, dim3 grid, const LfSegTable& seg, hipStream_t st) {
  auto kern = lora_da_kernel<T, RT>;
  constexpr int RP = RT * 32 + 32;
  const int smem = 2 * TILE_BYTES + 2 * ROWS * RP;
  static LfLdsFlags lds_ok;
  if (!lf_allow_lds(kern, smem, lds_ok)) return LF_ELAUNCH;
  return lf_launch(kern, grid, dim3(256), smem, st, (const T*)X, mask, mask_bits, (const T*)dS, part, M, K, R, group, max_chunks, seg);
}

template <typename T, int RT, int MASK>
static int da_ring_launch(const void* X, const uint8_t* mask, const void* dS, float* part, int M, int K, int R, const DaPlan& pl,
                          int nseg, const LfSegTable& seg, hipStream_t st) {
  auto kern = lora_da_ring_kernel<T, RT, da_tpw(RT), da_ns(RT, MASK), MASK>;
  const int smem = da_ring_smem(RT, MASK);
  static LfLdsFlags lds_ok;
  if (!lf_allow_lds(kern, smem, lds_ok)) return LF_ELAUNCH;
  return lf_launch(kern, dim3(pl.n_slices, pl.max_chunks, nseg), dim3(256), smem, st, (const T*)X, mask, (const T*)dS, part, M, K, R,
                   pl.n_slices, pl.group, pl.max_chunks, seg);
}

template <typename T>
static int da_impl(const void* X, const uint8_t* mask, int mask_bits, const void* dS, void* ws, int M, int K, int R, const LfSegTable& seg, hipStream_t st) {
  const int nseg = seg.table ? seg.n_seg : 1;
  float* part = (float*)ws;
  int group, max_chunks, rc;
  if (rt_of(R) <= 4) {
    const int fmt = mask == nullptr ? 0 : mask_bits ? 2 : 1;
    const DaPlan pl = da_plan(M, K, R, fmt, seg);
    group = pl.group;
    max_chunks = pl.max_chunks;
#define LF_DA_RING(RTV)                                                                                                   \
  rc = fmt == 2   ? da_ring_launch<T, RTV, 2>(X, mask, dS, part, M, K, R, pl, nseg, seg, st)                              \
       : fmt == 1 ? da_ring_launch<T, RTV, 1>(X, mask, dS, part, M, K, R, pl, nseg, seg, st)                              \
                  : da_ring_launch<T, RTV, 0>(X, mask, dS, part, M, K, R, pl, nseg, seg, st)
    switch (rt_of(R)) {
      case 1: LF_DA_RING(1); break;
      case 2: LF_DA_RING(2); break;
      default: LF_DA_RING(4); break;
    }
#undef LF_DA_RING
  } else {
    da_shape(M, K, R, seg, group, max_chunks);
    rc = da_launch<T, 8>(X, mask, mask_bits, dS, part, M, K, R, group, max_chunks, dim3(K / 64, max_chunks, nseg), seg, st);
  }
  if (rc != LF_OK) return rc;
  int maxrank = 0;
  for (int s = 0; s < nseg; s++) maxrank = seg.rank[s] > maxrank ? seg.rank[s] : maxrank;
  const int64_t nout = (int64_t)K * maxrank;
  return lf_launch((reduce_segments_kernel<T>), dim3((unsigned)((nout + 1023) / 1024), nseg), dim3(256), 0, st, (const float*)part, K, R, 1, mask != nullptr ? 1 : 2, M, group, max_chunks, seg);
}

int lf_launch_da(const void* X, const uint8_t* mask, int mask_bits, const void* dS, void* ws, size_t ws_bytes, int M, int K, int R,
                 const LfSegTable& seg, int dtype, hipStream_t st) {
  if (!X || !dS || M <= 0 || K <= 0) return LF_EINVAL;
  if (K % 128 != 0 || R % 16 != 0 || R <= 0 || R > LF_MAX_RANK) return LF_ESHAPE;
  if (seg.table && seg.block_size_m != ROWS) return LF_ESHAPE;
  const int nseg = seg.table ? seg.n_seg : 1;
  for (int s = 0; s < nseg; s++) if (!seg.out[s] || seg.rank[s] % 8 != 0 || seg.rank[s] > R) return LF_EINVAL;
  for (int s = 0; s < nseg; s++) if (((uintptr_t)seg.out[s] & 7) != 0) return LF_ESHAPE;  // 8-byte stores of dA
  if (!ws || ws_bytes < lf_da_workspace(M, K, R, seg)) return LF_EWORKSPACE;
  if (mask != nullptr && mask_bits && ((uintptr_t)mask & 3) != 0) return LF_ESHAPE;   // 4-byte loads of the keep bits
  if (dtype == LF_BF16) return da_impl<__bf16>(X, mask, mask_bits, dS, ws, M, K, R, seg, st);
  if (dtype == LF_F16) return da_impl<_Float16>(X, mask, mask_bits, dS, ws, M, K, R, seg, st);
  return LF_EINVAL;
}

