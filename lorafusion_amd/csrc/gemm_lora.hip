// MFMA GEMM with a LoRA term seeded into the accumulator, for gfx950 (MI355X).
//
//   C[M,N] = A[M,K] * op(B) + mult * (L[M,R] * Rop) (+ bias)
//
// NT (forward,  Y  = X W^T + scale * S B^T + bias):  B = W [N,K], Rop rows = B_lora [N,rank]
// NN (backward, dX = dY W + mask * (dS A)/(1-p)):     B = W [K,N] (W is [N_out,K_in] and the
//     contraction runs over N_out), Rop = A_lora [rank, N]
//
// This replaces the Triton kernels fused_lora_xw_sb / fused_multi_lora_xw_sb
// (lorafusion/ops/triton_ops/fused_lora_xw_sb.py:74-206, fused_multi_lora_xw_sb.py:66-218) and
// fused_lora_dyw_dsa / fused_multi_lora_dyw_dsa (fused_lora_dyw_dsa.py:69-181,
// fused_multi_lora_dyw_dsa.py:60-185).  As there, the accumulator starts from the LoRA product
// and the dense K-loop adds on top of it in fp32.
//
// Structure: one workgroup per BMxBN tile, 64-wide wavefronts each owning a WMxWN sub-tile of
// 16x16x32 MFMA blocks (under the power limit of the chip this shape sustains about 10 % more
// than 32x32x16: 2.13 vs 1.93 PFLOP/s in a register-only loop with random operands).  The K loop advances in steps of BK = 32 through a ring of NSTAGE LDS
// stages; both operand tiles go global -> LDS with 16-byte direct-to-LDS buffer loads (no VGPR
// staging, no vector ALU address work: the per-lane row offset is loop invariant and the K
// position is a scalar offset).  NSTAGE-1 stages of loads are in flight while one stage is
// consumed: with a single stage in flight the tile round trip under MFMA load (about twice
// the unloaded one) is longer than the MFMA time of a K step and every step stalls on it
// (measured: 1.18 -> 1.5 PFLOP/s on a loads+MFMA skeleton when a second stage may stay in
// flight).  LDS rows are 64 bytes (4 granules of 16 bytes); granule g of row r is stored at
// slot g ^ ((r>>1)&3).  A ds_read_b128 is served 16 lanes at a time, and the lanes served
// together are {0-3, 12-15, 20-27} and {4-11, 16-19, 28-31} of each half wave (probed on
// hardware): with this swizzle each such set (rows 0-3 and 12-15 of one granule column, rows
// 4-11 of the next) touches all 64 banks exactly once.  The swizzle is applied on the global
// side of the direct load (each lane fetches the granule whose LDS slot it owns).
// The NN operand is stored untransposed and read with ds_read_b64_tr_b16, which hands each
// lane four consecutive contraction elements of its column.  MFMA operands are swapped (B
// fragment as the "a" operand) so each lane ends with four consecutive output columns of one
// row.
#include "lf_common.h"
#include <algorithm>
#include <type_traits>

namespace {

constexpr int BK = 32;
#ifndef LF_STAG
#define LF_STAG 15
#endif
#ifndef LF_NSTAGE_SMALL
#define LF_NSTAGE_SMALL 10
#endif
#ifndef LF_NSTAGE
#define LF_NSTAGE 5
#endif
#ifndef LF_MEMPHASE_LOADS
#define LF_MEMPHASE_LOADS 1
#endif

template <typename T> struct MfmaOp;
template <> struct MfmaOp<__bf16> {
  static __device__ __forceinline__ lf_f32x4 run(lf_u32x4 a, lf_u32x4 b, lf_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(lf_bf16x8, a), __builtin_bit_cast(lf_bf16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    bf2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  static __device__ __forceinline__ float to_float(uint16_t bits) { return __builtin_bit_cast(float, (uint32_t)bits << 16); }
};
template <> struct MfmaOp<_Float16> {
  static __device__ __forceinline__ lf_f32x4 run(lf_u32x4 a, lf_u32x4 b, lf_f32x4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(lf_f16x8, a), __builtin_bit_cast(lf_f16x8, b), c, 0, 0, 0);
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  static __device__ __forceinline__ float to_float(uint16_t bits) { return (float)__builtin_bit_cast(_Float16, bits); }
};

typedef __attribute__((address_space(3))) void* lds_ptr_t;
typedef const __attribute__((address_space(1))) void* gbl_ptr_t;

__device__ __forceinline__ void load_g2l_16(const void* g, char* lds_wave_base) {
  // 16 bytes per lane, global -> LDS; the LDS destination is lds_wave_base + lane*16.
  __builtin_amdgcn_global_load_lds((gbl_ptr_t)g, (lds_ptr_t)lds_wave_base, 16, 0, 0);
}

// ds_read_b64_tr_b16 as inline assembly: through the builtin the compiler cannot tell the read
// from the direct-to-LDS loads still in flight and puts s_waitcnt vmcnt(0) in front of it, which
// serialises the whole load ring.  The result is valid only after a later s_waitcnt lgkmcnt(0)
// (the main loop has one before every barrier).
__device__ __forceinline__ lf_u32x2 lds_read_tr16(const char* p) {
  lf_u32x2 v;
  const uint32_t a = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
  asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(v) : "v"(a) : "memory");
  return v;
}

template <typename T, int BM, int BN, int WM, int WN, bool NN, int NSTAGE>
__global__ void __launch_bounds__((BM / WM) * (BN / WN) * 64, 1)
gemm_lora_kernel(const LfGemmParams p, const LfSegTable seg) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub (buffer-resource types are device-only)
  constexpr int NWM = BM / WM, NWN = BN / WN, NWAVES = NWM * NWN, NTHREADS = NWAVES * 64;
  constexpr int TM = WM / 16, TN = WN / 16;  // 16x16 accumulator blocks per wave
  static_assert(WM % 32 == 0 && WN % 32 == 0, "sub-tile shape");
  constexpr int A_STAGE = BM * BK * 2, B_STAGE = BN * BK * 2;
  constexpr int NLA = BM * 4 / NTHREADS;  // 16-byte loads per thread per A tile (rows of 4 granules)
  constexpr int NLB = BN * 4 / NTHREADS;
  static_assert(NLA >= 1 && NLB >= 1 && (NTHREADS / 4) % 16 == 0, "tile/thread shape");
  constexpr int GPR = BN / 8;             // NN: granules per LDS row of the B tile
  constexpr int BPITCH = BN * 2;          // NN: bytes per LDS row of the B tile
  constexpr int BKEY = BPITCH / 32 >= 8 ? 7 : BPITCH / 32 - 1;  // NN: swizzle key mask over 32-byte units

  extern __shared__ __attribute__((aligned(1024))) char smem[];
  char* ldsA = smem;
  char* ldsB = smem + NSTAGE * A_STAGE;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / NWN, wn = wave % NWN;
  const int l16 = lane & 15, kg = lane >> 4;  // row / column within a 16x16 block, group of 8 contraction elements

  // ---- tile mapping: XCD-aware (consecutive tiles stay on one XCD's L2) + grouped along M
  int pid = blockIdx.x;
  const int total = p.grid_m * p.grid_n;
  if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
  constexpr int GROUP_M = 8;
  const int width = GROUP_M * p.grid_n;
  const int group = pid / width;
  const int first_m = group * GROUP_M;
  const int gsz = min(p.grid_m - first_m, GROUP_M);
  const int pid_m = first_m + (pid % width) % gsz;
  const int pid_n = (pid % width) / gsz;
  const int m0 = pid_m * BM, n0 = pid_n * BN;

  // ---- staggered start of the K loop: workgroups that run side by side walk K from different
  // offsets (one 128-byte step apart) so their tile loads spread over the memory channels
  // instead of all hitting the same channel when the row pitch is a power of two.  The offset
  // depends on the tile column only: the tiles of a column, which stream the same B panel and
  // run on one XCD, stay aligned in K and meet each other's lines in the L2 (1.5 % faster at
  // 8192x4096x4096 than an offset by row + column).
  // (split contraction: this workgroup's share of the K steps is [kbeg, kbeg + nk); an even count, like K / BK)
  const int kbeg = p.ksplit > 1 ? (int)blockIdx.y * p.ks_steps : 0;
  const int nk = p.ksplit > 1 ? min(p.ks_steps, p.K / BK - kbeg) : p.K / BK;
  const int kstart = (2 * (pid_n & LF_STAG)) % nk;

  // ---- direct-to-LDS buffer loads: per thread one 32-bit byte offset per 16-byte granule (row part,
  // clamped at the matrix edge); the K position of a tile is a scalar offset shared by the wave.
  // The buffer of an operand with K-contiguous rows starts at the tile's first row, so the 32-bit
  // offsets span one panel of the tile and the operand itself may exceed 2 GiB.
  const char* a_base = (const char*)p.A + (int64_t)m0 * p.lda * 2;
  const char* b_base = NN ? (const char*)p.B : (const char*)p.B + (int64_t)n0 * p.ldb * 2;
  const __amdgpu_buffer_rsrc_t rsrcA = __builtin_amdgcn_make_buffer_rsrc((void*)a_base, 0, 0x7fffffff, 0x00020000);
  const __amdgpu_buffer_rsrc_t rsrcB = __builtin_amdgcn_make_buffer_rsrc((void*)b_base, 0, 0x7fffffff, 0x00020000);
  uint32_t avoff[NLA], bvoff[NLB];
  {
    // LDS slot (tid&3) of row r holds source granule slot ^ ((r>>1)&3); r>>1 = tid>>3 (mod 4)
    const int srcg = (tid & 3) ^ ((tid >> 3) & 3);
#pragma unroll
    for (int i = 0; i < NLA; i++) {
      int row = i * (NTHREADS / 4) + (tid >> 2);
      int gm = min(m0 + row, p.M - 1) - m0;  // row within the tile, clamped at the matrix edge
      avoff[i] = (uint32_t)((int64_t)gm * p.lda * 2 + srcg * 16);
    }
    if constexpr (!NN) {
#pragma unroll
      for (int i = 0; i < NLB; i++) {
        int row = i * (NTHREADS / 4) + (tid >> 2);
        int gn = min(n0 + row, p.N - 1) - n0;
        bvoff[i] = (uint32_t)((int64_t)gn * p.ldb * 2 + srcg * 16);
      }
    } else {
#pragma unroll
      for (int i = 0; i < NLB; i++) {
        // 32-byte unit u of LDS row r holds source unit u ^ key(r), key(r) = (r&3)*2 + ((r>>3)&1): the
        // 8 rows that 32 lanes of a transposed read touch (r, r+8 for four consecutive r) then cover
        // all 64 banks.  Rows of 128 bytes (64-column tiles) hold four units and their parity already
        // picks the half of the banks: there key(r) = ((r>>1)&1)*2 + ((r>>3)&1) separates the four
        // rows of one parity (the general key, cut to two bits, left two of them on the same unit)
        int gid = i * NTHREADS + tid;
        int row = gid / GPR, g = gid % GPR;
        int srcunit = (g >> 1) ^ (BPITCH == 128 ? ((((row >> 1) & 1) << 1) | ((row >> 3) & 1))
                                                : ((((row & 3) << 1) | ((row >> 3) & 1)) & BKEY));
        int col = min(n0 + (srcunit * 2 + (g & 1)) * 8, p.N - 8);
        bvoff[i] = (uint32_t)((int64_t)row * p.ldb * 2 + col * 2);
      }
    }
  }

  constexpr int NL = NLA + NLB;  // loads per thread per K step
  auto issue_loads = [&](int stage, int tile) {
    char* la = ldsA + stage * A_STAGE + wave * 1024;
    char* lb = ldsB + stage * B_STAGE + wave * 1024;
    int kt_pos = kstart + tile;
    if (kt_pos >= nk) kt_pos -= nk;
    kt_pos += kbeg;
    const int a_soff = kt_pos * (BK * 2);
    const int b_soff = NN ? kt_pos * BK * (int)p.ldb * 2 : a_soff;
#pragma unroll
    for (int i = 0; i < NLA; i++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, (lds_ptr_t)(la + i * NTHREADS * 16), 16, avoff[i], a_soff, 0, 0);
#pragma unroll
    for (int i = 0; i < NLB; i++)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcB, (lds_ptr_t)(lb + i * NTHREADS * 16), 16, bvoff[i], b_soff, 0, 0);
  };
  // one of the NL loads of a step (idx < NLA: operand A)
  auto issue_load_one = [&](int stage, int tile, int idx) {
    int kt_pos = kstart + tile;
    if (kt_pos >= nk) kt_pos -= nk;
    kt_pos += kbeg;
    const int a_soff = kt_pos * (BK * 2);
    if (idx < NLA) {
      char* la = ldsA + stage * A_STAGE + wave * 1024;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcA, (lds_ptr_t)(la + idx * NTHREADS * 16), 16, avoff[idx < NLA ? idx : 0], a_soff, 0, 0);
    } else {
      const int i = idx - NLA;
      char* lb = ldsB + stage * B_STAGE + wave * 1024;
      const int b_soff = NN ? kt_pos * BK * (int)p.ldb * 2 : a_soff;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrcB, (lds_ptr_t)(lb + i * NTHREADS * 16), 16, bvoff[i >= 0 && i < NLB ? i : 0], b_soff, 0, 0);
    }
  };
  // s_waitcnt vmcnt(n) with the other counters untouched (vmcnt = bits 3:0 and 15:14): wait until
  // at most STEPS whole K steps of this thread's loads are outstanding
  auto wait_loads = [&](auto STEPS) {
    constexpr int n = STEPS.value * NL;
    static_assert(n >= 0 && n < 64, "vmcnt is a 6-bit counter");
    __builtin_amdgcn_s_waitcnt(0x0f70 | (n & 15) | ((n >> 4) << 14));
  };
  using std::integral_constant;
  using Steps0 = integral_constant<int, 0>;

  lf_f32x4 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++) acc[i][j] = lf_f32x4{0.f, 0.f, 0.f, 0.f};

  // K steps are loaded in pairs (2T, 2T+1): the two 64-byte halves of the same 128-byte lines,
  // issued back to back so that the second request for a line meets the first in the L1 instead
  // of fetching the line from L2 again a step later (half the L2 read requests; 1.25 -> 1.35
  // PFLOP/s at 8192x4096x4096, at a higher clock: the kernel is power limited).  PAIR0 = steps
  // issued before the loop.
  constexpr int PAIR0 = (NSTAGE - 1) & ~1;
  auto issue_first_tiles = [&]() {
#pragma unroll
    for (int t = 0; t < PAIR0; t++)
      if (t < nk) issue_loads(t, t);
  };

  // ---- LoRA term seeds the accumulator.  Its loads go out ahead of the first tile loads: the
  // term needs two dependent round trips (routing table, then the operands) where the tiles need
  // one, and behind PAIR0 stages of tile loads in the texture addresser it would start a
  // microsecond late; the seeding MFMAs then run while the tiles land.
  const int wrow0 = m0 + wm * WM;  // first row of this wave's sub-tile
  if (p.L == nullptr || wrow0 >= p.M || kbeg != 0) {   // (split contraction: the first slice carries the term)
    issue_first_tiles();
  } else {
    const T* __restrict__ L = (const T*)p.L;
    const T* rp = (const T*)seg.ptr[0];
    int rank = seg.rank[0];
    // mult_mode 1 without a keep-mask means no dropout, whatever p says: the term is not rescaled
    bool use_mask = p.mask != nullptr && p.mult_mode == 1 && seg.p > 0.f;
    float mult = p.mult_mode == 0 ? seg.scale : (use_mask ? 1.f / (1.f - seg.p) : 1.f);
    if (seg.table != nullptr) {
      int blk = (p.row0 + wrow0) / seg.block_size_m;
      blk = min(blk, seg.n_blocks - 1);
      rank = seg.table[3 * blk + 0];
      int fb = seg.table[3 * blk + 2];
      int s = 0;
      for (int i = 1; i < seg.n_seg; i++) s = (seg.first_block[i] == fb) ? i : s;
      rp = (const T*)seg.ptr[s];
      if (p.mult_mode == 0) {
        mult = seg.block_scale[blk];
      } else {
        float pb = seg.block_p[blk];
        use_mask = p.mask != nullptr && pb > 0.f;
        mult = use_mask ? 1.f / (1.f - pb) : 1.f;
      }
    }
    // Keep-mask of this wave's sub-tile: 16-byte loads that cover whole rows of the sub-tile (issued
    // here so that their latency overlaps the seeding MFMAs), handed to the lanes that own the
    // accumulator elements through the wave's slice of the last ring stage, which no tile load
    // targets before the main loop.  Granule g of row r sits at slot g ^ ((r / MRW) & (MLPR-1)):
    // the 4-byte reads of 32 rows then spread over the banks (2-way instead of 16-way conflicts).
    constexpr int MLPR = WN / 16, MRPI = 64 / MLPR, MNI = 32 / MRPI, MRW = 256 / WN;
    constexpr int TM32 = WM / 32;  // 32-row bands of the sub-tile
    static_assert(NWM == 2 && MNI >= 1, "mask staging: 32 rows x WN bytes per wave fit B_STAGE / NWAVES");
    char* mreg = ldsB + (NSTAGE - 1) * B_STAGE + wave * (B_STAGE / NWAVES);
    const int mrow = lane / MLPR, mg = lane % MLPR;
    constexpr bool MEARLY = TM32 * MNI <= 8 && TM * TN <= 16;  // all mask loads up front while they fit next to the operands of a chunk
    lf_u32x4 mv[TM32][MNI];
    const int mcol = min(n0 + wn * WN + mg * 16, p.N - 16);
    auto load_mask_band = [&](int ib) {
#pragma unroll
      for (int ii = 0; ii < MNI; ii++) {
        const int gm = min(wrow0 + ib * 32 + ii * MRPI + mrow, p.M - 1);
        mv[ib][ii] = *(const lf_u32x4*)(p.mask + (int64_t)gm * p.ldmask + mcol);
      }
    };
    // (a bit-packed mask is read directly, one dword per accumulator block pair, below: these tiles serve short
    // row ranges and small shapes, where its few bytes come from L2)
    const bool bytes_mask = use_mask && !p.mask_bits, bits_mask = use_mask && p.mask_bits;
    if (bytes_mask && MEARLY) {
#pragma unroll
      for (int ib = 0; ib < TM32; ib++) load_mask_band(ib);
    }
    const __amdgpu_buffer_rsrc_t rsrcR = __builtin_amdgcn_make_buffer_rsrc((void*)rp, 0, 0x7fffffff, 0x00020000);
    // Bit-packed keep-mask: the dword that holds the lane's four columns of each accumulator block (element n of a
    // mask row = bit n & 7 of byte n >> 3).  Requested with the operands of the first chunk where the registers allow
    // (up to 16 blocks per wave), else in one batch behind the MFMAs.
    constexpr int GI = TM * TN <= 16 ? TM : (16 / TN > 0 ? 16 / TN : 1);   // block rows per batch of mask words
    constexpr bool BITS_EARLY = GI == TM;
    static_assert(TM % GI == 0, "whole batches");
    uint32_t mw[GI][TN];
    auto load_bits = [&](int i0) {
#pragma unroll
      for (int i = 0; i < GI; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) {
          const int gm = min(wrow0 + (i0 + i) * 16 + l16, p.M - 1);
          const int col0 = min(n0 + wn * WN + j * 16 + kg * 4, p.N - 4);
          mw[i][j] = *(const uint32_t*)(p.mask + (int64_t)gm * p.ldmask + ((col0 >> 5) << 2)) >> (col0 & 31);
        }
    };
    // one MFMA k-step covers 32 rank columns; lanes whose 8 columns lie beyond R (or the rank) feed zeros.
    // All loads of a chunk are requested before the first is used (the conditions sit outside the loops over the
    // fragments): the term costs one memory round trip per chunk, not one per fragment -- with a branch and a wait
    // per fragment the NN seed of a 128x256 tile took 17 us of an 80 us launch.
    for (int t = 0; t < (p.R + 31) / 32; t++) {
      const int r0 = t * 32 + kg * 8;
      lf_u32x4 rf[TN], lf[TM];
      uint32_t e[NN ? TN : 1][8];
#pragma unroll
      for (int j = 0; j < TN; j++) rf[j] = lf_u32x4{0, 0, 0, 0};
#pragma unroll
      for (int i = 0; i < TM; i++) lf[i] = lf_u32x4{0, 0, 0, 0};
      if (r0 < rank) {
#pragma unroll
        for (int j = 0; j < TN; j++) {
          const int gn = min(n0 + wn * WN + j * 16 + l16, p.N - 1);
          if constexpr (!NN) {
            rf[j] = *(const lf_u32x4*)(rp + (int64_t)gn * rank + r0);
          } else {
            // eight rows of one column: buffer loads that share a per-lane offset (row kg*8 of the
            // step, column gn) and take the row as a scalar offset, so the 8 x TN loads in flight
            // need no address registers of their own
            const uint32_t voff = (uint32_t)((kg * 8 * p.N + gn) * 2);
#pragma unroll
            for (int k = 0; k < 8; k++) e[j][k] = __builtin_amdgcn_raw_buffer_load_b16(rsrcR, voff, (t * 32 + k) * p.N * 2, 0);
          }
        }
      }
      if (r0 < p.R) {
#pragma unroll
        for (int i = 0; i < TM; i++) {
          const int gm = min(wrow0 + i * 16 + l16, p.M - 1);
          lf[i] = *(const lf_u32x4*)(L + (int64_t)gm * p.R + r0);
        }
      }
      if (t == 0) {
        if (bits_mask && BITS_EARLY) load_bits(0);
        __builtin_amdgcn_sched_barrier(0);
        issue_first_tiles();
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (NN) {
        if (r0 < rank) {
#pragma unroll
          for (int j = 0; j < TN; j++)
            rf[j] = lf_u32x4{e[j][0] | (e[j][1] << 16), e[j][2] | (e[j][3] << 16), e[j][4] | (e[j][5] << 16), e[j][6] | (e[j][7] << 16)};
        }
      }
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++) acc[i][j] = MfmaOp<T>::run(rf[j], lf[i], acc[i][j]);
    }
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int ib = i >> 1, h = i & 1;  // band of 32 rows, half of the band
      if (bytes_mask && h == 0) {
        if constexpr (!MEARLY) load_mask_band(ib);
#pragma unroll
        for (int ii = 0; ii < MNI; ii++) {
          const int r = ii * MRPI + mrow;
          *(lf_u32x4*)(mreg + r * WN + ((mg ^ ((r / MRW) & (MLPR - 1))) << 4)) = mv[ib][ii];
        }
      }
      const int r = h * 16 + l16;  // this lane's row of the band
      if constexpr (!BITS_EARLY) {
        if (bits_mask && i % GI == 0) load_bits(i);   // the next batch of block rows, all its words at once
      }
#pragma unroll
      for (int j = 0; j < TN; j++) {
        acc[i][j] *= mult;
        if (bits_mask) {
          const uint32_t bits = mw[i % GI][j];
#pragma unroll
          for (int e = 0; e < 4; e++) acc[i][j][e] = ((bits >> e) & 1u) ? acc[i][j][e] : 0.f;
        } else if (use_mask) {
          const int dw = j * 4 + kg;  // dword of the 4 columns j*16 + kg*4 ..
          const uint32_t mk = *(const uint32_t*)(mreg + r * WN + (((dw >> 2) ^ ((r / MRW) & (MLPR - 1))) << 4) + (dw & 3) * 4);
#pragma unroll
          for (int e = 0; e < 4; e++) acc[i][j][e] = ((mk >> (8 * e)) & 0xffu) ? acc[i][j][e] : 0.f;
        }
      }
    }
  }

  // ---- per-lane LDS fragment offsets: a lane reads 8 contraction elements (granule kg) of row l16
  int a_off[TM], b_off[TN];
  const int slot = (kg ^ ((l16 >> 1) & 3)) << 4;
#pragma unroll
  for (int i = 0; i < TM; i++) a_off[i] = (wm * WM + i * 16 + l16) * 64 + slot;
  if constexpr (!NN) {
#pragma unroll
    for (int j = 0; j < TN; j++) b_off[j] = (wn * WN + j * 16 + l16) * 64 + slot;
  } else {
    // ds_read_b64_tr_b16: within a 16-lane group, lane 4j+c addresses row j, columns 4c..4c+3 and
    // receives column (lane&15), rows 0..3.  Group kg takes contraction rows kg*8.. (two reads).
    const int j4 = l16 >> 2, c = l16 & 3;
    const int row0 = kg * 8 + j4;
    const int key = BPITCH == 128 ? (((j4 >> 1) << 1) | (kg & 1)) : (((j4 << 1) | (kg & 1)) & BKEY);
#pragma unroll
    for (int j = 0; j < TN; j++) {
      int colb = (wn * WN + j * 16 + 4 * c) * 2;  // byte offset within the row
      b_off[j] = row0 * BPITCH + (((colb >> 5) ^ key) << 5) + (colb & 31);
    }
  }

  lf_u32x4 fa[2][TM], fb[2][TN];  // two register sets; the anti-phase loop uses one
  lf_u32x2 fbt[2][TN][2];  // NN: halves of the B fragments, joined only after the wait that completes them
  // one fragment of a K step (idx < TM: A fragment idx, else B fragment idx - TM)
  auto read_one = [&](int set, int stage, int idx) {
    if (idx < TM) {
      fa[set][idx < TM ? idx : 0] = *(const lf_u32x4*)(ldsA + stage * A_STAGE + a_off[idx < TM ? idx : 0]);
    } else {
      const int j = idx - TM < TN ? idx - TM : 0;
      const char* sb = ldsB + stage * B_STAGE;
      if constexpr (!NN) {
        fb[set][j] = *(const lf_u32x4*)(sb + b_off[j]);
      } else {
        fbt[set][j][0] = lds_read_tr16(sb + b_off[j]);
        fbt[set][j][1] = lds_read_tr16(sb + b_off[j] + 4 * BPITCH);
      }
    }
  };
  auto read_frags = [&](int set, int stage) {
#pragma unroll
    for (int f = 0; f < TM + TN; f++) read_one(set, stage, f);
  };
  auto mfma_one = [&](int set, int idx) {
    const int i = idx / TN, j = idx % TN;
    if constexpr (NN) fb[set][j] = lf_u32x4{fbt[set][j][0][0], fbt[set][j][0][1], fbt[set][j][1][0], fbt[set][j][1][1]};
    acc[i][j] = MfmaOp<T>::run(fb[set][j], fa[set][i], acc[i][j]);
  };
  auto join_b = [&](int set) {
    if constexpr (NN) {
#pragma unroll
      for (int j = 0; j < TN; j++) fb[set][j] = lf_u32x4{fbt[set][j][0][0], fbt[set][j][0][1], fbt[set][j][1][0], fbt[set][j][1][1]};
    }
  };
  auto mfma_range = [&](int set, int m0_, int m1_) {
#pragma unroll
    for (int m = m0_; m < m1_; m++) acc[m / TN][m % TN] = MfmaOp<T>::run(fb[set][m % TN], fa[set][m / TN], acc[m / TN][m % TN]);
  };
  if constexpr (NWAVES <= 4) {
    // ---- main loop, one wave per SIMD: no neighbour to hide behind, so the fragments of step
    // kt+1 are read into a second register set while the MFMAs of step kt run; one barrier per
    // step.  At the top of step kt: tile kt is in registers, tile kt+1 has landed and is visible,
    // every wave has finished reading the stages of tiles kt-1 and kt.  Even steps issue the pair
    // (kt+PAIR0, kt+PAIR0+1) into those two stages and, at their end, wait for the pair
    // (kt+2, kt+3), issued two steps earlier.
    int stage = 0, kt = 0;
    auto k_step = [&](auto SET, auto LOAD, auto NEXT) {
      constexpr int cur = SET.value, nxt = 1 - SET.value;
      const int s1 = stage + 1 == NSTAGE ? 0 : stage + 1;
      // Source order is the issue order (a scheduling fence after every MFMA): the LDS reads of the
      // next step go out with the first half of the MFMAs, so that the second half covers the read
      // latency, and the tile loads spread evenly over the step -- the texture addresser takes
      // 16 cycles per load, and a wave that cannot issue a load cannot issue the MFMAs behind it.
      constexpr int NR = TM + TN, NM = TM * TN;  // fragment reads and MFMAs per step
      constexpr int NLD = LOAD.value ? 2 * NL : 0;  // lo/hi halves alternate: load l is half l&1 of load l>>1
      constexpr int LSTEP = NLD > 0 && NM / NLD > 0 ? NM / NLD : 1;
      constexpr int HALF = NM / 2 > 0 ? NM / 2 : 1, RPS = (NR + HALF - 1) / HALF;  // reads per MFMA slot
      int st_lo = stage + PAIR0, st_hi = stage + PAIR0 + 1;  // stage of unit u is u % NSTAGE
      st_lo = st_lo >= NSTAGE ? st_lo - NSTAGE : st_lo;
      st_hi = st_hi >= NSTAGE ? st_hi - NSTAGE : st_hi;
      st_hi = st_hi >= NSTAGE ? st_hi - NSTAGE : st_hi;
      auto load_l = [&](int l) { issue_load_one((l & 1) ? st_hi : st_lo, kt + PAIR0 + (l & 1), l >> 1); };
#pragma unroll
      for (int m = 0; m < NM; m++) {
        if (m % LSTEP == 0 && m / LSTEP < NLD) load_l(m / LSTEP);
        if constexpr (NEXT.value) {
#pragma unroll
          for (int r = m * RPS; r < (m + 1) * RPS && r < NR; r++) read_one(nxt, s1, r);
        }
        mfma_one(cur, m);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int l = (NM + LSTEP - 1) / LSTEP; l < NLD; l++) load_l(l);  // more loads than MFMA slots
      __builtin_amdgcn_sched_barrier(0);   // the waits stay behind the MFMAs that cover the read latency
      if constexpr (cur == 0) wait_loads(integral_constant<int, LOAD.value ? PAIR0 - 2 : 0>{});  // the pair (kt+2, kt+3) has landed
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): next fragments are in registers
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      stage = s1;
      kt++;
    };
    using T_ = integral_constant<bool, true>;
    using F_ = integral_constant<bool, false>;
    // tiles 0 and 1 must have landed.  PAIR0 steps are in flight only when the K loop has that many;
    // a shorter loop has fewer loads outstanding than the count allows, so it waits for all of them
    if (nk >= PAIR0) wait_loads(integral_constant<int, PAIR0 - 2>{});
    else wait_loads(Steps0{});
    __syncthreads();
    read_frags(0, 0);
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __syncthreads();  // every wave has read stage 0: step 0 may refill it
    while (kt + PAIR0 + 1 < nk) {  // two steps per trip: the register sets swap roles
      k_step(integral_constant<int, 0>{}, T_{}, T_{});
      k_step(integral_constant<int, 1>{}, F_{}, T_{});
    }
    // tail (an even number of steps is left: nk is even): no more loads, wait for everything
    while (kt + 2 < nk) {
      k_step(integral_constant<int, 0>{}, F_{}, T_{});
      k_step(integral_constant<int, 1>{}, F_{}, T_{});
    }
    k_step(integral_constant<int, 0>{}, F_{}, T_{});
    k_step(integral_constant<int, 1>{}, F_{}, F_{});
  } else {
  // ---- main loop, two wave groups in anti-phase.  Each K step of a wave is a memory phase (read all
  // fragments of the current tile into registers) followed by a compute phase (the MFMAs of the
  // step, in odd steps with its share of a later pair of tile loads between them); every
  // phase ends in a workgroup barrier.  The second half of the waves runs one phase behind the
  // first, so on every SIMD one wave feeds the MFMA pipe while its neighbour moves data: LDS
  // latency never sits between two MFMAs of a wave, and the barriers keep the two groups from
  // drifting into computing (or reading) at the same time -- with fewer barriers per step the
  // loop measured slower.
  //   phase 2k   : group 0 reads tile k        | group 1 computes tile k-1
  //   phase 2k+1 : group 0 computes tile k     | group 1 reads tile k
  // Tile k is read in phases 2k and 2k+1; every wave waits for its own share of it in a memory
  // phase that ends no later than phase 2k-1, so the barrier closing that phase publishes the tile.
  // Tile loads are issued in every odd step kt: the pair (kt+3, kt+4) goes into the stages of steps
  // kt-2 and kt-1 (last read in phase 2kt-1).  The texture addresser takes 16 cycles per 64-lane
  // 16-byte load, and a wave whose load has to wait for it cannot issue the MFMAs behind it: with
  // all loads of a step between the MFMAs of the compute phase that phase grows from 570 to 715
  // cycles.  The memory phase has some slack behind its fragment reads, enough for one of the four
  // loads of a step (LF_MEMPHASE_LOADS; measured per value at 8192x4096x4096: 0: 196 us, 1: 190,
  // 2: 192, 3: 194, 4: 196); the others stay in the compute phase, spread between the MFMAs.  At
  // the end of the memory phase of an odd step the pair (kt+1, kt+2), issued two steps earlier,
  // must have landed.
  const int grp = wave >= NWAVES / 2 ? 1 : 0;
  auto phase_barrier = [&]() {
    __builtin_amdgcn_sched_barrier(0);
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_sched_barrier(0);
  };
  int stage = 0, kt = 0;
  static_assert(NSTAGE == 5, "the anti-phase loop is written for a ring of five stages");
  constexpr int NM = TM * TN;
  constexpr int ML = LF_MEMPHASE_LOADS < NL ? LF_MEMPHASE_LOADS : NL;  // loads of a step issued from the memory phase
  auto compute_phase = [&](auto LOADC) {
    __builtin_amdgcn_s_setprio(1);
    if constexpr (LOADC.value) {
      const int s3 = stage + 3 >= NSTAGE ? stage + 3 - NSTAGE : stage + 3;
      const int s4 = stage + 4 >= NSTAGE ? stage + 4 - NSTAGE : stage + 4;
#pragma unroll
      for (int i = ML; i < NL; i++) {
        issue_load_one(s3, kt + 3, i);
        issue_load_one(s4, kt + 4, i);
      }
    }
    join_b(0);
    mfma_range(0, 0, NM);
    if constexpr (LOADC.value && NL > ML) {
      constexpr int NLC = NL - ML > 0 ? NL - ML : 1, PER = NM / (2 * NLC);
#pragma unroll
      for (int r = 0; r < 2 * NLC; r++) {
        __builtin_amdgcn_sched_group_barrier(0x008, PER, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, NM - PER * 2 * NLC, 0);
    }
    __builtin_amdgcn_s_setprio(0);
    phase_barrier();
    stage = stage + 1 == NSTAGE ? 0 : stage + 1;
    kt++;
  };
  auto step_pair = [&](auto LOAD) {
    // even step
    read_frags(0, stage);
    __builtin_amdgcn_s_waitcnt(0xc07f);
    phase_barrier();
    compute_phase(integral_constant<bool, false>{});
    // odd step: the pair (kt+1, kt+2) must have landed; issue the pair (kt+3, kt+4)
    read_frags(0, stage);
    wait_loads(Steps0{});
    if constexpr (LOAD.value && ML > 0) {
      __builtin_amdgcn_sched_barrier(0);
      const int s3 = stage + 3 >= NSTAGE ? stage + 3 - NSTAGE : stage + 3;
      const int s4 = stage + 4 >= NSTAGE ? stage + 4 - NSTAGE : stage + 4;
#pragma unroll
      for (int i = 0; i < ML; i++) {
        issue_load_one(s3, kt + 3, i);
        issue_load_one(s4, kt + 4, i);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
    phase_barrier();
    compute_phase(LOAD);
  };
  if (nk > 2) wait_loads(integral_constant<int, 2>{});
  else wait_loads(Steps0{});
  __syncthreads();
  if (grp == 1) phase_barrier();
  while (kt + 5 < nk) step_pair(integral_constant<bool, true>{});
  while (kt < nk) step_pair(integral_constant<bool, false>{});
  if (grp == 0) phase_barrier();
  }

  // ---- epilogue: bias, convert, then one 32-row band of the wave's sub-tile at a time through the
  // wave's own LDS region so that global stores are 16 bytes per lane and cover whole rows of
  // the sub-tile (WN*2 contiguous bytes) instead of 8-byte pieces scattered over 16 rows.
  // Granule g (16 bytes) of band row r sits at slot g ^ ((r / EP_RPW) & EP_KEY): EP_RPW rows span
  // the 64 banks once, so the 16 rows that write together land on different banks.
  if (p.ksplit > 1) {
    // split contraction: the fp32 sums of this slice, 16 bytes per lane (row l16 of a block, columns kg*4 .. +3)
    float* __restrict__ part = p.ks_ws + (int64_t)blockIdx.y * p.M * p.N;
#pragma unroll
    for (int i = 0; i < TM; i++)
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const int gm = wrow0 + i * 16 + l16, gn = n0 + wn * WN + j * 16 + kg * 4;
        if (gm < p.M && gn < p.N) *(lf_f32x4*)(part + (int64_t)gm * p.N + gn) = acc[i][j];
      }
    return;
  }
  T* __restrict__ C = (T*)p.C;
  const uint16_t* bias16 = (const uint16_t*)p.bias;
  constexpr int EP_PITCH = WN * 2;              // bytes per band row
  constexpr int EP_BAND = 32 * EP_PITCH;        // bytes per band
  constexpr int LPR = EP_PITCH / 16;            // lanes per row on the way out
  constexpr int RPI = 64 / LPR;                 // rows per store instruction
  constexpr int EP_RPW = 256 / EP_PITCH > 0 ? 256 / EP_PITCH : 1;
  constexpr int EP_KEY = LPR - 1;
  static_assert(2 * NWAVES * EP_BAND <= NSTAGE * (A_STAGE + B_STAGE), "epilogue staging fits the ring");
  __syncthreads();  // every wave is done with the ring
  char* ep = smem + wave * (2 * EP_BAND);
  float bv[TN][4];
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int gn = min(n0 + wn * WN + j * 16 + kg * 4, p.N - 4);
#pragma unroll
    for (int e = 0; e < 4; e++) bv[j][e] = bias16 != nullptr ? MfmaOp<T>::to_float(bias16[gn + e]) : 0.f;
  }
  const int out_col = n0 + wn * WN + (lane % LPR) * 8;
#pragma unroll
  for (int ib = 0; ib < TM / 2; ib++) {
    char* band = ep + (ib & 1) * EP_BAND;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int r = h * 16 + l16;
#pragma unroll
      for (int j = 0; j < TN; j++) {
        const lf_f32x4 a = acc[ib * 2 + h][j];
        lf_u32x2 o = {MfmaOp<T>::pack2(a[0] + bv[j][0], a[1] + bv[j][1]), MfmaOp<T>::pack2(a[2] + bv[j][2], a[3] + bv[j][3])};
        const int g = j * 2 + (kg >> 1);  // granule of the 4 columns j*16 + kg*4 ..; kg&1 selects its half
        *(lf_u32x2*)(band + r * EP_PITCH + ((g ^ ((r / EP_RPW) & EP_KEY)) << 4) + (kg & 1) * 8) = o;
      }
    }
#pragma unroll
    for (int r = 0; r < 32 / RPI; r++) {
      const int row = r * RPI + lane / LPR;
      const int g = lane % LPR;
      lf_u32x4 v = *(const lf_u32x4*)(band + row * EP_PITCH + ((g ^ ((row / EP_RPW) & EP_KEY)) << 4));
      const int gm = wrow0 + ib * 32 + row;
      if (gm < p.M && out_col < p.N) *(lf_u32x4*)(C + (int64_t)gm * p.ldc + out_col) = v;
    }
  }
#endif
}

// Second stage of a split contraction: C[m][n] = cast(sum over the slices, in index order, + bias[n]).  Eight columns
// per thread.
template <typename T>
__global__ void __launch_bounds__(256)
ksplit_reduce_kernel(const float* __restrict__ part, int nslices, const uint16_t* __restrict__ bias, T* __restrict__ C,
                     int M, int N, int64_t ldc) {
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 8;
  if (idx >= (int64_t)M * N) return;
  const int row = (int)(idx / N), col = (int)(idx % N);
  lf_f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = lo;
  for (int s = 0; s < nslices; s++) {
    const float* q = part + (int64_t)s * M * N + idx;
    lo += *(const lf_f32x4*)q;
    hi += *(const lf_f32x4*)(q + 4);
  }
  if (bias != nullptr) {
#pragma unroll
    for (int e = 0; e < 4; e++) {
      lo[e] += MfmaOp<T>::to_float(bias[col + e]);
      hi[e] += MfmaOp<T>::to_float(bias[col + 4 + e]);
    }
  }
  const lf_u32x4 o = {MfmaOp<T>::pack2(lo[0], lo[1]), MfmaOp<T>::pack2(lo[2], lo[3]), MfmaOp<T>::pack2(hi[0], hi[1]),
                      MfmaOp<T>::pack2(hi[2], hi[3])};
  *(lf_u32x4*)((uint16_t*)C + (int64_t)row * ldc + col) = o;
}

template <typename T>
int launch_ksplit_reduce(const LfGemmParams& p, hipStream_t st) {
  const int64_t n8 = (int64_t)p.M * p.N / 8, blocks = (n8 + 255) / 256;
  return lf_launch(ksplit_reduce_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, st, (const float*)p.ks_ws, p.ksplit,
                   (const uint16_t*)p.bias, (T*)p.C, p.M, p.N, p.ldc);
}

template <typename T, int BM, int BN, int WM, int WN, bool NN, int NSTAGE>
int launch_cfg(LfGemmParams p, const LfSegTable& seg, hipStream_t st) {
  constexpr int NTHREADS = (BM / WM) * (BN / WN) * 64;
  constexpr int SMEM = NSTAGE * (BM + BN) * BK * 2;
  p.grid_m = (p.M + BM - 1) / BM;
  p.grid_n = (p.N + BN - 1) / BN;
  auto kern = gemm_lora_kernel<T, BM, BN, WM, WN, NN, NSTAGE>;
  static LfLdsFlags lds_ok;
  if (!lf_allow_lds(kern, SMEM, lds_ok)) return LF_ELAUNCH;
  return lf_launch(kern, dim3(p.grid_m * p.grid_n, p.ksplit > 1 ? p.ksplit : 1), dim3(NTHREADS), SMEM, st, p, seg);
}

template <typename T, bool NN>
int launch_dtype(const LfGemmParams& p, const LfSegTable& seg, int cfg, hipStream_t st) {
  // Rows of one routing block must not straddle a wave's sub-tile: WM divides block_size_m.
  switch (cfg) {
    case 0: return launch_cfg<T, 256, 256, 128, 128, NN, LF_NSTAGE>(p, seg, st);
    case 1: return launch_cfg<T, 256, 256, 128, 64, NN, LF_NSTAGE>(p, seg, st);
    case 2: return launch_cfg<T, 128, 256, 64, 128, NN, LF_NSTAGE>(p, seg, st);
    case 3: return launch_cfg<T, 128, 256, 64, 64, NN, LF_NSTAGE>(p, seg, st);
    case 4: return launch_cfg<T, 128, 128, 64, 64, NN, LF_NSTAGE>(p, seg, st);
    case 5: return launch_cfg<T, 64, 64, 32, 32, NN, LF_NSTAGE_SMALL>(p, seg, st);
    case 6: return launch_cfg<T, 128, 64, 64, 32, NN, 9>(p, seg, st);
    default: return LF_EINVAL;
  }
}

}  // namespace

// Tile choice from a measured cost model.  A launch runs in "rounds" of resident workgroups
// (256 CUs x workgroups per CU).  Costs are microseconds measured at K = 4096: the first round
// costs lat0 + first_b * fill^2 (a lone tile per CU runs latency bound at boost clock, a full round
// is power limited), every further round next_a + next_b * fill, where fill is the occupied
// fraction of the round's slots.  For another K every term scales with K / 4096 except kRamp
// microseconds of lat0 (launch, first loads, epilogue), which a launch pays once whatever its K:
// a second launch for left-over rows pays off at a long K and does not at a short one.
struct TileCand { int cfg, bm, bn, slots; double lat0, first_b, next_a, next_b; };
static const TileCand kCands[] = {
    {7, 256, 256, 256, 70.0, 40.0, 50.0, 30.0},   // persistent, 4 waves of 128x128 (gemm_big.hip): rounds = tiles per workgroup
    {1, 256, 256, 256, 66.0, 50.0, 44.0, 60.0},   // 8 waves, 128x64 per wave
    {3, 128, 256, 256, 48.0, 28.0, 28.0, 38.0},   // 8 waves, 64x64 per wave
    {4, 128, 128, 512, 38.0, 47.0, 5.0, 70.0},    // 4 waves, two workgroups per CU
    {5, 64, 64, 512, 19.0, 17.0, 13.0, 18.0},     // 4 waves, 32x32 per wave: spreads a short row range
    {6, 128, 64, 256, 22.5, 4.5, 13.0, 14.0},     // 4 waves, 64x32 per wave: less operand traffic per flop than 64x64
    {8, 128, 256, 256, 41.5, 15.0, 45.0, 30.0},   // persistent, 4 waves of 64x128 (gemm_big.hip): 2048 x 4096 outputs are one round of it
};
constexpr double kRamp = 6.0;
static double launch_cost(const TileCand& c, int M, int N, int K) {
  const long tiles = (long)((M + c.bm - 1) / c.bm) * ((N + c.bn - 1) / c.bn);
  if (tiles <= 0) return 0.0;
  const long full = tiles / c.slots;
  const double fill = (double)(tiles % c.slots) / c.slots;
  double at4096;
  if (full == 0) at4096 = c.lat0 + c.first_b * fill * fill;
  else at4096 = c.lat0 + c.first_b + (full - 1) * (c.next_a + c.next_b) + (fill > 0 ? c.next_a + c.next_b * fill : 0.0);
  return kRamp + (at4096 - kRamp) * (K / 4096.0);
}
static int choose_cfg(int M, int N, int K, bool allow_big, double* cost_out = nullptr, bool allow_mid = true) {
  int best = 1;
  double best_cost = 1e30;
  for (const TileCand& c : kCands) {
    if (c.cfg == 7 && (!allow_big || M < 256 || N < 256)) continue;
    // (a lone 128x256 tile per CU takes 41 us whatever the fill, the same for both operand layouts: below half a round
    // the smaller tiles are faster)
    if (c.cfg == 8 && (!allow_big || !allow_mid || M < 128 || N < 256 || K < 256 || 2 * (long)((M + 127) / 128) * ((N + 255) / 256) <= c.slots)) continue;
    const double cost = launch_cost(c, M, N, K);
    if (cost < best_cost) { best_cost = cost; best = c.cfg; }
  }
  if (cost_out) *cost_out = best_cost;
  return best;
}
// Rows [0, m_main) as 256x256 tiles, the rest as a second launch with the tile that spreads it best, when that beats
// one launch (a nearly empty last round of big tiles costs a full tile time).  m_main is the multiple of 256 rows
// with the lowest modelled cost of both launches: usually the one whose tiles fill whole rounds of the chip
// (32 tile rows of 40 tiles are exactly five rounds; 30 rows of 40 are five rounds too, and leave a longer tail).
// Returns m_main (0: single launch).
static int choose_split(int M, int N, int K, bool allow_big, int* cfg_head, int* cfg_tail) {
  constexpr double kLaunch = 4.0;  // a second launch
  const int grid_n = (N + 255) / 256;
  if (grid_n > 256) return 0;
  const bool big = allow_big && N >= 256;
  const TileCand& head = kCands[big ? 0 : 1];
  double best;
  choose_cfg(M, N, K, allow_big, &best);
  int best_m = 0;
  for (int r = 1; r * 256 < M; r++) {
    double tail;
    // (left-over rows behind whole rounds of 256x256 tiles: small tiles or a split contraction, not the 128-row persistent tile)
    const int ct = choose_cfg(M - r * 256, N, K, allow_big, &tail, false);
    const double cost = launch_cost(head, r * 256, N, K) + tail + kLaunch;
    if (cost < best) { best = cost; best_m = r * 256; *cfg_tail = ct; }
  }
  *cfg_head = big ? 7 : 1;
  return best_m;
}

// Split contraction for a launch of few tiles over a long K (left-over rows of a packed batch, short batches): K is
// cut into slices, workgroup (tile, slice) keeps fp32 sums, a second kernel adds the slices.  Measured on the left-over
// rows of the 8B and 70B layers (128 and 384 rows; microseconds with the second kernel, unsplit first):
//   128 x 4096 over 28672 (NN): 64x64 tiles 134 -> 128x64 tiles in 4 slices 52;  over 6144: 31 -> 18
//   128 x 4096 over 14336 (NT): 54 -> 35;   384 x 8192 over 57344 (NN): 128x128 tiles 580 -> 256x256 tiles in 4 slices 399
//   384 x 8192 over 28672 (NT): 300 -> 203; 384 x 10240 over 8192: 64 unsplit, 95 in 2 slices of 256x256 tiles
// So: when the planned tiles fill less than half of the chip's workgroup slots, the launch moves to the 128x64 tile (up
// to 256 rows) or the eight-wave 256x256 tile (more rows) in as many slices as give every compute unit a workgroup,
// provided a slice keeps at least 48 K steps on the small tile and 192 on the large one (their fixed cost per
// workgroup: pipeline fill and an fp32 store of the tile) and the small tile gets at least three slices, at most 16
// slices and at most kKsplitMaxBytes of partial tiles.  A function of the shape, the planned tile and the routing block alone: a call that is given the workspace
// lf_workspace_bytes names always makes the same split, so its result does not depend on who calls.
constexpr size_t kKsplitMaxBytes = (size_t)64 << 20;
struct KSplit { int cfg, n, steps; };
static long tiles_of(int M, int N, int cfg, int* slots = nullptr) {
  int bm = 256, bn = 256, sl = 256;      // configurations 0, 1, 7
  for (const TileCand& k : kCands) if (k.cfg == cfg) { bm = k.bm; bn = k.bn; sl = k.slots; }
  if (cfg == 2) { bm = 128; bn = 256; }
  if (slots != nullptr) *slots = sl;
  return (long)((M + bm - 1) / bm) * ((N + bn - 1) / bn);
}
static KSplit ksplit_for(int M, int N, int K, int cfg, int routing_block) {
  const int nk = K / BK;
  const KSplit none = {cfg, 1, nk};
  int slots = 256;
  if (cfg == 7 || 2 * tiles_of(M, N, cfg, &slots) > slots) return none;   // the planned launch fills half of its slots
  const bool big_ok = routing_block <= 0 || routing_block % 128 == 0;
  const int cand = M <= 256 ? 6 : (big_ok ? 1 : 2);
  const int min_steps = cand == 6 ? 48 : 192;
  const long tiles = tiles_of(M, N, cand);
  long n = 256 / tiles;
  n = std::min(n, (long)16);
  n = std::min(n, (long)(nk / min_steps));
  const size_t slice = (size_t)M * N * sizeof(float);
  n = std::min(n, (long)(kKsplitMaxBytes / slice));
  if (n < (cand == 6 ? 3 : 2)) return none;   // two slices of the small tile only pay for the second kernel (22 -> 24 us at K = 4096)
  int steps = (int)((nk + n - 1) / n);
  steps += steps & 1;                                         // an even number of steps per slice (K / BK is even)
  return {cand, (nk + steps - 1) / steps, steps};             // no empty slice
}

static std::atomic<int> pinned_cfg{-1};
int lf_pin_tile_cfg(int cfg) {
  if (cfg < -1 || cfg > 8) return LF_EINVAL;
  pinned_cfg.store(cfg, std::memory_order_relaxed);
  return LF_OK;
}

// The launches lf_launch_gemm makes for an M x N product over K when no configuration is pinned: rows [0, *rows_head)
// with *cfg_head and, when *rows_head < M, the remaining rows with *cfg_tail (-1 otherwise).
void lf_plan_gemm(int M, int N, int K, int routing_block, int* rows_head, int* cfg_head, int* cfg_tail) {
  const bool allow_big = routing_block <= 0 || (routing_block % 128 == 0 && M % 128 == 0);
  int ch = 1, ct = 1;
  const int m_main = choose_split(M, N, K, allow_big, &ch, &ct);
  // A long contraction under a wide output runs faster on the eight-wave 256x256 tile than on the persistent kernel
  // (8192 x 8192 over 28672: 3.08 against 3.24 ms, over 57344: 5.74 against 5.85; at 4096 columns the two are level, and
  // at shorter contractions the persistent kernel is 3-8 % ahead): its long K loops let the tiles of an XCD drift apart
  // and lose the L2 hits on the panels they share.
  auto long_k = [&](int cfg) { return (cfg == 7 && K >= 16384 && N >= 8192) ? 1 : cfg; };
  auto demote = [&](int cfg0) {
    const int cfg = long_k(cfg0);
    return (routing_block > 0 && routing_block % 128 != 0 && (cfg == 0 || cfg == 1 || cfg == 7)) ? 2 : cfg;
  };
  if (m_main == 0) {
    *rows_head = M;
    *cfg_head = demote(choose_cfg(M, N, K, allow_big));
    *cfg_tail = -1;
  } else {
    *rows_head = m_main;
    *cfg_head = demote(ch);
    *cfg_tail = demote(ct);
  }
}

// Bytes of fp32 partial tiles the split contraction of an M x N product over K may write: the largest need over the
// launches of the plan and over the configurations a launch can be moved to at run time (the eight-wave 256x256 tile
// and the 128x256 tile stand in for the persistent kernel where it does not apply).
size_t lf_gemm_ksplit_bytes(int M, int N, int K, int routing_block) {
  if (M <= 0 || N <= 0 || K < BK) return 0;
  int rows = 0, ch = 1, ct = -1;
  lf_plan_gemm(M, N, K, routing_block, &rows, &ch, &ct);
  size_t need = 0;
  auto part = [&](int m, int cfg) {
    for (int c : {cfg, 1, 2, choose_cfg(m, N, K, false)}) {
      const KSplit ks = ksplit_for(m, N, K, c, routing_block);
      if (ks.n > 1) need = std::max(need, (size_t)ks.n * m * N * sizeof(float));
    }
  };
  part(rows, ch);
  if (ct >= 0) part(M - rows, ct);
  return need;
}

int lf_launch_gemm(const LfGemmParams& p, const LfSegTable& seg, bool nn, int dtype, int force_cfg, hipStream_t st) {
  if (force_cfg < 0) force_cfg = pinned_cfg.load(std::memory_order_relaxed);
  if (p.M <= 0 || p.N <= 0 || p.K <= 0) return LF_EINVAL;
  if (p.K % 64 != 0 || p.N % 8 != 0 || p.N < 8) return LF_ESHAPE;
  // 16-byte output stores
  if (p.ldc % 8 != 0 || ((uintptr_t)p.C & 15) != 0) return LF_ESHAPE;
  if (p.L != nullptr && (p.R % 16 != 0 || p.R <= 0 || p.R > LF_MAX_RANK)) return LF_ESHAPE;
  // the keep-mask is read 16 bytes at a time
  if (p.mask != nullptr && !p.mask_bits && (p.N % 16 != 0 || p.ldmask % 16 != 0 || ((uintptr_t)p.mask & 15) != 0)) return LF_ESHAPE;
  // bit-packed: read 4 bytes at a time (the persistent kernel: 16), rows of whole dwords
  if (p.mask != nullptr && p.mask_bits && (p.N % 32 != 0 || p.ldmask % 4 != 0 || ((uintptr_t)p.mask & 15) != 0)) return LF_ESHAPE;
  // tile loads address a panel of 256 rows (the K-major operand of the NN product: all of it) with 32-bit byte offsets
  if (256 * p.lda * 2 >= 0x7fffffffLL || (int64_t)(nn ? p.K : 256) * p.ldb * 2 >= 0x7fffffffLL) return LF_ESHAPE;
  if (seg.table != nullptr && (seg.block_size_m % 64 != 0)) return LF_ESHAPE;
  const bool planned = force_cfg < 0;
  auto launch = [&](const LfGemmParams& q, int cfg) {
    if (seg.table != nullptr && seg.block_size_m % 128 != 0 && (cfg == 0 || cfg == 1 || cfg == 7)) cfg = 2;
    // what the persistent kernel does not take goes to the eight-wave 256x256 tile: a keep-mask with one byte per
    // element, a dX term of more than 32 rank columns and (when the library chose the tile) a contraction of one K step
    if (cfg == 7 && ((q.mask != nullptr && (!q.mask_bits || q.N % 128 != 0)) || (nn && q.L != nullptr && q.R > 32) || (planned && q.K < 128))) cfg = 1;
    // the 128-row persistent tile has the same limits; a product it was planned for then runs on the small tile the
    // cost model likes best (pinned: on the four-wave 128x256 tile)
    if (cfg == 8 && ((q.mask != nullptr && (!q.mask_bits || q.N % 128 != 0)) || (nn && q.L != nullptr && q.R > 32)))
      cfg = planned ? choose_cfg(q.M, q.N, q.K, false) : 2;
    if (cfg == 7) return lf_launch_gemm_big(q, seg, nn, dtype, 256, st);
    if (cfg == 8) return lf_launch_gemm_big(q, seg, nn, dtype, 128, st);
    if (dtype != LF_BF16 && dtype != LF_F16) return (int)LF_EINVAL;
    LfGemmParams r = q;
    r.ksplit = 1;
    if (planned && r.ks_ws != nullptr && ((uintptr_t)r.ks_ws & 15) == 0) {   // (a pinned tile configuration stays as pinned)
      const KSplit ks = ksplit_for(r.M, r.N, r.K, cfg, seg.table != nullptr ? seg.block_size_m : 0);
      if (ks.n > 1 && (size_t)ks.n * r.M * r.N * sizeof(float) <= r.ks_ws_bytes) { cfg = ks.cfg; r.ksplit = ks.n; r.ks_steps = ks.steps; }
    }
    int rc;
    if (dtype == LF_BF16) rc = nn ? launch_dtype<__bf16, true>(r, seg, cfg, st) : launch_dtype<__bf16, false>(r, seg, cfg, st);
    else rc = nn ? launch_dtype<_Float16, true>(r, seg, cfg, st) : launch_dtype<_Float16, false>(r, seg, cfg, st);
    if (rc != LF_OK || r.ksplit <= 1) return rc;
    return dtype == LF_BF16 ? launch_ksplit_reduce<__bf16>(r, st) : launch_ksplit_reduce<_Float16>(r, st);
  };
  if (force_cfg >= 0) return launch(p, force_cfg);
  int m_main = 0, cfg_head = 1, cfg_tail = -1;
  lf_plan_gemm(p.M, p.N, p.K, seg.table != nullptr ? seg.block_size_m : 0, &m_main, &cfg_head, &cfg_tail);
  if (cfg_tail < 0) return launch(p, cfg_head);
  LfGemmParams head = p, tail = p;
  head.M = m_main;
  tail.M = p.M - m_main;
  tail.row0 = p.row0 + m_main;
  tail.A = (const char*)p.A + (int64_t)m_main * p.lda * 2;
  tail.C = (char*)p.C + (int64_t)m_main * p.ldc * 2;
  if (p.L != nullptr) tail.L = (const char*)p.L + (int64_t)m_main * p.R * 2;
  if (p.mask != nullptr) tail.mask = p.mask + (int64_t)m_main * p.ldmask;
  const int rc = launch(head, cfg_head);
  return rc != LF_OK ? rc : launch(tail, cfg_tail);
}
