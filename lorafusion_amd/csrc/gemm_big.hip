// Persistent MFMA GEMM in tiles of 256x256 or 128x256 with the LoRA term added to the accumulator, for gfx950 (MI355X).
//
//   C[M,N] = A[M,K] * op(B) + mult * (L[M,R] * Rop) (+ bias)        (operands as in gemm_lora.hip)
//
// The large-shape instance of the kernels that stand in for fused_lora_xw_sb / fused_multi_lora_xw_sb
// (lorafusion/ops/triton_ops/fused_lora_xw_sb.py:74-206, fused_multi_lora_xw_sb.py:66-218; the reference's
// persistent forward is fused_lora_xw_sb_tma.py:314,351-357) and fused_lora_dyw_dsa / fused_multi_lora_dyw_dsa
// (fused_lora_dyw_dsa.py:69-181, fused_multi_lora_dyw_dsa.py:60-185).
//
// Structure (of the 256x256 tile, TI = 8; what the 128x256 tile, TI = 4, does differently comes last)
//  * One workgroup per CU (at most), four 64-lane waves, each owning a 128x128 sub-tile (8x8 blocks of
//    16x16x32 MFMA, 256 accumulator registers).  One wave per SIMD: a K step of 32 costs 16 LDS fragment
//    reads per wave for 64 MFMAs, a third less LDS traffic than eight waves of 128x64.
//  * Persistent: workgroup b walks tiles b, b+G, b+2G, ... (G = workgroups launched).  The K loops of
//    successive tiles form one software pipeline: while a tile's last K steps run, the first stages of
//    the next tile are already on their way into LDS, and they land during the epilogue.
//  * K advances in stages of 64 (128-byte rows: every 16-byte lane of a load instruction belongs to a
//    whole cache line) through two LDS stages of 64 KB, filled by 16-byte direct-to-LDS buffer loads.
//    Stage s+1 is loaded while stage s is consumed; one workgroup barrier per stage, placed between
//    the two MFMA sub-steps (k 0-31, k 32-63) of a stage:
//        sub-step 0: MFMAs on fragment set 0; LDS reads of set 1 (same stage, k 32-63)
//        wait for this wave's loads of the next stage, barrier  (next stage visible, current stage dead)
//        sub-step 1: MFMAs on set 1; LDS reads of set 0 of the next stage; 16 tile loads of the stage
//                    after next into the dead stage, one every four MFMAs (the texture addresser takes
//                    16 cycles per 64-lane 16-byte load, and four waves issue in lockstep)
//    All memory instructions of the loop carry hand-placed s_waitcnt: fragment reads are inline assembly,
//    because the compiler's own counter bookkeeping gives up across the loop edge and waits for reads
//    and loads that were issued a few cycles earlier.
//  * LDS rows are 128 bytes (8 granules); granule g of row r sits at slot g ^ ((r>>1)&7), applied on the
//    global side of the direct load.  Fragment reads (ds_read_b128) are conflict free with it.  The NN
//    operand (W read as [K,N]) is stored untransposed and unpermuted in 512-byte rows (a permuted fetch order
//    measured twice as slow), two rows per load instruction with 32 bytes of padding after each pair, and
//    read with ds_read_b64_tr_b16: the rows that lanes read together sit in different pairs, hence on
//    different banks.
//  * The LoRA product is added at the end of a tile: the forward's 64 MFMAs per 16 rank columns go onto the
//    accumulators right behind the K loop; the dX product's term is formed block row by block row inside the
//    epilogue, multiplied by 1/(1-p) and masked with the wave's keep bits on the way out.  The operands that
//    are slow to fetch (keep bits from HBM, A_i rows that need a transposing read) land in the wave's own LDS
//    area as direct-to-LDS loads during the tile's first K step.  The forward scale is folded into the 16-bit L
//    fragments (exact for powers of two).
//  * Epilogue: 16-row bands of a wave's sub-tile go through 4 KB of LDS per wave (beside the two stages) and
//    leave as 16-byte non-temporal stores that cover whole 256-byte rows of the sub-tile.
//  * TI = 4: four waves of 64x128 (one round of 128x256 tiles is what 2048 x 4096 outputs give 256 CUs).  A K step
//    is half as long but loads three quarters as much, so the stages are three: step s issues the second half of
//    step s+2's loads in its first sub-step and the first half of step s+3's in its second, one load per five MFMAs,
//    and waits with vmcnt(12) before its barrier (see k_step3).  Nothing fits behind three stages: a wave's band /
//    landing area lies inside the stage of the tile's last K step, and the dX product's operands are requested in
//    that step's second sub-step.
#include "lf_common.h"
#include <type_traits>
#include <utility>

namespace {

// workgroup tile: 32 TI rows x 256 columns (TI = 8: 256x256, a wave owns 128x128; TI = 4: 128x256, a wave owns 64x128)
constexpr int BN = 256, BK = 64;
// NN operand B [64 k-rows, 256 columns]: rows of 512 bytes stored in pairs (k-rows r and r+4: the 1024 bytes one wave
// instruction of the direct load fills), 32 bytes of padding after every pair
constexpr int PAIR_NN = 1024 + 32;
template <bool NN, int TI> struct Lds {
  static constexpr int STAGE_A = TI * 32 * BK * 2;
  static constexpr int STAGE_B = NN ? 32 * PAIR_NN : BN * BK * 2;
  static constexpr int STAGE = STAGE_A + STAGE_B;
  // 256-row tile: two stages; per wave behind them 6 KB: the epilogue's band buffer (4 KB), before that the landing
  // area of a tile's LoRA operands (dX product: 4 KB of A_i rows + 2 KB of keep bits).
  // 128-row tile: three stages (a K step is half as long, so a stage's loads are given two steps to land) and nothing
  // behind them: a wave's 5 KB (4 KB of A_i rows or the band, 1 KB of keep bits) lie in the stage of the tile's last K
  // step, in the part that no load writes to between that step's barrier and the next tile's first step.
  static constexpr int NST = TI == 8 ? 2 : 3;
  static constexpr int EP_OFF = NST * STAGE, EP_WAVE = TI == 8 ? 6144 : 5120;
  static constexpr int BYTES = TI == 8 ? EP_OFF + 4 * EP_WAVE : EP_OFF;
  static_assert(BYTES <= 160 * 1024, "stages, landing area and epilogue bands fit the LDS of a CU");
};

template <typename T> struct BigOp;
// The MFMAs are inline assembly with the accumulator block constrained to the accumulation registers ("+a"): all 256
// of them hold the tile for the whole kernel, and the register allocator can neither park accumulator blocks in
// ordinary vector registers nor use accumulation registers as spill space for other values (both happened with the
// builtin: copies between the two files inside the K loop).  The compiler's hazard recogniser does not look inside
// inline assembly: the wait states between these MFMAs and compiler-generated code that touches the accumulator
// (v_accvgpr_write before, v_accvgpr_read after) are the explicit s_nop of mfma_fence() below.
template <> struct BigOp<__bf16> {
  static __device__ __forceinline__ void mfma(lf_f32x4& c, lf_u32x4 a, lf_u32x4 b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  // d = a b into ordinary vector registers (for a product that vector instructions pick up next)
  static __device__ __forceinline__ void mfma0(lf_f32x4& d, lf_u32x4 a, lf_u32x4 b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
  }
  // c = a b: the first product of a tile needs no zeroed accumulator
  static __device__ __forceinline__ void mfma_first(lf_f32x4& c, lf_u32x4 a, lf_u32x4 b) {
    asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
  }
  // the LoRA term: 16 rank columns per step (two registers per operand), into the accumulators / into (d = a b) and
  // onto (d += a b) ordinary vector registers
  static __device__ __forceinline__ void mfma16(lf_f32x4& c, lf_u32x2 a, lf_u32x2 b) {
    asm volatile("v_mfma_f32_16x16x16_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma16_v0(lf_f32x4& d, lf_u32x2 a, lf_u32x2 b) {
    asm volatile("v_mfma_f32_16x16x16_bf16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma16_v(lf_f32x4& d, lf_u32x2 a, lf_u32x2 b) {
    asm volatile("v_mfma_f32_16x16x16_bf16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    bf2 v = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  static __device__ __forceinline__ float to_float(uint16_t bits) { return __builtin_bit_cast(float, (uint32_t)bits << 16); }
};
template <> struct BigOp<_Float16> {
  static __device__ __forceinline__ void mfma(lf_f32x4& c, lf_u32x4 a, lf_u32x4 b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma0(lf_f32x4& d, lf_u32x4 a, lf_u32x4 b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma_first(lf_f32x4& c, lf_u32x4 a, lf_u32x4 b) {
    asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, 0" : "=a"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma16(lf_f32x4& c, lf_u32x2 a, lf_u32x2 b) {
    asm volatile("v_mfma_f32_16x16x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma16_v0(lf_f32x4& d, lf_u32x2 a, lf_u32x2 b) {
    asm volatile("v_mfma_f32_16x16x16_f16 %0, %1, %2, 0" : "=&v"(d) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ void mfma16_v(lf_f32x4& d, lf_u32x2 a, lf_u32x2 b) {
    asm volatile("v_mfma_f32_16x16x16_f16 %0, %1, %2, %0" : "+v"(d) : "v"(a), "v"(b));
  }
  static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
    typedef _Float16 h2 __attribute__((ext_vector_type(2)));
    h2 v = {(_Float16)lo, (_Float16)hi};
    return __builtin_bit_cast(uint32_t, v);
  }
  static __device__ __forceinline__ float to_float(uint16_t bits) { return (float)__builtin_bit_cast(_Float16, bits); }
};

// 24 wait states: more than any MFMA-to-VALU / VALU-to-MFMA distance the hardware asks for on an accumulator register
__device__ __forceinline__ void mfma_fence() { asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7" ::: "memory"); }

typedef __attribute__((address_space(3))) void* lds_ptr_t;

template <int N, typename F>
__device__ __forceinline__ void sfor(F&& f) {
  [&]<int... I>(std::integer_sequence<int, I...>) { (f(std::integral_constant<int, I>{}), ...); }(std::make_integer_sequence<int, N>{});
}

// LORA = false: the instance for calls without a LoRA term (the seed code is compiled out, which also keeps that
// instance free of register spills: a kernel that needs scratch memory pays for it at every launch).
template <typename T, bool NN, bool LORA, int TI>
__global__ void __launch_bounds__(256, 1)
gemm_big_kernel(const LfGemmParams p, const LfSegTable seg) {
#if defined(__HIP_DEVICE_COMPILE__)  // the host pass only needs the launch stub (buffer-resource types are device-only)
  using std::integral_constant;
  extern __shared__ __attribute__((aligned(1024))) char smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  constexpr int BM = TI * 32, WROWS = TI * 16;   // rows of the workgroup's tile, of a wave's sub-tile
  constexpr int NL = TI + 8;                     // tile loads per wave and stage (TI of A, 8 of B)
  constexpr int NM = TI * 8;                     // MFMAs per wave and sub-step
  constexpr int STAGE_A = Lds<NN, TI>::STAGE_A, STAGE = Lds<NN, TI>::STAGE, EP_OFF = Lds<NN, TI>::EP_OFF, EP_WAVE = Lds<NN, TI>::EP_WAVE;
  constexpr int NST = Lds<NN, TI>::NST;          // LDS stages
  constexpr int NH1 = TI + 2;                    // three stages: loads [0, NH1) of a stage (A, the first two of B) are its first half

  const int total = p.grid_m * p.grid_n;
  const int G = gridDim.x, wg = blockIdx.x;
  const int n_my = (total - wg + G - 1) / G;
  const int nk = p.K / BK;

  // Tile `it` of this workgroup -> first row / column and the start of its K walk.  XCD-aware (workgroup ids that
  // differ by a multiple of 8 share an XCD and its L2: they get neighbouring tiles), grouped 8 tile rows deep.  A tile
  // that would cross the matrix edge is shifted inwards instead (M, N >= 256): it recomputes a few rows / columns of
  // its neighbour -- identical values, since both walk K from the same start -- and no load or store needs a guard.
  struct Tile { int m0, n0, kstart; };
  auto tile_of = [&](int it) __attribute__((always_inline)) {
    int pid = it * G + wg;
    if ((total & 7) == 0) pid = (pid & 7) * (total >> 3) + (pid >> 3);
    const int GROUP_M = p.group_m;   // tile rows per group: 8, or 2 for a long K over few tile columns (see the launcher)
    const int width = GROUP_M * p.grid_n;
    const int group = pid / width;
    const int first_m = group * GROUP_M;
    const int gsz = min(p.grid_m - first_m, GROUP_M);
    const int pid_m = first_m + (pid % width) % gsz;
    const int pid_n = (pid % width) / gsz;
    Tile t;
    t.m0 = min(pid_m * BM, p.M - BM);
    t.n0 = min(pid_n * BN, p.N - BN);
    // tile columns that run side by side start one 128-byte step apart, so their loads spread over the memory
    // channels; the tiles of one column stay aligned and share the lines of their B panel in L2.  A shifted last
    // column starts where the column it overlaps starts.
    const int kcol = (pid_n == p.grid_n - 1 && p.N % BN != 0 && pid_n > 0) ? pid_n - 1 : pid_n;
    t.kstart = (kcol & 15) % nk;
    return t;
  };

  // ---------------------------------------------------------------- tile loads
  // Direct-to-LDS loads: one wave instruction fills 1024 contiguous LDS bytes.  Operands with K-contiguous rows
  // (A; B of the NT product): 8 rows of 128 B, lane -> (row tid>>3, slot tid&7) fetches granule slot ^ ((row>>1)&7);
  // load i of an operand covers rows i*32 .. i*32+31 (a scalar offset).  NN operand B [K,N]: wave w, load i fills
  // the pair of k-rows 8i+w (lanes 0-31) and 8i+w+4 (lanes 32-63), 512 contiguous bytes each, unpermuted.
  uint32_t a_voff, b_voff;
  {
    const int lrow = tid >> 3, lg = tid & 7;
    const int srcg = lg ^ ((lrow >> 1) & 7);
    a_voff = (uint32_t)((int64_t)lrow * p.lda * 2 + srcg * 16);
    if constexpr (!NN) {
      b_voff = (uint32_t)((int64_t)lrow * p.ldb * 2 + srcg * 16);
    } else {
      b_voff = (uint32_t)((int64_t)(wave + 4 * (lane >> 5)) * p.ldb * 2 + (lane & 31) * 16);
    }
  }
  const int a_istride = 32 * (int)p.lda * 2;
  const int b_istride = NN ? 8 * (int)p.ldb * 2 : 32 * (int)p.ldb * 2;
  // A wave issues one instruction per four cycles: behind every MFMA (16 cycles) there is room for three others.  The
  // loop therefore keeps scalar work per load to one instruction where the loads are issued: the buffer descriptors
  // of a tile sit in scalar registers, the scalar offsets of a stage's 16 loads are prepared one per MFMA during the
  // previous sub-step, and M0 (the LDS destination of a direct load) is written one MFMA ahead of its load, which also
  // covers the wait state between the two.
  struct LoadSrc { lf_u32x4 ra, rb; int kstart; };
  auto src_of = [&](const Tile& t) __attribute__((always_inline)) {
    const char* a_base = (const char*)p.A + (int64_t)t.m0 * p.lda * 2;
    const char* b_base = NN ? (const char*)p.B + (int64_t)t.n0 * 2 : (const char*)p.B + (int64_t)t.n0 * p.ldb * 2;
    LoadSrc s;
    s.ra = lf_u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uintptr_t)a_base),
                    (uint32_t)__builtin_amdgcn_readfirstlane((int)((uintptr_t)a_base >> 32)) & 0xffffu, 0x7fffffffu, 0x00020000u};
    s.rb = lf_u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)(uintptr_t)b_base),
                    (uint32_t)__builtin_amdgcn_readfirstlane((int)((uintptr_t)b_base >> 32)) & 0xffffu, 0x7fffffffu, 0x00020000u};
    s.kstart = t.kstart;
    return s;
  };
  const uint32_t lds0 = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) char*)smem;
  // LDS destination of load idx in stage 0: m0a / m0b + a compile-time offset
  const uint32_t m0a = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + wave * 1024));
  const uint32_t m0b = (uint32_t)__builtin_amdgcn_readfirstlane((int)(lds0 + STAGE_A + wave * (NN ? PAIR_NN : 1024)));
  constexpr int M0B_STEP = NN ? 4 * PAIR_NN : 4096;
  int istr[NL];  // scalar offset of load idx (idx < TI: operand A, else B) relative to the stage's first byte of its operand
#pragma unroll
  for (int i = 0; i < TI; i++) istr[i] = __builtin_amdgcn_readfirstlane(i * a_istride);
#pragma unroll
  for (int i = 0; i < 8; i++) istr[TI + i] = __builtin_amdgcn_readfirstlane(i * b_istride);
  // Scalars the K loop uses come through an empty asm: the compiler then waits for the kernel-argument loads behind
  // them here, once, instead of keeping a "scalar load may be pending" wait inside the loop, where it would also wait
  // for the fragment reads in flight (which it cannot see).
  int nk_s = nk, kb_mul = BK * (int)p.ldb * 2;
  asm volatile("" : "+s"(nk_s), "+s"(kb_mul));
#pragma unroll
  for (int i = 0; i < NL; i++) asm volatile("" : "+s"(istr[i]));
  // byte offsets (operand A, operand B) of K step k of a tile whose walk starts at kstart
  auto kbase = [&](int kstart, int k, int& ka, int& kb) __attribute__((always_inline)) {
    int kp = kstart + k;
    kp = kp >= nk_s ? kp - nk_s : kp;
    ka = kp * (BK * 2);
    kb = NN ? kp * kb_mul : ka;
  };
  auto set_m0 = [&](uint32_t base, auto OFF) __attribute__((always_inline)) {
    asm volatile("s_add_u32 m0, %0, %1" ::"s"(base), "n"(OFF.value) : "memory", "scc");
  };
  auto issue_load = [&](lf_u32x4 rsrc, uint32_t voff, int soff) __attribute__((always_inline)) {
    asm volatile("buffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(voff), "s"(rsrc), "s"(soff) : "memory");
  };
  // all loads of K step k of the tile behind `src` into stage `stage` (prologue only: no MFMAs to hide behind)
  auto load_stage = [&](const LoadSrc& src, int k, int stage, auto COUNT) __attribute__((always_inline)) {
    int ka, kb;
    kbase(src.kstart, k, ka, kb);
    sfor<COUNT.value>([&](auto I) {
      constexpr int idx = I.value;
      if constexpr (idx < TI) set_m0(m0a + stage * STAGE, std::integral_constant<int, idx * 4096>{});
      else set_m0(m0b + stage * STAGE, std::integral_constant<int, (idx - TI) * M0B_STEP>{});
      asm volatile("s_nop 0" ::: "memory");
      issue_load(idx < TI ? src.ra : src.rb, idx < TI ? a_voff : b_voff, (idx < TI ? ka : kb) + istr[idx]);
    });
  };

  auto lgkm0 = [&]() __attribute__((always_inline)) { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); };
  auto barrier = [&]() __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    lgkm0();
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
  };
  using S0 = integral_constant<int, 0>;
  using S1 = integral_constant<int, 1>;
  constexpr int RDS = TI == 8 ? 3 : 2;   // a fragment read every RDS MFMAs
  constexpr int LDP = NM / NL;           // a tile load every LDP MFMAs of sub-step 1 (256x256 tile: 4; denser issue queues up in the texture addresser there: 2 and 3 measured 2-6 % slower)
  static_assert(RDS * NL <= NM && LDP >= 2, "a sub-step has a gap for every fragment read and two for every tile load");
  const T* __restrict__ Lp = (const T*)p.L;
  T* __restrict__ C = (T*)p.C;
  const uint16_t* bias16 = (const uint16_t*)p.bias;

  // the first two stages of the first tile (three stages: and the first half of the third)
  Tile tile = tile_of(0);
  LoadSrc src = src_of(tile);
  load_stage(src, 0, 0, integral_constant<int, NL>{});
  load_stage(src, 1, 1, integral_constant<int, NL>{});
  if constexpr (NST == 3) load_stage(src, 2, 2, integral_constant<int, NH1>{});

  // Adapter of a wave's rows: rank, skinny operand, multiplier, whether a keep-mask applies.  With a routing table
  // these are two dependent scalar loads (table row, then the segment's pointer), so a tile's lookup is issued while
  // the previous tile computes and costs a latency only for a workgroup's first tile.
  struct Route { int rank; const T* rp; float mult; bool use_mask; };
  auto route_of = [&](int wave_row0) __attribute__((always_inline)) {
    Route r;
    r.rp = (const T*)seg.ptr[0];
    r.rank = seg.rank[0];
    // mult_mode 1 without a keep-mask means no dropout, whatever p says: the term is not rescaled
    r.use_mask = p.mask != nullptr && p.mult_mode == 1 && seg.p > 0.f;
    r.mult = p.mult_mode == 0 ? seg.scale : (r.use_mask ? 1.f / (1.f - seg.p) : 1.f);
    if (seg.table != nullptr) {
      int blk = (p.row0 + wave_row0) / seg.block_size_m;
      blk = min(blk, seg.n_blocks - 1);
      r.rank = seg.table[3 * blk + 0];
      const int fbk = seg.table[3 * blk + 2];
      int sidx = 0;
      for (int i = 1; i < seg.n_seg; i++) sidx = (seg.first_block[i] == fbk) ? i : sidx;
      r.rp = (const T*)seg.ptr[sidx];
      if (p.mult_mode == 0) {
        r.mult = seg.block_scale[blk];
      } else {
        const float pb = seg.block_p[blk];
        r.use_mask = p.mask != nullptr && pb > 0.f;
        r.mult = r.use_mask ? 1.f / (1.f - pb) : 1.f;
      }
    }
    return r;
  };
  constexpr bool has_lora = LORA;   // the launcher picks the LORA instance exactly when there is a term (p.L != nullptr)
  Route route{};
  if (has_lora) route = route_of(tile.m0 + wm * WROWS);
  const int n16 = p.R >> 4;   // chunks of 16 rank columns (one 16x16x16 MFMA step each)

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the first tile's two stages (later tiles: waited for before the epilogue's stores)
  int par = 0;  // LDS stage of the current tile's K step 0 (tiles follow each other through the stages without a gap)
  for (int it = 0; it < n_my; it++) {
    // everything below is scoped to one tile: fragments, accumulators and LoRA operands do not live across tiles
    const Tile nxt_tile = it + 1 < n_my ? tile_of(it + 1) : tile;
    const LoadSrc nxt_src = src_of(nxt_tile);
    const int m0 = tile.m0, n0 = tile.n0;
    const int wrow0 = m0 + wm * WROWS;
    const Route rt = route;
    if (has_lora) route = route_of(nxt_tile.m0 + wm * WROWS);  // in flight during this tile's K loop

    lf_u32x4 fa[2][TI], fb[2][8];
    lf_f32x4 acc[TI][8];
    uint32_t fa_off[2], fb_off[2];
    // one fragment read of sub-step KS of the stage at LDS byte offset `st`, the o-th of its sub-step: first the 8 B
    // fragments, then the TI A fragments
    auto read_one = [&](auto SET, auto KS, uint32_t st, auto ORD) __attribute__((always_inline)) {
      constexpr int idx = ORD.value < 8 ? ORD.value + 8 : ORD.value - 8, set = SET.value, ks = KS.value;   // idx < 8: A fragment idx; else B fragment idx - 8
      if constexpr (idx < 8) {
        const uint32_t ad = fa_off[ks] + st;
        lf_u32x4 tmp;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(tmp) : "v"(ad), "n"(idx * 2048) : "memory");
        fa[set][idx] = tmp;
      } else if constexpr (!NN) {
        const uint32_t ad = fb_off[ks] + st;
        lf_u32x4 tmp;
        asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(tmp) : "v"(ad), "n"((idx - 8) * 2048) : "memory");
        fb[set][idx - 8] = tmp;
      } else {
        const uint32_t ad = fb_off[0] + st;
        lf_u32x2 lo, hi;
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(lo) : "v"(ad), "n"(ks * 16 * PAIR_NN + (idx - 8) * 32) : "memory");
        asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(hi) : "v"(ad), "n"(ks * 16 * PAIR_NN + (idx - 8) * 32 + 512) : "memory");
        fb[set][idx - 8] = lf_u32x4{lo[0], lo[1], hi[0], hi[1]};
      }
    };
    // FIRST: the first MFMA into an accumulator block of a tile takes the constant 0 as its addend and writes the
    // block: no zeroing pass, and nothing of the previous tile has to be cleared
    auto mfma_one = [&](int set, int m, auto FIRST) __attribute__((always_inline)) {
      const int i = m >> 3, j = m & 7;
      if constexpr (FIRST.value) BigOp<T>::mfma_first(acc[i][j], fb[set][j], fa[set][i]);
      else BigOp<T>::mfma(acc[i][j], fb[set][j], fa[set][i]);
    };

    // ------------------------------------------------------------ operands of the LoRA term
    // The term is added at the END of a tile (masked: inside the epilogue's conversion).  Nothing of it may be
    // requested behind the epilogue's stores: loads and stores share one counter and complete out of order with
    // respect to each other, so a wait for such a load would be a wait for the 128 KB of output stored just before.
    // The dX product (NN) therefore requests, during the tile's first K sub-step (the texture addresser is idle
    // there), what it cannot fetch quickly afterwards -- the keep-mask bits of the wave's block, which come
    // from HBM, and the first 16 rows of A_i over the wave's columns, which the MFMA needs transposed -- as
    // direct-to-LDS loads into the wave's own 6 KB behind the stages (the epilogue's band buffer, idle until then):
    // no registers are involved, and the data has landed by the vmcnt(0) of the tile's second K step (K >= 128).
    // The L fragments and the forward's B_i fragments are plain 8-byte loads issued right behind the K loop; they come
    // from L2, and their wait coincides with the wait for the next tile's stages that precedes the first store anyway.
    const bool sel = NN && LORA && p.mult_mode == 1 && rt.use_mask;   // keep-mask applies to this wave's rows
    // This wave's area.  Three stages: in the stage of the tile's last step, behind the first half of a stage's loads
    // (operand B from its third load on): the last step's own reads of it end at its barrier, and the next load that
    // writes there is issued in the next tile's first step.  The dX product's operands are requested into it during
    // the last step's second sub-step and waited for right behind the K loop.
    const uint32_t last_stage = (uint32_t)((par + nk - 1) % 3) * STAGE;
    const uint32_t area = NST == 2 ? lds0 + EP_OFF + wave * EP_WAVE : lds0 + last_stage + STAGE_A + 2 * M0B_STEP + wave * EP_WAVE;
    static_assert(NST == 2 || 4 * EP_WAVE <= 6 * 4096, "the four areas fit the second half of a stage's B part");
    const uint32_t area_r = area, area_m = area + 4096;   // A_i rows, keep bits
    uint32_t rfl_voff = 0, mk_voff = 0;
    lf_u32x4 rsrcR{}, rsrcM{};
    int rfl_s0 = 0, rfl_step = 0, mk_step = 0;
    if constexpr (NN && LORA) {
      int sl = lane;
      asm volatile("" : "+v"(sl));   // lane-dependent offsets are derived inside the tile loop (not hoisted and spilled)
      // A_i [rank, N]: load q covers rank rows 4q .. 4q+3 (lane>>4) x 128 columns (16 bytes per lane); rows beyond
      // the adapter's rank lie beyond the buffer's end and read as zeros
      const uint64_t rb = (uint64_t)(uintptr_t)rt.rp;
      rsrcR = lf_u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)rb), (uint32_t)__builtin_amdgcn_readfirstlane((int)(rb >> 32)) & 0xffffu,
                       (uint32_t)__builtin_amdgcn_readfirstlane(rt.rank * p.N * 2), 0x00020000u};
      rfl_voff = (uint32_t)(((sl >> 4) * p.N + (sl & 15) * 8) * 2);
      rfl_s0 = (n0 + wn * 128) * 2;
      rfl_step = 4 * p.N * 2;
      // keep bits: load q covers rows 64q + lane, 16 bytes (128 columns) each (TI / 4 loads).  Without a mask they read the
      // head of L (an inline-assembly statement under a run-time condition does not compile inside a generic lambda)
      const uint64_t mb = sel ? (uint64_t)(uintptr_t)(p.mask + (int64_t)wrow0 * p.ldmask + ((n0 + wn * 128) >> 3)) : (uint64_t)(uintptr_t)Lp;
      rsrcM = lf_u32x4{(uint32_t)__builtin_amdgcn_readfirstlane((int)mb), (uint32_t)__builtin_amdgcn_readfirstlane((int)(mb >> 32)) & 0xffffu, 0x7fffffffu, 0x00020000u};
      mk_voff = sel ? (uint32_t)(sl * (int)p.ldmask) : 0u;
      mk_step = sel ? 64 * (int)p.ldmask : 0;
    }
    constexpr int N_LORA_LOADS = (NN && LORA) ? 4 + TI / 4 : 0;
    // load `q` of the list above, issued in gaps 2q (M0) and 2q+1 of the tile's first sub-step
    auto lora_m0 = [&](auto Q) __attribute__((always_inline)) {
      if constexpr (Q.value < 4) set_m0(area_r, integral_constant<int, Q.value * 1024>{});
      else set_m0(area_m, integral_constant<int, (Q.value - 4) * 1024>{});
    };
    auto lora_load = [&](auto Q) __attribute__((always_inline)) {
      constexpr int q = Q.value;
      // named once outside inline assembly: this clang does not capture a variable that a generic lambda uses in
      // assembly operands only.  The nop in front of each load: its scalar operands may have been restored from a
      // vector register lane (v_readlane) by the instruction before, and a scalar register written by the vector ALU
      // needs five wait states before a memory instruction reads it -- a hazard the compiler resolves for its own
      // instructions but cannot see inside inline assembly (the load would go out with the register's old value: a
      // wild address).  The K loop's loads take their scalar operands from scalar arithmetic only.
      const uint32_t rfl_voff_ = rfl_voff, mk_voff_ = mk_voff;
      const lf_u32x4 rsrcR_ = rsrcR, rsrcM_ = rsrcM;
      if constexpr (q < 4) {
        const int so = rfl_s0 + q * rfl_step;
        asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(rfl_voff_), "s"(rsrcR_), "s"(so) : "memory");
      } else {
        const int so = (q - 4) * mk_step;
        asm volatile("s_nop 4\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" ::"v"(mk_voff_), "s"(rsrcM_), "s"(so) : "memory");
      }
    };

    // ------------------------------------------------------------ fragment addresses
    // A (and NT B): lane reads granule ks*4+kg of row l16 of a 16-row block; blocks are 2048 bytes apart.  Derived
    // from an opaque copy of the lane id, every tile
    {
      int fl = lane;
      asm volatile("" : "+v"(fl));
      const int l16 = fl & 15, kg = fl >> 4;
      const int key = (l16 >> 1) & 7;
#pragma unroll
      for (int ks = 0; ks < 2; ks++) fa_off[ks] = lds0 + (wm * WROWS + l16) * 128 + (((ks * 4 + kg) ^ key) << 4);
      if constexpr (!NN) {
#pragma unroll
        for (int ks = 0; ks < 2; ks++) fb_off[ks] = lds0 + STAGE_A + (wn * 128 + l16) * 128 + (((ks * 4 + kg) ^ key) << 4);
      } else {
        // ds_read_b64_tr_b16: within a 16-lane group, lane 4j+c addresses row j, columns 4c..4c+3 and receives column
        // (lane&15), rows 0..3.  Group kg takes k-rows kg*8 + j4 (and +4: the other row of the pair, 512 bytes on);
        // sub-step ks: +32 rows.  k-row r = 32 ks + 16 b4 + 8 b3 + 4 hh + j4 lives in pair j4 + 4 b3 + 8 (b4 + 2 ks): the
        // eight rows that 32 lanes read together sit in eight pairs, whose paddings put them on different banks
        const int j4 = l16 >> 2, c = l16 & 3;
        fb_off[0] = lds0 + STAGE_A + (j4 + 4 * (kg & 1) + 8 * (kg >> 1)) * PAIR_NN + (wn * 128 + 4 * c) * 2;
        fb_off[1] = fb_off[0];
      }
    }

    // ------------------------------------------------------------ K loop
    barrier();   // both stages of this tile's first two K steps are in LDS (every wave has waited for its loads)
    {
      const uint32_t st = par * STAGE;
      sfor<NL>([&](auto I) { read_one(S0{}, S0{}, st, I); });
    }
    lgkm0();
    // K step s lives in stage (par + s) & 1.  Sub-step 1 of step s refills that stage with step s+2 of this tile; the
    // last two steps prefetch the first two steps of the next tile instead (of this tile again when none follows:
    // loads that nothing consumes keep the step body uniform).  Gap schedule of a step (one MFMA = one gap of three
    // issue slots): sub-step 0: a fragment read every third gap, the scalar offset of one load of the coming stage
    // every fourth (first step of a tile: a load of the LoRA operands in every gap that has one); sub-step 1: a
    // fragment read every third gap, M0 in gap 4i, load i in gap 4i+1.
    // FIRST (a tile's step 0): its MFMAs of sub-step 0 write the accumulators, and there is nothing to wait for at the
    // barrier -- step 1's stage was waited for before the previous tile's stores; a vmcnt(0) here would wait for those
    // stores, which by the second step's wait have long been acknowledged.
    auto k_step = [&](int s, const LoadSrc& ld, int lk, auto FIRST) __attribute__((always_inline)) {
      const int cs = (par + s) & 1;
      const uint32_t cur = cs * STAGE, nxt = STAGE - cur;
      int ka, kb;
      kbase(ld.kstart, lk, ka, kb);
      const uint32_t ma = m0a + cur, mb = m0b + cur;
      int soff[NL];
      sfor<NM>([&](auto MM) {
        constexpr int m = MM.value;
        if constexpr (m % RDS == 0 && m / RDS < NL) read_one(S1{}, S1{}, cur, integral_constant<int, m / RDS>{});
        if constexpr (m % LDP == LDP / 2 && m / LDP < NL) soff[m / LDP] = (m / LDP < TI ? ka : kb) + istr[m / LDP];
        if constexpr (FIRST.value && m < 2 * N_LORA_LOADS) {
          if constexpr (m % 2 == 0) lora_m0(integral_constant<int, m / 2>{});
          else lora_load(integral_constant<int, m / 2>{});
        }
        mfma_one(0, m, FIRST);
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (!FIRST.value) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this wave's loads of step s+1 (issued a sub-step ago) have landed
      barrier();
      sfor<NM>([&](auto MM) {
        constexpr int m = MM.value;
        if constexpr (m % RDS == 0 && m / RDS < NL) read_one(S0{}, S0{}, nxt, integral_constant<int, m / RDS>{});
        if constexpr (m % LDP == 0 && m / LDP < NL) {
          if constexpr (m / LDP < TI) set_m0(ma, integral_constant<int, (m / LDP) * 4096>{});
          else set_m0(mb, integral_constant<int, (m / LDP - TI) * M0B_STEP>{});
        }
        if constexpr (m % LDP == 1 && m / LDP < NL) issue_load(m / LDP < TI ? ld.ra : ld.rb, m / LDP < TI ? a_voff : b_voff, soff[m / LDP]);
        mfma_one(1, m, std::false_type{});
        __builtin_amdgcn_sched_barrier(0);
      });
      __builtin_amdgcn_sched_barrier(0);
      lgkm0();
      __builtin_amdgcn_sched_barrier(0);
    };
    // ------------------------------------------------------------ K loop over three stages (128-row tile)
    // Step s lives in stage (par + s) % 3.  Its sub-step 0 issues the second half of step s+2's loads into the stage
    // that died at the barrier of step s-1, its sub-step 1 the first half of step s+3's into its own stage, dead since
    // this step's barrier: a stage's loads are issued over a whole step and have another step to land.  At the barrier
    // of step s the loads of step s+1 must have landed: all but the 12 issued last.  Steps beyond the tile's last one
    // are the next tile's first ones.  FIRST (a tile's step 0) waits for nothing: what it needs was waited for before
    // the previous tile's stores (or the kernel's first loads), and a counted wait here would wait for those stores.
    uint32_t cst = (uint32_t)par * STAGE;   // byte offset of the current step's stage
    auto k_step3 = [&](const LoadSrc& l2, int k2, const LoadSrc& l3, int k3, auto FIRST, auto LAST) __attribute__((always_inline)) {
      const uint32_t cur = cst;
      const uint32_t nx1 = cur + STAGE >= 3 * STAGE ? cur + STAGE - 3 * STAGE : cur + STAGE;
      const uint32_t nx2 = nx1 + STAGE >= 3 * STAGE ? nx1 + STAGE - 3 * STAGE : nx1 + STAGE;
      int ka2, kb2, ka3, kb3;
      kbase(l2.kstart, k2, ka2, kb2);
      kbase(l3.kstart, k3, ka3, kb3);
      const uint32_t mb2 = m0b + nx2, ma3 = m0a + cur, mb3 = m0b + cur;
      int so = 0;
      sfor<NM>([&](auto MM) {
        constexpr int m = MM.value;
        if constexpr (m % RDS == 0 && m / RDS < NL) read_one(S1{}, S1{}, cur, integral_constant<int, m / RDS>{});
        // second half of step s+2: loads NH1 .. NL-1 (all of operand B), M0 and the scalar offset in gap 5i+1, the load in gap 5i+2
        if constexpr (m % 5 == 1 && m / 5 < NL - NH1) {
          constexpr int idx = NH1 + m / 5;
          so = kb2 + istr[idx];
          set_m0(mb2, integral_constant<int, (idx - TI) * M0B_STEP>{});
        }
        if constexpr (m % 5 == 2 && m / 5 < NL - NH1) issue_load(l2.rb, b_voff, so);
        mfma_one(0, m, FIRST);
        __builtin_amdgcn_sched_barrier(0);
      });
      if constexpr (!FIRST.value) asm volatile("s_waitcnt vmcnt(12)" ::: "memory");
      barrier();
      sfor<NM>([&](auto MM) {
        constexpr int m = MM.value;
        if constexpr (m % RDS == 0 && m / RDS < NL) read_one(S0{}, S0{}, nx1, integral_constant<int, m / RDS>{});
        // first half of step s+3: loads 0 .. NH1-1
        if constexpr (m % 5 == 1 && m / 5 < NH1) {
          constexpr int idx = m / 5;
          so = (idx < TI ? ka3 : kb3) + istr[idx];
          if constexpr (idx < TI) set_m0(ma3, integral_constant<int, idx * 4096>{});
          else set_m0(mb3, integral_constant<int, (idx - TI) * M0B_STEP>{});
        }
        if constexpr (m % 5 == 2 && m / 5 < NH1) issue_load(m / 5 < TI ? l3.ra : l3.rb, m / 5 < TI ? a_voff : b_voff, so);
        // the tile's last step: the dX product's LoRA operands, M0 in gap 5q+3, the load in gap 5q+4
        if constexpr (LAST.value && m % 5 >= 3 && m / 5 < N_LORA_LOADS) {
          if constexpr (m % 5 == 3) lora_m0(integral_constant<int, m / 5>{});
          else lora_load(integral_constant<int, m / 5>{});
        }
        mfma_one(1, m, std::false_type{});
        __builtin_amdgcn_sched_barrier(0);
      });
      __builtin_amdgcn_sched_barrier(0);
      lgkm0();
      __builtin_amdgcn_sched_barrier(0);
      cst = nx1;
    };
    // K step q of this tile, or, beyond its last, step q - nk of the next: descriptors picked with scalar selects
    auto pick = [&](int q, LoadSrc& l, int& k) __attribute__((always_inline)) {
      const bool own = q < nk;
#pragma unroll
      for (int d = 0; d < 4; d++) { l.ra[d] = own ? src.ra[d] : nxt_src.ra[d]; l.rb[d] = own ? src.rb[d] : nxt_src.rb[d]; }
      l.kstart = own ? src.kstart : nxt_src.kstart;
      k = own ? q : q - nk;
    };
    if constexpr (NST == 2) {
      // step 0 loads this tile's step 2, or (nk == 2) the next tile's step 0; descriptors picked with scalar selects
      const bool own = nk > 2;
      LoadSrc l0;
#pragma unroll
      for (int d = 0; d < 4; d++) { l0.ra[d] = own ? src.ra[d] : nxt_src.ra[d]; l0.rb[d] = own ? src.rb[d] : nxt_src.rb[d]; }
      l0.kstart = own ? src.kstart : nxt_src.kstart;
      k_step(0, l0, own ? 2 : 0, std::true_type{});
      int s = 1;
      for (; s + 2 < nk; s++) k_step(s, src, s + 2, std::false_type{});
      for (; s < nk; s++) k_step(s, nxt_src, s + 2 - nk, std::false_type{});
      par = (par + nk) & 1;
    } else {
      // (nk >= 4: the launcher's condition for this tile)
      k_step3(src, 2, src, 3, std::true_type{}, std::false_type{});
      int s = 1;
      for (; s + 3 < nk; s++) k_step3(src, s + 2, src, s + 3, std::false_type{}, std::false_type{});
      for (; s + 1 < nk; s++) {
        LoadSrc l2, l3;
        int k2, k3;
        pick(s + 2, l2, k2);
        pick(s + 3, l3, k3);
        k_step3(l2, k2, l3, k3, std::false_type{}, std::false_type{});
      }
      k_step3(nxt_src, 1, nxt_src, 2, std::false_type{}, std::true_type{});   // step nk-1
      par = (par + nk) % 3;
      // the operands requested in the last sub-step (and with them the next tile's first loads)
      if constexpr (N_LORA_LOADS > 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    mfma_fence();

    // ------------------------------------------------------------ LoRA term: operands; forward: 64 MFMAs per chunk onto the
    // accumulators (dX: the term is formed per block row inside the epilogue below, from up to two chunks = 32 rank columns)
    lf_u32x2 rf0[8], lv0[TI], rf1[8], lv1[TI];
    lf_u32x4 mw[TI];
    if constexpr (LORA) {
      int sl = lane;
      asm volatile("" : "+v"(sl));
      const int l16 = sl & 15, kg = sl >> 4;
      const T* rp = rt.rp;
      const int rank = rt.rank;
      const __amdgpu_buffer_rsrc_t rsrcRc = __builtin_amdgcn_make_buffer_rsrc((void*)rp, 0, 0x7fffffff, 0x00020000);
      // chunk t of the operands: 16 rank columns, two registers per 16x16x16 fragment.  FROM_LDS: the A_i fragments of
      // chunk 0 of the dX product are transposing reads of the rows that landed in the wave's LDS area (within a
      // 16-lane group, lane 4j+c addresses row j, columns 4c..4c+3 and receives column lane&15, rows 0..3).
      auto load_chunk = [&](int t, lf_u32x2 (&rf)[8], lf_u32x2 (&lv)[TI], auto FROM_LDS) __attribute__((always_inline)) {
        const int r0 = t * 16 + kg * 4;
        const int rcc = r0 < rank ? r0 : 0;   // lanes beyond the rank re-read the first columns; zeroed in prep_chunk
#pragma unroll
        for (int i = 0; i < TI; i++) lv[i] = *(const lf_u32x2*)(Lp + (int64_t)(wrow0 + i * 16 + l16) * p.R + r0);
        if constexpr (FROM_LDS.value) {
          const uint32_t ad = area_r + (kg * 4 + (l16 >> 2)) * 256 + (l16 & 3) * 8;
          lf_u32x2 t0, t1, t2, t3, t4, t5, t6, t7;
          asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(t0) : "v"(ad) : "memory");
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:32" : "=v"(t1) : "v"(ad) : "memory");
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:64" : "=v"(t2) : "v"(ad) : "memory");
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:96" : "=v"(t3) : "v"(ad) : "memory");
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:128" : "=v"(t4) : "v"(ad) : "memory");
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:160" : "=v"(t5) : "v"(ad) : "memory");
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:192" : "=v"(t6) : "v"(ad) : "memory");
          asm volatile("ds_read_b64_tr_b16 %0, %1 offset:224" : "=v"(t7) : "v"(ad) : "memory");
          asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(t0), "+v"(t1), "+v"(t2), "+v"(t3), "+v"(t4), "+v"(t5), "+v"(t6), "+v"(t7) :: "memory");
          rf[0] = t0; rf[1] = t1; rf[2] = t2; rf[3] = t3; rf[4] = t4; rf[5] = t5; rf[6] = t6; rf[7] = t7;
        } else {
#pragma unroll
          for (int j = 0; j < 8; j++) {
            const int gn = n0 + wn * 128 + j * 16 + l16;
            if constexpr (!NN) {
              rf[j] = *(const lf_u32x2*)(rp + (int64_t)gn * rank + rcc);
            } else {
              const uint32_t voff = (uint32_t)((rcc * p.N + gn) * 2);
              uint32_t e[4];
#pragma unroll
              for (int k = 0; k < 4; k++) e[k] = __builtin_amdgcn_raw_buffer_load_b16(rsrcRc, voff, k * p.N * 2, 0);
              rf[j] = lf_u32x2{e[0] | (e[1] << 16), e[2] | (e[3] << 16)};
            }
          }
        }
      };
      // lanes whose rank columns lie beyond the adapter's rank feed zeros; the forward scale goes into the 16-bit L
      // fragment (fp32 product, one rounding; exact for powers of two)
      auto prep_chunk = [&](int t, lf_u32x2 (&rf)[8], lf_u32x2 (&lv)[TI]) __attribute__((always_inline)) {
        const bool in_r = t * 16 + kg * 4 < rank;
#pragma unroll
        for (int j = 0; j < 8; j++)
#pragma unroll
          for (int d = 0; d < 2; d++) rf[j][d] = in_r ? rf[j][d] : 0u;
        if (p.mult_mode == 0 && rt.mult != 1.f) {
#pragma unroll
          for (int i = 0; i < TI; i++)
#pragma unroll
            for (int d = 0; d < 2; d++)
              lv[i][d] = BigOp<T>::pack2(BigOp<T>::to_float((uint16_t)(lv[i][d] & 0xffffu)) * rt.mult, BigOp<T>::to_float((uint16_t)(lv[i][d] >> 16)) * rt.mult);
        }
        // The MFMAs are inline assembly, which the compiler's hazard recogniser does not see: a vector ALU result
        // needs wait states before an MFMA reads it.  The nop takes the operands as in/outs, so every instruction
        // that produces them stays in front of it and every MFMA behind.
        if constexpr (TI == 8) {
          asm volatile("s_nop 3" : "+v"(rf[0]), "+v"(rf[1]), "+v"(rf[2]), "+v"(rf[3]), "+v"(rf[4]), "+v"(rf[5]), "+v"(rf[6]), "+v"(rf[7]),
                                   "+v"(lv[0]), "+v"(lv[1]), "+v"(lv[2]), "+v"(lv[3]), "+v"(lv[4]), "+v"(lv[5]), "+v"(lv[6]), "+v"(lv[7]));
        } else {
          asm volatile("s_nop 3" : "+v"(rf[0]), "+v"(rf[1]), "+v"(rf[2]), "+v"(rf[3]), "+v"(rf[4]), "+v"(rf[5]), "+v"(rf[6]), "+v"(rf[7]),
                                   "+v"(lv[0]), "+v"(lv[1]), "+v"(lv[2]), "+v"(lv[3]));
        }
      };
      if constexpr (NN) {
        // dX product: the term is formed in the epilogue, block row by block row, under the keep bits of the wave's
        // block (one 16-byte row piece per block row, from the LDS area; all ones where no mask applies)
        const uint32_t ad = area_m + l16 * 16;
        lf_u32x4 m0_, m1_, m2_, m3_, m4_{}, m5_{}, m6_{}, m7_{};
        asm volatile("ds_read_b128 %0, %1" : "=v"(m0_) : "v"(ad) : "memory");
        asm volatile("ds_read_b128 %0, %1 offset:256" : "=v"(m1_) : "v"(ad) : "memory");
        asm volatile("ds_read_b128 %0, %1 offset:512" : "=v"(m2_) : "v"(ad) : "memory");
        asm volatile("ds_read_b128 %0, %1 offset:768" : "=v"(m3_) : "v"(ad) : "memory");
        if constexpr (TI == 8) {
          asm volatile("ds_read_b128 %0, %1 offset:1024" : "=v"(m4_) : "v"(ad) : "memory");
          asm volatile("ds_read_b128 %0, %1 offset:1280" : "=v"(m5_) : "v"(ad) : "memory");
          asm volatile("ds_read_b128 %0, %1 offset:1536" : "=v"(m6_) : "v"(ad) : "memory");
          asm volatile("ds_read_b128 %0, %1 offset:1792" : "=v"(m7_) : "v"(ad) : "memory");
        }
        load_chunk(0, rf0, lv0, std::true_type{});
        if constexpr (TI == 8) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(m0_), "+v"(m1_), "+v"(m2_), "+v"(m3_), "+v"(m4_), "+v"(m5_), "+v"(m6_), "+v"(m7_) :: "memory");
        else asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(m0_), "+v"(m1_), "+v"(m2_), "+v"(m3_) :: "memory");
        const lf_u32x4 ones = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
        mw[0] = sel ? m0_ : ones; mw[1] = sel ? m1_ : ones; mw[2] = sel ? m2_ : ones; mw[3] = sel ? m3_ : ones;
        if constexpr (TI == 8) { mw[4] = sel ? m4_ : ones; mw[5] = sel ? m5_ : ones; mw[6] = sel ? m6_ : ones; mw[7] = sel ? m7_ : ones; }
        prep_chunk(0, rf0, lv0);
        if (n16 > 1) { load_chunk(1, rf1, lv1, std::false_type{}); prep_chunk(1, rf1, lv1); }
      } else {
        load_chunk(0, rf0, lv0, std::false_type{});
        prep_chunk(0, rf0, lv0);
#pragma unroll
        for (int i = 0; i < TI; i++)
#pragma unroll
          for (int j = 0; j < 8; j++) BigOp<T>::mfma16(acc[i][j], rf0[j], lv0[i]);
        for (int t = 1; t < n16; t++) {
          load_chunk(t, rf1, lv1, std::false_type{});
          prep_chunk(t, rf1, lv1);
#pragma unroll
          for (int i = 0; i < TI; i++)
#pragma unroll
            for (int j = 0; j < 8; j++) BigOp<T>::mfma16(acc[i][j], rf1[j], lv1[i]);
        }
        mfma_fence();
      }
    }

    // ------------------------------------------------------------ epilogue: (masked LoRA term,) bias, convert, 16-row bands through LDS
    auto epilogue = [&](auto MASKED) __attribute__((always_inline)) {
      // lane-dependent addresses are derived from an opaque copy of the lane id: computed here, every tile, in a few
      // instructions -- otherwise the compiler hoists a hundred address registers out of the tile loop and spills them
      int ln = lane;
      asm volatile("" : "+v"(ln));
      const int e16 = ln & 15, ekg = ln >> 4;
      const uint32_t ep_lds = area;
      lf_u32x2 bvp[8];
#pragma unroll
      for (int j = 0; j < 8; j++) bvp[j] = lf_u32x2{0u, 0u};
      if (bias16 != nullptr) {
#pragma unroll
        for (int j = 0; j < 8; j++) bvp[j] = *(const lf_u32x2*)(bias16 + n0 + wn * 128 + j * 16 + ekg * 4);
      }
      const int orow = ln >> 4, og = ln & 15;  // on the way out: 16 lanes per 256-byte row, 4 rows per instruction
      T* crow = C + (int64_t)(wrow0 + orow) * p.ldc + n0 + wn * 128 + og * 8;
      // Masked term: the product of block row i (8 blocks, 16x16x16 MFMAs per chunk of 16 rank columns) goes to
      // ordinary vector registers, P[i & 1]; block row i+1 is multiplied while block row i is converted, which also
      // covers the wait states between an MFMA and the vector instructions that read its result.  The lane's keep
      // bits of block (i, j) are bits (j&1)*16 + kg*4 .. +3 of dword j>>1 of the row piece mw[i].
      lf_f32x4 P[2][8];
      const float mult = p.mult_mode == 1 ? rt.mult : 1.f;   // (a forward scale is already in the L fragments)
      const uint32_t bsh = (uint32_t)ekg * 4;
      auto p_row = [&](auto I) __attribute__((always_inline)) {
        constexpr int i = I.value;
#pragma unroll
        for (int j = 0; j < 8; j++) BigOp<T>::mfma16_v0(P[i & 1][j], rf0[j], lv0[i]);
        if (n16 > 1) {
#pragma unroll
          for (int j = 0; j < 8; j++) BigOp<T>::mfma16_v(P[i & 1][j], rf1[j], lv1[i]);
        }
      };
      if constexpr (MASKED.value) p_row(integral_constant<int, 0>{});
      sfor<TI>([&](auto I) {
        constexpr int i = I.value;
        uint32_t mws[4] = {0u, 0u, 0u, 0u};
        if constexpr (MASKED.value) {
          if constexpr (i + 1 < TI) p_row(integral_constant<int, i + 1>{});
          lf_f32x4(&tm)[8] = P[i & 1];
          // wait states between the MFMAs of this block row (a block row of MFMAs ago, except for the last) and the
          // vector instructions that read their results
          asm volatile("s_nop 7\n\ts_nop 7\n\ts_nop 7"
                       : "+v"(tm[0]), "+v"(tm[1]), "+v"(tm[2]), "+v"(tm[3]), "+v"(tm[4]), "+v"(tm[5]), "+v"(tm[6]), "+v"(tm[7]));
#pragma unroll
          for (int q = 0; q < 4; q++) mws[q] = mw[i][q] >> bsh;
        }
        // band = the 16 rows of accumulator block row i; band row r, granule g (16 bytes = 8 columns) at slot g ^ r
#pragma unroll
        for (int j = 0; j < 8; j++) {
          // a definition right in front of the use: the copies out of the accumulation registers cannot rise above it
          // (without it the masked variant reads all 256 up front, into registers it does not have)
          if constexpr (MASKED.value) asm volatile("" : "+a"(acc[i][j]));
          lf_f32x4 a = acc[i][j];
          if constexpr (MASKED.value) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
              const uint32_t keep = (uint32_t)__builtin_amdgcn_sbfe((int)mws[j >> 1], (j & 1) * 16 + e, 1);   // 0 or all ones
              // (the element goes through a scalar first: __builtin_bit_cast applied directly to an element expression of
              // a vector reads element 0 for every index with this compiler)
              const float pe = P[i & 1][j][e];
              const float pm = __builtin_bit_cast(float, __builtin_bit_cast(uint32_t, pe) & keep);
              a[e] = __builtin_fmaf(pm, mult, a[e]);   // 1/(1-p) in fp32
            }
          }
          const float b0 = BigOp<T>::to_float((uint16_t)(bvp[j][0] & 0xffffu)), b1 = BigOp<T>::to_float((uint16_t)(bvp[j][0] >> 16));
          const float b2 = BigOp<T>::to_float((uint16_t)(bvp[j][1] & 0xffffu)), b3 = BigOp<T>::to_float((uint16_t)(bvp[j][1] >> 16));
          const lf_u32x2 o = {BigOp<T>::pack2(a[0] + b0, a[1] + b1), BigOp<T>::pack2(a[2] + b2, a[3] + b3)};
          const int g = j * 2 + (ekg >> 1);
          const uint32_t ad = ep_lds + e16 * 256 + ((g ^ e16) << 4) + (ekg & 1) * 8;
          asm volatile("ds_write_b64 %0, %1" ::"v"(ad), "v"(o) : "memory");
        }
        lf_u32x4 v[4];
#pragma unroll
        for (int rr = 0; rr < 4; rr++) {
          const int row = rr * 4 + orow;
          const uint32_t ad = ep_lds + row * 256 + ((og ^ row) << 4);
          asm volatile("ds_read_b128 %0, %1" : "=v"(v[rr]) : "v"(ad) : "memory");
        }
        lgkm0();
        // Before the first store: the next tile's first two stages have landed (requested in this tile's last two K
        // steps).  Waiting here, not at the next tile's start, keeps the stores out of the wait.
        if constexpr (i == 0) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
        // non-temporal: the output is not read again by this kernel; stored this way it leaves the L2 to the operand
        // panels
        for (int rr = 0; rr < 4; rr++) __builtin_nontemporal_store(v[rr], (lf_u32x4*)(crow + (int64_t)(i * 16 + rr * 4) * p.ldc));
        __builtin_amdgcn_sched_barrier(0);  // one band at a time: the scheduler otherwise reads all 256 accumulators up front
      });
    };
    epilogue(std::bool_constant<NN && LORA>{});
    tile = nxt_tile;
    src = nxt_src;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the last, unconsumed prefetches
#endif
}

template <typename T, bool NN, bool LORA, int TI>
int launch_big(LfGemmParams p, const LfSegTable& seg, int max_wgs, hipStream_t st) {
  constexpr int BM = TI * 32;
  p.grid_m = (p.M + BM - 1) / BM;
  p.grid_n = (p.N + BN - 1) / BN;
  auto kern = gemm_big_kernel<T, NN, LORA, TI>;
  static LfLdsFlags lds_ok;
  constexpr int SMEM_BYTES = Lds<NN, TI>::BYTES;
  if (!lf_allow_lds(kern, SMEM_BYTES, lds_ok)) return LF_ELAUNCH;
  // Tile order: an XCD's 32 concurrent tiles form a block of group_m tile rows x 32 / group_m columns.  8 x 4 fetches
  // the fewest operand panels (8 + 4).  With a long K and at most 16 tile columns the left operand does not fit the
  // 256 MB memory-side cache and every pass over it is an HBM pass: 2 rows x 16 columns read it once per round
  // (and as 16 neighbouring 128-byte pieces per row at a time) and leave the re-reads to the right operand, which the
  // cache holds (16384x4096x14336: 1614 -> 1554 us; 16384x4096x28672: 3010 -> 2964 us; at K = 6144 it loses 8 %).
  p.group_m = (p.K >= 8192 && p.grid_n <= 16) ? 2 : 8;
  const long total = (long)p.grid_m * p.grid_n;
  const int grid = (int)(total < max_wgs ? total : max_wgs);
  return lf_launch(kern, dim3(grid), dim3(256), SMEM_BYTES, st, p, seg);
}

std::atomic<int> cu_count[64];

}  // namespace

// Compute units of the current device (one persistent workgroup each), looked up once per device.
int lf_cu_count() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  int n = cu_count[dev].load(std::memory_order_acquire);
  if (n <= 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    cu_count[dev].store(n, std::memory_order_release);
  }
  return n;
}

template <typename T, int TI>
int launch_big_ti(const LfGemmParams& p, const LfSegTable& seg, bool nn, int wgs, hipStream_t st) {
  if (p.L != nullptr) return nn ? launch_big<T, true, true, TI>(p, seg, wgs, st) : launch_big<T, false, true, TI>(p, seg, wgs, st);
  return nn ? launch_big<T, true, false, TI>(p, seg, wgs, st) : launch_big<T, false, false, TI>(p, seg, wgs, st);
}

int lf_launch_gemm_big(const LfGemmParams& p, const LfSegTable& seg, bool nn, int dtype, int tile_rows, hipStream_t st) {
  if (tile_rows != 256 && tile_rows != 128) return LF_EINVAL;
  // edge tiles are shifted inwards; the K loop runs over two stages (256 rows) or three (128 rows: at least four K steps)
  if (p.K % BK != 0 || p.K < (tile_rows == 256 ? 2 : 4) * BK || p.M < tile_rows || p.N < BN || p.N % 8 != 0) return LF_ESHAPE;
  // the rows of a wave (half a tile's) lie in one routing block, also in a shifted edge tile
  const int wrows = tile_rows / 2;
  if (seg.table != nullptr && (seg.block_size_m % wrows != 0 || p.M % wrows != 0)) return LF_ESHAPE;
  // the keep-mask comes bit-packed (16 bytes per 128 columns of a row); the dX product forms its term from up to 32 rank columns
  if (p.mask != nullptr && (!p.mask_bits || p.N % 128 != 0 || p.ldmask % 4 != 0)) return LF_ESHAPE;
  if (nn && p.L != nullptr && p.R > 32) return LF_ESHAPE;
  const int wgs = lf_cu_count();
  if (dtype == LF_BF16) return tile_rows == 256 ? launch_big_ti<__bf16, 8>(p, seg, nn, wgs, st) : launch_big_ti<__bf16, 4>(p, seg, nn, wgs, st);
  if (dtype == LF_F16) return tile_rows == 256 ? launch_big_ti<_Float16, 8>(p, seg, nn, wgs, st) : launch_big_ti<_Float16, 4>(p, seg, nn, wgs, st);
  return LF_EINVAL;
}
