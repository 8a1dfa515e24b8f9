// Shared declarations for the gfx950 LoRA-linear kernels (internal; the public C ABI is
// include/lorafusion_hip.h).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <atomic>
#include "../../include/lorafusion_hip.h"  // error codes, dtype ids, LF_MAX_SEG

#define LF_MAX_RANK 128

typedef __bf16 lf_bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 lf_f16x8 __attribute__((ext_vector_type(8)));
typedef float lf_f32x16 __attribute__((ext_vector_type(16)));
typedef float lf_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t lf_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t lf_u32x2 __attribute__((ext_vector_type(2)));
typedef short lf_s16x4 __attribute__((ext_vector_type(4)));

// Per-launch routing of token blocks to adapters.  `table` == nullptr means one adapter
// over all rows (ptr[0], rank[0]); otherwise block b = row / block_size_m has
// (rank, valid_rows, first_block) = table[3b..3b+2] and belongs to the segment s with
// first_block[s] == table[3b+2].
struct LfSegTable {
  const void* ptr[LF_MAX_SEG];   // per-segment skinny operand (B_i, A_i, ...)
  void* out[LF_MAX_SEG];         // per-segment output (dA_i, dB_i) where a kernel has one
  int first_block[LF_MAX_SEG];
  int rank[LF_MAX_SEG];
  int n_seg;
  int block_size_m;
  int n_blocks;
  const int32_t* table;          // device int32 [n_blocks,3] or nullptr
  const float* block_scale;      // device f32 [n_blocks] or nullptr
  const float* block_p;          // device f32 [n_blocks] or nullptr
  float scale;                   // used when table == nullptr
  float p;                       // used when table == nullptr
};

struct LfGemmParams {
  const void* A;      // [M,K] row-major, lda
  const void* B;      // NT: [N,K] row-major; NN: [K,N] row-major; ldb
  void* C;            // [M,N], ldc
  const void* bias;   // [N] or nullptr
  int M, N, K;
  int64_t lda, ldb, ldc;
  const void* L;      // [M,R] skinny left operand of the LoRA term (S or dS), or nullptr
  int R;              // columns of L (multiple of 16)
  const uint8_t* mask;  // [M,N] keep-mask applied to the LoRA term (dX path) or nullptr
  int64_t ldmask;     // bytes between mask rows
  int mask_bits;      // 0: one byte per element; 1: one bit per element (element n of a row = bit n & 7 of byte n >> 3)
  int mult_mode;      // 0: LoRA term * scale ; 1: LoRA term * 1/(1-p), masked where p > 0
  int grid_m, grid_n;
  int row0;           // global row of local row 0 (routing lookup when a launch covers a row range)
  int group_m;        // persistent kernel: tile rows per group of its tile order (set by its launcher)
  // Split contraction (launches with few tiles and a long K; set by lf_launch_gemm): workgroup (x, y) contracts the
  // K steps [y * ks_steps, (y + 1) * ks_steps) of tile x and writes its fp32 sums to ks_ws[y][M][N]; a second
  // kernel adds the ksplit slices in index order.  ks_ws / ks_ws_bytes come from the caller (nullptr: never split).
  float* ks_ws;
  size_t ks_ws_bytes;
  int ksplit, ks_steps;
};

// launchers (one per translation unit)
int lf_launch_gemm(const LfGemmParams& p, const LfSegTable& seg, bool nn, int dtype, int force_cfg, hipStream_t st);
int lf_launch_gemm_big(const LfGemmParams& p, const LfSegTable& seg, bool nn, int dtype, int tile_rows, hipStream_t st);  // persistent tiles of 256 or 128 rows x 256 columns
int lf_cu_count();
int lf_pin_tile_cfg(int cfg);  // -1: automatic choice
void lf_plan_gemm(int M, int N, int K, int routing_block, int* rows_head, int* cfg_head, int* cfg_tail);
size_t lf_gemm_ksplit_bytes(int M, int N, int K, int routing_block);  // workspace of the split contraction for this product

// Raise a kernel's dynamic-LDS limit once per device (the attribute belongs to the device's copy of
// the function; one flag array per kernel instantiation; threads that race here repeat the same call).
struct LfLdsFlags { std::atomic<bool> done[64]; };
template <typename Kern>
static inline bool lf_allow_lds(Kern kern, int bytes, LfLdsFlags& flags) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
  if (!flags.done[dev].load(std::memory_order_acquire)) {
    if (hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, bytes) != hipSuccess) return false;
    flags.done[dev].store(true, std::memory_order_release);
  }
  return true;
}

// Launch `kern` and report this launch's own status: the return code of hipLaunchKernel, not the
// thread's last-error slot, which may hold (and would lose) an error of the caller's earlier HIP calls.
template <typename... KArgs, typename... Args>
static inline int lf_launch(void (*kern)(KArgs...), dim3 grid, dim3 block, size_t smem, hipStream_t st, Args&&... args) {
  auto go = [&](KArgs... ka) {
    void* argv[] = {(void*)&ka...};
    return hipLaunchKernel((const void*)kern, grid, block, argv, smem, st);
  };
  return go(args...) == hipSuccess ? LF_OK : LF_ELAUNCH;
}
