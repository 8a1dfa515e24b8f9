// RMSNorm and SiLU-multiply for gfx950: the two elementwise steps either side of the LoRA linears of a decoder
// layer (RMSNorm before the q/k/v projections and before the MLP, SiLU(gate) * up before the down projection).
//
// The reference takes both from the liger-kernel package (lorafusion/utils/module.py:41-71, requirements.txt:20);
// the arithmetic here is that package's "llama" mode:
//   rstd = 1/sqrt(mean(x^2) + eps) in fp32;  y = round16(round16(x * rstd) * w)
//   dx = rstd * (m - x * rstd^2 * mean(m * x)),  m = dy * w;   dw = sum_rows dy * round16(x * rstd)   (fp32 sums)
//   c = round16(round16(silu(a)) * b);  db = dc * silu(a);  da = dc * (silu(a) * (1 - sig(a)) + sig(a)) * b
//
// All four kernels are HBM-bound streams.  RMSNorm: one wavefront owns a row and keeps it in registers between
// the sum of squares and the scaling (lane l holds the 16-byte pieces l, l+64, ... of the row, so every load and
// store instruction of a wave covers 1 KiB of contiguous memory); the weight vector stays in registers over the
// rows a wave visits.  The backward kernel is persistent over rows and keeps its share of dw in fp32 registers;
// the four waves of a workgroup add their shares through LDS, each workgroup writes one partial row, and a second
// small kernel sums the partial rows in a fixed order (no atomics: the result does not depend on timing).
// SiLU-multiply takes row strides, so gate and up may be the two halves of one merged [M, 2I] projection output and
// da / db the two halves of its gradient.
#include "lf_common.h"
#include "act_math.h"

namespace {

// Makes the compiler treat a packed vector as changed: the fp32 values unpacked from it cannot be kept alive across
// this point (or hoisted out of a loop), only the packed registers are.  Emits no instruction.
__device__ __forceinline__ void keep_packed(lf_u32x4& v) {
  asm volatile("" : "+v"(v));
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

constexpr int NORM_THREADS = 256;
constexpr int NORM_WAVES = NORM_THREADS / 64;

// CH = 16-byte pieces of a row per lane: rows of up to CH * 512 elements; FULL: exactly that many (no guards).
template <typename T, int CH, bool FULL>
__global__ void __launch_bounds__(NORM_THREADS)
rmsnorm_fwd_kernel(const lf_u32x4* __restrict__ x, const lf_u32x4* __restrict__ w, lf_u32x4* __restrict__ y,
                   float* __restrict__ rstd_out, int M, int hc /* H / 8 */, float h, float eps) {
  const int lane = threadIdx.x & 63;
  const int gw = blockIdx.x * NORM_WAVES + (threadIdx.x >> 6), nw = gridDim.x * NORM_WAVES;
  const lf_u32x4 zero = {0u, 0u, 0u, 0u};
  lf_u32x4 wv[CH];
#pragma unroll
  for (int c = 0; c < CH; c++) wv[c] = (FULL || c * 64 + lane < hc) ? w[c * 64 + lane] : zero;
  for (int row = gw; row < M; row += nw) {
    const lf_u32x4* xr = x + (int64_t)row * hc;
    lf_u32x4 xv[CH];
#pragma unroll
    for (int c = 0; c < CH; c++) xv[c] = (FULL || c * 64 + lane < hc) ? xr[c * 64 + lane] : zero;
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CH; c++) {
      float f[8];
      unpack8<T>(xv[c], f);
#pragma unroll
      for (int e = 0; e < 8; e++) ss += f[e] * f[e];
    }
    ss = wave_sum(ss);
#pragma unroll
    for (int c = 0; c < CH; c++) {
      keep_packed(xv[c]);
      keep_packed(wv[c]);
    }
    const float r = 1.0f / sqrtf(ss / h + eps);
    if (lane == 0) rstd_out[row] = r;
    lf_u32x4* yr = y + (int64_t)row * hc;
#pragma unroll
    for (int c = 0; c < CH; c++) {
      float f[8], g[8];
      unpack8<T>(xv[c], f);
      unpack8<T>(wv[c], g);
#pragma unroll
      for (int e = 0; e < 8; e++) f[e] = round16<T>(f[e] * r) * g[e];
      if (FULL || c * 64 + lane < hc) __builtin_nontemporal_store(pack8<T>(f), yr + c * 64 + lane);
    }
  }
}

// Widest rows with dw: the weight vector is read from LDS instead (registers go to the row, its gradient and the sums).
constexpr bool bwd_w_in_regs(int ch, bool dw) { return !(dw && ch >= 12); }

// dX may alias dY: a wave holds the whole row of dY in registers before it writes that row of dX (neither pointer
// is restrict-qualified, so the compiler may not move a load of dY below a store to dX either).
template <typename T, int CH, bool DW, bool FULL>
__global__ void __launch_bounds__(NORM_THREADS)
rmsnorm_bwd_kernel(const lf_u32x4* dy, const lf_u32x4* __restrict__ x, const lf_u32x4* __restrict__ w,
                   const float* __restrict__ rstd, lf_u32x4* dx, float* __restrict__ dw_partial /* [gridDim.x, H] */,
                   int M, int hc, float h) {
  // LDS: one row of fp32 partial sums (DW), then the weight vector where it is not kept in registers
  extern __shared__ __align__(16) float red[];
  constexpr bool WREG = bwd_w_in_regs(CH, DW);
  lf_u32x4* wl = (lf_u32x4*)(red + (DW ? hc * 8 : 0));
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int gw = blockIdx.x * NORM_WAVES + wave, nw = gridDim.x * NORM_WAVES;
  const lf_u32x4 zero = {0u, 0u, 0u, 0u};
  lf_u32x4 wv[WREG ? CH : 1];
  if constexpr (WREG) {
#pragma unroll
    for (int c = 0; c < CH; c++) wv[c] = (FULL || c * 64 + lane < hc) ? w[c * 64 + lane] : zero;
  } else {
    for (int i = threadIdx.x; i < CH * 64; i += NORM_THREADS) wl[i] = (FULL || i < hc) ? w[i] : zero;
    __syncthreads();
  }
  auto w_piece = [&](int c) -> lf_u32x4 {
    if constexpr (WREG) return wv[c];
    else return wl[c * 64 + lane];
  };
  float acc[DW ? CH : 1][8];
#pragma unroll
  for (int c = 0; c < (DW ? CH : 1); c++)
#pragma unroll
    for (int e = 0; e < 8; e++) acc[c][e] = 0.f;
  for (int row = gw; row < M; row += nw) {
    const lf_u32x4* xr = x + (int64_t)row * hc;
    const lf_u32x4* dyr = dy + (int64_t)row * hc;
    lf_u32x4 xv[CH], dv[CH];
#pragma unroll
    for (int c = 0; c < CH; c++) {
      const bool in = FULL || c * 64 + lane < hc;
      xv[c] = in ? xr[c * 64 + lane] : zero;
      dv[c] = in ? dyr[c * 64 + lane] : zero;
    }
    const float r = rstd[row];
    if constexpr (WREG) {
#pragma unroll
      for (int c = 0; c < CH; c++) keep_packed(wv[c]);
    }
    float dot = 0.f;
#pragma unroll
    for (int c = 0; c < CH; c++) {
      float f[8], d[8], g[8];
      unpack8<T>(xv[c], f);
      unpack8<T>(dv[c], d);
      unpack8<T>(w_piece(c), g);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        dot += d[e] * g[e] * f[e];
        if (DW) acc[c][e] += d[e] * round16<T>(f[e] * r);
      }
      __builtin_amdgcn_sched_barrier(0);  // piece by piece: unpacking all pieces at once costs 3 x 8 registers each
    }
    dot = wave_sum(dot);
#pragma unroll
    for (int c = 0; c < CH; c++) {
      keep_packed(xv[c]);
      keep_packed(dv[c]);
      if constexpr (WREG) keep_packed(wv[c]);
    }
    const float coef = r * r * (dot / h);
    lf_u32x4* dxr = dx + (int64_t)row * hc;
#pragma unroll
    for (int c = 0; c < CH; c++) {
      float f[8], d[8], g[8];
      unpack8<T>(xv[c], f);
      unpack8<T>(dv[c], d);
      unpack8<T>(w_piece(c), g);
#pragma unroll
      for (int e = 0; e < 8; e++) d[e] = r * (d[e] * g[e] - f[e] * coef);
      if (FULL || c * 64 + lane < hc) __builtin_nontemporal_store(pack8<T>(d), dxr + c * 64 + lane);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  if (DW) {
    // waves 1..3 hand their sums to wave 0 one after the other through one row of LDS
    for (int src = 1; src < NORM_WAVES; src++) {
      if (wave == src) {
#pragma unroll
        for (int c = 0; c < CH; c++)
          if (FULL || c * 64 + lane < hc) {
            float* p = red + (c * 64 + lane) * 8;
            *(lf_f32x4*)p = lf_f32x4{acc[c][0], acc[c][1], acc[c][2], acc[c][3]};
            *(lf_f32x4*)(p + 4) = lf_f32x4{acc[c][4], acc[c][5], acc[c][6], acc[c][7]};
          }
      }
      __syncthreads();
      if (wave == 0) {
#pragma unroll
        for (int c = 0; c < CH; c++)
          if (FULL || c * 64 + lane < hc) {
            const float* p = red + (c * 64 + lane) * 8;
            const lf_f32x4 lo = *(const lf_f32x4*)p, hi = *(const lf_f32x4*)(p + 4);
#pragma unroll
            for (int e = 0; e < 4; e++) {
              acc[c][e] += lo[e];
              acc[c][4 + e] += hi[e];
            }
          }
      }
      __syncthreads();
    }
    if (wave == 0) {
      float* out = dw_partial + (int64_t)blockIdx.x * hc * 8;
#pragma unroll
      for (int c = 0; c < CH; c++)
        if (FULL || c * 64 + lane < hc) {
          float* p = out + (c * 64 + lane) * 8;
          *(lf_f32x4*)p = lf_f32x4{acc[c][0], acc[c][1], acc[c][2], acc[c][3]};
          *(lf_f32x4*)(p + 4) = lf_f32x4{acc[c][4], acc[c][5], acc[c][6], acc[c][7]};
        }
    }
  }
}

// dw[col] = sum over the partial rows in a fixed order: 64 strided groups, then the 64 group sums in order.
// 16 columns per workgroup, so that a 4096-wide row gives every compute unit one workgroup.
constexpr int DWR_COLS = 16, DWR_GROUPS = 64;
template <typename T>
__global__ void __launch_bounds__(DWR_COLS * DWR_GROUPS)
rmsnorm_dw_reduce_kernel(const float* __restrict__ partial, int n_partial, int H, T* __restrict__ dw) {
  __shared__ float part[DWR_GROUPS][DWR_COLS];
  const int colx = threadIdx.x & (DWR_COLS - 1), grp = threadIdx.x / DWR_COLS;
  const int col = blockIdx.x * DWR_COLS + colx;
  float s = 0.f;
  if (col < H)
    for (int g = grp; g < n_partial; g += DWR_GROUPS) s += partial[(int64_t)g * H + col];
  part[grp][colx] = s;
  __syncthreads();
  if (grp == 0 && col < H) {
    float t = 0.f;
#pragma unroll
    for (int g = 0; g < DWR_GROUPS; g++) t += part[g][colx];
    dw[col] = (T)t;
  }
}


constexpr int ACT_THREADS = 256;

// One thread: one 16-byte column piece of ROWS consecutive rows.  Strides in 16-byte units.
template <typename T, int ROWS>
__global__ void __launch_bounds__(ACT_THREADS)
silu_mul_fwd_kernel(const lf_u32x4* __restrict__ a, const lf_u32x4* __restrict__ b, lf_u32x4* __restrict__ c, int M,
                    int ic /* I / 8 */, int col_blocks, int64_t lda, int64_t ldb, int64_t ldc) {
  const int cb = blockIdx.x % col_blocks, rb = blockIdx.x / col_blocks;
  const int col = cb * ACT_THREADS + threadIdx.x;
  if (col >= ic) return;
  const int row0 = rb * ROWS;
  lf_u32x4 av[ROWS], bv[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; i++)
    if (row0 + i < M) {
      // (streams read once and written once: neither loads nor stores allocate in the caches)
      av[i] = __builtin_nontemporal_load(a + (int64_t)(row0 + i) * lda + col);
      bv[i] = __builtin_nontemporal_load(b + (int64_t)(row0 + i) * ldb + col);
    }
#pragma unroll
  for (int i = 0; i < ROWS; i++)
    if (row0 + i < M) {
      __builtin_nontemporal_store(silu_mul8<T>(av[i], bv[i]), c + (int64_t)(row0 + i) * ldc + col);
    }
}

// dA may alias A and dB may alias B (every thread reads its pieces before it writes them).
template <typename T, int ROWS>
__global__ void __launch_bounds__(ACT_THREADS)
silu_mul_bwd_kernel(const lf_u32x4* __restrict__ dc, const lf_u32x4* a, const lf_u32x4* b, lf_u32x4* da, lf_u32x4* db,
                    int M, int ic, int col_blocks, int64_t lddc, int64_t lda, int64_t ldb, int64_t ldda, int64_t lddb) {
  const int cb = blockIdx.x % col_blocks, rb = blockIdx.x / col_blocks;
  const int col = cb * ACT_THREADS + threadIdx.x;
  if (col >= ic) return;
  const int row0 = rb * ROWS;
  lf_u32x4 av[ROWS], bv[ROWS], cv[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; i++)
    if (row0 + i < M) {
      cv[i] = __builtin_nontemporal_load(dc + (int64_t)(row0 + i) * lddc + col);
      av[i] = __builtin_nontemporal_load(a + (int64_t)(row0 + i) * lda + col);
      bv[i] = __builtin_nontemporal_load(b + (int64_t)(row0 + i) * ldb + col);
    }
#pragma unroll
  for (int i = 0; i < ROWS; i++)
    if (row0 + i < M) {
      float fa[8], fb[8], fc[8], ga[8], gb[8];
      unpack8<T>(av[i], fa);
      unpack8<T>(bv[i], fb);
      unpack8<T>(cv[i], fc);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float sig = sigmoid_f32(fa[e]);
        const float silu = fa[e] * sig;
        gb[e] = fc[e] * silu;
        ga[e] = fc[e] * (silu * (1.0f - sig) + sig) * fb[e];
      }
      __builtin_nontemporal_store(pack8<T>(ga), da + (int64_t)(row0 + i) * ldda + col);
      __builtin_nontemporal_store(pack8<T>(gb), db + (int64_t)(row0 + i) * lddb + col);
    }
}

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

constexpr int NORM_MAX_H = 8192;  // 16 pieces of 16 bytes per lane
constexpr int BWD_MAX_WGS_PER_CU = 4;

// Row widths that are a multiple of 512 elements get the kernel with exactly that many pieces per lane and no
// guards; other widths the next of 1, 2, 4, 8, 16 pieces with guards.
struct NormShape {
  int ch;
  bool full;
};
inline NormShape norm_shape(int hc) {
  if (hc % 64 == 0) return {hc / 64, true};
  int ch = 1;
  while (ch * 64 < hc) ch *= 2;
  return {ch, false};
}

using FwdKern = void (*)(const lf_u32x4*, const lf_u32x4*, lf_u32x4*, float*, int, int, float, float);
using BwdKern = void (*)(const lf_u32x4*, const lf_u32x4*, const lf_u32x4*, const float*, lf_u32x4*, float*, int, int, float);

#define LF_CH_CASES(X) X(1) X(2) X(3) X(4) X(5) X(6) X(7) X(8) X(9) X(10) X(11) X(12) X(13) X(14) X(15) X(16)
#define LF_CH_POW2(X) X(1) X(2) X(4) X(8) X(16)

template <typename T>
FwdKern fwd_kernel(NormShape sh) {
  if (sh.full) {
    switch (sh.ch) {
#define X(CH) case CH: return rmsnorm_fwd_kernel<T, CH, true>;
      LF_CH_CASES(X)
#undef X
    }
  } else {
    switch (sh.ch) {
#define X(CH) case CH: return rmsnorm_fwd_kernel<T, CH, false>;
      LF_CH_POW2(X)
#undef X
    }
  }
  return nullptr;
}

template <typename T, bool DW>
BwdKern bwd_kernel(NormShape sh) {
  if (sh.full) {
    switch (sh.ch) {
#define X(CH) case CH: return rmsnorm_bwd_kernel<T, CH, DW, true>;
      LF_CH_CASES(X)
#undef X
    }
  } else {
    switch (sh.ch) {
#define X(CH) case CH: return rmsnorm_bwd_kernel<T, CH, DW, false>;
      LF_CH_POW2(X)
#undef X
    }
  }
  return nullptr;
}

inline BwdKern bwd_kernel_of(int dtype, bool dw, NormShape sh) {
  if (dtype == LF_BF16) return dw ? bwd_kernel<__bf16, true>(sh) : bwd_kernel<__bf16, false>(sh);
  if (dtype == LF_F16) return dw ? bwd_kernel<_Float16, true>(sh) : bwd_kernel<_Float16, false>(sh);
  return nullptr;
}

inline size_t bwd_smem(int H, bool dw, NormShape sh) {
  return (dw ? (size_t)H * sizeof(float) : 0) + (bwd_w_in_regs(sh.ch, dw) ? 0 : (size_t)sh.ch * 64 * 16);
}

// Workgroups of the persistent backward kernel: what is resident at once (its registers decide), at most
// BWD_MAX_WGS_PER_CU per compute unit (which bounds the partial rows of dw), never more than the rows need.
inline int bwd_grid(int M, BwdKern kern, size_t smem) {
  int occ = 0;
  if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, (const void*)kern, NORM_THREADS, smem) != hipSuccess || occ < 1) occ = 1;
  if (occ > BWD_MAX_WGS_PER_CU) occ = BWD_MAX_WGS_PER_CU;
  const int64_t need = ((int64_t)M + NORM_WAVES - 1) / NORM_WAVES;
  const int64_t cap = (int64_t)lf_cu_count() * occ;
  return (int)(need < cap ? need : cap);
}

}  // namespace

extern "C" {

int lf_rmsnorm_fwd(const void* X, const void* W, void* Y, float* rstd, int M, int H, float eps, int dtype,
                   void* stream) {
  if (!X || !W || !Y || !rstd || M <= 0 || H <= 0) return LF_EINVAL;
  if (H % 8 != 0 || !aligned16(X) || !aligned16(W) || !aligned16(Y)) return LF_ESHAPE;
  if (H > NORM_MAX_H) return LF_ELIMIT;
  const int hc = H / 8;
  const NormShape sh = norm_shape(hc);
  const FwdKern kern = dtype == LF_BF16 ? fwd_kernel<__bf16>(sh) : dtype == LF_F16 ? fwd_kernel<_Float16>(sh) : nullptr;
  if (!kern) return LF_EINVAL;
  const int64_t need = ((int64_t)M + NORM_WAVES - 1) / NORM_WAVES;
  const int64_t cap = (int64_t)lf_cu_count() * 16;
  const unsigned grid = (unsigned)(need < cap ? need : cap);
  return lf_launch(kern, dim3(grid), dim3(NORM_THREADS), 0, (hipStream_t)stream, (const lf_u32x4*)X,
                   (const lf_u32x4*)W, (lf_u32x4*)Y, rstd, M, hc, (float)H, eps);
}

size_t lf_rmsnorm_bwd_workspace(int M, int H) {
  if (M <= 0 || H <= 0 || H % 8 != 0 || H > NORM_MAX_H) return 0;
  const int64_t need = ((int64_t)M + NORM_WAVES - 1) / NORM_WAVES;
  const int64_t cap = (int64_t)lf_cu_count() * BWD_MAX_WGS_PER_CU;
  return (size_t)(need < cap ? need : cap) * (size_t)H * sizeof(float);
}

int lf_rmsnorm_bwd(const void* dY, const void* X, const void* W, const float* rstd, void* dX, void* dW, int M, int H,
                   int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  if (!dY || !X || !W || !rstd || !dX || M <= 0 || H <= 0) return LF_EINVAL;
  if (H % 8 != 0 || !aligned16(dY) || !aligned16(X) || !aligned16(W) || !aligned16(dX)) return LF_ESHAPE;
  if (H > NORM_MAX_H) return LF_ELIMIT;
  const int hc = H / 8;
  const NormShape sh = norm_shape(hc);
  const bool with_dw = dW != nullptr;
  const BwdKern kern = bwd_kernel_of(dtype, with_dw, sh);
  if (!kern) return LF_EINVAL;
  const size_t smem = bwd_smem(H, with_dw, sh);
  const int grid = bwd_grid(M, kern, smem);
  if (with_dw && (!workspace || !aligned16(workspace) || workspace_bytes < (size_t)grid * H * sizeof(float)))
    return LF_EWORKSPACE;
  float* partial = (float*)workspace;
  const int rc = lf_launch(kern, dim3((unsigned)grid), dim3(NORM_THREADS), smem, (hipStream_t)stream,
                           (const lf_u32x4*)dY, (const lf_u32x4*)X, (const lf_u32x4*)W, rstd, (lf_u32x4*)dX, partial, M,
                           hc, (float)H);
  if (rc != LF_OK || !with_dw) return rc;
  const unsigned rgrid = (unsigned)((H + DWR_COLS - 1) / DWR_COLS);
  if (dtype == LF_BF16)
    return lf_launch((rmsnorm_dw_reduce_kernel<__bf16>), dim3(rgrid), dim3(DWR_COLS * DWR_GROUPS), 0,
                     (hipStream_t)stream, (const float*)partial, grid, H, (__bf16*)dW);
  return lf_launch((rmsnorm_dw_reduce_kernel<_Float16>), dim3(rgrid), dim3(DWR_COLS * DWR_GROUPS), 0,
                   (hipStream_t)stream, (const float*)partial, grid, H, (_Float16*)dW);
}

static int act_check(int M, int I, std::initializer_list<const void*> ptrs, std::initializer_list<int64_t> lds) {
  if (M <= 0 || I <= 0) return LF_EINVAL;
  for (const void* p : ptrs) {
    if (!p) return LF_EINVAL;
    if (!aligned16(p)) return LF_ESHAPE;
  }
  if (I % 8 != 0) return LF_ESHAPE;
  for (int64_t ld : lds)
    if (ld < I || ld % 8 != 0) return LF_ESHAPE;
  return LF_OK;
}

int lf_silu_mul_fwd(const void* A, const void* B, void* C, int M, int I, int64_t lda, int64_t ldb, int64_t ldc,
                    int dtype, void* stream) {
  const int rc = act_check(M, I, {A, B, C}, {lda, ldb, ldc});
  if (rc != LF_OK) return rc;
  constexpr int ROWS = 2;
  const int ic = I / 8, col_blocks = (ic + ACT_THREADS - 1) / ACT_THREADS;
  const int64_t grid = (int64_t)col_blocks * ((M + ROWS - 1) / ROWS);
  if (grid > 0x7fffffffLL) return LF_ELIMIT;
  if (dtype == LF_BF16)
    return lf_launch((silu_mul_fwd_kernel<__bf16, ROWS>), dim3((unsigned)grid), dim3(ACT_THREADS), 0, (hipStream_t)stream,
                     (const lf_u32x4*)A, (const lf_u32x4*)B, (lf_u32x4*)C, M, ic, col_blocks, lda / 8, ldb / 8, ldc / 8);
  if (dtype == LF_F16)
    return lf_launch((silu_mul_fwd_kernel<_Float16, ROWS>), dim3((unsigned)grid), dim3(ACT_THREADS), 0, (hipStream_t)stream,
                     (const lf_u32x4*)A, (const lf_u32x4*)B, (lf_u32x4*)C, M, ic, col_blocks, lda / 8, ldb / 8, ldc / 8);
  return LF_EINVAL;
}

int lf_silu_mul_bwd(const void* dC, const void* A, const void* B, void* dA, void* dB, int M, int I, int64_t lddc,
                    int64_t lda, int64_t ldb, int64_t ldda, int64_t lddb, int dtype, void* stream) {
  const int rc = act_check(M, I, {dC, A, B, dA, dB}, {lddc, lda, ldb, ldda, lddb});
  if (rc != LF_OK) return rc;
  constexpr int ROWS = 2;
  const int ic = I / 8, col_blocks = (ic + ACT_THREADS - 1) / ACT_THREADS;
  const int64_t grid = (int64_t)col_blocks * ((M + ROWS - 1) / ROWS);
  if (grid > 0x7fffffffLL) return LF_ELIMIT;
  if (dtype == LF_BF16)
    return lf_launch((silu_mul_bwd_kernel<__bf16, ROWS>), dim3((unsigned)grid), dim3(ACT_THREADS), 0, (hipStream_t)stream,
                     (const lf_u32x4*)dC, (const lf_u32x4*)A, (const lf_u32x4*)B, (lf_u32x4*)dA, (lf_u32x4*)dB, M, ic,
                     col_blocks, lddc / 8, lda / 8, ldb / 8, ldda / 8, lddb / 8);
  if (dtype == LF_F16)
    return lf_launch((silu_mul_bwd_kernel<_Float16, ROWS>), dim3((unsigned)grid), dim3(ACT_THREADS), 0, (hipStream_t)stream,
                     (const lf_u32x4*)dC, (const lf_u32x4*)A, (const lf_u32x4*)B, (lf_u32x4*)dA, (lf_u32x4*)dB, M, ic,
                     col_blocks, lddc / 8, lda / 8, ldb / 8, ldda / 8, lddb / 8);
  return LF_EINVAL;
}

}  // extern "C"
