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
// MFMA 16x16x32 operand layout (64 lanes): lane l holds row/col (l & 15) and the 8
// contraction elements of chunk (l >> 4).  Where the contraction index is the slow memory
// dimension, tiles are staged in LDS and read with ds_read_b64_tr_b16 (16 lanes read a
// 4-row x 16-column patch; lane 4j+c addresses row j, columns 4c..4c+3; each lane receives
// its column's 4 rows).
#include "lf_common.h"

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

__device__ __forceinline__ lf_u32x4 tr_read8(const char* p, int pitch) {
  // 8 contraction elements (rows r..r+3 and r+4..r+7) of this lane's column
  lf_s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(p));
  lf_s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) lf_s16x4*)(p + 4 * pitch));
  lf_u32x2 a = __builtin_bit_cast(lf_u32x2, lo), b = __builtin_bit_cast(lf_u32x2, hi);
  return lf_u32x4{a[0], a[1], b[0], b[1]};
}

// ------------------------------------------------------------------------------------ xa
// grid (n_blocks, ksplit); 4 waves, wave w owns rows 32w..32w+31 of the block.
// part[ks][row][R] (fp32) = sum over this K slice of mask*X*A^T  (unscaled).
template <typename T, int RT>
__global__ void __launch_bounds__(256)
lora_xa_kernel(const T* __restrict__ X, const uint8_t* __restrict__ mask, float* __restrict__ part,
               int M, int K, int R, int kslice, const LfSegTable seg) {
  const int blk = blockIdx.x, ks = blockIdx.y;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int li = lane & 15, qq = lane >> 4;
  const BlockInfo bi = block_info(seg, blk, M);
  const T* __restrict__ A = (const T*)seg.ptr[bi.seg];
  const bool use_mask = mask != nullptr && bi.p > 0.f;
  const int Mrows = seg.table ? seg.n_blocks * ROWS : M;

  lf_f32x4 acc[2][RT];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int c = 0; c < RT; c++) acc[a][c] = lf_f32x4{0.f, 0.f, 0.f, 0.f};

  int64_t xrow[2];
#pragma unroll
  for (int rt = 0; rt < 2; rt++) xrow[rt] = min(blk * ROWS + wave * 32 + rt * 16 + li, Mrows - 1);

  const int k_begin = ks * kslice, k_end = min(K, k_begin + kslice);
  for (int kb = k_begin; kb < k_end; kb += 128) {
    const int kc = kb + qq * 32;  // this lane's 32 contiguous k
    lf_u32x4 xf[2][4];
#pragma unroll
    for (int rt = 0; rt < 2; rt++) {
      const T* xp = X + xrow[rt] * K + kc;
#pragma unroll
      for (int j = 0; j < 4; j++) xf[rt][j] = __builtin_nontemporal_load((const lf_u32x4*)(xp + 8 * j));
      if (use_mask) {
        const lf_u32x2* mp = (const lf_u32x2*)(mask + xrow[rt] * K + kc);
#pragma unroll
        for (int j = 0; j < 4; j++) xf[rt][j] = apply_mask8(xf[rt][j], __builtin_nontemporal_load(mp + j));
      }
    }
#pragma unroll
    for (int c = 0; c < RT; c++) {
      const int r = c * 16 + li;
      lf_u32x4 af[4];
      if (r < bi.rank) {
        const T* ap = A + (int64_t)r * K + kc;
#pragma unroll
        for (int j = 0; j < 4; j++) af[j] = *(const lf_u32x4*)(ap + 8 * j);
      } else {
#pragma unroll
        for (int j = 0; j < 4; j++) af[j] = lf_u32x4{0, 0, 0, 0};
      }
#pragma unroll
      for (int rt = 0; rt < 2; rt++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[rt][c] = Mfma16<T>::run(xf[rt][j], af[j], acc[rt][c]);
    }
  }
  // C layout: lane holds column (lane & 15), rows 4*(lane >> 4) + e
  float* out = part + (int64_t)ks * Mrows * R;
#pragma unroll
  for (int rt = 0; rt < 2; rt++)
#pragma unroll
    for (int c = 0; c < RT; c++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int row = blk * ROWS + wave * 32 + rt * 16 + qq * 4 + e;
        if (row < Mrows) out[(int64_t)row * R + c * 16 + li] = acc[rt][c][e];
      }
}

// S[row][col] = cast( 1/(1-p) * sum_ks part[ks][row][col] ), zero for padded rows / rank columns.
template <typename T>
__global__ void __launch_bounds__(256)
reduce_rows_kernel(const float* __restrict__ part, T* __restrict__ out, int nparts, int M, int R,
                   int mode /*0: times 1/(1-p); 1: times scale*/, const LfSegTable seg) {
  const int Mrows = seg.table ? seg.n_blocks * ROWS : M;
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (int64_t)Mrows * R) return;
  const int row = (int)(idx / R), col = (int)(idx % R);
  const int blk = row / ROWS;
  const BlockInfo bi = block_info(seg, blk, M);
  float v = 0.f;
  if (row - blk * ROWS < bi.valid && col < bi.rank) {
    for (int p = 0; p < nparts; p++) v += part[(int64_t)p * Mrows * R + idx];
    v *= (mode == 0) ? (bi.p > 0.f ? 1.f / (1.f - bi.p) : 1.f) : bi.scale;
  }
  ((uint16_t*)out)[idx] = Mfma16<T>::cvt(v);
}

// ------------------------------------------------------------------------------- dys_dyb
// grid (n_blocks, nsplit).  Each workgroup walks its N slice in 128-column chunks:
//   dS partial  [128 rows, R]  += dY_chunk * B_chunk          (accumulated over the slice)
//   dB partial  [128 cols, R]   = dY_chunk^T * S_block        (complete per chunk)
// LDS: dY chunk [128][128] pitch 288 B, B chunk [128][R] and S block [128][R] pitch 2R+32 B
// (pitches keep the 4-row transpose reads on distinct banks).
template <typename T, int RT>
__global__ void __launch_bounds__(256)
lora_dys_dyb_kernel(const T* __restrict__ dY, const T* __restrict__ S, float* __restrict__ ds_part,
                    float* __restrict__ db_part, int M, int N, int R, int nslice, const LfSegTable seg) {
  constexpr int DYP = 288;
  constexpr int RP = RT * 32 + 32;
  __shared__ __attribute__((aligned(16))) char lds_dy[ROWS * DYP];
  __shared__ __attribute__((aligned(16))) char lds_b[128 * RP];
  __shared__ __attribute__((aligned(16))) char lds_s[ROWS * RP];

  const int blk = blockIdx.x, ns = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, qq = lane >> 4, j4 = li >> 2, c4 = li & 3;
  const BlockInfo bi = block_info(seg, blk, M);
  const T* __restrict__ Bl = (const T*)seg.ptr[bi.seg];
  const int Mrows = seg.table ? seg.n_blocks * ROWS : M;

  // S block -> LDS (rows beyond `valid` as zeros so they add nothing to dB)
  for (int g = tid; g < ROWS * RT * 2; g += 256) {  // 16-byte granules, RT*2 per row
    const int row = g / (RT * 2), gc = g % (RT * 2);
    lf_u32x4 v = {0, 0, 0, 0};
    if (row < bi.valid) v = *(const lf_u32x4*)(S + (int64_t)(blk * ROWS + row) * R + gc * 8);
    *(lf_u32x4*)(lds_s + row * RP + gc * 16) = v;
  }

  lf_f32x4 acc_ds[2][RT];
#pragma unroll
  for (int a = 0; a < 2; a++)
#pragma unroll
    for (int c = 0; c < RT; c++) acc_ds[a][c] = lf_f32x4{0.f, 0.f, 0.f, 0.f};

  int64_t yrow[2];
#pragma unroll
  for (int rt = 0; rt < 2; rt++) yrow[rt] = min(blk * ROWS + wave * 32 + rt * 16 + li, Mrows - 1);

  const int n_begin = ns * nslice, n_end = min(N, n_begin + nslice);
  for (int nb = n_begin; nb < n_end; nb += 128) {
    // dY chunk: this lane's fragments (row li of each 16-row tile, 32 contiguous columns)
    lf_u32x4 yf[2][4];
#pragma unroll
    for (int rt = 0; rt < 2; rt++) {
      const T* yp = dY + yrow[rt] * N + nb + qq * 32;
#pragma unroll
      for (int j = 0; j < 4; j++) yf[rt][j] = __builtin_nontemporal_load((const lf_u32x4*)(yp + 8 * j));
    }
    __syncthreads();  // previous chunk's LDS reads are done
#pragma unroll
    for (int rt = 0; rt < 2; rt++)
#pragma unroll
      for (int j = 0; j < 4; j++)
        *(lf_u32x4*)(lds_dy + (wave * 32 + rt * 16 + li) * DYP + (qq * 32 + j * 8) * 2) = yf[rt][j];
    // B chunk rows nb..nb+127 (rank columns, zero padded to R)
    for (int g = tid; g < 128 * RT * 2; g += 256) {
      const int row = g / (RT * 2), gc = g % (RT * 2);
      lf_u32x4 v = {0, 0, 0, 0};
      if (gc * 8 < bi.rank) v = *(const lf_u32x4*)(Bl + (int64_t)(nb + row) * bi.rank + gc * 8);
      *(lf_u32x4*)(lds_b + row * RP + gc * 16) = v;
    }
    __syncthreads();

    // dS += dY_chunk * B_chunk : a = dY fragment (registers), b = B^T via transpose read
#pragma unroll
    for (int c = 0; c < RT; c++) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const lf_u32x4 bf = tr_read8(lds_b + (qq * 32 + j * 8 + j4) * RP + (c * 16 + 4 * c4) * 2, RP);
#pragma unroll
        for (int rt = 0; rt < 2; rt++) acc_ds[rt][c] = Mfma16<T>::run(yf[rt][j], bf, acc_ds[rt][c]);
      }
    }
    // dB chunk: D[n][r] = sum_m dY[m][n] S[m][r]; wave w owns columns 32w..32w+31 of the chunk
    lf_f32x4 acc_db[2][RT];
#pragma unroll
    for (int a = 0; a < 2; a++)
#pragma unroll
      for (int c = 0; c < RT; c++) acc_db[a][c] = lf_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; kk++) {
      const int mrow = kk * 32 + qq * 8 + j4;
      lf_u32x4 sf[RT];
#pragma unroll
      for (int c = 0; c < RT; c++) sf[c] = tr_read8(lds_s + mrow * RP + (c * 16 + 4 * c4) * 2, RP);
#pragma unroll
      for (int nt = 0; nt < 2; nt++) {
        const lf_u32x4 yt = tr_read8(lds_dy + mrow * DYP + (wave * 32 + nt * 16 + 4 * c4) * 2, DYP);
#pragma unroll
        for (int c = 0; c < RT; c++) acc_db[nt][c] = Mfma16<T>::run(yt, sf[c], acc_db[nt][c]);
      }
    }
    float* dbo = db_part + ((int64_t)blk * N + nb) * R;
#pragma unroll
    for (int nt = 0; nt < 2; nt++)
#pragma unroll
      for (int c = 0; c < RT; c++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          dbo[(int64_t)(wave * 32 + nt * 16 + qq * 4 + e) * R + c * 16 + li] = acc_db[nt][c][e];
  }
  float* dso = ds_part + (int64_t)ns * Mrows * R;
#pragma unroll
  for (int rt = 0; rt < 2; rt++)
#pragma unroll
    for (int c = 0; c < RT; c++)
#pragma unroll
      for (int e = 0; e < 4; e++) {
        const int row = blk * ROWS + wave * 32 + rt * 16 + qq * 4 + e;
        if (row < Mrows) dso[(int64_t)row * R + c * 16 + li] = acc_ds[rt][c][e];
      }
}

// out_s[n][r] (r < rank_s) = cast( mult * sum over the segment's blocks of part[b][n][r] )
//   mult_mode 0: block scale ; 1: 1/(1-p) of the block.  part is [n_blocks][rows][R].
// Used for dB (rows = N, out [N, rank]) and dA (transposed flag: part [b][R][K], out [rank, K]).
template <typename T>
__global__ void __launch_bounds__(256)
reduce_segments_kernel(const float* __restrict__ part, int rows, int R, int transposed, int mult_mode, int M,
                       const LfSegTable seg) {
  const int s = blockIdx.y;
  const int rank = seg.table ? seg.rank[s] : seg.rank[0];
  const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // index into the output [rows, rank] or [rank, rows]
  if (idx >= (int64_t)rows * rank) return;
  int b0 = 0, b1;
  float mult;
  if (seg.table == nullptr) {
    b1 = (M + ROWS - 1) / ROWS;
    mult = mult_mode == 0 ? seg.scale : (seg.p > 0.f ? 1.f / (1.f - seg.p) : 1.f);
  } else {
    b0 = seg.first_block[s];
    b1 = (s + 1 < seg.n_seg) ? seg.first_block[s + 1] : seg.n_blocks;
    mult = mult_mode == 0 ? (seg.block_scale ? seg.block_scale[b0] : 1.f)
                          : ((seg.block_p && seg.block_p[b0] > 0.f) ? 1.f / (1.f - seg.block_p[b0]) : 1.f);
  }
  int64_t pidx;
  if (!transposed) {
    const int n = (int)(idx / rank), r = (int)(idx % rank);
    pidx = (int64_t)n * R + r;
  } else {
    const int r = (int)(idx / rows), k = (int)(idx % rows);
    pidx = (int64_t)r * rows + k;
  }
  float v = 0.f;
  for (int b = b0; b < b1; b++) v += part[(int64_t)b * rows * R + pidx];
  ((uint16_t*)seg.out[s])[idx] = Mfma16<T>::cvt(v * mult);
}

// ------------------------------------------------------------------------------------ da
// grid (n_blocks, K / kslice).  part[b][r][k] = sum over the block's rows of dS[m][r] * mask*X[m][k]
// (without 1/(1-p); the reduce applies it).  dS block and X chunk are staged in LDS and both
// read through the transpose path since the contraction index m is the slow dimension of both.
template <typename T, int RT>
__global__ void __launch_bounds__(256)
lora_da_kernel(const T* __restrict__ X, const uint8_t* __restrict__ mask, const T* __restrict__ dS,
               float* __restrict__ part, int M, int K, int R, int kslice, const LfSegTable seg) {
  constexpr int XP = 288;
  constexpr int RP = RT * 32 + 32;
  __shared__ __attribute__((aligned(16))) char lds_x[ROWS * XP];
  __shared__ __attribute__((aligned(16))) char lds_ds[ROWS * RP];
  const int blk = blockIdx.x;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, qq = lane >> 4, j4 = li >> 2, c4 = li & 3;
  const BlockInfo bi = block_info(seg, blk, M);
  const bool use_mask = mask != nullptr && bi.p > 0.f;
  const int Mrows = seg.table ? seg.n_blocks * ROWS : M;

  for (int g = tid; g < ROWS * RT * 2; g += 256) {
    const int row = g / (RT * 2), gc = g % (RT * 2);
    lf_u32x4 v = {0, 0, 0, 0};
    if (row < bi.valid) v = *(const lf_u32x4*)(dS + (int64_t)(blk * ROWS + row) * R + gc * 8);
    *(lf_u32x4*)(lds_ds + row * RP + gc * 16) = v;
  }
  int64_t xrow[2];
#pragma unroll
  for (int rt = 0; rt < 2; rt++) xrow[rt] = min(blk * ROWS + wave * 32 + rt * 16 + li, Mrows - 1);

  const int k_begin = blockIdx.y * kslice, k_end = min(K, k_begin + kslice);
  for (int kb = k_begin; kb < k_end; kb += 128) {
    lf_u32x4 xf[2][4];
#pragma unroll
    for (int rt = 0; rt < 2; rt++) {
      const T* xp = X + xrow[rt] * K + kb + qq * 32;
#pragma unroll
      for (int j = 0; j < 4; j++) xf[rt][j] = __builtin_nontemporal_load((const lf_u32x4*)(xp + 8 * j));
      if (use_mask) {
        const lf_u32x2* mp = (const lf_u32x2*)(mask + xrow[rt] * K + kb + qq * 32);
#pragma unroll
        for (int j = 0; j < 4; j++) xf[rt][j] = apply_mask8(xf[rt][j], __builtin_nontemporal_load(mp + j));
      }
    }
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < 2; rt++)
#pragma unroll
      for (int j = 0; j < 4; j++)
        *(lf_u32x4*)(lds_x + (wave * 32 + rt * 16 + li) * XP + (qq * 32 + j * 8) * 2) = xf[rt][j];
    __syncthreads();

    // D[r][k] = sum_m dS[m][r] X~[m][k]; wave w owns columns 32w..32w+31 of the chunk
    lf_f32x4 acc[RT][2];
#pragma unroll
    for (int c = 0; c < RT; c++)
#pragma unroll
      for (int a = 0; a < 2; a++) acc[c][a] = lf_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; kk++) {
      const int mrow = kk * 32 + qq * 8 + j4;
      lf_u32x4 df[RT];
#pragma unroll
      for (int c = 0; c < RT; c++) df[c] = tr_read8(lds_ds + mrow * RP + (c * 16 + 4 * c4) * 2, RP);
#pragma unroll
      for (int kt = 0; kt < 2; kt++) {
        const lf_u32x4 xt = tr_read8(lds_x + mrow * XP + (wave * 32 + kt * 16 + 4 * c4) * 2, XP);
#pragma unroll
        for (int c = 0; c < RT; c++) acc[c][kt] = Mfma16<T>::run(df[c], xt, acc[c][kt]);
      }
    }
    // C layout: column (k) = lane & 15, rows (r) = 4*(lane >> 4) + e
    float* po = part + (int64_t)blk * R * K;
#pragma unroll
    for (int c = 0; c < RT; c++)
#pragma unroll
      for (int kt = 0; kt < 2; kt++)
#pragma unroll
        for (int e = 0; e < 4; e++)
          po[(int64_t)(c * 16 + qq * 4 + e) * K + kb + wave * 32 + kt * 16 + li] = acc[c][kt][e];
  }
}

int rt_of(int R) { return R <= 16 ? 1 : R <= 32 ? 2 : R <= 64 ? 4 : 8; }

}  // namespace

static int n_row_blocks(int M, const LfSegTable& seg) { return seg.table ? seg.n_blocks : (M + ROWS - 1) / ROWS; }

// Split factor so that blocks * split fills the chip; slices are multiples of 128.
static int pick_split(int nblk, int len) {
  int split = 1;
  while (nblk * split < 512 && len / (split * 2) >= 128 && (len % (split * 2 * 128)) == 0) split *= 2;
  return split;
}

size_t lf_xa_workspace(int M, int K, int R, const LfSegTable& seg) {
  const int nblk = n_row_blocks(M, seg);
  const int64_t rows = seg.table ? (int64_t)nblk * ROWS : M;
  return (size_t)pick_split(nblk, K) * rows * R * sizeof(float);
}

template <typename T>
static int xa_impl(const void* X, const uint8_t* mask, void* S, void* ws, int M, int K, int R, const LfSegTable& seg, hipStream_t st) {
  const int nblk = n_row_blocks(M, seg);
  const int64_t rows = seg.table ? (int64_t)nblk * ROWS : M;
  const int split = pick_split(nblk, K);
  const int kslice = K / split;
  float* part = (float*)ws;
  dim3 grid(nblk, split);
#define LF_XA(RT) hipLaunchKernelGGL((lora_xa_kernel<T, RT>), grid, dim3(256), 0, st, (const T*)X, mask, part, M, K, R, kslice, seg)
  switch (rt_of(R)) { case 1: LF_XA(1); break; case 2: LF_XA(2); break; case 4: LF_XA(4); break; default: LF_XA(8); break; }
#undef LF_XA
  if (lf_check_launch() != LF_OK) return LF_ELAUNCH;
  const int64_t n = rows * R;
  hipLaunchKernelGGL((reduce_rows_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (const float*)part, (T*)S, split, M, R, 0, seg);
  return lf_check_launch();
}

int lf_launch_xa(const void* X, const uint8_t* mask, void* S, void* ws, size_t ws_bytes, int M, int K, int R,
                 const LfSegTable& seg, int dtype, hipStream_t st) {
  if (!X || !S || M <= 0 || K <= 0) return LF_EINVAL;
  if (K % 128 != 0 || R % 16 != 0 || R <= 0 || R > LF_MAX_RANK) return LF_ESHAPE;
  if (seg.table && seg.block_size_m != ROWS) return LF_ESHAPE;
  if (!ws || ws_bytes < lf_xa_workspace(M, K, R, seg)) return LF_EWORKSPACE;
  if (dtype == LF_BF16) return xa_impl<__bf16>(X, mask, S, ws, M, K, R, seg, st);
  if (dtype == LF_F16) return xa_impl<_Float16>(X, mask, S, ws, M, K, R, seg, st);
  return LF_EINVAL;
}

size_t lf_dys_dyb_workspace(int M, int N, int R, const LfSegTable& seg) {
  const int nblk = n_row_blocks(M, seg);
  const int64_t rows = seg.table ? (int64_t)nblk * ROWS : M;
  return ((size_t)pick_split(nblk, N) * rows * R + (size_t)nblk * N * R) * sizeof(float);
}

template <typename T>
static int dys_dyb_impl(const void* dY, const void* S, void* dS, void* ws, int M, int N, int R, const LfSegTable& seg, hipStream_t st) {
  const int nblk = n_row_blocks(M, seg);
  const int64_t rows = seg.table ? (int64_t)nblk * ROWS : M;
  const int split = pick_split(nblk, N);
  const int nslice = N / split;
  float* ds_part = (float*)ws;
  float* db_part = ds_part + (int64_t)split * rows * R;
  dim3 grid(nblk, split);
#define LF_DYS(RT) hipLaunchKernelGGL((lora_dys_dyb_kernel<T, RT>), grid, dim3(256), 0, st, (const T*)dY, (const T*)S, ds_part, db_part, M, N, R, nslice, seg)
  switch (rt_of(R)) { case 1: LF_DYS(1); break; case 2: LF_DYS(2); break; case 4: LF_DYS(4); break; default: LF_DYS(8); break; }
#undef LF_DYS
  if (lf_check_launch() != LF_OK) return LF_ELAUNCH;
  const int64_t n = rows * R;
  hipLaunchKernelGGL((reduce_rows_kernel<T>), dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, (const float*)ds_part, (T*)dS, split, M, R, 1, seg);
  if (lf_check_launch() != LF_OK) return LF_ELAUNCH;
  const int nseg = seg.table ? seg.n_seg : 1;
  int maxrank = 0;
  for (int s = 0; s < nseg; s++) maxrank = seg.rank[s] > maxrank ? seg.rank[s] : maxrank;
  const int64_t nout = (int64_t)N * maxrank;
  hipLaunchKernelGGL((reduce_segments_kernel<T>), dim3((unsigned)((nout + 255) / 256), nseg), dim3(256), 0, st, (const float*)db_part, N, R, 0, 0, M, seg);
  return lf_check_launch();
}

int lf_launch_dys_dyb(const void* dY, const void* S, void* dS, void* ws, size_t ws_bytes, int M, int N, int R,
                      const LfSegTable& seg, int dtype, hipStream_t st) {
  if (!dY || !S || !dS || M <= 0 || N <= 0) return LF_EINVAL;
  if (N % 128 != 0 || R % 16 != 0 || R <= 0 || R > LF_MAX_RANK) return LF_ESHAPE;
  if (seg.table && seg.block_size_m != ROWS) return LF_ESHAPE;
  const int nseg = seg.table ? seg.n_seg : 1;
  for (int s = 0; s < nseg; s++) if (!seg.out[s] || !seg.ptr[s] || seg.rank[s] % 8 != 0 || seg.rank[s] > R) return LF_EINVAL;
  if (!ws || ws_bytes < lf_dys_dyb_workspace(M, N, R, seg)) return LF_EWORKSPACE;
  if (dtype == LF_BF16) return dys_dyb_impl<__bf16>(dY, S, dS, ws, M, N, R, seg, st);
  if (dtype == LF_F16) return dys_dyb_impl<_Float16>(dY, S, dS, ws, M, N, R, seg, st);
  return LF_EINVAL;
}

size_t lf_da_workspace(int M, int K, int R, const LfSegTable& seg) {
  return (size_t)n_row_blocks(M, seg) * R * K * sizeof(float);
}

template <typename T>
static int da_impl(const void* X, const uint8_t* mask, const void* dS, void* ws, int M, int K, int R, const LfSegTable& seg, hipStream_t st) {
  const int nblk = n_row_blocks(M, seg);
  const int split = pick_split(nblk, K);
  const int kslice = K / split;
  float* part = (float*)ws;
  dim3 grid(nblk, split);
#define LF_DA(RT) hipLaunchKernelGGL((lora_da_kernel<T, RT>), grid, dim3(256), 0, st, (const T*)X, mask, (const T*)dS, part, M, K, R, kslice, seg)
  switch (rt_of(R)) { case 1: LF_DA(1); break; case 2: LF_DA(2); break; case 4: LF_DA(4); break; default: LF_DA(8); break; }
#undef LF_DA
  if (lf_check_launch() != LF_OK) return LF_ELAUNCH;
  const int nseg = seg.table ? seg.n_seg : 1;
  int maxrank = 0;
  for (int s = 0; s < nseg; s++) maxrank = seg.rank[s] > maxrank ? seg.rank[s] : maxrank;
  const int64_t nout = (int64_t)K * maxrank;
  hipLaunchKernelGGL((reduce_segments_kernel<T>), dim3((unsigned)((nout + 255) / 256), nseg), dim3(256), 0, st, (const float*)part, K, R, 1, 1, M, seg);
  return lf_check_launch();
}

int lf_launch_da(const void* X, const uint8_t* mask, const void* dS, void* ws, size_t ws_bytes, int M, int K, int R,
                 const LfSegTable& seg, int dtype, hipStream_t st) {
  if (!X || !dS || M <= 0 || K <= 0) return LF_EINVAL;
  if (K % 128 != 0 || R % 16 != 0 || R <= 0 || R > LF_MAX_RANK) return LF_ESHAPE;
  if (seg.table && seg.block_size_m != ROWS) return LF_ESHAPE;
  const int nseg = seg.table ? seg.n_seg : 1;
  for (int s = 0; s < nseg; s++) if (!seg.out[s] || seg.rank[s] % 8 != 0 || seg.rank[s] > R) return LF_EINVAL;
  if (!ws || ws_bytes < lf_da_workspace(M, K, R, seg)) return LF_EWORKSPACE;
  if (dtype == LF_BF16) return da_impl<__bf16>(X, mask, dS, ws, M, K, R, seg, st);
  if (dtype == LF_F16) return da_impl<_Float16>(X, mask, dS, ws, M, K, R, seg, st);
  return LF_EINVAL;
}
