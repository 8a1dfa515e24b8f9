// NF4 block dequantisation for gfx950: packed 4-bit codes -> bf16/fp16, HBM-bandwidth bound.
//
// Replaces dequantize_16bit_nf4_kernel / dequantize_16bit_nf4_tiled_kernel
// (lorafusion/ops/triton_ops/dequantize_nf4.py:77-161,180-268).  Same arithmetic, bit for bit:
//   absmax = fma(code2[absq[blk]], absmax2[blk / blocksize2], offset)     (nested, :129-138)
//   out[2i] = NF4[q[i] >> 4] * absmax ; out[2i+1] = NF4[q[i] & 15] * absmax   (:154-158)
// with one fp32 rounding per operation and round-to-nearest-even on the final cast.
//
// Layout: the weight is one flat run of packed bytes, so the kernel is 1-D, and every wavefront works alone: no
// barrier after the set-up of the two tables.  A wave takes chunks of 64*U packed dwords (U steps; each lane 4 packed
// bytes = 8 elements per step, so a step reads 256 contiguous bytes and writes 1 KiB contiguous bytes); chunk c
// goes to wave c mod (waves of the grid), so the addresses in flight form one compact window that moves through
// the weight.  The block scales of a chunk are computed once by its first lanes (one byte load and one table
// lookup per quantisation block, not per lane and step: the texture addresser's time goes to the data) and handed
// to the lanes of each step by a cross-lane read.  The loads of a wave's next chunk are issued before the stores
// of the current one.  The 16 NF4 values and the 256-entry second-level table live in LDS (a wave's lookups hit
// distinct banks or broadcast).
//
// Stores are non-temporal: the output is 4 of every 5 bytes this kernel moves and is written exactly once, and
// with stores that do not allocate in the caches the [14336, 4096] weight takes 21.5 us instead of 23.5, the
// [57344, 8192] weight 165 us instead of 220 (7.15 TB/s; a fill of the same output alone: 137 us).  Non-temporal
// loads of the packed bytes measured slower (26.5 us at [14336, 4096]).
#include "lf_common.h"

namespace {

__constant__ float kNf4Code[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f, 0.33791524171829224f,
    0.44070982933044434f, 0.5626170039176941f, 0.7229568362236023f, 1.0f};

template <typename T> __device__ __forceinline__ uint32_t pack2(float lo, float hi);
template <> __device__ __forceinline__ uint32_t pack2<__bf16>(float lo, float hi) {
  typedef __bf16 v2 __attribute__((ext_vector_type(2)));
  v2 v = {(__bf16)lo, (__bf16)hi};
  return __builtin_bit_cast(uint32_t, v);
}
template <> __device__ __forceinline__ uint32_t pack2<_Float16>(float lo, float hi) {
  typedef _Float16 v2 __attribute__((ext_vector_type(2)));
  v2 v = {(_Float16)lo, (_Float16)hi};
  return __builtin_bit_cast(uint32_t, v);
}

constexpr int NF4_THREADS = 256;
constexpr int NF4_WAVES = NF4_THREADS / 64;

template <typename T, bool NESTED, int U>
__global__ void __launch_bounds__(NF4_THREADS)
nf4_dequant_kernel(const uint32_t* __restrict__ packed, const void* __restrict__ absmax_in,
                   const float* __restrict__ code2, const float* __restrict__ absmax2,
                   const float* __restrict__ offset_p, lf_u32x4* __restrict__ out, int64_t n_words /* packed dwords */,
                   int shift /* log2(blocksize) - 3: packed dword -> block */, int shift2 /* log2(blocksize2) */,
                   int64_t n_chunks /* of 64*U packed dwords */) {
  __shared__ float lut[16];
  __shared__ float lut2[256];
  const int tid = threadIdx.x, lane = tid & 63;
  if (tid < 16) lut[tid] = kNf4Code[tid];
  if (NESTED) lut2[tid] = code2[tid];
  __syncthreads();
  const float offset = NESTED ? offset_p[0] : 0.f;
  const int64_t wave0 = (int64_t)blockIdx.x * NF4_WAVES + (tid >> 6), n_waves = (int64_t)gridDim.x * NF4_WAVES;
  // quantisation blocks per chunk (a block larger than a chunk holds whole chunks: the launcher picks U so that
  // there are at most 64), and the lane that holds the scale of this lane's dword in each step
  const int n_lead = ((64 * U) >> shift) > 0 ? (64 * U) >> shift : 1;
  const int64_t nblk_total = (n_words + ((int64_t)1 << shift) - 1) >> shift;
  int src[U];
#pragma unroll
  for (int s = 0; s < U; s++) src[s] = ((s * 64 + lane) >> shift) * 4;

  uint32_t w_next[U], aq_next = 0;
  float a2_next = 0.f;
  auto request = [&](int64_t c) {
    const int64_t base = c * (64 * U);
#pragma unroll
    for (int s = 0; s < U; s++) {
      const int64_t i = base + s * 64 + lane;
      w_next[s] = i < n_words ? packed[i] : 0u;
    }
    const int64_t blk = (base >> shift) + lane;
    aq_next = 0;
    a2_next = 0.f;
    if (lane < n_lead && blk < nblk_total) {
      if (NESTED) {
        aq_next = ((const uint8_t*)absmax_in)[blk];
        a2_next = absmax2[blk >> shift2];
      } else {
        a2_next = ((const float*)absmax_in)[blk];
      }
    }
  };
  int64_t c = wave0;
  if (c < n_chunks) request(c);
  for (; c < n_chunks; c += n_waves) {
    uint32_t w[U];
#pragma unroll
    for (int s = 0; s < U; s++) w[s] = w_next[s];
    const uint32_t aq = aq_next;
    const float a2 = a2_next;
    if (c + n_waves < n_chunks) request(c + n_waves);
    // single-rounding fused multiply-add, as tl.fma in the reference
    const float scale = NESTED ? __builtin_fmaf(lut2[aq], a2, offset) : a2;
    const int64_t base = c * (64 * U);
#pragma unroll
    for (int s = 0; s < U; s++) {
      // (all 64 lanes take part in the cross-lane read: the bounds check comes after it)
      const float am = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src[s], __builtin_bit_cast(int, scale)));
      const int64_t i = base + s * 64 + lane;
      if (i < n_words) {
        lf_u32x4 o;
#pragma unroll
        for (int b = 0; b < 4; b++) {
          const uint32_t byte = (w[s] >> (8 * b)) & 0xffu;  // memory order: byte b of the dword
          const float hi = lut[byte >> 4] * am;
          const float lo = lut[byte & 15u] * am;
          o[b] = pack2<T>(hi, lo);
        }
        __builtin_nontemporal_store(o, out + i);
      }
    }
  }
}

}  // namespace

int lf_launch_nf4_dequant(const uint8_t* packed, const void* absmax, const float* code2, const float* absmax2,
                          const float* offset, void* out, int64_t n_elems, int blocksize, int blocksize2,
                          int out_dtype, hipStream_t st) {
  if (!packed || !absmax || !out || n_elems <= 0) return LF_EINVAL;
  if (blocksize < 8 || (blocksize & (blocksize - 1)) != 0 || n_elems % blocksize != 0) return LF_ESHAPE;
  const bool nested = blocksize2 > 0;
  if (nested && (!code2 || !absmax2 || !offset || (blocksize2 & (blocksize2 - 1)) != 0)) return LF_EINVAL;
  if (((uintptr_t)packed & 3) != 0 || ((uintptr_t)out & 15) != 0) return LF_ESHAPE;
  int shift = 0, shift2 = 0;
  while ((1 << shift) < blocksize) shift++;
  shift -= 3;  // 8 elements per packed dword
  while (nested && (1 << shift2) < blocksize2) shift2++;
  const int64_t n_words = n_elems / 8;
  // four steps per chunk; one for blocksizes 8 and 16, whose chunk of four steps would hold more than 64 blocks
  const int u = shift >= 2 ? 4 : 1;
  const int64_t n_chunks = (n_words + 64 * u - 1) / (64 * u);
  int64_t grid = (n_chunks + NF4_WAVES - 1) / NF4_WAVES;   // one chunk per wave up to 2^20 workgroups, then several
  if (grid > (1 << 20)) grid = 1 << 20;
#define LF_NF4_LAUNCH_U(T, NESTED, U)                                                                    \
  return lf_launch((nf4_dequant_kernel<T, NESTED, U>), dim3((unsigned)grid), dim3(NF4_THREADS), 0, st,   \
                   (const uint32_t*)packed, absmax, code2, absmax2, offset, (lf_u32x4*)out, n_words, shift, shift2, n_chunks)
#define LF_NF4_LAUNCH(T, NESTED)                                                                         \
  do { if (u == 4) LF_NF4_LAUNCH_U(T, NESTED, 4); else LF_NF4_LAUNCH_U(T, NESTED, 1); } while (0)
  if (out_dtype == LF_BF16) {
    if (nested) LF_NF4_LAUNCH(__bf16, true); else LF_NF4_LAUNCH(__bf16, false);
  } else if (out_dtype == LF_F16) {
    if (nested) LF_NF4_LAUNCH(_Float16, true); else LF_NF4_LAUNCH(_Float16, false);
  } else {
    return LF_EINVAL;
  }
#undef LF_NF4_LAUNCH
#undef LF_NF4_LAUNCH_U
}
