// NF4 block dequantisation for gfx950: packed 4-bit codes -> bf16/fp16, HBM-bandwidth bound.
//
// Replaces dequantize_16bit_nf4_kernel / dequantize_16bit_nf4_tiled_kernel
// (lorafusion/ops/triton_ops/dequantize_nf4.py:77-161,180-268).  Same arithmetic, bit for bit:
//   absmax = fma(code2[absq[blk]], absmax2[blk / blocksize2], offset)     (nested, :129-138)
//   out[2i] = NF4[q[i] >> 4] * absmax ; out[2i+1] = NF4[q[i] & 15] * absmax   (:154-158)
// with one fp32 rounding per operation and round-to-nearest-even on the final cast.
//
// Layout: the weight is one flat run of packed bytes, so the kernel is 1-D.  Each lane takes 4
// packed bytes (8 elements) per step and writes one 16-byte vector; a wavefront therefore
// reads 256 contiguous bytes and writes 1 KiB contiguous bytes per step.  The 16 NF4 values
// and the 256-entry second-level table live in LDS (a wave's lookups hit distinct banks or
// broadcast).  Each workgroup covers STEPS*2048 elements so several loads are in flight per lane.
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

#ifndef LF_NF4_STEPS
#define LF_NF4_STEPS 16
#endif
constexpr int NF4_THREADS = 256;
constexpr int NF4_STEPS = LF_NF4_STEPS;

template <typename T, bool NESTED>
__global__ void __launch_bounds__(NF4_THREADS)
nf4_dequant_kernel(const uint32_t* __restrict__ packed, const void* __restrict__ absmax_in,
                   const float* __restrict__ code2, const float* __restrict__ absmax2,
                   const float* __restrict__ offset_p, lf_u32x4* __restrict__ out, int64_t n_words /* packed dwords */,
                   int shift /* log2(blocksize) - 3: packed dword -> block */, int shift2 /* log2(blocksize2) */) {
  __shared__ float lut[16];
  __shared__ float lut2[256];
  __shared__ float am_lds[NF4_THREADS * NF4_STEPS];  // block scales of this workgroup's span (at most one per packed dword)
  const int tid = threadIdx.x;
  if (tid < 16) lut[tid] = kNf4Code[tid];
  if (NESTED) lut2[tid] = code2[tid];
  const int64_t wg_base = (int64_t)blockIdx.x * (NF4_THREADS * NF4_STEPS);
  const int64_t base = wg_base + tid;
  // packed data first: these are the loads the stores wait for
  uint32_t w[NF4_STEPS];
#pragma unroll
  for (int s = 0; s < NF4_STEPS; s++) {
    const int64_t i = base + (int64_t)s * NF4_THREADS;
        w[s] = i < n_words ? packed[i] : 0u;
  }
  if (NESTED) __syncthreads();  // lut2 is complete
  // One scale per quantisation block of the span, computed once (a lane-per-dword lookup would
  // issue a byte load and a float load per lane and step: twice the vector-memory instructions
  // of the data itself, and the texture addresser takes 16 cycles for each).
  const int64_t blk0 = wg_base >> shift;
  const int nblk = ((NF4_THREADS * NF4_STEPS) >> shift) > 0 ? (NF4_THREADS * NF4_STEPS) >> shift : 1;
  const int64_t nblk_total = (n_words + ((int64_t)1 << shift) - 1) >> shift;
  float offset = 0.f;
  if (NESTED) offset = offset_p[0];
  for (int j = tid; j < nblk; j += NF4_THREADS) {
    const int64_t blk = blk0 + j;
    float a = 0.f;
    if (blk < nblk_total) {
      if (NESTED) {
        const uint8_t aq = ((const uint8_t*)absmax_in)[blk];
        // single-rounding fused multiply-add, as tl.fma in the reference
        a = __builtin_fmaf(lut2[aq], absmax2[blk >> shift2], offset);
      } else {
        a = ((const float*)absmax_in)[blk];
      }
    }
    am_lds[j] = a;
  }
  __syncthreads();
  float am[NF4_STEPS];
#pragma unroll
  for (int s = 0; s < NF4_STEPS; s++) am[s] = am_lds[(s * NF4_THREADS + tid) >> shift];
#pragma unroll
  for (int s = 0; s < NF4_STEPS; s++) {
    const int64_t i = base + (int64_t)s * NF4_THREADS;
    if (i < n_words) {
      lf_u32x4 o;
#pragma unroll
      for (int b = 0; b < 4; b++) {
        const uint32_t byte = (w[s] >> (8 * b)) & 0xffu;  // memory order: byte b of the dword
        const float hi = lut[byte >> 4] * am[s];
        const float lo = lut[byte & 15u] * am[s];
        o[b] = pack2<T>(hi, lo);
      }
      out[i] = o;  // a plain store: the non-temporal kind fills 117 MB at 5.6 TB/s, this one at 6.45
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
  const int64_t per_wg = (int64_t)NF4_THREADS * NF4_STEPS;
  const int64_t grid = (n_words + per_wg - 1) / per_wg;
  if (grid > 0x7fffffffLL) return LF_ESHAPE;
#define LF_NF4_LAUNCH(T, NESTED)                                                                         \
  return lf_launch((nf4_dequant_kernel<T, NESTED>), dim3((unsigned)grid), dim3(NF4_THREADS), 0, st,      \
                     (const uint32_t*)packed, absmax, code2, absmax2, offset, (lf_u32x4*)out, n_words, shift, shift2)
  if (out_dtype == LF_BF16) {
    if (nested) LF_NF4_LAUNCH(__bf16, true); else LF_NF4_LAUNCH(__bf16, false);
  } else if (out_dtype == LF_F16) {
    if (nested) LF_NF4_LAUNCH(_Float16, true); else LF_NF4_LAUNCH(_Float16, false);
  } else {
    return LF_EINVAL;
  }
#undef LF_NF4_LAUNCH
}
