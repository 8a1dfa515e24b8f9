// Seeded dropout keep-mask for gfx950: the mask half of seeded_dropout
// (lorafusion/ops/triton_ops/dropout.py:19-68) and of blocked_seeded_dropout with one p per
// 128-row block (lorafusion/ops/triton_ops/blocked_dropout.py:16-75).  The dropped tensor itself
// is never materialised here: the rank-r kernels rebuild it from X and this mask.
//
// Generator: Philox4x32 with 10 rounds (Salmon et al., SC'11), key = the 64-bit seed, counter =
// (element index / 8, 0, 0); the 16-bit draw (element index % 8) of the 128 output bits belongs to
// the element, which is kept when draw >= floor(p * 2^16).  The stream is a function of (seed, element index) only, so it is
// independent of the launch shape; it is not the reference's stream (Triton's rand4x with 7
// rounds and a float compare).  HBM bound: one byte written per element.
#include "lf_common.h"
#include "philox.h"

namespace {

// Each thread writes 16 consecutive mask bytes (two Philox calls); K % 16 == 0 keeps them in one row.
__global__ void __launch_bounds__(256)
dropout_mask_kernel(uint8_t* __restrict__ mask, int64_t n16, int K, uint32_t thr, const float* __restrict__ block_p,
                    int block_size_m, uint32_t seed_lo, uint32_t seed_hi) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= n16) return;
  const int64_t e0 = t * 16;
  if (block_p != nullptr) thr = lf_keep_threshold(block_p[(e0 / K) / block_size_m]);
  lf_u32x4 o;
#pragma unroll
  for (int c = 0; c < 2; c++) {
    uint32_t lo, hi;
    lf_keep8((uint64_t)(e0 >> 3) + c, thr, seed_lo, seed_hi, lo, hi);
    o[2 * c] = lo;
    o[2 * c + 1] = hi;
  }
  __builtin_nontemporal_store(o, (lf_u32x4*)(mask + e0));   // a write-only stream: no reason to keep it in the caches
}

// Keep-mask formats: one byte per element (the reference's bool tensor, lorafusion/ops/triton_ops/dropout.py:79) and
// one bit per element (element k of a row = bit k & 7 of byte k >> 3).  Each thread converts 16 elements.
__global__ void __launch_bounds__(256)
mask_pack_kernel(const lf_u32x4* __restrict__ bytes, uint16_t* __restrict__ bits, int64_t n16) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= n16) return;
  const lf_u32x4 v = bytes[t];
  uint32_t o = 0;
#pragma unroll
  for (int d = 0; d < 4; d++) {
    // any nonzero byte keeps: normalise to 0/1, then one multiply gathers the four bits (no carries: see lf_keep8)
    const uint32_t w = v[d];
    const uint32_t nz = ((w | ((w & 0x7f7f7f7fu) + 0x7f7f7f7fu)) >> 7) & 0x01010101u;
    o |= ((nz * 0x01020408u) >> 24) << (4 * d);
  }
  bits[t] = (uint16_t)o;
}

__global__ void __launch_bounds__(256)
mask_unpack_kernel(const uint16_t* __restrict__ bits, lf_u32x4* __restrict__ bytes, int64_t n16) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= n16) return;
  const uint32_t b = bits[t];
  lf_u32x4 o;
#pragma unroll
  for (int d = 0; d < 4; d++) o[d] = (((b >> (4 * d)) & 0xfu) * 0x00204081u) & 0x01010101u;
  __builtin_nontemporal_store(o, bytes + t);
}

}  // namespace

int lf_launch_mask_pack(const uint8_t* bytes, uint8_t* bits, int64_t n, hipStream_t st) {
  const int64_t n16 = n / 16, blocks = (n16 + 255) / 256;
  if (blocks > 0x7fffffffLL) return LF_ELIMIT;
  return lf_launch(mask_pack_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const lf_u32x4*)bytes, (uint16_t*)bits, n16);
}

int lf_launch_mask_unpack(const uint8_t* bits, uint8_t* bytes, int64_t n, hipStream_t st) {
  const int64_t n16 = n / 16, blocks = (n16 + 255) / 256;
  if (blocks > 0x7fffffffLL) return LF_ELIMIT;
  return lf_launch(mask_unpack_kernel, dim3((unsigned)blocks), dim3(256), 0, st, (const uint16_t*)bits, (lf_u32x4*)bytes, n16);
}

int lf_launch_dropout_mask(uint8_t* mask, int M, int K, float p, const float* block_p, int block_size_m, uint64_t seed,
                           hipStream_t st) {
  if (!mask || M <= 0 || K <= 0) return LF_EINVAL;
  if (K % 16 != 0 || ((uintptr_t)mask & 15) != 0) return LF_ESHAPE;
  if (!(p >= 0.f && p < 1.f)) return LF_EINVAL;
  if (block_p != nullptr && block_size_m <= 0) return LF_EINVAL;
  const uint32_t thr = lf_keep_threshold(p);
  const int64_t n16 = (int64_t)M * K / 16;
  const int64_t blocks = (n16 + 255) / 256;
  if (blocks > 0x7fffffffLL) return LF_ELIMIT;
  return lf_launch(dropout_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, st, mask, n16, K, thr, block_p, block_size_m,
                     (uint32_t)seed, (uint32_t)(seed >> 32));
}
