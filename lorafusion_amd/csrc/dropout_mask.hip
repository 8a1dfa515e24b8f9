// Seeded dropout keep-mask for gfx950: the mask half of seeded_dropout
// (lorafusion/ops/triton_ops/dropout.py:19-68) and of blocked_seeded_dropout with one p per
// 128-row block (lorafusion/ops/triton_ops/blocked_dropout.py:16-75).  The dropped tensor itself
// is never materialised here: the rank-r kernels rebuild it from X and this mask.
//
// Generator: Philox4x32 with 10 rounds (Salmon et al., SC'11), key = the 64-bit seed, counter =
// (element index / 4, 0, 0); output word (element index % 4) belongs to the element, which is kept
// when word >= floor(p * 2^32).  The stream is a function of (seed, element index) only, so it is
// independent of the launch shape; it is not the reference's stream (Triton's rand4x with 7
// rounds and a float compare).  HBM bound: one byte written per element.
#include "lf_common.h"

namespace {

__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
                                              uint32_t k1, uint32_t (&out)[4]) {
#pragma unroll
  for (int r = 0; r < 10; r++) {
    // one 32x32->64 multiply per product (v_mad_u64_u32) instead of separate high and low halves
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c0 = n0; c1 = (uint32_t)p1; c2 = n2; c3 = (uint32_t)p0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// Each thread writes 16 consecutive mask bytes (four Philox calls); K % 16 == 0 keeps them in one row.
__global__ void __launch_bounds__(256)
dropout_mask_kernel(uint8_t* __restrict__ mask, int64_t n16, int K, uint32_t thr, const float* __restrict__ block_p,
                    int block_size_m, uint32_t seed_lo, uint32_t seed_hi) {
  const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (t >= n16) return;
  const int64_t e0 = t * 16;
  if (block_p != nullptr) {
    const float p = block_p[(e0 / K) / block_size_m];
    const double s = (double)p * 4294967296.0;
    thr = s >= 4294967295.0 ? 0xffffffffu : (uint32_t)s;
  }
  lf_u32x4 o;
#pragma unroll
  for (int c = 0; c < 4; c++) {
    const uint64_t ctr = (uint64_t)(e0 >> 2) + c;
    uint32_t w[4];
    philox4x32_10((uint32_t)ctr, (uint32_t)(ctr >> 32), 0u, 0u, seed_lo, seed_hi, w);
    o[c] = (w[0] >= thr ? 1u : 0u) | (w[1] >= thr ? 0x100u : 0u) | (w[2] >= thr ? 0x10000u : 0u) | (w[3] >= thr ? 0x1000000u : 0u);
  }
  __builtin_nontemporal_store(o, (lf_u32x4*)(mask + e0));
}

}  // namespace

int lf_launch_dropout_mask(uint8_t* mask, int M, int K, float p, const float* block_p, int block_size_m, uint64_t seed,
                           hipStream_t st) {
  if (!mask || M <= 0 || K <= 0) return LF_EINVAL;
  if (K % 16 != 0 || ((uintptr_t)mask & 15) != 0) return LF_ESHAPE;
  if (!(p >= 0.f && p < 1.f)) return LF_EINVAL;
  if (block_p != nullptr && block_size_m <= 0) return LF_EINVAL;
  const double s = (double)p * 4294967296.0;
  const uint32_t thr = s >= 4294967295.0 ? 0xffffffffu : (uint32_t)s;
  const int64_t n16 = (int64_t)M * K / 16;
  const int64_t blocks = (n16 + 255) / 256;
  if (blocks > 0x7fffffffLL) return LF_ELIMIT;
  hipLaunchKernelGGL(dropout_mask_kernel, dim3((unsigned)blocks), dim3(256), 0, st, mask, n16, K, thr, block_p, block_size_m,
                     (uint32_t)seed, (uint32_t)(seed >> 32));
  return lf_check_launch();
}
