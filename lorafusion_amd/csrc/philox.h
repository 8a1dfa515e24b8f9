// Philox4x32-10 (Salmon et al., SC'11) and the keep rule of the seeded dropout mask, shared by the
// standalone mask kernel and the rank-r forward pass that draws its mask on the fly.
// Element e of the [M, K] mask uses counter (e / 8, 0, 0), key = the 64-bit seed, and the 16-bit
// draw e % 8 of the call's 128 output bits (word (e % 8) / 2, low half for even e, high half for odd
// e); it is kept when draw >= floor(p * 2^16).  Sixteen bits per element resolve p to 1.5e-5 and halve
// the integer multiplies per element, which are what bounds the generation (20 quarter-rate 32x32
// multiplies per call).
#pragma once
#include <stdint.h>

__device__ __forceinline__ void lf_philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0,
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

__host__ __device__ __forceinline__ uint32_t lf_keep_threshold(float p) {
  const double s = (double)p * 65536.0;
  return s >= 65535.0 ? 65535u : (uint32_t)s;
}

// Keep bytes (0/1) of the eight elements 8*ctr .. 8*ctr+7 in memory order: `lo` holds the first four.
__device__ __forceinline__ void lf_keep8(uint64_t ctr, uint32_t thr, uint32_t seed_lo, uint32_t seed_hi, uint32_t& lo,
                                         uint32_t& hi) {
  uint32_t w[4];
  lf_philox4x32_10((uint32_t)ctr, (uint32_t)(ctr >> 32), 0u, 0u, seed_lo, seed_hi, w);
  lo = ((w[0] & 0xffffu) >= thr ? 1u : 0u) | ((w[0] >> 16) >= thr ? 0x100u : 0u) | ((w[1] & 0xffffu) >= thr ? 0x10000u : 0u) |
       ((w[1] >> 16) >= thr ? 0x1000000u : 0u);
  hi = ((w[2] & 0xffffu) >= thr ? 1u : 0u) | ((w[2] >> 16) >= thr ? 0x100u : 0u) | ((w[3] & 0xffffu) >= thr ? 0x10000u : 0u) |
       ((w[3] >> 16) >= thr ? 0x1000000u : 0u);
}
