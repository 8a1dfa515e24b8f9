/* CPU restatement of the seeded dropout keep-mask (test infrastructure, never linked into the
 * product).  The reference draws its mask with Triton's rand4x (Philox, 7 rounds, float compare;
 * lorafusion/ops/triton_ops/dropout.py:49-50, blocked_dropout.py:57-60); the build defines its own
 * stream -- Philox4x32 with the standard 10 rounds (Salmon, Moraes, Dror, Shaw: "Parallel random
 * numbers: as easy as 1, 2, 3", SC'11), sixteen bits per element, integer compare -- and this
 * file is its scalar definition.  Pinned by the published known-answer vectors of Philox4x32-10. */
#include <stdint.h>

void philox4x32_10_ref(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3], k0 = key[0], k1 = key[1];
  for (int r = 0; r < 10; r++) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0, p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0, n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c0 = n0; c1 = (uint32_t)p1; c2 = n2; c3 = (uint32_t)p0;
    k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

uint32_t keep_threshold_ref(float p) {
  const double s = (double)p * 65536.0;
  return s >= 65535.0 ? 65535u : (uint32_t)s;
}

/* mask[m][k] = draw(e % 8) of philox(counter = (e / 8, 0, 0), key = seed) >= floor(p_row[m] * 2^16),
 * e = m * K + k; draw j is the low (even j) or high (odd j) 16 bits of output word j / 2. */
void keep_mask_ref(uint8_t* mask, int64_t M, int64_t K, const float* row_p, uint64_t seed) {
  const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  for (int64_t m = 0; m < M; m++) {
    const uint32_t thr = keep_threshold_ref(row_p[m]);
    for (int64_t k = 0; k < K; k++) {
      const uint64_t e = (uint64_t)(m * K + k), c = e >> 3;
      const uint32_t ctr[4] = {(uint32_t)c, (uint32_t)(c >> 32), 0u, 0u};
      uint32_t w[4];
      philox4x32_10_ref(ctr, key, w);
      const uint32_t word = w[(e & 7) >> 1];
      const uint32_t draw = (e & 1) ? word >> 16 : word & 0xffffu;
      mask[m * K + k] = draw >= thr ? 1 : 0;
    }
  }
}
