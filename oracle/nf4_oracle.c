/* NF4 block dequantisation oracle (test infrastructure; never linked into the product).
 *
 * Restates /root/reference/lorafusion/ops/triton_ops/dequantize_nf4.py:
 *   - the 16 code values              :16-33
 *   - flat byte offset -> block index :124-126, 288-315  (block = byte >> (log2(bs)-1))
 *   - nested absmax                   :129-138  absmax = fma(code[absq[blk]], absmax2[blk / bs2], offset)
 *   - nibble order and product        :154-158  byte i -> element 2i (high nibble), 2i+1 (low nibble)
 *   - interleave + cast on store      :251-268
 * Build: gcc -O2 -ffp-contract=off -shared -fPIC (see Makefile).  fmaf() is the single-rounding
 * fused multiply-add; -ffp-contract=off keeps the compiler from fusing the LUT*absmax product
 * with anything else.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

static const float NF4_CODE[16] = {
    -1.0f, -0.6961928009986877f, -0.5250730514526367f, -0.39491748809814453f,
    -0.28444138169288635f, -0.18477343022823334f, -0.09105003625154495f, 0.0f,
    0.07958029955625534f, 0.16093020141124725f, 0.24611230194568634f, 0.33791524171829224f,
    0.44070982933044434f, 0.5626170039176941f, 0.7229568362236023f, 1.0f};

const float* nf4_code_table(void) { return NF4_CODE; }

/* fp32 -> bf16, round to nearest even (NaN kept quiet). */
static uint16_t f32_to_bf16_rne(float f) {
  uint32_t u;
  memcpy(&u, &f, 4);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

/* absq: uint8 [n/blocksize] when nested (absmax2 != NULL), else absmax_f32 is used.
 * out_f32 (optional) gets the unrounded fp32 products; out_bf16 (optional) their RNE bf16 bits. */
void nf4_dequant_ref(const uint8_t* q, const uint8_t* absq, const float* absmax_f32, const float* code,
                     const float* absmax2, const float* offset, float* out_f32, uint16_t* out_bf16,
                     int64_t n_elems, int blocksize, int blocksize2) {
  int shift = 0, shift2 = 0;
  while ((1 << shift) < blocksize) shift++;
  shift -= 1; /* per packed byte: two elements */
  if (absmax2) {
    while ((1 << shift2) < blocksize2) shift2++;
    shift2 += shift;
  }
  for (int64_t i = 0; i < n_elems / 2; i++) {
    float absmax;
    if (absmax2) {
      float dq = code[absq[i >> shift]];
      absmax = fmaf(dq, absmax2[i >> shift2], offset[0]);
    } else {
      absmax = absmax_f32[i >> shift];
    }
    float hi = NF4_CODE[q[i] >> 4] * absmax;
    float lo = NF4_CODE[q[i] & 15] * absmax;
    if (out_f32) { out_f32[2 * i] = hi; out_f32[2 * i + 1] = lo; }
    if (out_bf16) { out_bf16[2 * i] = f32_to_bf16_rne(hi); out_bf16[2 * i + 1] = f32_to_bf16_rne(lo); }
  }
}

/* Per-block routing triple (rank, valid_rows, first_block): lorafusion/ops/multi_lora.py:369-435. */
int64_t routing_table_ref(const int32_t* seq_len, const int32_t* rank, int n_seg, int block_size_m,
                          int32_t* lookup /* [nb,3] */, int64_t max_blocks) {
  int64_t blk = 0;
  for (int s = 0; s < n_seg; s++) {
    int32_t padded = ((seq_len[s] - 1) / block_size_m + 1) * block_size_m;
    int64_t start = blk;
    for (int32_t i = 0; i < padded / block_size_m; i++) {
      if (blk >= max_blocks) return -1;
      int32_t valid = seq_len[s] - i * block_size_m;
      if (valid > block_size_m) valid = block_size_m;
      lookup[3 * blk + 0] = rank[s];
      lookup[3 * blk + 1] = valid;
      lookup[3 * blk + 2] = (int32_t)start;
      blk++;
    }
  }
  return blk;
}
