/* lorafusion_hip.h -- C ABI of liblorafusion_hip.so (MI355X / gfx950).
 *
 * Drop-in boundary for the `lorafusion.ops` LoRA-linear hot path of CentML/lorafusion.  The
 * reference's boundary is Python (Triton wrappers); each entry point below names the
 * reference wrapper it stands in for.  A Python layer (lorafusion_amd/ops) keeps the
 * reference's call signatures and calls these through ctypes.
 *
 * Conventions
 *  - Every tensor pointer is a DEVICE pointer owned by the caller; tensors are dense row-major.
 *    `lf_routing` and the `*_ptrs` arrays are HOST memory, read during the call only.
 *  - dtype: LF_BF16 or LF_F16 for all 16-bit tensors of a call; accumulation is fp32.
 *  - Return 0 on success, a negative LF_E* code otherwise (lf_strerror gives the text).  The
 *    library may be called from several host threads: the state it keeps is set once per device
 *    and then only read (per-kernel LDS limits, the compute-unit count, the address of the static
 *    scratch buffer), plus the one process-wide test knob of lf_set_tile_cfg (an atomic int);
 *    lf_lora_bwd_static is the one entry point whose calls share memory (see there).
 *  - Work is enqueued on `stream` (a hipStream_t, passed as void*); nothing synchronises.
 *  - The library allocates nothing: scratch memory comes in through `workspace`
 *    (size from lf_workspace_bytes), 256-byte aligned.
 *  - Shape limits: K % 128 == 0, N % 128 == 0, R % 16 == 0, 16 <= R <= 128, rank_i % 8 == 0,
 *    at most LF_MAX_SEG adapter segments per call, routing block size 128.
 *
 * Notation: X [M,K], W [N,K], A_i [r_i,K], B_i [N,r_i], S [M,R] = drop(X) A^T (1/(1-p) applied,
 * zero beyond rank_i and in padded rows), dS [M,R] = scale dY B, mask uint8 [M,K] keep-mask
 * (non-zero = keep), R = max rank rounded up to 16.  Wherever an entry point takes a keep-mask,
 * mask == NULL means "no dropout" for the whole call: p of the routing is then ignored and
 * nothing is rescaled by 1/(1-p).
 *
 * Keep-mask formats.  Every keep-mask argument (read or written) comes in one of two formats, chosen
 * per call by OR-ing LF_MASK_BITS into `dtype`:
 *  - bytes (default): uint8 [M,K], one byte per element, non-zero = keep -- the reference's bool
 *    tensor (lorafusion/ops/triton_ops/dropout.py:79, read back by
 *    fused_lora_dyw_dsa.py:144-153);
 *  - bits (dtype | LF_MASK_BITS): uint8 [M,K/8], element k of a row = bit (k & 7) of byte (k >> 3)
 *    of that row, 1 = keep; rows K/8 bytes apart, base 16-byte aligned.  An eighth of the traffic in
 *    every kernel that touches the mask; the format the Python layer uses for masks the library
 *    draws itself.  lf_mask_pack / lf_mask_unpack convert.  The large-shape GEMM kernel reads
 *    bits only: a dX call with a byte mask (or with more than 32 rank columns) runs on the older
 *    eight-wave tile, a few per cent slower.
 */
#ifndef LORAFUSION_HIP_H
#define LORAFUSION_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LF_OK 0
#define LF_EINVAL (-1)
#define LF_ESHAPE (-2)
#define LF_EWORKSPACE (-3)
#define LF_ELAUNCH (-4)
#define LF_ELIMIT (-5)
#define LF_ESTATIC (-6)

#define LF_BF16 0
#define LF_F16 1
#define LF_MASK_BITS 0x100 /* OR into dtype: the call's keep-masks are bit-packed (see above) */

#define LF_MAX_SEG 32

/* Routing of token rows to adapters.  Single adapter: n_seg = 1, block_table = NULL, `scale`
 * and `p` apply to all M rows.  Multi-LoRA: the per-block tables built by
 * prepare_multi_lora_batch_info (lorafusion/ops/multi_lora.py:348-453): block_table[b] =
 * (rank, valid_rows, first_block_of_segment); segment s owns blocks
 * [seg_first_block[s], seg_first_block[s+1]) and M must equal n_blocks * block_size_m.
 * One segment per adapter: dA_i / dB_i of a segment are written, not accumulated, so an adapter
 * whose tokens sit in two separate row ranges of one call would keep the second range's gradient
 * only -- pack each adapter's tokens contiguously, as prepare_multi_lora_batch_info's callers do
 * (lorafusion/train/training_utils.py:1304-1334 sorts by adapter), or give the two segments their own
 * outputs and sum them (the Python autograd layer does that by itself when one adapter's tensors are
 * passed for two segments: each occurrence receives its segment's gradient and autograd adds them). */
typedef struct lf_routing {
  int32_t n_seg;
  int32_t block_size_m;
  int32_t n_blocks;
  int32_t reserved;
  const int32_t* block_table; /* device int32 [n_blocks,3] or NULL */
  const float* block_scale;   /* device f32 [n_blocks] */
  const float* block_p;       /* device f32 [n_blocks] */
  float scale;
  float p;
  int32_t seg_first_block[LF_MAX_SEG];
  int32_t seg_rank[LF_MAX_SEG];
} lf_routing;

#define LF_OP_XA 0
#define LF_OP_DYS_DYB 1
#define LF_OP_DA 2
#define LF_OP_FWD 3
#define LF_OP_BWD 4
#define LF_OP_NF4_FWD 5
#define LF_OP_NF4_BWD 6

int lf_version(void);
const char* lf_strerror(int code);
/* Bytes of `workspace` the entry point(s) behind `op` use for this shape: the fp32 partial sums of
 * the rank-r passes, which a call must be given, and for LF_OP_FWD / BWD / NF4_* the fp32 partial
 * tiles of a split contraction (launches with few tiles and a long K: left-over rows of a packed
 * batch, short batches), which a call skips when the workspace is smaller or NULL.  0 also for a
 * shape or routing the entry point itself would refuse (M <= 0, R not a multiple of 16 in 16..128, a tiled dimension
 * -- N for DYS_DYB / BWD / NF4_*, K for XA / DA / FWD / BWD / NF4_* -- that is not a positive multiple
 * of 128, bad routing): the size query never fails harder than the call. */
size_t lf_workspace_bytes(int op, int M, int N, int K, int R, const lf_routing* routing);

/* S = drop(X) A^T.  Stands in for seeded_dropout + `masked_scaled_x @ lora_a.T`
 * (lorafusion/ops/lora_v1.py:111-119) and fused_dropout_matmul
 * (lorafusion/ops/triton_ops/fused_dropout_matmul.py:280-354); multi-LoRA: the `full_s` product
 * (lorafusion/ops/multi_lora.py:481-513).  mask may be NULL (no dropout). */
int lf_lora_xa(const void* X, const uint8_t* mask, const void* const* a_ptrs, void* S, void* workspace,
               size_t ws_bytes, int M, int K, int R, const lf_routing* routing, int dtype, void* stream);

/* lf_lora_xa with the keep-mask drawn inside the kernel instead of read: the reference's default
 * forward, where seeded_dropout makes the mask and the dropped input in one pass
 * (lorafusion/ops/lora_v1.py:111-116; fused_dropout_matmul with store_mask,
 * fused_dropout_matmul.py:300-352).  mask_out [M,K] receives exactly the bytes lf_dropout_mask
 * writes for the same (seed, routing): rows of a block with p = 0 are all ones. */
int lf_lora_xa_seeded(const void* X, uint8_t* mask_out, const void* const* a_ptrs, void* S, int M, int K, int R,
                      const lf_routing* routing, uint64_t seed, int dtype, void* stream);

/* Y = X W^T + scale * S B^T + bias.  Stands in for fused_lora_xw_sb / fused_lora_xw_sb_tma
 * (lorafusion/ops/triton_ops/fused_lora_xw_sb.py:209-316, fused_lora_xw_sb_tma.py:244-392) and
 * fused_multi_lora_xw_sb (fused_multi_lora_xw_sb.py:221-339).  bias may be NULL.  With S = NULL
 * the LoRA term is skipped (plain GEMM). */
int lf_lora_xw_sb(const void* X, const void* W, const void* bias, const void* S, const void* const* b_ptrs,
                  void* Y, int M, int N, int K, int R, const lf_routing* routing, int dtype, void* stream);

/* dS = scale dY B  and  dB_i = scale dY^T S over segment i.  Stands in for fused_lora_dys_dyb
 * (lorafusion/ops/triton_ops/fused_lora_dys_dyb.py:182-301) and fused_multi_lora_dys_dyb
 * (fused_multi_lora_dys_dyb.py:188-321).  Sums are two-stage and deterministic. */
int lf_lora_dys_dyb(const void* dY, const void* S, const void* const* b_ptrs, void* dS, void* const* db_ptrs,
                    void* workspace, size_t ws_bytes, int M, int N, int R, const lf_routing* routing, int dtype,
                    void* stream);

/* dA_i = dS^T drop(X) over segment i.  Stands in for `ds.T @ masked_scaled_x`
 * (lorafusion/ops/lora_v1.py:153, lorafusion/ops/multi_lora.py:576-581). */
int lf_lora_da(const void* X, const uint8_t* mask, const void* dS, void* const* da_ptrs, void* workspace,
               size_t ws_bytes, int M, int K, int R, const lf_routing* routing, int dtype, void* stream);

/* dX = dY W + where(mask, (dS A)/(1-p), 0).  Stands in for fused_lora_dyw_dsa(_tma)
 * (lorafusion/ops/triton_ops/fused_lora_dyw_dsa.py:184-297) and fused_multi_lora_dyw_dsa
 * (fused_multi_lora_dyw_dsa.py:188-305).  mask is [M,K]; NULL or p == 0 means no dropout. */
int lf_lora_dyw_dsa(const void* dY, const void* W, const void* dS, const void* const* a_ptrs, const uint8_t* mask,
                    void* dX, int M, int N, int K, int R, const lf_routing* routing, int dtype, void* stream);

/* Whole forward: lf_lora_xa then lf_lora_xw_sb.  Stands in for _fused_linear_lora_forward
 * (lorafusion/ops/lora_v1.py:87-129) and _fused_linear_multi_lora_forward
 * (lorafusion/ops/multi_lora.py:456-536).  S_out [M,R] is the tensor to keep for backward. */
int lf_lora_fwd(const void* X, const void* W, const void* bias, const uint8_t* mask, const void* const* a_ptrs,
                const void* const* b_ptrs, void* Y, void* S_out, void* workspace, size_t ws_bytes, int M, int N,
                int K, int R, const lf_routing* routing, int dtype, void* stream);

/* Whole forward with the mask drawn from `seed`: lf_lora_xa_seeded then lf_lora_xw_sb
 * (lorafusion/ops/lora_v1.py:87-129 called without a precomputed mask).  workspace as for lf_lora_fwd
 * (lf_workspace_bytes(LF_OP_FWD, ...); may be NULL: the product then never splits its contraction). */
int lf_lora_fwd_seeded(const void* X, const void* W, const void* bias, uint8_t* mask_out, const void* const* a_ptrs,
                       const void* const* b_ptrs, void* Y, void* S_out, void* workspace, size_t ws_bytes, int M, int N,
                       int K, int R, const lf_routing* routing, uint64_t seed, int dtype, void* stream);

/* Whole backward: lf_lora_dys_dyb, lf_lora_da, and (dX != NULL) lf_lora_dyw_dsa.  Stands in
 * for _fused_linear_lora_backward (lorafusion/ops/lora_v1.py:132-166) and
 * _fused_linear_multi_lora_backward (lorafusion/ops/multi_lora.py:539-599).  dS_out [M,R] is
 * scratch owned by the caller. */
int lf_lora_bwd(const void* dY, const void* X, const void* W, const uint8_t* mask, const void* S,
                const void* const* a_ptrs, const void* const* b_ptrs, void* dX, void* const* da_ptrs,
                void* const* db_ptrs, void* dS_out, void* workspace, size_t ws_bytes, int M, int N, int K, int R,
                const lf_routing* routing, int dtype, void* stream);

/* lf_lora_bwd without a workspace argument, for callers that cannot allocate device memory (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  It has no
 * counterpart in the reference.  The fp32 partial sums of the rank-r passes (and the partial tiles
 * of the dX product's split contraction, where it has one) go to a buffer of
 * LF_STATIC_SCRATCH_BYTES that is part of the library's device image (one copy per GPU, held until
 * the process ends); the call allocates and frees nothing.  A call that needs more than the buffer
 * holds (lf_workspace_bytes(LF_OP_BWD, ...) > LF_STATIC_SCRATCH_BYTES) returns LF_ESTATIC and
 * enqueues nothing.  All calls on one GPU share the buffer: calls that may overlap on one GPU
 * (different streams, or several host threads) race -- serialise them.  Nothing in the buffer has
 * to start at zero (every partial sum is written before it is read within the call), and its
 * contents after a call are unspecified.  The first call on a device looks up the buffer's
 * address, which loads the library's device code if no kernel of it has run there yet; make that
 * call outside a graph capture.  Outputs are bit-identical to lf_lora_bwd's. */
#define LF_STATIC_SCRATCH_BYTES (32u << 20)
int lf_lora_bwd_static(const void* dY, const void* X, const void* W, const uint8_t* mask, const void* S,
                       const void* const* a_ptrs, const void* const* b_ptrs, void* dX, void* const* da_ptrs,
                       void* const* db_ptrs, void* dS_out, int M, int N, int K, int R, const lf_routing* routing,
                       int dtype, void* stream);

/* C = A op(B) (+bias): trans_b = 1: B is [N,K] (C = A B^T); trans_b = 0: B is [K,N].  The same
 * MFMA kernel as above without the LoRA term; used to time the plain base GEMMs.  tile_cfg
 * = -1 lets the library choose. */
int lf_gemm(const void* A, const void* B, const void* bias, void* C, int M, int N, int K, int trans_b, int dtype,
            int tile_cfg, void* stream);

/* Tile configuration of every later MFMA GEMM launch of this process that does not name one itself
 * (the fused entry points, lf_gemm with tile_cfg = -1): 0..8 pins it, -1 (the initial state)
 * returns to the library's own choice.  A process-wide setting meant for tests and tuning runs --
 * parity of every tile shape at small sizes; the reference has the same kind of knob in the
 * Triton autotune configs of its kernels (lorafusion/ops/triton_ops/config.py).  A launch whose
 * shape the pinned configuration cannot take fails with LF_ESHAPE (7, the persistent kernel's
 * 256x256 tile, needs M, N >= 256 and K >= 128; 8, its 128x256 tile, M >= 128, N >= 256 and
 * K >= 256).  Returns LF_EINVAL outside -1..8. */
int lf_set_tile_cfg(int tile_cfg);

/* The launches the library makes for an M x N output contracted over K when no configuration is pinned: rows
 * [0, *rows_head) as one launch of tile configuration *cfg_head and, when *rows_head < M, the rest
 * as a second launch of *cfg_tail (-1 when there is none).  routing_block_size_m: 0 for a
 * single-adapter call, else the routing block size.  For benchmarks that time one kernel of a
 * fused call on its own; no counterpart in the reference (Triton's autotuner picks there). */
int lf_gemm_plan(int M, int N, int K, int routing_block_size_m, int* rows_head, int* cfg_head, int* cfg_tail);

/* NF4 block dequantisation.  Stands in for dequantize_nf4_triton
 * (lorafusion/ops/triton_ops/dequantize_nf4.py:271-346).  packed: uint8 [n/2] (element 2i in the
 * high nibble of byte i); absmax: uint8 [n/blocksize] when blocksize2 > 0 (double quantised:
 * absmax = fma(code2[absmax[b]], absmax2[b / blocksize2], offset)), else float32
 * [n/blocksize]; out: 16-bit [n]. */
int lf_nf4_dequant(const uint8_t* packed, const void* absmax, const float* code2, const float* absmax2,
                   const float* offset, void* out, int64_t n_elems, int blocksize, int blocksize2, int out_dtype,
                   void* stream);

/* An NF4 base weight [N,K] in the layout lf_nf4_dequant reads (the tensors of a bitsandbytes
 * QuantState: lorafusion/ops/triton_ops/dequantize_nf4.py:288-315). */
typedef struct lf_nf4_weight {
  const uint8_t* packed;  /* uint8 [N*K/2] */
  const void* absmax;     /* uint8 [N*K/blocksize] when blocksize2 > 0, else float32 */
  const float* code2;     /* float32 [256] or NULL */
  const float* absmax2;   /* float32 [N*K/blocksize/blocksize2] or NULL */
  const float* offset;    /* float32 [1] or NULL */
  int32_t blocksize;
  int32_t blocksize2;     /* 0: absmax is float32 (not nested) */
  void* dense;            /* optional: caller-owned 16-bit [N,K] buffer, 256-byte aligned, or NULL */
  int32_t dense_valid;    /* with `dense`: 0 = this call dequantises into it; 1 = it already holds the
                             dequantised weight (of this call's dtype) and nothing is dequantised */
  int32_t reserved;
} lf_nf4_weight;

/* QLoRA forward / backward: the base weight is stored as NF4, dequantised into the head of
 * `workspace` (2*N*K bytes, rounded up to 256) and fed to lf_lora_fwd / lf_lora_bwd, whose own
 * workspace follows it; sizes from lf_workspace_bytes(LF_OP_NF4_FWD / LF_OP_NF4_BWD, ...).  Stands
 * in for dequantize_nf4_triton followed by the fused LoRA linear, the flow the reference sketches
 * in lorafusion/ops/experimental/fused_quantized_nf4_lora_xw_sb_tma.py:280-428.
 * With W->dense the dequantised weight lives in the caller's buffer instead: the forward fills it
 * (dense_valid = 0) and a backward that follows while it is still live reuses it (dense_valid = 1)
 * -- one dequantisation per step instead of two, for 2*N*K bytes held in between; the workspace
 * is then that of lf_lora_fwd / lf_lora_bwd (LF_OP_FWD / LF_OP_BWD).  With dX == NULL the backward
 * needs no weight: it dequantises nothing and its workspace is that of LF_OP_BWD. */
int lf_nf4_lora_fwd(const void* X, const lf_nf4_weight* W, const void* bias, const uint8_t* mask,
                    const void* const* a_ptrs, const void* const* b_ptrs, void* Y, void* S_out, void* workspace,
                    size_t ws_bytes, int M, int N, int K, int R, const lf_routing* routing, int dtype, void* stream);
int lf_nf4_lora_bwd(const void* dY, const void* X, const lf_nf4_weight* W, const uint8_t* mask, const void* S,
                    const void* const* a_ptrs, const void* const* b_ptrs, void* dX, void* const* da_ptrs,
                    void* const* db_ptrs, void* dS_out, void* workspace, size_t ws_bytes, int M, int N, int K, int R,
                    const lf_routing* routing, int dtype, void* stream);

/* Seeded dropout keep-mask (1 = keep), uint8 [M, K], K % 16 == 0.  Stands in for the mask output of
 * seeded_dropout (lorafusion/ops/triton_ops/dropout.py:71-93) and, with `routing` carrying
 * block_p (n_blocks entries, one per block_size_m rows; the block table itself is not read), of
 * blocked_seeded_dropout (lorafusion/ops/triton_ops/blocked_dropout.py:78-135); routing == NULL
 * uses `p` for every row.
 * Philox4x32-10 keyed by `seed`, sixteen bits per element (element e: counter e/8, 16-bit draw e%8 of
 * the 128 output bits, low half of a word first), kept when draw >= floor(p * 2^16): a function of
 * (seed, element index) only. */
int lf_dropout_mask(uint8_t* mask, int M, int K, float p, const lf_routing* routing, uint64_t seed, void* stream);

/* Keep-mask format conversion: bytes [M,K] (non-zero = keep) -> bits [M,K/8] and back (to 0/1
 * bytes); K % 128 == 0, both buffers 16-byte aligned.  The reference has one format only (its bool
 * tensor, lorafusion/ops/triton_ops/dropout.py:79); these exist so that a caller holding such a
 * tensor can use the bit-packed entry points, and read back a mask the library drew. */
int lf_mask_pack(const uint8_t* mask_bytes, uint8_t* mask_bits, int M, int K, void* stream);
int lf_mask_unpack(const uint8_t* mask_bits, uint8_t* mask_bytes, int M, int K, void* stream);

/* RMSNorm and SiLU-multiply: the elementwise steps either side of the LoRA linears of a decoder layer.  The
 * reference takes them from the liger-kernel package (apply_liger_kernel, lorafusion/utils/module.py:41-71;
 * liger-kernel==0.5.6, requirements.txt:20); these stand in for that package's LigerRMSNormFunction ("llama"
 * casting mode, offset 0) and LigerSiLUMulFunction.  HBM-bound streams; X, Y, dY, dX dense [M,H] and W [H] of one
 * 16-bit dtype, 16-byte aligned, H % 8 == 0, H <= 8192 (LF_ELIMIT beyond).
 *   forward:  rstd[m] = 1/sqrt(mean_h X[m,h]^2 + eps) (fp32, kept for the backward);
 *             Y = round16(round16(X * rstd) * W)
 *   backward: dX = rstd * (dY*W - X * rstd^2 * mean_h(dY*W*X));  dW = sum_m dY * round16(X * rstd) (fp32 sums,
 *             summed in a fixed order: no atomics).  dX may alias dY.  dW == NULL skips the weight gradient (frozen
 *             norm weights, the LoRA fine-tuning case) and needs no workspace; otherwise `workspace` holds
 *             lf_rmsnorm_bwd_workspace(M, H) bytes. */
int lf_rmsnorm_fwd(const void* X, const void* W, void* Y, float* rstd, int M, int H, float eps, int dtype,
                   void* stream);
size_t lf_rmsnorm_bwd_workspace(int M, int H);
int lf_rmsnorm_bwd(const void* dY, const void* X, const void* W, const float* rstd, void* dX, void* dW, int M, int H,
                   int dtype, void* workspace, size_t workspace_bytes, void* stream);
/*   C = round16(round16(silu(A)) * B), silu in fp32;  dB = dC * silu(A),  dA = dC * (silu(A) * (1 - sig(A)) + sig(A)) * B.
 * All operands [M,I] with their own row strides in elements (ld >= I, ld % 8 == 0, I % 8 == 0, 16-byte aligned
 * bases), so A and B may be the two halves of a merged gate/up projection output [M,2I] and dA, dB the two halves
 * of its gradient.  dA may alias A and dB may alias B. */
int lf_silu_mul_fwd(const void* A, const void* B, void* C, int M, int I, int64_t lda, int64_t ldb, int64_t ldc,
                    int dtype, void* stream);
/* SiLU-multiply as the prologue of the LoRA linear that follows it (the down projection of a SwiGLU MLP: liger-kernel's
 * LigerSwiGLUMLP computes down_proj(silu(gate) * up), and the reference's patched down_proj then starts with the
 * rank-r pass of lorafusion/ops/lora_v1.py:111-119 / multi_lora.py:502-513 on that product).  lf_lora_xa_silu_mul is
 * lf_lora_xa / lf_lora_xa_seeded whose input X = round16(round16(silu(G)) * U) is computed on the fly from the gate and
 * up tensors [M,K] (rows `ld` elements apart: the halves of a merged projection output, or two tensors; ld >= K,
 * ld % 8 == 0, 16-byte aligned) and written once to X_out [M,K] for the base GEMM and the backward: the activation
 * pass and the rank-r pass's own read of X disappear.  X_out is bit-identical to lf_silu_mul_fwd's output and S to
 * lf_lora_xa's on it.  mask: explicit keep-mask [M,K] or NULL; mask_out != NULL: the mask is drawn from `seed` as
 * lf_lora_xa_seeded draws it and written there (mask and mask_out exclude each other); both NULL: no dropout.
 * lf_swiglu_lora_fwd adds the fused GEMM of lf_lora_xw_sb on X_out: Y = X_out W^T + scale S B^T + bias
 * (workspace as for lf_lora_fwd: lf_workspace_bytes(LF_OP_FWD, ...), or NULL).
 * The backward is lf_lora_bwd with X = X_out followed by lf_silu_mul_bwd on its dX. */
int lf_lora_xa_silu_mul(const void* G, const void* U, int64_t ld, void* X_out, const uint8_t* mask, uint8_t* mask_out,
                        uint64_t seed, const void* const* a_ptrs, void* S, int M, int K, int R, const lf_routing* routing,
                        int dtype, void* stream);
int lf_swiglu_lora_fwd(const void* G, const void* U, int64_t ld, void* X_out, const void* W, const void* bias,
                       const uint8_t* mask, uint8_t* mask_out, uint64_t seed, const void* const* a_ptrs,
                       const void* const* b_ptrs, void* Y, void* S_out, void* workspace, size_t ws_bytes, int M, int N,
                       int K, int R, const lf_routing* routing, int dtype, void* stream);
int lf_silu_mul_bwd(const void* dC, const void* A, const void* B, void* dA, void* dB, int M, int I, int64_t lddc,
                    int64_t lda, int64_t ldb, int64_t ldda, int64_t lddb, int dtype, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* LORAFUSION_HIP_H */
