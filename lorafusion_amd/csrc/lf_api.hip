// extern "C" entry points of liblorafusion_hip.so: argument checks, workspace carving, launches.
#include "lf_common.h"
#include <atomic>
#include <algorithm>

int lf_launch_nf4_dequant(const uint8_t*, const void*, const float*, const float*, const float*, void*, int64_t,
                          int, int, int, hipStream_t);
int lf_launch_xa(const void*, const void*, int64_t, void*, const uint8_t*, uint8_t*, int, uint64_t, void*, int, int, int, const LfSegTable&, int,
                 hipStream_t);
int lf_launch_mask_pack(const uint8_t*, uint8_t*, int64_t, hipStream_t);
int lf_launch_mask_unpack(const uint8_t*, uint8_t*, int64_t, hipStream_t);
int lf_launch_dys_dyb(const void*, const void*, void*, void*, size_t, int, int, int, const LfSegTable&, int, hipStream_t);
int lf_launch_da(const void*, const uint8_t*, int, const void*, void*, size_t, int, int, int, const LfSegTable&, int, hipStream_t);
int lf_launch_dropout_mask(uint8_t*, int, int, float, const float*, int, uint64_t, hipStream_t);
size_t lf_xa_workspace(int, int, int, const LfSegTable&);
size_t lf_dys_dyb_workspace(int, int, int, const LfSegTable&);
size_t lf_da_workspace(int, int, int, const LfSegTable&);

// Scratch of lf_lora_bwd_static: part of the device image, one copy per GPU at its own address.  In
// host code the array's name is only a handle for hipGetSymbolAddress; kernels and launch code
// receive the looked-up device address.
static __device__ __align__(256) unsigned char scratch[LF_STATIC_SCRATCH_BYTES];
static constexpr int kMaxDevices = 64;
static std::atomic<void*> scratch_addr[kMaxDevices];

// Device address of `scratch` on the current device, looked up once per device (two threads that
// race here store the same value).
static int static_scratch(void** out) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return LF_ELAUNCH;
  void* p = scratch_addr[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return LF_ELAUNCH;
    scratch_addr[dev].store(p, std::memory_order_release);
  }
  *out = p;
  return LF_OK;
}

namespace {

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

// Host routing description -> kernel-argument table.
int make_seg(const lf_routing* r, int M, const void* const* ptrs, void* const* outs, LfSegTable& t) {
  if (!r) return LF_EINVAL;
  if (r->n_seg < 1) return LF_EINVAL;
  if (r->n_seg > LF_MAX_SEG) return LF_ELIMIT;
  t = LfSegTable{};
  t.n_seg = r->n_seg;
  t.block_size_m = r->block_size_m;
  t.n_blocks = r->n_blocks;
  t.table = r->block_table;
  t.block_scale = r->block_scale;
  t.block_p = r->block_p;
  t.scale = r->scale;
  t.p = r->p;
  if (r->block_table) {
    if (r->block_size_m != 128) return LF_ESHAPE;
    if (r->n_blocks < 1 || (int64_t)r->n_blocks * r->block_size_m != M) return LF_ESHAPE;
    if (!r->block_scale || !r->block_p) return LF_EINVAL;
  } else {
    if (r->n_seg != 1) return LF_EINVAL;
    if (!(r->p >= 0.f && r->p < 1.f)) return LF_EINVAL;
  }
  for (int s = 0; s < r->n_seg; s++) {
    t.first_block[s] = r->seg_first_block[s];
    t.rank[s] = r->seg_rank[s];
    t.ptr[s] = ptrs ? ptrs[s] : nullptr;
    t.out[s] = outs ? outs[s] : nullptr;
    if (t.rank[s] < 8 || t.rank[s] % 8 != 0 || t.rank[s] > LF_MAX_RANK) return LF_ESHAPE;
    if (s > 0 && t.first_block[s] <= t.first_block[s - 1]) return LF_EINVAL;
  }
  return LF_OK;
}

bool bad_dtype(int d) { return d != LF_BF16 && d != LF_F16; }
// `dtype` arguments carry the keep-mask format in LF_MASK_BITS: returns that flag and leaves the element type
int take_mask_bits(int& dtype) {
  const int bits = (dtype & LF_MASK_BITS) != 0;
  dtype &= ~LF_MASK_BITS;
  return bits;
}

// What the rank-r passes and their planners assume of a dimension they tile (N of dys_dyb, K of xa / da) and of R.
bool bad_tiled_dim(int v) { return v <= 0 || v % 128 != 0; }
bool bad_rank_cols(int R) { return R <= 0 || R % 16 != 0 || R > LF_MAX_RANK; }

}  // namespace

extern "C" {

int lf_version(void) { return 2; }

const char* lf_strerror(int code) {
  switch (code) {
    case LF_OK: return "ok";
    case LF_EINVAL: return "invalid argument (null pointer, non-positive size, unknown dtype or bad routing)";
    case LF_ESHAPE: return "shape not supported (need K % 128 == 0, N % 128 == 0, R % 16 == 0, R <= 128, rank % 8 == 0, routing block 128)";
    case LF_EWORKSPACE: return "workspace missing or too small (see lf_workspace_bytes)";
    case LF_ELAUNCH: return "HIP reported an error at kernel launch";
    case LF_ELIMIT: return "too many adapter segments in one call";
    case LF_ESTATIC: return "the call needs more scratch than the library's static buffer holds (LF_STATIC_SCRATCH_BYTES); use the entry point with a workspace argument";
    default: return "unknown error code";
  }
}

size_t lf_workspace_bytes(int op, int M, int N, int K, int R, const lf_routing* routing) {
  LfSegTable t;
  const void* dummy_ptrs[LF_MAX_SEG] = {};
  if (make_seg(routing, M, dummy_ptrs, nullptr, t) != LF_OK) return 0;
  // shapes the launch itself would refuse need no workspace; the planners are only asked about shapes they tile
  if (M <= 0 || bad_rank_cols(R)) return 0;
  const bool reads_n = op == LF_OP_DYS_DYB || op == LF_OP_BWD || op == LF_OP_NF4_BWD || op == LF_OP_NF4_FWD;
  const bool reads_k = op == LF_OP_XA || op == LF_OP_DA || op == LF_OP_FWD || op == LF_OP_BWD || op == LF_OP_NF4_FWD ||
                       op == LF_OP_NF4_BWD;
  if ((reads_n && bad_tiled_dim(N)) || (reads_k && bad_tiled_dim(K))) return 0;
  const int rb = t.table != nullptr ? t.block_size_m : 0;
  switch (op) {
    case LF_OP_XA: return align256(lf_xa_workspace(M, K, R, t));
    case LF_OP_DYS_DYB: return align256(lf_dys_dyb_workspace(M, N, R, t));
    case LF_OP_DA: return align256(lf_da_workspace(M, K, R, t));
    // (the products of the whole-pass entry points may split their contraction: Y = [M,N] over K, dX = [M,K] over N)
    case LF_OP_FWD: return align256(std::max(lf_xa_workspace(M, K, R, t), lf_gemm_ksplit_bytes(M, N, K, rb)));
    case LF_OP_BWD: {
      size_t a = lf_dys_dyb_workspace(M, N, R, t), b = lf_da_workspace(M, K, R, t);
      return align256(std::max(std::max(a, b), lf_gemm_ksplit_bytes(M, K, N, rb)));
    }
    case LF_OP_NF4_FWD:
      return align256((size_t)N * K * 2) + align256(std::max(lf_xa_workspace(M, K, R, t), lf_gemm_ksplit_bytes(M, N, K, rb)));
    case LF_OP_NF4_BWD: {
      size_t a = lf_dys_dyb_workspace(M, N, R, t), b = lf_da_workspace(M, K, R, t);
      return align256((size_t)N * K * 2) + align256(std::max(std::max(a, b), lf_gemm_ksplit_bytes(M, K, N, rb)));
    }
    default: return 0;
  }
}

int lf_lora_xa(const void* X, const uint8_t* mask, const void* const* a_ptrs, void* S, void* workspace,
               size_t ws_bytes, int M, int K, int R, const lf_routing* routing, int dtype, void* stream) {
  const int mb = take_mask_bits(dtype);
  if (bad_dtype(dtype) || !a_ptrs) return LF_EINVAL;
  LfSegTable t;
  int rc = make_seg(routing, M, a_ptrs, nullptr, t);
  if (rc != LF_OK) return rc;
  for (int s = 0; s < t.n_seg; s++) if (!t.ptr[s]) return LF_EINVAL;
  (void)workspace; (void)ws_bytes;  // no partial sums leave the workgroups
  return lf_launch_xa(X, nullptr, 0, nullptr, mask, nullptr, mb, 0, S, M, K, R, t, dtype, (hipStream_t)stream);
}

int lf_lora_xa_seeded(const void* X, uint8_t* mask_out, const void* const* a_ptrs, void* S, int M, int K, int R,
                      const lf_routing* routing, uint64_t seed, int dtype, void* stream) {
  const int mb = take_mask_bits(dtype);
  if (bad_dtype(dtype) || !a_ptrs || !mask_out) return LF_EINVAL;
  LfSegTable t;
  int rc = make_seg(routing, M, a_ptrs, nullptr, t);
  if (rc != LF_OK) return rc;
  for (int s = 0; s < t.n_seg; s++) if (!t.ptr[s]) return LF_EINVAL;
  return lf_launch_xa(X, nullptr, 0, nullptr, nullptr, mask_out, mb, seed, S, M, K, R, t, dtype, (hipStream_t)stream);
}

int lf_lora_xa_silu_mul(const void* G, const void* U, int64_t ld, void* X_out, const uint8_t* mask, uint8_t* mask_out,
                        uint64_t seed, const void* const* a_ptrs, void* S, int M, int K, int R, const lf_routing* routing,
                        int dtype, void* stream) {
  const int mb = take_mask_bits(dtype);
  if (bad_dtype(dtype) || !a_ptrs || !G || !U || !X_out) return LF_EINVAL;
  if (mask && mask_out) return LF_EINVAL;
  LfSegTable t;
  int rc = make_seg(routing, M, a_ptrs, nullptr, t);
  if (rc != LF_OK) return rc;
  for (int s = 0; s < t.n_seg; s++) if (!t.ptr[s]) return LF_EINVAL;
  return lf_launch_xa(G, U, ld, X_out, mask, mask_out, mb, seed, S, M, K, R, t, dtype, (hipStream_t)stream);
}

// lf_lora_xw_sb / lf_lora_dyw_dsa with a workspace for the split contraction of under-filled launches (the whole
// forward / backward entry points pass theirs on; the single-product entry points have none and never split)
static int xw_sb_ws(const void* X, const void* W, const void* bias, const void* S, const void* const* b_ptrs, void* Y,
                    void* workspace, size_t ws_bytes, int M, int N, int K, int R, const lf_routing* routing, int dtype,
                    void* stream) {
  if (bad_dtype(dtype) || !X || !W || !Y) return LF_EINVAL;
  LfSegTable t{};
  if (S) {
    if (!b_ptrs) return LF_EINVAL;
    int rc = make_seg(routing, M, b_ptrs, nullptr, t);
    if (rc != LF_OK) return rc;
    for (int s = 0; s < t.n_seg; s++) if (!t.ptr[s]) return LF_EINVAL;
  }
  if (K % 128 != 0 || N % 128 != 0) return LF_ESHAPE;
  LfGemmParams p{};
  p.A = X; p.B = W; p.C = Y; p.bias = bias;
  p.M = M; p.N = N; p.K = K; p.lda = K; p.ldb = K; p.ldc = N;
  p.L = S; p.R = R; p.mask = nullptr; p.ldmask = 0; p.mult_mode = 0;
  p.ks_ws = (float*)workspace; p.ks_ws_bytes = workspace ? ws_bytes : 0;
  return lf_launch_gemm(p, t, /*nn=*/false, dtype, -1, (hipStream_t)stream);
}

int lf_lora_xw_sb(const void* X, const void* W, const void* bias, const void* S, const void* const* b_ptrs,
                  void* Y, int M, int N, int K, int R, const lf_routing* routing, int dtype, void* stream) {
  return xw_sb_ws(X, W, bias, S, b_ptrs, Y, nullptr, 0, M, N, K, R, routing, dtype, stream);
}

int lf_swiglu_lora_fwd(const void* G, const void* U, int64_t ld, void* X_out, const void* W, const void* bias,
                       const uint8_t* mask, uint8_t* mask_out, uint64_t seed, const void* const* a_ptrs,
                       const void* const* b_ptrs, void* Y, void* S_out, void* workspace, size_t ws_bytes, int M, int N,
                       int K, int R, const lf_routing* routing, int dtype, void* stream) {
  int rc = lf_lora_xa_silu_mul(G, U, ld, X_out, mask, mask_out, seed, a_ptrs, S_out, M, K, R, routing, dtype, stream);
  if (rc != LF_OK) return rc;
  return xw_sb_ws(X_out, W, bias, S_out, b_ptrs, Y, workspace, ws_bytes, M, N, K, R, routing, dtype & ~LF_MASK_BITS, stream);
}

int lf_lora_dys_dyb(const void* dY, const void* S, const void* const* b_ptrs, void* dS, void* const* db_ptrs,
                    void* workspace, size_t ws_bytes, int M, int N, int R, const lf_routing* routing, int dtype,
                    void* stream) {
  if (bad_dtype(dtype) || !b_ptrs || !db_ptrs) return LF_EINVAL;
  LfSegTable t;
  int rc = make_seg(routing, M, b_ptrs, db_ptrs, t);
  if (rc != LF_OK) return rc;
  return lf_launch_dys_dyb(dY, S, dS, workspace, ws_bytes, M, N, R, t, dtype, (hipStream_t)stream);
}

int lf_lora_da(const void* X, const uint8_t* mask, const void* dS, void* const* da_ptrs, void* workspace,
               size_t ws_bytes, int M, int K, int R, const lf_routing* routing, int dtype, void* stream) {
  const int mb = take_mask_bits(dtype);
  if (bad_dtype(dtype) || !da_ptrs) return LF_EINVAL;
  LfSegTable t;
  int rc = make_seg(routing, M, nullptr, da_ptrs, t);
  if (rc != LF_OK) return rc;
  return lf_launch_da(X, mask, mb, dS, workspace, ws_bytes, M, K, R, t, dtype, (hipStream_t)stream);
}

static int dyw_dsa_ws(const void* dY, const void* W, const void* dS, const void* const* a_ptrs, const uint8_t* mask,
                      void* dX, void* workspace, size_t ws_bytes, int M, int N, int K, int R, const lf_routing* routing,
                      int dtype, void* stream) {
  const int mb = take_mask_bits(dtype);
  if (bad_dtype(dtype) || !dY || !W || !dX) return LF_EINVAL;
  LfSegTable t{};
  if (dS) {
    if (!a_ptrs) return LF_EINVAL;
    int rc = make_seg(routing, M, a_ptrs, nullptr, t);
    if (rc != LF_OK) return rc;
    for (int s = 0; s < t.n_seg; s++) if (!t.ptr[s]) return LF_EINVAL;
  }
  if (K % 128 != 0 || N % 128 != 0) return LF_ESHAPE;
  // dX[M,K] = dY[M,N] * W[N,K]: output columns = K, contraction = N
  LfGemmParams p{};
  p.A = dY; p.B = W; p.C = dX; p.bias = nullptr;
  p.M = M; p.N = K; p.K = N; p.lda = N; p.ldb = K; p.ldc = K;
  p.L = dS; p.R = R; p.mask = mask; p.ldmask = mb ? K / 8 : K; p.mask_bits = mb; p.mult_mode = 1;
  p.ks_ws = (float*)workspace; p.ks_ws_bytes = workspace ? ws_bytes : 0;
  return lf_launch_gemm(p, t, /*nn=*/true, dtype, -1, (hipStream_t)stream);
}

int lf_lora_dyw_dsa(const void* dY, const void* W, const void* dS, const void* const* a_ptrs, const uint8_t* mask,
                    void* dX, int M, int N, int K, int R, const lf_routing* routing, int dtype, void* stream) {
  return dyw_dsa_ws(dY, W, dS, a_ptrs, mask, dX, nullptr, 0, M, N, K, R, routing, dtype, stream);
}

int lf_lora_fwd(const void* X, const void* W, const void* bias, const uint8_t* mask, const void* const* a_ptrs,
                const void* const* b_ptrs, void* Y, void* S_out, void* workspace, size_t ws_bytes, int M, int N,
                int K, int R, const lf_routing* routing, int dtype, void* stream) {
  int rc = lf_lora_xa(X, mask, a_ptrs, S_out, workspace, ws_bytes, M, K, R, routing, dtype, stream);
  if (rc != LF_OK) return rc;
  // (the rank-r pass is done with the workspace: the product's split contraction may have it)
  return xw_sb_ws(X, W, bias, S_out, b_ptrs, Y, workspace, ws_bytes, M, N, K, R, routing, dtype & ~LF_MASK_BITS, stream);
}

int lf_lora_fwd_seeded(const void* X, const void* W, const void* bias, uint8_t* mask_out, const void* const* a_ptrs,
                       const void* const* b_ptrs, void* Y, void* S_out, void* workspace, size_t ws_bytes, int M, int N,
                       int K, int R, const lf_routing* routing, uint64_t seed, int dtype, void* stream) {
  int rc = lf_lora_xa_seeded(X, mask_out, a_ptrs, S_out, M, K, R, routing, seed, dtype, stream);
  if (rc != LF_OK) return rc;
  return xw_sb_ws(X, W, bias, S_out, b_ptrs, Y, workspace, ws_bytes, M, N, K, R, routing, dtype & ~LF_MASK_BITS, stream);
}

int lf_lora_bwd(const void* dY, const void* X, const void* W, const uint8_t* mask, const void* S,
                const void* const* a_ptrs, const void* const* b_ptrs, void* dX, void* const* da_ptrs,
                void* const* db_ptrs, void* dS_out, void* workspace, size_t ws_bytes, int M, int N, int K, int R,
                const lf_routing* routing, int dtype, void* stream) {
  int rc = lf_lora_dys_dyb(dY, S, b_ptrs, dS_out, db_ptrs, workspace, ws_bytes, M, N, R, routing, dtype & ~LF_MASK_BITS, stream);
  if (rc != LF_OK) return rc;
  rc = lf_lora_da(X, mask, dS_out, da_ptrs, workspace, ws_bytes, M, K, R, routing, dtype, stream);
  if (rc != LF_OK) return rc;
  // (stream order: the partial sums of the two rank-r passes are consumed by now, so the product's split contraction
  // may reuse the workspace from its start)
  if (dX) rc = dyw_dsa_ws(dY, W, dS_out, a_ptrs, mask, dX, workspace, ws_bytes, M, N, K, R, routing, dtype, stream);
  return rc;
}

int lf_lora_bwd_static(const void* dY, const void* X, const void* W, const uint8_t* mask, const void* S,
                       const void* const* a_ptrs, const void* const* b_ptrs, void* dX, void* const* da_ptrs,
                       void* const* db_ptrs, void* dS_out, int M, int N, int K, int R, const lf_routing* routing,
                       int dtype, void* stream) {
  if (bad_dtype(dtype & ~LF_MASK_BITS) || !dY || !X || !S || !b_ptrs || !da_ptrs || !db_ptrs || !dS_out) return LF_EINVAL;
  if (dX && (!W || !a_ptrs)) return LF_EINVAL;
  if (M <= 0 || N <= 0 || K <= 0 || R <= 0) return LF_EINVAL;
  if (bad_tiled_dim(N) || bad_tiled_dim(K) || bad_rank_cols(R)) return LF_ESHAPE;
  LfSegTable t;
  int rc = make_seg(routing, M, nullptr, nullptr, t);
  if (rc != LF_OK) return rc;
  // what lf_workspace_bytes(LF_OP_BWD, ...) names: the rank-r passes' partial sums or the dX product's partial tiles,
  // whichever is larger (with less, the product would not split its contraction and its sums would differ in order)
  const size_t a = lf_dys_dyb_workspace(M, N, R, t), b = lf_da_workspace(M, K, R, t);
  const size_t need = align256(std::max(std::max(a, b), lf_gemm_ksplit_bytes(M, K, N, t.table != nullptr ? t.block_size_m : 0)));
  if (need > (size_t)LF_STATIC_SCRATCH_BYTES) return LF_ESTATIC;
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc != LF_OK) return rc;
  return lf_lora_bwd(dY, X, W, mask, S, a_ptrs, b_ptrs, dX, da_ptrs, db_ptrs, dS_out, ws, LF_STATIC_SCRATCH_BYTES, M, N, K,
                     R, routing, dtype, stream);
}

int lf_set_tile_cfg(int tile_cfg) { return lf_pin_tile_cfg(tile_cfg); }

int lf_gemm_plan(int M, int N, int K, int routing_block_size_m, int* rows_head, int* cfg_head, int* cfg_tail) {
  if (M <= 0 || N <= 0 || K <= 0 || rows_head == nullptr || cfg_head == nullptr || cfg_tail == nullptr) return LF_EINVAL;
  lf_plan_gemm(M, N, K, routing_block_size_m, rows_head, cfg_head, cfg_tail);
  return LF_OK;
}

int lf_gemm(const void* A, const void* B, const void* bias, void* C, int M, int N, int K, int trans_b, int dtype,
            int tile_cfg, void* stream) {
  if (bad_dtype(dtype) || !A || !B || !C) return LF_EINVAL;
  LfSegTable t{};
  LfGemmParams p{};
  p.A = A; p.B = B; p.C = C; p.bias = bias;
  p.M = M; p.N = N; p.K = K; p.lda = K; p.ldb = trans_b ? K : N; p.ldc = N;
  return lf_launch_gemm(p, t, /*nn=*/!trans_b, dtype, tile_cfg, (hipStream_t)stream);
}

int lf_nf4_dequant(const uint8_t* packed, const void* absmax, const float* code2, const float* absmax2,
                   const float* offset, void* out, int64_t n_elems, int blocksize, int blocksize2, int out_dtype,
                   void* stream) {
  return lf_launch_nf4_dequant(packed, absmax, code2, absmax2, offset, out, n_elems, blocksize, blocksize2,
                               out_dtype, (hipStream_t)stream);
}

// Where the dequantised weight of an NF4 call lives: the caller's W->dense, or the head of the workspace.
static int nf4_dense(const lf_nf4_weight* W, bool needed, void* workspace, size_t ws_bytes, int N, int K, int dtype,
                     hipStream_t st, const void** dense, size_t* head) {
  *dense = nullptr;
  *head = 0;
  if (!needed) return LF_OK;
  if (!W || N <= 0 || K <= 0) return LF_EINVAL;
  void* dst = W->dense;
  if (dst != nullptr) {
    if (((uintptr_t)dst & 255) != 0) return LF_EINVAL;
    *dense = dst;
    if (W->dense_valid) return LF_OK;
  } else {
    *head = align256((size_t)N * K * 2);
    if (!workspace || ws_bytes < *head || ((uintptr_t)workspace & 255) != 0) return LF_EWORKSPACE;
    dst = workspace;
    *dense = dst;
  }
  if (!W->packed || !W->absmax) return LF_EINVAL;
  return lf_launch_nf4_dequant(W->packed, W->absmax, W->code2, W->absmax2, W->offset, dst, (int64_t)N * K, W->blocksize,
                               W->blocksize2, dtype, st);
}

int lf_nf4_lora_fwd(const void* X, const lf_nf4_weight* W, const void* bias, const uint8_t* mask,
                    const void* const* a_ptrs, const void* const* b_ptrs, void* Y, void* S_out, void* workspace,
                    size_t ws_bytes, int M, int N, int K, int R, const lf_routing* routing, int dtype, void* stream) {
  if (bad_dtype(dtype & ~LF_MASK_BITS)) return LF_EINVAL;
  const void* dense;
  size_t head;
  int rc = nf4_dense(W, true, workspace, ws_bytes, N, K, dtype & ~LF_MASK_BITS, (hipStream_t)stream, &dense, &head);
  if (rc != LF_OK) return rc;
  return lf_lora_fwd(X, dense, bias, mask, a_ptrs, b_ptrs, Y, S_out, workspace ? (char*)workspace + head : nullptr,
                     ws_bytes - head, M, N, K, R, routing, dtype, stream);
}

int lf_nf4_lora_bwd(const void* dY, const void* X, const lf_nf4_weight* W, const uint8_t* mask, const void* S,
                    const void* const* a_ptrs, const void* const* b_ptrs, void* dX, void* const* da_ptrs,
                    void* const* db_ptrs, void* dS_out, void* workspace, size_t ws_bytes, int M, int N, int K, int R,
                    const lf_routing* routing, int dtype, void* stream) {
  if (bad_dtype(dtype & ~LF_MASK_BITS)) return LF_EINVAL;
  const void* dense;
  size_t head;
  int rc = nf4_dense(W, dX != nullptr, workspace, ws_bytes, N, K, dtype & ~LF_MASK_BITS, (hipStream_t)stream, &dense, &head);
  if (rc != LF_OK) return rc;
  return lf_lora_bwd(dY, X, dense, mask, S, a_ptrs, b_ptrs, dX, da_ptrs, db_ptrs, dS_out,
                     workspace ? (char*)workspace + head : nullptr, ws_bytes - head, M, N, K, R, routing, dtype, stream);
}

int lf_mask_pack(const uint8_t* mask_bytes, uint8_t* mask_bits, int M, int K, void* stream) {
  if (!mask_bytes || !mask_bits || M <= 0 || K <= 0) return LF_EINVAL;
  if (K % 128 != 0 || (((uintptr_t)mask_bytes | (uintptr_t)mask_bits) & 15) != 0) return LF_ESHAPE;
  return lf_launch_mask_pack(mask_bytes, mask_bits, (int64_t)M * K, (hipStream_t)stream);
}

int lf_mask_unpack(const uint8_t* mask_bits, uint8_t* mask_bytes, int M, int K, void* stream) {
  if (!mask_bytes || !mask_bits || M <= 0 || K <= 0) return LF_EINVAL;
  if (K % 128 != 0 || (((uintptr_t)mask_bytes | (uintptr_t)mask_bits) & 15) != 0) return LF_ESHAPE;
  return lf_launch_mask_unpack(mask_bits, mask_bytes, (int64_t)M * K, (hipStream_t)stream);
}

int lf_dropout_mask(uint8_t* mask, int M, int K, float p, const lf_routing* routing, uint64_t seed, void* stream) {
  const float* block_p = nullptr;
  int bs = 0;
  if (routing != nullptr && (routing->block_table != nullptr || routing->block_p != nullptr)) {
    if (!routing->block_p || routing->block_size_m <= 0) return LF_EINVAL;
    if ((int64_t)routing->n_blocks * routing->block_size_m != M) return LF_ESHAPE;
    block_p = routing->block_p;
    bs = routing->block_size_m;
  }
  return lf_launch_dropout_mask(mask, M, K, p, block_p, bs, seed, (hipStream_t)stream);
}

}  // extern "C"
