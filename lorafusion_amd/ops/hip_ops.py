"""Kernel-level wrappers: one Python function per reference Triton wrapper, backed by HIP.

Names, argument meaning and error behaviour (``ValueError`` with a message for every
shape / dtype / contiguity violation) follow ``lorafusion/ops/triton_ops/*.py``; the work is
done by liblorafusion_hip.so through ctypes.  Single-adapter functions take plain tensors;
``*_multi_*`` functions take the per-block routing tables of ``prepare_multi_lora_batch_info``.
"""

from __future__ import annotations

import ctypes
import random

import torch

from lorafusion_amd import _lib as L

FUSED_MULTI_LORA_BLOCK_SIZE_M = 128


# --------------------------------------------------------------------------- validation


def _check_2d(t: torch.Tensor, name: str, dtype: torch.dtype | None = None) -> None:
    if t.ndim != 2:
        raise ValueError(f"{name} must be a 2D tensor, but got {t.ndim}D.")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous.")
    if dtype is not None and t.dtype != dtype:
        raise ValueError(f"{name} must have dtype {dtype}, but got {t.dtype}.")
    L.require_gpu(t, name)


def _check_mask(mask: torch.Tensor | None, shape, name: str = "dropout_mask") -> torch.Tensor | None:
    """A keep-mask for a ``shape = (M, K)`` input: bool / uint8 ``[M, K]`` (one byte per element, the reference's
    format) or uint8 ``[M, K // 8]`` (bit-packed: element k of a row = bit k & 7 of byte k >> 3; ``pack_mask``)."""
    if mask is None:
        return None
    if mask.dtype not in (torch.bool, torch.uint8):
        raise ValueError(f"{name} must be a bool (or uint8) tensor, but got {mask.dtype}.")
    M, K = tuple(shape)
    if tuple(mask.shape) != (M, K) and not (mask.dtype == torch.uint8 and tuple(mask.shape) == (M, K // 8)):
        raise ValueError(f"{name} must have shape {tuple(shape)}, but got {tuple(mask.shape)}.")
    if not mask.is_contiguous():
        raise ValueError(f"{name} must be contiguous.")
    L.require_gpu(mask, name)
    return mask


def _dt(t: torch.Tensor, mask: torch.Tensor | None, K: int) -> int:
    """The C ABI's dtype argument of a call whose keep-mask is ``mask``: the element type, plus the flag that says
    the mask is bit-packed (told apart by its row length: K // 8 bytes instead of K)."""
    bits = mask is not None and mask.shape[-1] * 8 == K and mask.dtype == torch.uint8
    return L.dtype_id(t.dtype) | (L.LF_MASK_BITS if bits else 0)


def is_packed_mask(mask: torch.Tensor | None, K: int) -> bool:
    return mask is not None and mask.dtype == torch.uint8 and mask.shape[-1] * 8 == K


def pack_mask(mask: torch.Tensor) -> torch.Tensor:
    """bool / uint8 ``[M, K]`` keep-mask -> bit-packed uint8 ``[M, K // 8]`` (K % 128 == 0), on the GPU."""
    if mask.ndim != 2 or mask.dtype not in (torch.bool, torch.uint8) or not mask.is_contiguous():
        raise ValueError("pack_mask takes a contiguous 2D bool (or uint8) tensor.")
    L.require_gpu(mask, "mask")
    M, K = mask.shape
    _check_dims(M, None, K)
    bits = torch.empty((M, K // 8), dtype=torch.uint8, device=mask.device)
    L.check(L.lib().lf_mask_pack(L.ptr(mask), L.ptr(bits), M, K, L.stream_of(mask)), "lf_mask_pack")
    return bits


def unpack_mask(bits: torch.Tensor) -> torch.Tensor:
    """bit-packed uint8 ``[M, K // 8]`` -> bool ``[M, K]``."""
    if bits.ndim != 2 or bits.dtype != torch.uint8 or not bits.is_contiguous():
        raise ValueError("unpack_mask takes a contiguous 2D uint8 tensor.")
    L.require_gpu(bits, "bits")
    M, K = bits.shape[0], bits.shape[1] * 8
    _check_dims(M, None, K)
    mask = torch.empty((M, K), dtype=torch.bool, device=bits.device)
    L.check(L.lib().lf_mask_unpack(L.ptr(bits), L.ptr(mask), M, K, L.stream_of(bits)), "lf_mask_unpack")
    return mask


def _check_dims(M: int, N: int | None, K: int | None) -> None:
    if M <= 0:
        raise ValueError(f"M must be positive, got {M}.")
    if K is not None and K % 128 != 0:
        raise ValueError(f"K must be a multiple of 128, got {K}.")
    if N is not None and N % 128 != 0:
        raise ValueError(f"N must be a multiple of 128, got {N}.")


def _check_rank(r: int) -> None:
    if r < 8 or r % 8 != 0 or r > 128:
        raise ValueError(f"LoRA rank must be a multiple of 8 in [8, 128], got {r}.")


def _check_p(p: float) -> None:
    if not (0.0 <= p < 1.0):
        raise ValueError(f"dropout_p must be in [0, 1), got {p}.")


class MultiRouting:
    """Host + device description of a packed multi-LoRA batch, shared by all multi kernels."""

    def __init__(self, padded_seq_len_list, rank_list, block_to_lookup_table, block_to_alpha,
                 block_to_dropout_p, *, enable_dropout: bool = True,
                 block_size_m: int = FUSED_MULTI_LORA_BLOCK_SIZE_M):
        if block_size_m != FUSED_MULTI_LORA_BLOCK_SIZE_M:
            raise ValueError(
                f"block_size_m must be {FUSED_MULTI_LORA_BLOCK_SIZE_M} for the fused multi-LoRA kernels, got {block_size_m}."
            )
        tbl = block_to_lookup_table
        if tbl.ndim != 2 or tbl.shape[1] != 3 or tbl.dtype != torch.int32:
            raise ValueError("block_to_lookup_table must be an int32 tensor of shape [num_blocks, 3].")
        L.require_gpu(tbl, "block_to_lookup_table")
        nb = tbl.shape[0]
        if sum(padded_seq_len_list) != nb * block_size_m:
            raise ValueError(
                f"sum(padded_seq_len_list)={sum(padded_seq_len_list)} does not match {nb} blocks of {block_size_m} rows."
            )
        if any(p % block_size_m for p in padded_seq_len_list):
            raise ValueError("every padded sequence length must be a multiple of block_size_m.")
        for r in rank_list:
            _check_rank(r)
        self.table = tbl.contiguous()
        self.scale = block_to_alpha.to(device=tbl.device, dtype=torch.float32).contiguous()
        if enable_dropout:
            self.p = block_to_dropout_p.to(device=tbl.device, dtype=torch.float32).contiguous()
        else:
            self.p = torch.zeros(nb, dtype=torch.float32, device=tbl.device)
        if self.scale.numel() != nb or self.p.numel() != nb:
            raise ValueError("block_to_alpha and block_to_dropout_p must have one entry per block.")
        self.padded_seq_len_list = list(padded_seq_len_list)
        self.rank_list = list(rank_list)
        self.block_size_m = block_size_m
        self.enable_dropout = bool(enable_dropout)
        self.n_blocks = nb
        self.M = nb * block_size_m
        self.R = L.round_rank(max(rank_list))
        self.c = L.multi_routing(self.padded_seq_len_list, self.rank_list, self.table, self.scale, self.p, block_size_m)


def _routing_single(rank: int, scale: float, p: float):
    _check_rank(rank)
    _check_p(p)
    return L.single_routing(rank, scale, p)


def _ws(op: int, M: int, N: int, K: int, R: int, routing, device):
    n = L.lib().lf_workspace_bytes(op, M, N, K, R, routing)
    return L.workspace(n, device), n


# --------------------------------------------------------------------------- forward pieces


def _xa(x, mask, a_list, routing, M, K, R):
    s = torch.empty((M, R), dtype=x.dtype, device=x.device)
    ws, nbytes = _ws(L.LF_OP_XA, M, 0, K, R, routing, x.device)
    rc = L.lib().lf_lora_xa(L.ptr(x), L.ptr(mask), L.ptr_array(a_list), L.ptr(s), L.ptr(ws), nbytes, M, K, R,
                            routing, _dt(x, mask, K), L.stream_of(x))
    L.check(rc, "lf_lora_xa")
    return s


def make_dropout_mask(shape, p, seed: int | None, device, routing: "MultiRouting | None" = None) -> torch.Tensor:
    """Bernoulli(1-p) keep-mask, bool ``[M, K]``, drawn on the device by the HIP Philox kernel.

    The mask half of ``seeded_dropout`` (lorafusion/ops/triton_ops/dropout.py:71-93); with
    ``routing`` the per-block p of the packed batch is used (blocked_seeded_dropout,
    lorafusion/ops/triton_ops/blocked_dropout.py:78-135) and ``p`` is ignored.  ``seed=None``
    draws a seed on the host, as the reference does (dropout.py:75-76).
    """
    M, K = int(shape[0]), int(shape[1])
    if K % 16 != 0:
        raise ValueError(f"the mask kernel needs K % 16 == 0, got K={K}.")
    if seed is None:
        seed = random.randrange(int(1e6))  # noqa: S311
    dev = torch.device(device)
    if dev.type != "cuda":
        raise ValueError("make_dropout_mask draws the mask on the GPU; got device " + str(device))
    if dev.index is None:
        dev = torch.device("cuda", torch.cuda.current_device())
    mask = torch.empty((M, K), dtype=torch.bool, device=dev)
    rc = None
    if routing is not None:
        if routing.M != M:
            raise ValueError(f"routing covers {routing.M} rows, mask has {M}.")
        rc, pv = ctypes.byref(routing.c), 0.0
    else:
        _check_p(float(p))
        pv = float(p)
    with torch.cuda.device(dev):
        L.check(L.lib().lf_dropout_mask(L.ptr(mask), M, K, ctypes.c_float(pv), rc, ctypes.c_uint64(int(seed) & 0xFFFFFFFFFFFFFFFF),
                                        L.stream_of(mask)), "lf_dropout_mask")
    return mask


def seeded_dropout(x: torch.Tensor, p: float, seed: int | None = None, *, store_mask: bool = True):
    """``(where(mask, x/(1-p), 0), mask)`` -- lorafusion/ops/triton_ops/dropout.py:71-93.

    Kept for API parity; the fused path never materialises the dropped tensor.  The mask comes
    from the HIP Philox4x32-10 kernel keyed by ``seed`` (a stream of its own, not Triton's).
    """
    _check_p(p)
    mask = make_dropout_mask(x.shape, p, seed, x.device)
    out = torch.where(mask, x * (1.0 / (1.0 - p)), torch.zeros((), dtype=x.dtype, device=x.device))
    return out, (mask if store_mask else None)


def blocked_seeded_dropout(x: torch.Tensor, block_to_dropout_p: torch.Tensor, block_size_m: int, seed: int | None = None,
                           *, store_mask: bool = True):
    """Dropout with one p per ``block_size_m`` rows -- lorafusion/ops/triton_ops/blocked_dropout.py:78-135.

    Returns ``(where(mask, x / (1 - p_block), 0), mask)``; the mask comes from the HIP Philox kernel
    keyed by ``seed`` (the same bytes ``make_dropout_mask`` gives a packed batch with these p).
    """
    if x.ndim != 2:
        raise ValueError("x must be a 2D tensor")
    L.require_gpu(x, "x")
    M, K = x.shape
    if block_size_m <= 0 or M % block_size_m != 0:
        raise ValueError(f"x has {M} rows, not a multiple of block_size_m = {block_size_m}.")
    if K % 16 != 0:
        raise ValueError(f"the mask kernel needs K % 16 == 0, got K={K}.")
    nb = M // block_size_m
    p = block_to_dropout_p.to(device=x.device, dtype=torch.float32).contiguous()
    if p.numel() != nb:
        raise ValueError(f"block_to_dropout_p must have {nb} entries, got {p.numel()}.")
    if seed is None:
        seed = random.randrange(int(1e6))  # noqa: S311
    r = L.Routing()
    r.n_seg, r.block_size_m, r.n_blocks = 1, int(block_size_m), nb
    r.block_table, r.block_scale, r.block_p = None, None, p.data_ptr()
    mask = torch.empty((M, K), dtype=torch.bool, device=x.device)
    with torch.cuda.device(x.device):
        L.check(L.lib().lf_dropout_mask(L.ptr(mask), M, K, ctypes.c_float(0.0), ctypes.byref(r),
                                        ctypes.c_uint64(int(seed) & 0xFFFFFFFFFFFFFFFF), L.stream_of(mask)), "lf_dropout_mask")
    scale = (1.0 / (1.0 - p)).repeat_interleave(block_size_m).unsqueeze(1)
    out = torch.where(mask, (x.float() * scale).to(x.dtype), torch.zeros((), dtype=x.dtype, device=x.device))
    return out, (mask if store_mask else None)


def fused_dropout_matmul(x: torch.Tensor, a: torch.Tensor, dropout_p: float, seed: int = 42, *,
                         store_mask: bool = False, store_masked_scaled_x: bool = False,
                         dropout_mask: torch.Tensor | None = None):
    """``S = drop(x) @ a.T`` -- lorafusion/ops/triton_ops/fused_dropout_matmul.py:280-354.

    Returns ``(s, mask, masked_scaled_x)``.  ``dropout_mask`` (extension) supplies the keep-mask
    explicitly; otherwise one is drawn from ``seed``.  ``s`` has ``round_up(r, 16)`` columns,
    zero beyond ``r``.
    """
    _check_2d(x, "x")
    _check_2d(a, "a", x.dtype)
    M, K = x.shape
    r = a.shape[0]
    if a.shape[1] != K:
        raise ValueError(f"a must have shape [r, {K}], but got {tuple(a.shape)}.")
    _check_dims(M, None, K)
    routing = _routing_single(r, 1.0, dropout_p)
    mask = None
    if dropout_p > 0:
        mask = _check_mask(dropout_mask, x.shape) if dropout_mask is not None else make_dropout_mask(x.shape, dropout_p, seed, x.device)
    s = _xa(x, mask, [a], routing, M, K, L.round_rank(r))
    xs = None
    if store_masked_scaled_x:
        mb = unpack_mask(mask) if is_packed_mask(mask, K) else mask
        xs = x if mask is None else torch.where(mb, x * (1.0 / (1.0 - dropout_p)), torch.zeros((), dtype=x.dtype, device=x.device))
    return s, (mask if store_mask else None), xs


def _pad_cols(t: torch.Tensor, R: int) -> torch.Tensor:
    """[M, r] -> [M, R] zero padded (no copy when r == R)."""
    if t.shape[1] == R:
        return t
    out = torch.zeros((t.shape[0], R), dtype=t.dtype, device=t.device)
    out[:, : t.shape[1]] = t
    return out


def fused_lora_xw_sb(x: torch.Tensor, w: torch.Tensor, s: torch.Tensor, b: torch.Tensor, alpha: float,
                     bias: torch.Tensor | None = None, *, config=None) -> torch.Tensor:
    """``y = x @ w.T + (s @ b.T) * alpha + bias`` -- fused_lora_xw_sb.py:209-316.

    x [M,K], w [N,K], s [M,r] (or [M, round_up(r,16)]), b [N,r].  ``config`` is accepted and ignored.
    """
    _check_2d(x, "x")
    _check_2d(w, "w", x.dtype)
    _check_2d(s, "s", x.dtype)
    _check_2d(b, "b", x.dtype)
    M, K = x.shape
    N, r = b.shape
    if w.shape != (N, K):
        raise ValueError(f"w must have shape [{N}, {K}], but got {tuple(w.shape)}.")
    R = L.round_rank(r)
    if s.shape[0] != M or s.shape[1] not in (r, R):
        raise ValueError(f"s must have shape [{M}, {r}], but got {tuple(s.shape)}.")
    if bias is not None and (bias.shape != (N,) or bias.dtype != x.dtype or not bias.is_contiguous()):
        raise ValueError(f"bias must be a contiguous [{N}] tensor of dtype {x.dtype}.")
    _check_dims(M, N, K)
    routing = _routing_single(r, alpha, 0.0)
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    s_p = _pad_cols(s, R)
    rc = L.lib().lf_lora_xw_sb(L.ptr(x), L.ptr(w), L.ptr(bias), L.ptr(s_p), L.ptr_array([b]), L.ptr(y),
                               M, N, K, R, routing, L.dtype_id(x.dtype), L.stream_of(x))
    L.check(rc, "lf_lora_xw_sb")
    return y


def fused_lora_dys_dyb(dy: torch.Tensor, b: torch.Tensor, s: torch.Tensor, alpha: float, *, config=None):
    """``db = alpha * dy.T @ s``, ``ds = alpha * dy @ b`` -- fused_lora_dys_dyb.py:182-301.

    Returns ``(db [N,r], ds [M, round_up(r,16)])``; sums are deterministic (no atomics).
    """
    _check_2d(dy, "dy")
    _check_2d(b, "b", dy.dtype)
    _check_2d(s, "s", dy.dtype)
    M, N = dy.shape
    r = b.shape[1]
    R = L.round_rank(r)
    if b.shape[0] != N:
        raise ValueError(f"b must have shape [{N}, r], but got {tuple(b.shape)}.")
    if s.shape[0] != M or s.shape[1] not in (r, R):
        raise ValueError(f"s must have shape [{M}, {r}], but got {tuple(s.shape)}.")
    _check_dims(M, N, None)
    routing = _routing_single(r, alpha, 0.0)
    db = torch.empty((N, r), dtype=dy.dtype, device=dy.device)
    ds = torch.empty((M, R), dtype=dy.dtype, device=dy.device)
    ws, nbytes = _ws(L.LF_OP_DYS_DYB, M, N, 0, R, routing, dy.device)
    s_p = _pad_cols(s, R)
    rc = L.lib().lf_lora_dys_dyb(L.ptr(dy), L.ptr(s_p), L.ptr_array([b]), L.ptr(ds), L.ptr_array([db]),
                                 L.ptr(ws), nbytes, M, N, R, routing, L.dtype_id(dy.dtype), L.stream_of(dy))
    L.check(rc, "lf_lora_dys_dyb")
    return db, ds


def fused_lora_da(x: torch.Tensor, ds: torch.Tensor, r: int, dropout_p: float = 0.0,
                  dropout_mask: torch.Tensor | None = None) -> torch.Tensor:
    """``da = ds.T @ drop(x)`` -- the cuBLAS call at lorafusion/ops/lora_v1.py:153, with the
    dropped input rebuilt from ``x`` and the keep-mask inside the kernel."""
    _check_2d(x, "x")
    _check_2d(ds, "ds", x.dtype)
    M, K = x.shape
    R = L.round_rank(r)
    if ds.shape[0] != M or ds.shape[1] not in (r, R):
        raise ValueError(f"ds must have shape [{M}, {r}], but got {tuple(ds.shape)}.")
    _check_dims(M, None, K)
    _check_p(dropout_p)
    if dropout_p > 0 and dropout_mask is None:
        raise ValueError("dropout_mask must be provided if dropout_p != 0")
    mask = _check_mask(dropout_mask, x.shape) if dropout_p > 0 else None
    routing = _routing_single(r, 1.0, dropout_p)
    da = torch.empty((r, K), dtype=x.dtype, device=x.device)
    ws, nbytes = _ws(L.LF_OP_DA, M, 0, K, R, routing, x.device)
    ds_p = _pad_cols(ds, R)
    rc = L.lib().lf_lora_da(L.ptr(x), L.ptr(mask), L.ptr(ds_p), L.ptr_array([da]), L.ptr(ws), nbytes,
                            M, K, R, routing, _dt(x, mask, K), L.stream_of(x))
    L.check(rc, "lf_lora_da")
    return da


def fused_lora_dyw_dsa(dy: torch.Tensor, w: torch.Tensor, ds: torch.Tensor, a: torch.Tensor, dropout_p: float,
                       dropout_mask: torch.Tensor | None = None, *, config=None) -> torch.Tensor:
    """``dx = dy @ w + where(mask, (ds @ a)/(1-p), 0)`` -- fused_lora_dyw_dsa.py:184-297."""
    _check_2d(dy, "dy")
    _check_2d(w, "w", dy.dtype)
    _check_2d(ds, "ds", dy.dtype)
    _check_2d(a, "a", dy.dtype)
    M, N = dy.shape
    r, K = a.shape
    R = L.round_rank(r)
    if w.shape != (N, K):
        raise ValueError(f"w must have shape [{N}, {K}], but got {tuple(w.shape)}.")
    if ds.shape[0] != M or ds.shape[1] not in (r, R):
        raise ValueError(f"ds must have shape [{M}, {r}], but got {tuple(ds.shape)}.")
    _check_dims(M, N, K)
    _check_p(dropout_p)
    if dropout_p > 0 and dropout_mask is None:  # as fused_lora_dyw_dsa.py:184-297 does
        raise ValueError("dropout_mask must be provided if dropout_p != 0")
    mask = _check_mask(dropout_mask, (M, K)) if dropout_p > 0 else None
    routing = _routing_single(r, 1.0, dropout_p)
    dx = torch.empty((M, K), dtype=dy.dtype, device=dy.device)
    ds_p = _pad_cols(ds, R)
    rc = L.lib().lf_lora_dyw_dsa(L.ptr(dy), L.ptr(w), L.ptr(ds_p), L.ptr_array([a]), L.ptr(mask), L.ptr(dx),
                                 M, N, K, R, routing, _dt(dy, mask, K), L.stream_of(dy))
    L.check(rc, "lf_lora_dyw_dsa")
    return dx


# --------------------------------------------------------------------------- multi-LoRA pieces


def _check_adapters(a_list, b_list, routing: MultiRouting, K: int | None, N: int | None, dtype):
    if a_list is not None:
        for a, r in zip(a_list, routing.rank_list, strict=True):
            _check_2d(a, "lora_a", dtype)
            if a.shape[0] != r or (K is not None and a.shape[1] != K):
                raise ValueError(f"lora_a must have shape [{r}, {K}], but got {tuple(a.shape)}.")
    if b_list is not None:
        for b, r in zip(b_list, routing.rank_list, strict=True):
            _check_2d(b, "lora_b", dtype)
            if b.shape[1] != r or (N is not None and b.shape[0] != N):
                raise ValueError(f"lora_b must have shape [{N}, {r}], but got {tuple(b.shape)}.")


def fused_multi_lora_xa(x, a_list, routing: MultiRouting, dropout_mask=None):
    """Packed ``S``: row m holds ``drop(x[m]) @ A_i.T`` for the adapter i owning row m
    (zero in padded rows and beyond rank_i).  Replaces ``full_s`` of
    lorafusion/ops/multi_lora.py:502-513, which multiplies every token by every adapter."""
    _check_2d(x, "x")
    M, K = x.shape
    if M != routing.M:
        raise ValueError(f"x has {M} rows but the routing tables cover {routing.M}.")
    _check_dims(M, None, K)
    _check_adapters(a_list, None, routing, K, None, x.dtype)
    mask = _check_mask(dropout_mask, x.shape)
    return _xa(x, mask, a_list, routing.c, M, K, routing.R)


def fused_multi_lora_xw_sb(x, w, s, b_list, routing: MultiRouting, bias=None):
    """Per-block ``y = x w^T + alpha_b * s B_b^T + bias`` -- fused_multi_lora_xw_sb.py:221-339.
    Padded rows receive the base GEMM (+bias) only."""
    _check_2d(x, "x")
    _check_2d(w, "w", x.dtype)
    _check_2d(s, "s", x.dtype)
    M, K = x.shape
    N = w.shape[0]
    if M != routing.M or w.shape[1] != K or s.shape != (M, routing.R):
        raise ValueError("x / w / s shapes do not match the routing tables.")
    _check_dims(M, N, K)
    _check_adapters(None, b_list, routing, None, N, x.dtype)
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    rc = L.lib().lf_lora_xw_sb(L.ptr(x), L.ptr(w), L.ptr(bias), L.ptr(s), L.ptr_array(b_list), L.ptr(y), M, N, K,
                               routing.R, routing.c, L.dtype_id(x.dtype), L.stream_of(x))
    L.check(rc, "lf_lora_xw_sb")
    return y


def fused_multi_lora_dys_dyb(dy, s, b_list, routing: MultiRouting):
    """Per-adapter ``db_i`` and packed ``ds`` -- fused_multi_lora_dys_dyb.py:188-321."""
    _check_2d(dy, "dy")
    _check_2d(s, "s", dy.dtype)
    M, N = dy.shape
    if M != routing.M or s.shape != (M, routing.R):
        raise ValueError("dy / s shapes do not match the routing tables.")
    _check_dims(M, N, None)
    _check_adapters(None, b_list, routing, None, N, dy.dtype)
    db_list = [torch.empty((N, r), dtype=dy.dtype, device=dy.device) for r in routing.rank_list]
    ds = torch.empty((M, routing.R), dtype=dy.dtype, device=dy.device)
    ws, nbytes = _ws(L.LF_OP_DYS_DYB, M, N, 0, routing.R, routing.c, dy.device)
    rc = L.lib().lf_lora_dys_dyb(L.ptr(dy), L.ptr(s), L.ptr_array(b_list), L.ptr(ds), L.ptr_array(db_list), L.ptr(ws),
                                 nbytes, M, N, routing.R, routing.c, L.dtype_id(dy.dtype), L.stream_of(dy))
    L.check(rc, "lf_lora_dys_dyb")
    return db_list, ds


def fused_multi_lora_da(x, ds, routing: MultiRouting, dropout_mask=None):
    """Per-adapter ``da_i = ds_i.T @ drop(x_i)`` -- lorafusion/ops/multi_lora.py:576-581."""
    _check_2d(x, "x")
    _check_2d(ds, "ds", x.dtype)
    M, K = x.shape
    if M != routing.M or ds.shape != (M, routing.R):
        raise ValueError("x / ds shapes do not match the routing tables.")
    _check_dims(M, None, K)
    mask = _check_mask(dropout_mask, x.shape)
    da_list = [torch.empty((r, K), dtype=x.dtype, device=x.device) for r in routing.rank_list]
    ws, nbytes = _ws(L.LF_OP_DA, M, 0, K, routing.R, routing.c, x.device)
    rc = L.lib().lf_lora_da(L.ptr(x), L.ptr(mask), L.ptr(ds), L.ptr_array(da_list), L.ptr(ws), nbytes, M, K,
                            routing.R, routing.c, _dt(x, mask, K), L.stream_of(x))
    L.check(rc, "lf_lora_da")
    return da_list


def fused_multi_lora_dyw_dsa(dy, w, ds, a_list, routing: MultiRouting, dropout_mask=None):
    """Per-block ``dx = dy w + where(mask, (ds A_b)/(1-p_b), 0)`` -- fused_multi_lora_dyw_dsa.py:188-305."""
    _check_2d(dy, "dy")
    _check_2d(w, "w", dy.dtype)
    _check_2d(ds, "ds", dy.dtype)
    M, N = dy.shape
    K = w.shape[1]
    if M != routing.M or w.shape[0] != N or ds.shape != (M, routing.R):
        raise ValueError("dy / w / ds shapes do not match the routing tables.")
    _check_dims(M, N, K)
    _check_adapters(a_list, None, routing, K, None, dy.dtype)
    mask = _check_mask(dropout_mask, (M, K))
    dx = torch.empty((M, K), dtype=dy.dtype, device=dy.device)
    rc = L.lib().lf_lora_dyw_dsa(L.ptr(dy), L.ptr(w), L.ptr(ds), L.ptr_array(a_list), L.ptr(mask), L.ptr(dx), M, N, K,
                                 routing.R, routing.c, _dt(dy, mask, K), L.stream_of(dy))
    L.check(rc, "lf_lora_dyw_dsa")
    return dx


# --------------------------------------------------------------------------- whole fwd / bwd


def lora_forward(x, w, a_list, b_list, routing_c, R, mask, bias):
    """One C call: S = drop(x) A^T, then y = x w^T + scale S B^T + bias.  Returns (y, s)."""
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    s = torch.empty((M, R), dtype=x.dtype, device=x.device)
    ws, nbytes = _ws(L.LF_OP_FWD, M, N, K, R, routing_c, x.device)
    rc = L.lib().lf_lora_fwd(L.ptr(x), L.ptr(w), L.ptr(bias), L.ptr(mask), L.ptr_array(a_list), L.ptr_array(b_list),
                             L.ptr(y), L.ptr(s), L.ptr(ws), nbytes, M, N, K, R, routing_c, _dt(x, mask, K),
                             L.stream_of(x))
    L.check(rc, "lf_lora_fwd")
    return y, s


def lora_forward_seeded(x, w, a_list, b_list, routing_c, R, seed: int, bias, *, packed: bool = True):
    """As ``lora_forward`` with the keep-mask drawn inside the rank-r kernel from ``seed``.
    Returns (y, s, mask).  The mask comes back bit-packed (uint8 ``[M, K // 8]``, the format the backward kernels read
    fastest; ``packed=False``: bool ``[M, K]``); unpacked it equals ``make_dropout_mask`` for the same seed and routing."""
    M, K = x.shape
    N = w.shape[0]
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    s = torch.empty((M, R), dtype=x.dtype, device=x.device)
    mask = torch.empty((M, K // 8), dtype=torch.uint8, device=x.device) if packed else torch.empty((M, K), dtype=torch.bool, device=x.device)
    ws, nbytes = _ws(L.LF_OP_FWD, M, N, K, R, routing_c, x.device)
    rc = L.lib().lf_lora_fwd_seeded(L.ptr(x), L.ptr(w), L.ptr(bias), L.ptr(mask), L.ptr_array(a_list), L.ptr_array(b_list),
                                    L.ptr(y), L.ptr(s), L.ptr(ws), nbytes, M, N, K, R, routing_c,
                                    ctypes.c_uint64(int(seed) & 0xFFFFFFFFFFFFFFFF), _dt(x, mask, K), L.stream_of(x))
    L.check(rc, "lf_lora_fwd_seeded")
    return y, s, mask


def lora_backward(dy, x, w, a_list, b_list, s, routing_c, R, mask, rank_list, requires_dx: bool = True):
    """One C call: dS/dB, dA and (optionally) dX.  Returns (dx | None, da_list, db_list)."""
    M, N = dy.shape
    K = x.shape[1]
    dx = torch.empty((M, K), dtype=dy.dtype, device=dy.device) if requires_dx else None
    da_list = [torch.empty((r, K), dtype=dy.dtype, device=dy.device) for r in rank_list]
    db_list = [torch.empty((N, r), dtype=dy.dtype, device=dy.device) for r in rank_list]
    ds = torch.empty((M, R), dtype=dy.dtype, device=dy.device)
    ws, nbytes = _ws(L.LF_OP_BWD, M, N, K, R, routing_c, dy.device)
    rc = L.lib().lf_lora_bwd(L.ptr(dy), L.ptr(x), L.ptr(w), L.ptr(mask), L.ptr(s), L.ptr_array(a_list),
                             L.ptr_array(b_list), L.ptr(dx), L.ptr_array(da_list), L.ptr_array(db_list), L.ptr(ds),
                             L.ptr(ws), nbytes, M, N, K, R, routing_c, _dt(dy, mask, K), L.stream_of(dy))
    L.check(rc, "lf_lora_bwd")
    return dx, da_list, db_list


def nf4_lora_forward(x, wref, a_list, b_list, routing_c, R, mask, bias, *, keep_dense: bool = False):
    """``lora_forward`` with the base weight given as NF4 (``nf4.NF4WeightRef``): one C call dequantises it
    and runs the forward on it.  Returns (y, s), or (y, s, dense) with ``keep_dense``: the dequantised
    weight then goes into a tensor of its own instead of the call's workspace, for a backward that
    follows while it is still around (``nf4_lora_backward(..., dense=dense)``)."""
    M, K = x.shape
    N = wref.shape[0]
    y = torch.empty((M, N), dtype=x.dtype, device=x.device)
    s = torch.empty((M, R), dtype=x.dtype, device=x.device)
    dense = torch.empty((N, K), dtype=x.dtype, device=x.device) if keep_dense else None
    wc = wref.with_dense(dense, valid=False)
    ws, nbytes = _ws(L.LF_OP_FWD if keep_dense else L.LF_OP_NF4_FWD, M, N, K, R, routing_c, x.device)
    rc = L.lib().lf_nf4_lora_fwd(L.ptr(x), ctypes.byref(wc), L.ptr(bias), L.ptr(mask), L.ptr_array(a_list),
                                 L.ptr_array(b_list), L.ptr(y), L.ptr(s), L.ptr(ws), nbytes, M, N, K, R, routing_c,
                                 _dt(x, mask, K), L.stream_of(x))
    L.check(rc, "lf_nf4_lora_fwd")
    return (y, s, dense) if keep_dense else (y, s)


def nf4_lora_backward(dy, x, wref, a_list, b_list, s, routing_c, R, mask, rank_list, requires_dx: bool = True,
                      dense: torch.Tensor | None = None):
    """``lora_backward`` with the base weight given as NF4.  ``dense``: the dequantised weight a forward with
    ``keep_dense`` left behind (nothing is dequantised then).  Returns (dx | None, da_list, db_list)."""
    M, N = dy.shape
    K = x.shape[1]
    dx = torch.empty((M, K), dtype=dy.dtype, device=dy.device) if requires_dx else None
    da_list = [torch.empty((r, K), dtype=dy.dtype, device=dy.device) for r in rank_list]
    db_list = [torch.empty((N, r), dtype=dy.dtype, device=dy.device) for r in rank_list]
    ds = torch.empty((M, R), dtype=dy.dtype, device=dy.device)
    if dense is not None and (tuple(dense.shape) != (N, K) or dense.dtype != dy.dtype or not dense.is_contiguous()):
        raise ValueError(f"dense must be a contiguous [{N}, {K}] tensor of dtype {dy.dtype}.")
    wc = wref.with_dense(dense, valid=True)
    # no weight-sized head in the workspace when the weight is handed over, or not needed at all (no dX)
    lean = dense is not None or not requires_dx
    ws, nbytes = _ws(L.LF_OP_BWD if lean else L.LF_OP_NF4_BWD, M, N, K, R, routing_c, dy.device)
    rc = L.lib().lf_nf4_lora_bwd(L.ptr(dy), L.ptr(x), ctypes.byref(wc), L.ptr(mask), L.ptr(s), L.ptr_array(a_list),
                                 L.ptr_array(b_list), L.ptr(dx), L.ptr_array(da_list), L.ptr_array(db_list), L.ptr(ds),
                                 L.ptr(ws), nbytes, M, N, K, R, routing_c, _dt(dy, mask, K), L.stream_of(dy))
    L.check(rc, "lf_nf4_lora_bwd")
    return dx, da_list, db_list


def gemm(a: torch.Tensor, b: torch.Tensor, *, trans_b: bool = True, bias=None, tile_cfg: int = -1) -> torch.Tensor:
    """Plain ``a @ b.T`` (trans_b) or ``a @ b`` with the same MFMA kernel, no LoRA term."""
    _check_2d(a, "a")
    _check_2d(b, "b", a.dtype)
    M, K = a.shape
    N = b.shape[0] if trans_b else b.shape[1]
    if (b.shape[1] if trans_b else b.shape[0]) != K:
        raise ValueError("inner dimensions do not match.")
    c = torch.empty((M, N), dtype=a.dtype, device=a.device)
    rc = L.lib().lf_gemm(L.ptr(a), L.ptr(b), L.ptr(bias), L.ptr(c), M, N, K, int(trans_b), L.dtype_id(a.dtype),
                         tile_cfg, L.stream_of(a))
    L.check(rc, "lf_gemm")
    return c
