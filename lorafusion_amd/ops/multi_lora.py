"""Multi-LoRA: several adapters' token segments in one launch.

Mirrors lorafusion/ops/multi_lora.py: ``MultiLoRABatchInfo`` / ``prepare_multi_lora_batch_info``
(:295-453), ``fused_linear_multi_lora`` / ``FusedLinearMultiLoRA`` (:602-830) and the batch-info
bookkeeping of ``MultiLoRAManager`` (:65-292; its DDP / optimizer-step part needs several GPUs
and is left out).

Differences from the reference, all deliberate:
 * ``S`` is computed per row with the row's own adapter (the reference multiplies every token by
   every adapter, multi_lora.py:502) and always from the *dropped* input, as in the single path;
 * per-block ``alpha`` / ``p`` are stored in ``output_dtype`` (bf16 by default, multi_lora.py:355,393-394) and
   widened to fp32 once per micro-batch, when the routing is built, not in every kernel;
 * heterogeneous dropout works (the reference's call raises TypeError, multi_lora.py:490-496);
 * any number of adapters up to 32 (the reference stops at 4);
 * padded rows of ``y`` hold the base GEMM (+bias) and padded rows of ``dx`` hold ``dy W``
   (the reference leaves them uninitialised).
"""

from __future__ import annotations

import random
from collections import deque
from dataclasses import dataclass
from typing import Any, Sequence

import numpy as np
import torch

from lorafusion_amd import _lib as L
from lorafusion_amd.ops import hip_ops
from lorafusion_amd.ops.hip_ops import FUSED_MULTI_LORA_BLOCK_SIZE_M, MultiRouting

THREE_DIM = 3


@dataclass
class MultiLoRABatchInfo:
    """Batch info for Multi-LoRA (field names as in lorafusion/ops/multi_lora.py:295-346).

    ``block_to_lookup_table`` is int32 ``[num_blocks, 3]``: per ``block_size_m``-row block
    ``(lora_rank, valid_rows_in_block, first_block_of_its_segment)``.
    """

    seq_len_list: list[int]
    lora_idx_list: list[int]
    lora_rank_list: list[int]
    dropout_p_list: list[float]
    alpha_list: list[float]
    block_size_m: int
    padded_seq_len_list: list[int]
    block_to_lookup_table: torch.Tensor
    block_to_dropout_p: torch.Tensor
    block_to_alpha: torch.Tensor
    enable_dropout: bool
    same_dropout_p_value: float | None
    max_r: int
    microbatch_idx: int | None = None
    micro_batch_info: Any | None = None
    allow_empty_micro_batch_info: bool = False

    @property
    def num_active_adapters(self) -> int:
        return len(set(self.lora_idx_list))

    def routing(self, *, enable_dropout: bool) -> MultiRouting:
        """The kernels' view of this micro-batch (fp32 copies of the per-block tables on the device plus
        the host struct of segment bounds and ranks), built on first use and kept: every LoRA linear of
        every layer that runs this micro-batch shares it, where the reference rebuilds its pointer lists in
        every layer call (lorafusion/ops/multi_lora.py:519-523)."""
        cache = self.__dict__.setdefault("_routing_cache", {})
        key = bool(enable_dropout)
        if key not in cache:
            cache[key] = MultiRouting(self.padded_seq_len_list, self.lora_rank_list, self.block_to_lookup_table,
                                      self.block_to_alpha, self.block_to_dropout_p, enable_dropout=key,
                                      block_size_m=self.block_size_m)
        return cache[key]


def build_block_tables(seq_len_list, lora_rank_list, dropout_p_list, alpha_list, block_size_m):
    """Vectorised routing tables (numpy): returns (padded_seq_len_list, lookup int32 [nb,3],
    block_p float64 [nb], block_alpha float64 [nb])."""
    n = len(seq_len_list)
    if not (len(lora_rank_list) == len(dropout_p_list) == len(alpha_list) == n):
        raise ValueError("seq_len_list, lora_rank_list, dropout_p_list and alpha_list must have the same length")
    if n == 0:
        raise ValueError("seq_len_list must not be empty")
    seq = np.asarray(seq_len_list, dtype=np.int64)
    if (seq <= 0).any():
        raise ValueError(f"every sequence length must be positive, got {list(seq_len_list)}")
    if block_size_m <= 0:
        raise ValueError(f"block_size_m must be positive, got {block_size_m}")
    nblk = (seq - 1) // block_size_m + 1
    padded = nblk * block_size_m
    first = np.concatenate(([0], np.cumsum(nblk)[:-1]))
    total = int(nblk.sum())
    seg_of_block = np.repeat(np.arange(n), nblk)
    idx_in_seg = np.arange(total) - first[seg_of_block]
    lookup = np.empty((total, 3), dtype=np.int32)
    lookup[:, 0] = np.asarray(lora_rank_list, dtype=np.int64)[seg_of_block]
    lookup[:, 1] = np.minimum(block_size_m, seq[seg_of_block] - idx_in_seg * block_size_m)
    lookup[:, 2] = first[seg_of_block]
    block_p = np.asarray(dropout_p_list, dtype=np.float64)[seg_of_block]
    block_alpha = np.asarray(alpha_list, dtype=np.float64)[seg_of_block]
    return [int(v) for v in padded], lookup, block_p, block_alpha


def prepare_multi_lora_batch_info(
    seq_len_list: list[int],
    lora_idx_list: list[int],
    lora_rank_list: list[int],
    dropout_p_list: list[float],
    alpha_list: list[float],
    block_size_m: int,
    output_dtype: torch.dtype = torch.bfloat16,
    micro_batch_info: Any | None = None,
    *,
    allow_empty_micro_batch_info: bool = False,
) -> MultiLoRABatchInfo:
    """Build the per-block tables of a packed batch (lorafusion/ops/multi_lora.py:348-453).

    The tensors live on ``"cuda"`` as in the reference (multi_lora.py:427-429); without a GPU they
    stay on the CPU, so the integer routing can be checked there.
    """
    padded, lookup, block_p, block_alpha = build_block_tables(
        seq_len_list, lora_rank_list, dropout_p_list, alpha_list, block_size_m
    )
    device = "cuda" if torch.cuda.is_available() else "cpu"
    same = all(p == dropout_p_list[0] for p in dropout_p_list)
    return MultiLoRABatchInfo(
        seq_len_list=seq_len_list,
        lora_idx_list=lora_idx_list,
        lora_rank_list=lora_rank_list,
        dropout_p_list=dropout_p_list,
        alpha_list=alpha_list,
        block_size_m=block_size_m,
        padded_seq_len_list=padded,
        block_to_lookup_table=torch.from_numpy(lookup).to(device=device),
        block_to_dropout_p=torch.from_numpy(block_p).to(dtype=output_dtype).to(device=device),
        block_to_alpha=torch.from_numpy(block_alpha).to(dtype=output_dtype).to(device=device),
        enable_dropout=any(p > 0 for p in dropout_p_list),
        same_dropout_p_value=dropout_p_list[0] if same else None,
        max_r=max(lora_rank_list),
        micro_batch_info=micro_batch_info,
        allow_empty_micro_batch_info=allow_empty_micro_batch_info,
    )


def batch_info_from_micro_batch(
    micro_batch_info: Any,
    lora_configs: "Sequence[Any] | dict[int, Any]",
    block_size_m: int = FUSED_MULTI_LORA_BLOCK_SIZE_M,
    output_dtype: torch.dtype = torch.bfloat16,
) -> MultiLoRABatchInfo:
    """Routing tables straight from a scheduler micro-batch descriptor.

    Restates the conversion the reference's data provider does before every micro-batch
    (lorafusion/train/training_utils.py:1250-1334): adapters in ascending index order, one segment per
    adapter with ``adapter_num_tokens_pairs[idx]`` tokens, rank / dropout / multiplier from
    ``lora_configs[idx]`` (``.r``, ``.lora_dropout``, ``.lora_alpha`` -- the reference hands the raw
    ``lora_alpha`` to the kernels as the multiplier there, training_utils.py:1323).  ``micro_batch_info``
    is duck-typed on the fields of ``MicroBatchInfo`` (lorafusion/solver/proposed_solver.py:51-131):
    ``adapter_group_info``, ``adapter_num_tokens_pairs``, ``padded_adapter_num_tokens_pairs``,
    ``adapter_padding_multiple``; the descriptor's own padding must be the kernels' block size.
    """
    if getattr(micro_batch_info, "is_empty_marker", False):
        raise ValueError("an empty-marker micro-batch carries no tokens; there is nothing to route.")
    pad = getattr(micro_batch_info, "adapter_padding_multiple", block_size_m)
    if pad != block_size_m:
        raise ValueError(
            f"micro-batch padding multiple {pad} differs from the kernels' block size {block_size_m}."
        )
    adapters = sorted(micro_batch_info.adapter_group_info)
    if not adapters:
        raise ValueError("the micro-batch names no adapter.")
    seq_len_list = [int(micro_batch_info.adapter_num_tokens_pairs[a]) for a in adapters]
    cfgs = [lora_configs[a] for a in adapters]
    info = prepare_multi_lora_batch_info(
        seq_len_list=seq_len_list,
        lora_idx_list=list(adapters),
        lora_rank_list=[int(c.r) for c in cfgs],
        dropout_p_list=[float(c.lora_dropout) for c in cfgs],
        alpha_list=[float(c.lora_alpha) for c in cfgs],
        block_size_m=block_size_m,
        output_dtype=output_dtype,
        micro_batch_info=micro_batch_info,
    )
    padded_pairs = getattr(micro_batch_info, "padded_adapter_num_tokens_pairs", None)
    if padded_pairs is not None:
        expect = [int(padded_pairs[a]) for a in adapters]
        if expect != info.padded_seq_len_list:
            raise ValueError(
                f"padded token counts of the micro-batch {expect} differ from the routing tables {info.padded_seq_len_list}."
            )
    return info


class FusedLinearMultiLoRA(torch.autograd.Function):
    """Packed multi-adapter LoRA linear.  Adapter tensors are passed as ``*a_list, *b_list``."""

    @staticmethod
    def forward(ctx, padded_x, linear_w, linear_bias, dropout_mask, seed, routing: MultiRouting, quant_state,
                keep_dequantized, n_adapters, *ab):
        if padded_x.ndim == THREE_DIM:
            if padded_x.shape[0] != 1:
                raise ValueError("currently, we only support batch size 1 for multi-linear LoRA")
            x2d = padded_x.reshape(padded_x.shape[1], padded_x.shape[2])
            lead = True
        elif padded_x.ndim == 2:
            x2d, lead = padded_x, False
        else:
            raise ValueError(f"padded_x must be a 3D tensor, but got {padded_x.ndim}")
        x2d = x2d.contiguous()
        linear_w = linear_w.contiguous()
        a_list = [t.contiguous() for t in ab[:n_adapters]]
        b_list = [t.contiguous() for t in ab[n_adapters:]]
        M, K = x2d.shape
        wref = None
        if quant_state is not None:
            # NF4 base weight: linear_w holds the packed codes, quant_state its bitsandbytes-style state
            from lorafusion_amd.ops.nf4 import NF4WeightRef

            wref = NF4WeightRef(linear_w, quant_state)
            w_shape, w_dtype = tuple(wref.shape), wref.dtype
        else:
            w_shape, w_dtype = tuple(linear_w.shape), linear_w.dtype
        if M != routing.M:
            raise ValueError(f"padded_x has {M} rows but the batch info covers {routing.M}.")
        if len(w_shape) != 2 or w_shape[1] != K or w_dtype != x2d.dtype:
            raise ValueError(f"linear_w must have shape [N, {K}] and dtype {x2d.dtype}.")
        N = w_shape[0]
        L.require_gpu(x2d, "padded_x")
        L.dtype_id(x2d.dtype)
        hip_ops._check_dims(M, N, K)
        hip_ops._check_adapters(a_list, b_list, routing, K, N, x2d.dtype)
        if linear_bias is not None and (tuple(linear_bias.shape) != (N,) or linear_bias.dtype != x2d.dtype):
            raise ValueError(f"linear_bias must have shape [{N}] and dtype {x2d.dtype}.")

        mask, dense = None, None
        bias = linear_bias.contiguous() if linear_bias is not None else None
        if wref is not None:
            if routing.enable_dropout:
                if dropout_mask is None:
                    dropout_mask = hip_ops.make_dropout_mask((M, K), 0.0, seed, x2d.device, routing=routing)
                mask = hip_ops._check_mask(dropout_mask.reshape(M, -1), (M, K))
                if not hip_ops.is_packed_mask(mask, K):
                    mask = hip_ops.pack_mask(mask)   # read three times (rank-r forward, dA, dX): an eighth of the bytes each
            if keep_dequantized:
                y, s, dense = hip_ops.nf4_lora_forward(x2d, wref, a_list, b_list, routing.c, routing.R, mask, bias,
                                                       keep_dense=True)
            else:
                y, s = hip_ops.nf4_lora_forward(x2d, wref, a_list, b_list, routing.c, routing.R, mask, bias)
        elif routing.enable_dropout and dropout_mask is None:
            # per-block p from the routing table, mask drawn inside the rank-r pass
            if seed is None:
                seed = random.randrange(int(1e6))  # noqa: S311
            y, s, mask = hip_ops.lora_forward_seeded(x2d, linear_w, a_list, b_list, routing.c, routing.R, seed, bias)
        else:
            if routing.enable_dropout:
                mask = hip_ops._check_mask(dropout_mask.reshape(M, -1), (M, K))
                if not hip_ops.is_packed_mask(mask, K):
                    mask = hip_ops.pack_mask(mask)   # read three times (rank-r forward, dA, dX): an eighth of the bytes each
            y, s = hip_ops.lora_forward(x2d, linear_w, a_list, b_list, routing.c, routing.R, mask, bias)

        ctx.save_for_backward(x2d, linear_w, mask, s, dense, *a_list, *b_list)
        ctx.routing = routing
        ctx.quant_state = quant_state
        ctx.n_adapters = n_adapters
        ctx.lead = lead
        return y.reshape(1, M, N) if lead else y

    @staticmethod
    def backward(ctx, dy):
        x2d, linear_w, mask, s, dense, *ab = ctx.saved_tensors
        n = ctx.n_adapters
        a_list, b_list = list(ab[:n]), list(ab[n:])
        routing = ctx.routing
        if dy.ndim == THREE_DIM:
            if dy.shape[0] != 1:
                raise ValueError("currently, we only support batch size 1 for multi-linear LoRA")
            dy2d = dy.reshape(dy.shape[1], dy.shape[2])
        elif dy.ndim == 2:
            dy2d = dy
        else:
            raise ValueError(f"dy must be a 3D tensor, but got {dy.ndim}")
        dy2d = dy2d.contiguous()
        if ctx.quant_state is not None:
            from lorafusion_amd.ops.nf4 import NF4WeightRef

            dx, da_list, db_list = hip_ops.nf4_lora_backward(
                dy2d, x2d, NF4WeightRef(linear_w, ctx.quant_state), a_list, b_list, s, routing.c, routing.R, mask,
                routing.rank_list, requires_dx=ctx.needs_input_grad[0], dense=dense,
            )
        else:
            dx, da_list, db_list = hip_ops.lora_backward(
                dy2d, x2d, linear_w, a_list, b_list, s, routing.c, routing.R, mask, routing.rank_list,
                requires_dx=ctx.needs_input_grad[0],
            )
        if dx is not None and ctx.lead:
            dx = dx.reshape(1, *dx.shape)
        return (dx, None, None, None, None, None, None, None, None, *da_list, *db_list)


def fused_linear_multi_lora(
    padded_x: torch.Tensor,
    linear_w: torch.Tensor,
    *,
    lora_a_list: list[torch.Tensor],
    lora_b_list: list[torch.Tensor],
    seq_len_list: list[int],
    padded_seq_len_list: list[int],
    block_to_lookup_table: torch.Tensor,
    block_to_dropout_p: torch.Tensor,
    block_to_alpha: torch.Tensor,
    enable_dropout: bool,
    same_dropout_p_value: float | None,
    max_r: int,
    linear_bias: torch.Tensor | None = None,
    dropout_mask: torch.Tensor | None = None,
    seed: int | None = None,
    quant_state=None,
    routing: MultiRouting | None = None,
    keep_dequantized: bool = False,
) -> torch.Tensor:
    """Fused multi-adapter LoRA linear (lorafusion/ops/multi_lora.py:762-830).

    ``padded_x`` is ``[1, sum(padded_seq_len_list), K]``; adapter i owns rows
    ``[cur_i, cur_i + seq_len_list[i])`` with ``cur`` advancing by the padded lengths.
    ``dropout_mask`` / ``seed`` are extensions for reproducible runs.  With ``quant_state`` (the
    bitsandbytes-style state ``dequantize_nf4_triton`` takes) ``linear_w`` holds packed NF4 codes and
    is dequantised inside the forward and backward calls.  ``routing`` (extension) is the cached
    ``MultiLoRABatchInfo.routing(...)`` of the micro-batch the table arguments come from; without it the same
    object is built here, per call.  ``keep_dequantized`` (extension, NF4 only): the forward's dequantised
    weight is kept for the backward, which then dequantises nothing (2*N*K bytes held in between).
    """
    if len(lora_a_list) != len(lora_b_list):
        raise ValueError("lora_a_list and lora_b_list must have the same length")
    if len(lora_a_list) == 0:
        raise ValueError("lora_a_list and lora_b_list must not be empty")
    if len(lora_a_list) > L.LF_MAX_SEG:
        raise ValueError(f"currently, we only support up to {L.LF_MAX_SEG} simultaneous LoRA adapters")
    if len(seq_len_list) != len(lora_a_list) or len(padded_seq_len_list) != len(lora_a_list):
        raise ValueError("seq_len_list / padded_seq_len_list must have one entry per adapter")
    rank_list = [a.shape[0] for a in lora_a_list]
    if max(rank_list) > max_r:
        raise ValueError(f"max_r={max_r} is smaller than the largest adapter rank {max(rank_list)}")
    if routing is None:
        routing = MultiRouting(padded_seq_len_list, rank_list, block_to_lookup_table, block_to_alpha,
                               block_to_dropout_p, enable_dropout=enable_dropout)
    elif (routing.padded_seq_len_list != list(padded_seq_len_list) or routing.rank_list != rank_list
          or routing.enable_dropout != bool(enable_dropout) or routing.table.data_ptr() != block_to_lookup_table.data_ptr()):
        raise ValueError("routing does not belong to the batch tables passed with it")
    return FusedLinearMultiLoRA.apply(padded_x, linear_w, linear_bias, dropout_mask, seed, routing, quant_state,
                                      bool(keep_dequantized), len(lora_a_list), *lora_a_list, *lora_b_list)


# --------------------------------------------------------------------------- manager

multi_lora_manager: "MultiLoRAManager | None" = None


def init_multi_lora_manager(lora_configs, num_pipeline_stages: int,
                            multi_lora_max_microbatch_tokens: int | None,
                            multi_lora_global_batch_sizes: list[int] | None = None) -> "MultiLoRAManager":
    """lorafusion/ops/multi_lora.py:40-57 (``multi_lora_global_batch_sizes`` has a default there too, and is
    rejected when left at None, multi_lora.py:92-94)."""
    global multi_lora_manager
    if multi_lora_manager is not None:
        raise ValueError("Multi-LoRA manager has already been initialized")
    multi_lora_manager = MultiLoRAManager(lora_configs, num_pipeline_stages, multi_lora_max_microbatch_tokens,
                                          multi_lora_global_batch_sizes)
    return multi_lora_manager


def get_multi_lora_manager() -> "MultiLoRAManager | None":
    return multi_lora_manager


def reset_multi_lora_manager() -> None:
    global multi_lora_manager
    multi_lora_manager = None


class MultiLoRAManager:
    """Queue of batch infos between forward and backward of in-flight microbatches.

    The forward pass reads the newest batch info, backward / recompute the oldest
    (lorafusion/ops/multi_lora.py:196-292).  Gradient all-reduce and per-adapter optimizer
    stepping (multi_lora.py:125-184) belong to the multi-GPU runtime and are not provided.
    """

    def __init__(self, lora_configs, num_pipeline_stages: int,
                 multi_lora_max_microbatch_tokens: int | None,
                 multi_lora_global_batch_sizes: list[int] | None = None) -> None:
        self.lora_configs = lora_configs
        self.num_pipeline_stages = num_pipeline_stages
        self.multi_lora_max_microbatch_tokens = multi_lora_max_microbatch_tokens
        self.multi_lora_global_batch_sizes = multi_lora_global_batch_sizes
        if multi_lora_global_batch_sizes is None:
            raise ValueError("multi_lora_global_batch_sizes is not provided")
        if len(multi_lora_global_batch_sizes) != len(lora_configs):
            raise ValueError(f"Expected {len(lora_configs)} batch sizes, got {len(multi_lora_global_batch_sizes)}")
        self.adapter_sample_counts = dict.fromkeys(range(len(lora_configs)), 0)
        self.batch_info_deque: deque = deque(maxlen=num_pipeline_stages)
        self.lora_linear_layers: dict[int, int] = {}
        self.lora_linear_counter = 0
        self.microbatch_idx = 0
        self.is_in_backward = False

    def register_lora_linear(self, lora_linear) -> int:
        layer_id = id(lora_linear)
        if layer_id not in self.lora_linear_layers:
            self.lora_linear_layers[layer_id] = self.lora_linear_counter
        self.lora_linear_counter += 1
        return self.lora_linear_layers[layer_id]

    def add_batch_info(self, batch_info: MultiLoRABatchInfo) -> None:
        if len(self.batch_info_deque) == self.num_pipeline_stages:
            raise ValueError(f"Batch info deque is full. Current size: {len(self.batch_info_deque)}")
        batch_info.microbatch_idx = self.microbatch_idx
        self.microbatch_idx += 1
        self.batch_info_deque.append(batch_info)
        if batch_info.block_to_lookup_table.is_cuda:
            # once per micro-batch, here, instead of once per LoRA linear per layer
            batch_info.routing(enable_dropout=batch_info.enable_dropout)
        micro = getattr(batch_info, "micro_batch_info", None)
        if micro is None:
            if batch_info.allow_empty_micro_batch_info:
                return
            raise ValueError("MicroBatchInfo is not available")
        for adapter_idx, num_samples in micro.adapter_num_samples_pairs.items():
            if adapter_idx not in self.adapter_sample_counts:
                raise ValueError(f"Adapter {adapter_idx} not found in adapter_sample_counts")
            self.adapter_sample_counts[adapter_idx] += num_samples

    def get_newest_batch_info(self) -> MultiLoRABatchInfo | None:
        return self.batch_info_deque[-1] if self.batch_info_deque else None

    def get_oldest_batch_info(self) -> MultiLoRABatchInfo | None:
        return self.batch_info_deque[0] if self.batch_info_deque else None

    def pop_oldest_batch_info(self) -> MultiLoRABatchInfo | None:
        return self.batch_info_deque.popleft() if self.batch_info_deque else None

    def clear_batch_info(self) -> None:
        self.batch_info_deque.clear()

    @property
    def is_in_forward(self) -> bool:
        return not self.is_in_backward

    def set_backward_pass_state(self, *, is_backward: bool) -> None:
        self.is_in_backward = is_backward

    def mark_backward_pass_started(self) -> None:
        self.set_backward_pass_state(is_backward=True)

    def mark_forward_pass_started(self) -> None:
        self.set_backward_pass_state(is_backward=False)


def get_lora_kernel_config(kernel_name: str):
    """Only the one tile constant that is part of the data contract is exposed
    (lorafusion/ops/triton_ops/config.py:149-152)."""
    if kernel_name == "fused_multi_lora_block_size_m":
        return FUSED_MULTI_LORA_BLOCK_SIZE_M
    raise ValueError(f"Unknown kernel config {kernel_name!r}; the HIP kernels choose their own tiles.")
