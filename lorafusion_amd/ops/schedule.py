"""Scheduler micro-batch descriptors and schedule files, without the scheduler.

The reference's planner emits a schedule as a list of ``AdapterGroupStepInfo`` whose ``micro_batch_infos`` are
``MicroBatchInfo`` records (lorafusion/solver/proposed_solver.py:51-131, 326-331); its training side loads the
pickled list and flattens it into micro-batches (lorafusion/train/training_utils.py:1142-1151).  A pickle of
those classes can only be opened with the reference importable, so the interchange format here is JSON: one
object per micro-batch with the *source* fields of ``MicroBatchInfo`` -- ``data_samples`` as
``[adapter_idx, global_batch_idx, sample_idx, num_tokens]`` rows, ``max_microbatch_size``,
``adapter_padding_multiple``, ``micro_batch_idx``, ``is_empty_marker`` -- optionally grouped in steps
(``{"micro_batch_infos": [...]}``, the shape of ``AdapterGroupStepInfo``).  ``MicroBatchDescriptor`` derives the
same fields from ``data_samples`` that ``MicroBatchInfo.update_from_data_samples`` derives
(proposed_solver.py:84-131), so ``batch_info_from_micro_batch`` and ``MultiLoRAManager`` take it as they take the
reference's own object.

A reference user dumps a schedule with::

    json.dump([{"micro_batch_infos": [
                    {"data_samples": [[a, g, s, n] for (a, g, s), n in mb.data_samples.items()],
                     "max_microbatch_size": mb.max_microbatch_size,
                     "adapter_padding_multiple": mb.adapter_padding_multiple,
                     "micro_batch_idx": mb.micro_batch_idx, "is_empty_marker": mb.is_empty_marker}
                    for mb in step.micro_batch_infos]} for step in adapter_group_step_infos], f)
"""

from __future__ import annotations

import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Iterable


def _round_up(x: int, multiple: int) -> int:
    return (x + multiple - 1) // multiple * multiple


@dataclass
class MicroBatchDescriptor:
    """The fields of ``MicroBatchInfo`` (proposed_solver.py:51-75), derived from ``data_samples`` on creation."""

    data_samples: dict[tuple[int, int, int], int]
    max_microbatch_size: int
    adapter_padding_multiple: int
    micro_batch_idx: int | None = None
    is_empty_marker: bool = False
    adapter_group_info: set[int] = field(init=False)
    adapter_global_batch_idx_pairs: set[tuple[int, int]] = field(init=False)
    adapter_token_lengths_pairs: dict[int, list[int]] = field(init=False)
    adapter_num_samples_pairs: dict[int, int] = field(init=False)
    adapter_num_tokens_pairs: dict[int, int] = field(init=False)
    total_tokens: int = field(init=False)
    padded_adapter_num_tokens_pairs: dict[int, int] = field(init=False)
    padded_total_tokens: int = field(init=False)

    def __post_init__(self) -> None:
        if self.adapter_padding_multiple <= 0:
            raise ValueError(f"adapter_padding_multiple must be positive, got {self.adapter_padding_multiple}.")
        samples = {(int(a), int(g), int(s)): int(n) for (a, g, s), n in self.data_samples.items()}
        if any(n < 0 for n in samples.values()):
            raise ValueError("a sample cannot have a negative number of tokens.")
        self.data_samples = samples
        self.adapter_group_info = {a for a, _, _ in samples}
        self.adapter_global_batch_idx_pairs = {(a, g) for a, g, _ in samples}
        self.adapter_token_lengths_pairs = {
            adapter: [n for (a, _, _), n in samples.items() if a == adapter] for adapter in self.adapter_group_info
        }
        self.adapter_num_samples_pairs = {a: len(v) for a, v in self.adapter_token_lengths_pairs.items()}
        self.adapter_num_tokens_pairs = {a: sum(v) for a, v in self.adapter_token_lengths_pairs.items()}
        self.total_tokens = sum(self.adapter_num_tokens_pairs.values())
        self.padded_adapter_num_tokens_pairs = {
            a: _round_up(n, self.adapter_padding_multiple) for a, n in self.adapter_num_tokens_pairs.items()
        }
        self.padded_total_tokens = sum(self.padded_adapter_num_tokens_pairs.values())

    @classmethod
    def from_json_object(cls, obj: dict[str, Any]) -> "MicroBatchDescriptor":
        rows = obj.get("data_samples")
        if not isinstance(rows, list):
            raise ValueError("a micro-batch needs 'data_samples': a list of [adapter, global_batch, sample, tokens] rows.")
        samples: dict[tuple[int, int, int], int] = {}
        for row in rows:
            if not isinstance(row, (list, tuple)) or len(row) != 4:
                raise ValueError(f"data_samples rows are [adapter, global_batch, sample, tokens], got {row!r}.")
            key = (int(row[0]), int(row[1]), int(row[2]))
            if key in samples:
                raise ValueError(f"sample {key} appears twice in one micro-batch.")
            samples[key] = int(row[3])
        try:
            return cls(samples, int(obj["max_microbatch_size"]), int(obj["adapter_padding_multiple"]),
                       obj.get("micro_batch_idx"), bool(obj.get("is_empty_marker", False)))
        except KeyError as e:
            raise ValueError(f"a micro-batch needs the field {e.args[0]!r}.") from None

    def to_json_object(self) -> dict[str, Any]:
        return {
            "data_samples": [[a, g, s, n] for (a, g, s), n in self.data_samples.items()],
            "max_microbatch_size": self.max_microbatch_size,
            "adapter_padding_multiple": self.adapter_padding_multiple,
            "micro_batch_idx": self.micro_batch_idx,
            "is_empty_marker": self.is_empty_marker,
        }


def micro_batches_from_json(obj: Any) -> list[MicroBatchDescriptor]:
    """A parsed schedule -> its micro-batches in order: a list of micro-batch objects, or a list of steps that each
    hold ``micro_batch_infos`` (flattened as lorafusion/train/training_utils.py:1147-1149 flattens the steps)."""
    if not isinstance(obj, list):
        raise ValueError("a schedule is a JSON list of micro-batches or of steps with 'micro_batch_infos'.")
    out: list[MicroBatchDescriptor] = []
    for item in obj:
        if isinstance(item, dict) and "micro_batch_infos" in item:
            out.extend(MicroBatchDescriptor.from_json_object(mb) for mb in item["micro_batch_infos"])
        elif isinstance(item, dict):
            out.append(MicroBatchDescriptor.from_json_object(item))
        else:
            raise ValueError(f"unexpected schedule entry {item!r}.")
    return out


def load_schedule(path: "str | Path") -> list[MicroBatchDescriptor]:
    """Micro-batches of the JSON schedule file at ``path``."""
    with Path(path).open("r", encoding="utf-8") as f:
        return micro_batches_from_json(json.load(f))


def dump_schedule(micro_batches: Iterable[Any], path: "str | Path") -> None:
    """Write micro-batches (these descriptors, or the reference's ``MicroBatchInfo`` objects: anything with
    ``data_samples``, ``max_microbatch_size``, ``adapter_padding_multiple``) as a JSON schedule."""
    rows = []
    for mb in micro_batches:
        rows.append({
            "data_samples": [[int(a), int(g), int(s), int(n)] for (a, g, s), n in mb.data_samples.items()],
            "max_microbatch_size": int(mb.max_microbatch_size),
            "adapter_padding_multiple": int(mb.adapter_padding_multiple),
            "micro_batch_idx": getattr(mb, "micro_batch_idx", None),
            "is_empty_marker": bool(getattr(mb, "is_empty_marker", False)),
        })
    with Path(path).open("w", encoding="utf-8") as f:
        json.dump(rows, f)
