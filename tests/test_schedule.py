"""Schedule files and micro-batch descriptors (host logic, CPU).

``MicroBatchDescriptor`` must derive from ``data_samples`` what the reference's ``MicroBatchInfo`` derives
(lorafusion/solver/proposed_solver.py:84-131): checked here against an independent tally of the same samples, through
a JSON round trip, and through ``batch_info_from_micro_batch`` against the routing oracle.
"""

import json
import random
from types import SimpleNamespace

import pytest
import torch

from lorafusion_amd.ops import schedule as sch
from oracle import routing


def _random_samples(rnd, n_adapters, n_samples):
    samples = {}
    for i in range(n_samples):
        samples[(rnd.randrange(n_adapters), rnd.randrange(3), i)] = rnd.randint(1, 900)
    return samples


@pytest.mark.parametrize("seed", range(8))
def test_descriptor_fields_follow_the_samples(seed):
    rnd = random.Random(seed)
    pad = rnd.choice([64, 128])
    samples = _random_samples(rnd, rnd.randint(1, 6), rnd.randint(1, 20))
    mb = sch.MicroBatchDescriptor(samples, max_microbatch_size=16384, adapter_padding_multiple=pad, micro_batch_idx=seed)
    # independent tally
    tokens, counts = {}, {}
    for (a, _, _), n in samples.items():
        tokens[a] = tokens.get(a, 0) + n
        counts[a] = counts.get(a, 0) + 1
    assert mb.adapter_group_info == set(tokens)
    assert mb.adapter_num_tokens_pairs == tokens and mb.adapter_num_samples_pairs == counts
    assert mb.total_tokens == sum(samples.values())
    assert mb.padded_adapter_num_tokens_pairs == {a: -(-n // pad) * pad for a, n in tokens.items()}
    assert mb.padded_total_tokens == sum(mb.padded_adapter_num_tokens_pairs.values())
    assert mb.adapter_global_batch_idx_pairs == {(a, g) for a, g, _ in samples}
    for a, lens in mb.adapter_token_lengths_pairs.items():
        assert sorted(lens) == sorted(n for (x, _, _), n in samples.items() if x == a)


def test_schedule_round_trip_and_step_grouping(tmp_path):
    rnd = random.Random(42)
    mbs = [sch.MicroBatchDescriptor(_random_samples(rnd, 4, 9), 8192, 128, micro_batch_idx=i) for i in range(5)]
    path = tmp_path / "schedule.json"
    sch.dump_schedule(mbs, path)
    back = sch.load_schedule(path)
    assert [b.to_json_object() for b in back] == [m.to_json_object() for m in mbs]
    assert [b.adapter_num_tokens_pairs for b in back] == [m.adapter_num_tokens_pairs for m in mbs]
    # the reference's grouping: steps that hold micro_batch_infos, flattened in order
    steps = [{"micro_batch_infos": [m.to_json_object() for m in mbs[:2]]}, {"micro_batch_infos": [m.to_json_object() for m in mbs[2:]]}]
    assert [b.micro_batch_idx for b in sch.micro_batches_from_json(steps)] == [0, 1, 2, 3, 4]
    # objects that only look like MicroBatchInfo can be dumped too
    duck = SimpleNamespace(data_samples={(0, 0, 0): 5, (2, 0, 1): 7}, max_microbatch_size=64, adapter_padding_multiple=128)
    sch.dump_schedule([duck], path)
    assert sch.load_schedule(path)[0].adapter_num_tokens_pairs == {0: 5, 2: 7}


def test_malformed_schedules_are_refused(tmp_path):
    with pytest.raises(ValueError):
        sch.micro_batches_from_json({"data_samples": []})
    with pytest.raises(ValueError):
        sch.micro_batches_from_json([{"data_samples": [[0, 0, 0]], "max_microbatch_size": 1, "adapter_padding_multiple": 128}])
    with pytest.raises(ValueError):
        sch.micro_batches_from_json([{"data_samples": [[0, 0, 0, 4], [0, 0, 0, 5]], "max_microbatch_size": 1, "adapter_padding_multiple": 128}])
    with pytest.raises(ValueError):
        sch.micro_batches_from_json([{"data_samples": [[0, 0, 0, 4]], "adapter_padding_multiple": 128}])
    with pytest.raises(ValueError):
        sch.MicroBatchDescriptor({(0, 0, 0): 4}, 16, 0)
    p = tmp_path / "bad.json"
    p.write_text(json.dumps([3]))
    with pytest.raises(ValueError):
        sch.load_schedule(p)


def test_descriptor_drives_the_routing_tables():
    """The op's routing from a descriptor equals the routing oracle's tables for the same per-adapter token counts
    (adapters in ascending order, one segment each)."""
    from lorafusion_amd.ops import multi_lora as ml

    cfgs = [SimpleNamespace(r=r, lora_alpha=a, lora_dropout=p) for r, a, p in ((16, 2.0, 0.0), (32, 1.0, 0.1), (8, 4.0, 0.05), (64, 0.5, 0.1))]
    samples = {(3, 0, 0): 150, (0, 0, 1): 120, (0, 1, 2): 180, (1, 0, 3): 129}
    mb = sch.micro_batches_from_json([sch.MicroBatchDescriptor(samples, 4096, 128).to_json_object()])[0]
    info = ml.batch_info_from_micro_batch(mb, cfgs)
    seq, ranks = [300, 129, 150], [16, 32, 64]
    padded, lookup, *_ = routing.block_tables(seq, ranks, [0.0, 0.1, 0.1], [2.0, 1.0, 0.5], 128)
    assert info.lora_idx_list == [0, 1, 3] and info.seq_len_list == seq and info.padded_seq_len_list == list(padded)
    assert torch.equal(info.block_to_lookup_table.cpu(), torch.as_tensor(lookup, dtype=torch.int32))
    # a descriptor padded for another block size is refused
    with pytest.raises(ValueError):
        ml.batch_info_from_micro_batch(sch.MicroBatchDescriptor(samples, 4096, 64), cfgs)
