"""GPU parity of the persistent GEMM kernel's fused paths at small sizes, for both of its tiles (256x256 over two
LDS stages, 128x256 over three).

The library picks that kernel by itself only for large products; here it is pinned
(lf_set_tile_cfg(7) / (8)) so that its LoRA seeding (rank chunks, per-wave routing lookups, the scale
folded into the skinny operand), its keep-mask select on the dX path, bias, fp16, edge tiles that
are shifted inwards and tiles that span two adapters all run against the CPU oracle at sizes the
oracle restates in full.  Tolerances as in test_gpu_lora_single.py / test_gpu_lora_multi.py.
"""

import pytest
import torch

from tests.test_gpu_lora_multi import _run as run_multi
from tests.test_gpu_lora_single import _run_case as run_single

pytestmark = pytest.mark.gpu


@pytest.fixture(params=[7, 8], ids=["256x256", "128x256"])
def big_tiles(request):
    from lorafusion_amd import _lib

    assert _lib.lib().lf_set_tile_cfg(request.param) == 0
    yield request.param
    assert _lib.lib().lf_set_tile_cfg(-1) == 0


@pytest.mark.parametrize(
    "M,K,N,r,p,scale",
    [
        (256, 256, 256, 16, 0.0, 2.0),     # one tile, no dropout
        (256, 256, 256, 16, 0.1, 1.0),     # scale 1: the skinny operand goes in unscaled
        (512, 1024, 768, 16, 0.1, 2.0),
        (384, 512, 1280, 32, 0.05, 0.5),   # last tile row shifted inwards by 128 rows
        (300, 256, 384, 8, 0.2, 4.0),      # ragged M, N = 1.5 tiles (both edge tiles shifted), rank 8
        (640, 768, 512, 64, 0.1, 3.0),     # two rank chunks; a scale that is not a power of two
        (300, 256, 256, 128, 0.1, 1.0),    # four rank chunks
        (257, 256, 384, 40, 0.3, 0.5),     # rank 40 inside 48 columns
        (520, 512, 640, 96, 0.1, 1.5),
    ],
)
def test_single_through_big_tiles(big_tiles, M, K, N, r, p, scale):
    run_single(M, K, N, r, p, scale)


def test_single_bias_3d_fp16_through_big_tiles(big_tiles):
    run_single(512, 512, 640, 16, 0.1, 2.0, bias=True, three_d=True)
    run_single(256, 512, 384, 16, 0.1, 2.0, dtype=torch.float16)
    run_single(768, 256, 512, 32, 0.0, 0.25, dtype=torch.float16, bias=True)


@pytest.mark.parametrize(
    "seq,ranks,p_list,scales",
    [
        ([256, 128], [16, 16], [0.1, 0.1], [2.0, 2.0]),
        ([129, 130, 128], [16, 16, 16], [0.1, 0.1, 0.1], [1.0, 2.0, 4.0]),        # tiles that span two adapters
        ([100, 300, 64, 257], [16, 16, 16, 16], [0.0, 0.05, 0.1, 0.1], [1.0, 2.0, 2.0, 4.0]),
        ([200, 50], [16, 64], [0.0, 0.0], [2.0, 0.5]),                             # mixed ranks, no dropout
        ([1, 127, 128, 129, 5, 300, 77, 64], [16, 32, 16, 8, 64, 16, 16, 32], [0.1] * 8, [1.0, 3.0] * 4),
        ([200, 130, 300], [16, 48, 8], [0.1, 0.0, 0.25], [1.0, 2.0, 0.5]),
        ([150, 260], [96, 40], [0.1, 0.1], [0.5, 2.0]),
    ],
)
def test_multi_through_big_tiles(big_tiles, seq, ranks, p_list, scales):
    run_multi(seq, 512, 384, ranks, p_list, scales)


def test_multi_bias_through_big_tiles(big_tiles):
    run_multi([256, 130, 384], 384, 512, [16, 16, 32], [0.125, 0.0, 0.25], [2.0, 1.0, 0.5], bias=True,
              explicit_dtype=torch.bfloat16)


def test_pinned_tile_rejects_small_products():
    """The persistent kernel shifts edge tiles inwards, so it needs at least one full tile: pinned to a 128-row
    product it fails with a shape error instead of falling back silently."""
    from lorafusion_amd import _lib
    from lorafusion_amd.ops import hip_ops

    a = torch.randn(128, 64, device="cuda").bfloat16()
    b = torch.randn(256, 64, device="cuda").bfloat16()
    assert _lib.lib().lf_set_tile_cfg(7) == 0
    try:
        with pytest.raises(RuntimeError):
            hip_ops.gemm(a, b)
    finally:
        assert _lib.lib().lf_set_tile_cfg(-1) == 0
    assert _lib.lib().lf_set_tile_cfg(9) != 0
    hip_ops.gemm(a, b)


def test_pinned_128_row_tile_rejects_a_short_contraction():
    """The 128-row tile runs its K loop over three stages: fewer than four K steps (K < 256) is a shape error when pinned
    (the library's own choice never lands there)."""
    from lorafusion_amd import _lib
    from lorafusion_amd.ops import hip_ops

    a = torch.randn(256, 192, device="cuda").bfloat16()
    b = torch.randn(256, 192, device="cuda").bfloat16()
    assert _lib.lib().lf_set_tile_cfg(8) == 0
    try:
        with pytest.raises(RuntimeError):
            hip_ops.gemm(a, b)
    finally:
        assert _lib.lib().lf_set_tile_cfg(-1) == 0
    assert torch.allclose(hip_ops.gemm(a, b).float(), a.float() @ b.float().T, rtol=2e-2, atol=0.5)
