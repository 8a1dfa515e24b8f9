"""The public ops keep the reference's call signatures.

tests/golden/reference_signatures.json holds the parameter lists of the reference's public
functions on this path, read from its source text (tests/golden/make_reference_signatures.py).
For each one the mirror in this package must take the same positional parameters in the same
order, the same keyword-only parameters, and the same defaults; what this package adds must be
optional (a default) and come after the reference's parameters, so every call written against the
reference binds the same way here.
"""

import importlib
import inspect
import json
import os

import pytest
import torch  # noqa: F401  (defaults such as torch.bfloat16 are evaluated against it)

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, "golden", "reference_signatures.json")) as f:
    SIGS = json.load(f)


def _default_value(src: str):
    from lorafusion_amd.utils.module import LigerKernelLevel

    # literals, torch dtypes and the level enum typed into the fixture
    return eval(src, {"torch": torch, "LigerKernelLevel": LigerKernelLevel})  # noqa: S307


@pytest.mark.parametrize("ref", SIGS, ids=[f"{s['module'].rsplit('.', 1)[1]}.{s['name']}" for s in SIGS])
def test_signature_matches_reference(ref):
    fn = getattr(importlib.import_module(ref["module"]), ref["name"])
    params = list(inspect.signature(fn).parameters.values())
    P = inspect.Parameter
    pos = [p for p in params if p.kind in (P.POSITIONAL_ONLY, P.POSITIONAL_OR_KEYWORD)]
    kwo = [p for p in params if p.kind == P.KEYWORD_ONLY]

    # positional parameters: the reference's, in order, first
    assert [p.name for p in pos[: len(ref["positional"])]] == ref["positional"], ref["reference"]
    for extra in pos[len(ref["positional"]):]:
        assert extra.default is not P.empty, f"added positional parameter {extra.name!r} has no default"
    # keyword-only parameters: every one of the reference's is accepted by keyword
    by_name = {p.name: p for p in params}
    for name in ref["keyword_only"]:
        assert name in by_name and by_name[name].kind in (P.KEYWORD_ONLY, P.POSITIONAL_OR_KEYWORD), \
            f"{ref['reference']}: keyword parameter {name!r} is missing"
    for extra in kwo:
        if extra.name not in ref["keyword_only"]:
            assert extra.default is not P.empty, f"added keyword parameter {extra.name!r} has no default"
    # defaults
    for name in ref["positional"] + ref["keyword_only"]:
        p = by_name[name]
        if name in ref["defaults"]:
            assert p.default is not P.empty, f"{ref['reference']}: {name!r} lost its default"
            assert p.default == _default_value(ref["defaults"][name]), \
                f"{ref['reference']}: default of {name!r} is {p.default!r}, reference has {ref['defaults'][name]}"
        else:
            assert p.default is P.empty, f"{ref['reference']}: {name!r} is required in the reference"
    if ref["var_positional"]:
        assert any(p.kind == P.VAR_POSITIONAL for p in params), f"{ref['reference']}: takes *args"
    if ref["var_keyword"]:
        assert any(p.kind == P.VAR_KEYWORD for p in params), f"{ref['reference']}: takes **kwargs"
