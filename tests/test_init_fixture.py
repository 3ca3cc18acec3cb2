"""The module constructor against the reference's own output (tests/golden/convblock_init.json, written by
tests/golden/make_init_fixture.py from the reference's ConvBlock under manual_seed(0)): same state_dict keys in the
same order, same shapes and dtypes, and the same values (order-sensitive checksums), which pins the draw order and the
initialisers of pyramid_dwconv/conv_block.py:25-34 and dwconv_triton.py:390-416."""
import json
from pathlib import Path

import pytest
import torch

FIX = json.loads((Path(__file__).parent / "golden" / "convblock_init.json").read_text())


def _checks(t):
    v = t.detach().double().flatten()
    idx = torch.arange(1, v.numel() + 1, dtype=torch.float64)
    return float(v.sum()), float(v.abs().sum()), float((v * idx).sum() / v.numel()), [float(x) for x in v[:4]]


@pytest.mark.parametrize("case", FIX, ids=lambda c: "-".join(f"{k}={v}" for k, v in c["kwargs"].items()))
def test_constructor_matches_reference(case):
    import pyramid_dwconv

    kw = {k: (tuple(v) if isinstance(v, list) else v) for k, v in case["kwargs"].items()}
    torch.manual_seed(0)
    m = pyramid_dwconv.ConvBlock(**kw)
    sd = m.state_dict()
    assert list(sd.keys()) == list(case["state_dict"].keys())
    for name, want in case["state_dict"].items():
        t = sd[name]
        assert list(t.shape) == want["shape"], name
        assert str(t.dtype) == want["dtype"], name
        s, a, w, head = _checks(t)
        assert head == want["head"], name
        assert s == pytest.approx(want["sum"], rel=1e-12, abs=1e-12), name
        assert a == pytest.approx(want["abs_sum"], rel=1e-12), name
        assert w == pytest.approx(want["weighted_sum"], rel=1e-12, abs=1e-12), name
