"""Host-side pieces of bench.py that need no GPU: the traffic table it reads from profiles/ and its byte counts."""
import importlib.util
from pathlib import Path

ROOT = Path(__file__).resolve().parents[1]


def _bench():
    spec = importlib.util.spec_from_file_location("bench_under_test", ROOT / "bench.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_traffic_table_parses():
    t = _bench().load_traffic()
    assert t, "profiles/hbm_traffic_by_kernel.txt gave no entries"
    for key in ("dwconv_fwd[32x56x56x64,k=13]", "dwconv_wgrad[32x56x56x64,k=13]", "dense_bwd_pair"):
        assert key in t and t[key] > 1e6


def test_algorithmic_bytes_of_the_headline_block():
    b = _bench()
    f, fb = b.block_alg_bytes(32, 56, 56, 128, 13, 2)
    assert round(f / 1e6, 1) == 260.2 and round(fb / 1e6, 1) == 658.6
    iss = b.conv_issue(13)
    assert iss["fwd"] == 8 * 32 and iss["useful"] == 169 and iss["wgrad"] == 256
    assert b.n_sets(32, 56, 56, 128, 13, 2) == 3
