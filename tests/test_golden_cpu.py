"""The committed golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py with the NumPy oracle)
against the independent C restatement, plus the integer tables and the vectors lyra's own tests hold."""
import glob
import os

import numpy as np
import pytest
import torch

from oracle import clib
from oracle import lyra_oracle as O

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


@pytest.mark.parametrize("name", sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLDEN, "attn_*.npz"))))
def test_c_attention_matches_golden(name):
    d = _load(name)
    fp8 = "k_codes" in d
    H = d["q"].shape[-1]
    k, v = (d["k_codes"], d["v_codes"]) if fp8 else (d["k"], d["v"])
    ks = d["k_scale"][..., 0] if fp8 else None
    vs = d["v_scale"][..., 0] if fp8 else None
    gate = O.bf16_from_bits(d["gate"]) if "gate" in d else None
    got = clib.decode_attention(d["q"], k, v, ks, vs, d["sinks"], d["position"], gate, H**-0.5, int(d["sliding_window"]))
    np.testing.assert_allclose(got, d["out_fp32"], atol=2e-5, rtol=2e-5)


@pytest.mark.parametrize("name", sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLDEN, "gemm_*.npz"))))
def test_c_gemm_matches_golden(name):
    d = _load(name)
    fp8 = "rhs_codes" in d
    rhs = d["rhs_codes"] if fp8 else d["rhs"]
    got = clib.decode_gemm(d["lhs"], rhs, d["rhs_scale"] if fp8 else None, tuple(d["block"]) if fp8 else None, d["group_sizes"],
                           d["bias"] if "bias" in d else None, fused_swiglu=bool(d["swiglu"]))
    np.testing.assert_allclose(got, d["out_fp32"], atol=1e-4, rtol=1e-4)


def test_fp8_table_fixture_is_torch_e4m3fn():
    table = _load("tables.npz")["fp8_e4m3fn"]
    want = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).to(torch.float32).numpy()
    finite = np.isfinite(want)
    assert np.array_equal(table[finite], want[finite]) and np.isnan(table[~finite]).all()
    assert table[finite].max() == 448.0


def test_window_table_fixture_brute_force():
    rows = _load("tables.npz")["window_rows"]
    S = 512
    keys = np.arange(S)
    for sw, pos, lo, hi, start, sliding in rows[:: 7]:
        mask = (keys <= pos) & ((keys > pos - sw) if sw > 0 else True)
        vis = keys[mask]
        assert (vis[0], vis[-1]) == (lo, hi) and len(vis) == (min(sw, pos + 1) if sw > 0 else pos + 1)
        if sliding:
            wlen = O.decode_window(sw)
            assert start % 128 == 0 or start == S - wlen
            assert start <= lo and hi < start + wlen  # every visible key lies inside the slab the reference slices


def test_routing_fixture_closed_forms():
    d = _load("routing.npz")
    # lyra tests/test_combine.py:13-17: assignments [0,2,4,7,1,3,4,7] sort stably to rows [0,4,1,5,2,6,3,7]
    assert d["assignments"].tolist() == [0, 2, 4, 7, 1, 3, 4, 7]
    assert d["permute"].tolist() == [0, 4, 1, 5, 2, 6, 3, 7]
    assert np.array_equal(d["permute"], np.argsort(d["assignments"], kind="stable"))
    assert np.array_equal(d["unpermute"][d["permute"]], np.arange(8))
    # routed part: indices of the 3 largest logits, lowest index first on ties; scores sum to 1 over the routed picks
    logits, active = d["logits"], d["active_map"].reshape(16, 4)
    assert active[3].tolist() == [0, 1, 2, 15]  # an all-tied row picks experts 0, 1, 2, then the shared expert
    for t in range(16):
        top = sorted(range(15), key=lambda e: (-logits[t, e], e))[:3]
        assert active[t, :3].tolist() == top and active[t, 3] == 15
    np.testing.assert_allclose(d["scores"][:, :3].sum(-1), 1.0, rtol=1e-6)
    assert (d["scores"][:, 3] == 1.0).all()
    assert np.array_equal(d["route_groups"], np.bincount(d["active_map"], minlength=16))
    assert np.array_equal(d["route_permute"], np.argsort(d["active_map"], kind="stable"))
