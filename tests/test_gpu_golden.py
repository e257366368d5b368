"""HIP kernels, called through the C ABI, against the committed golden fixtures (float32 oracle outputs):
|got - want| <= 2e-2 + 1e-2 * |want| on bf16 outputs."""
import glob
import os
import sys

import numpy as np
import pytest
import torch

from tests import gpu_util as U

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _names(prefix):
    return sorted(os.path.basename(p) for p in glob.glob(os.path.join(GOLDEN, prefix + "_*.npz")))


def _bits(a):
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).to(U.dev()).view(torch.bfloat16)


@pytest.mark.parametrize("name", _names("attn"))
def test_attention_golden(name):
    from lyra_amd import _lib

    print(f"golden {name}", file=sys.stderr, flush=True)
    d = np.load(os.path.join(GOLDEN, name), allow_pickle=False)
    fp8 = "k_codes" in d
    dev = U.dev()
    q = _bits(d["q"])
    B, N, _, H = q.shape
    if fp8:
        k, v = U.t_fp8(d["k_codes"]), U.t_fp8(d["v_codes"])
        ks, vs = U.t_f32(d["k_scale"][..., 0]), U.t_f32(d["v_scale"][..., 0])
    else:
        k, v, ks, vs = _bits(d["k"]), _bits(d["v"]), None, None
    K, S = k.shape[1], k.shape[2]
    sinks = U.t_f32(d["sinks"])
    pos = torch.from_numpy(d["position"]).to(dev)
    gate = _bits(d["gate"]) if "gate" in d else None
    out = torch.empty(B, N, 1, H, dtype=torch.bfloat16, device=dev)
    sw = int(d["sliding_window"])
    L = _lib.lib
    ws = torch.zeros(max(L.lyra_decode_attention_workspace(B, N, K, S, H, sw), 256), dtype=torch.uint8, device=dev)
    rc = L.lyra_decode_attention(q.data_ptr(), k.data_ptr(), v.data_ptr(), ks.data_ptr() if fp8 else None, vs.data_ptr() if fp8 else None,
                                 sinks.data_ptr(), pos.data_ptr(), 1, gate.data_ptr() if gate is not None else None, out.data_ptr(),
                                 ws.data_ptr(), ws.numel(), B, N, K, S, H, H**-0.5, sw, _lib.DTYPE_E4M3FN if fp8 else _lib.DTYPE_BF16,
                                 _lib.DTYPE_BF16, torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, name)
    torch.cuda.synchronize()
    U.assert_close(U.to_np(out), d["out_fp32"], what=name)
    assert int(ws[: 1 << 16].count_nonzero()) == 0  # arrival counters are back at zero


@pytest.mark.parametrize("name", _names("gemm"))
def test_gemm_golden(name):
    from lyra_amd import _lib

    print(f"golden {name}", file=sys.stderr, flush=True)
    d = np.load(os.path.join(GOLDEN, name), allow_pickle=False)
    fp8 = "rhs_codes" in d
    dev = U.dev()
    lhs = _bits(d["lhs"])
    M, K = lhs.shape
    if fp8:
        rhs, scale = U.t_fp8(d["rhs_codes"]), U.t_f32(d["rhs_scale"])
        bk, bn = (int(b) for b in d["block"])
    else:
        rhs, scale, bk, bn = _bits(d["rhs"]), None, 0, 0
    G, _, N = rhs.shape
    sizes = torch.from_numpy(d["group_sizes"]).to(dev)
    bias = U.t_f32(d["bias"]) if "bias" in d else None
    swiglu = int(d["swiglu"])
    out = torch.empty(M, N // 2 if swiglu else N, dtype=torch.bfloat16, device=dev)
    L = _lib.lib
    ws = torch.zeros(max(L.lyra_decode_gemm_workspace(M, G, K, N, swiglu), 256), dtype=torch.uint8, device=dev)
    rc = L.lyra_decode_gemm(lhs.data_ptr(), rhs.data_ptr(), scale.data_ptr() if fp8 else None, bk, bn, sizes.data_ptr(),
                            bias.data_ptr() if bias is not None else None, out.data_ptr(), ws.data_ptr(), ws.numel(), M, G, K, N,
                            _lib.DTYPE_E4M3FN if fp8 else _lib.DTYPE_BF16, _lib.DTYPE_BF16, swiglu, 1.702, 7.0,
                            torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, name)
    torch.cuda.synchronize()
    U.assert_close(U.to_np(out), d["out_fp32"], what=name)


def test_routing_golden():
    from lyra_amd.kernels import decode_fused as F

    d = np.load(os.path.join(GOLDEN, "routing.npz"), allow_pickle=False)
    scores, groups, row_map, dest = F.moe_route(U.t_f32(d["logits"]), 15, 1, 3)
    assert np.array_equal(groups.cpu().numpy(), d["route_groups"])
    assert np.array_equal(dest.cpu().numpy(), d["route_unpermute"])
    assert np.array_equal(row_map.cpu().numpy(), d["route_permute"] // 4)
    np.testing.assert_allclose(scores.cpu().numpy(), d["scores"], atol=1e-6, rtol=1e-5)
