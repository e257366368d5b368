"""lyra_decode_attention_static (the entry point that allocates nothing: partials and counters live in a device array of
the library) against lyra_decode_attention with a caller workspace, through the C ABI: bit-identical outputs on two calls
in a row, the second on a smaller input, plus the size limit.  Collected last: the static array is shared state."""
import sys

import numpy as np
import pytest
import torch

from oracle import lyra_oracle as O
from tests import gpu_util as U

pytestmark = pytest.mark.gpu


def _call(case, B, N, K, S, H, pos, sw, static, gate=None):
    from lyra_amd import _lib

    L = _lib.lib
    q, k, v, sinks = U.attention_torch_inputs(case)
    dev = U.dev()
    p = torch.tensor(pos, dtype=torch.int32, device=dev)
    out = torch.full((B, N, 1, H), float("nan"), dtype=torch.bfloat16, device=dev)
    g = None if gate is None else U.t_bf16(gate)
    stream = torch.cuda.current_stream().cuda_stream
    head = (q.data_ptr(), k.qval.data_ptr(), v.qval.data_ptr(), k.scale.data_ptr(), v.scale.data_ptr(), sinks.data_ptr(),
            p.data_ptr(), 1, g.data_ptr() if g is not None else None, out.data_ptr())
    tail = (B, N, K, S, H, H**-0.5, sw, _lib.DTYPE_E4M3FN, _lib.DTYPE_BF16, stream)
    if static:
        rc = L.lyra_decode_attention_static(*head, *tail)
    else:
        ws = torch.zeros(max(L.lyra_decode_attention_workspace(B, N, K, S, H, sw), 256), dtype=torch.uint8, device=dev)
        rc = L.lyra_decode_attention(*head, ws.data_ptr(), ws.numel(), *tail)
    _lib.check(rc, "static" if static else "workspace")
    torch.cuda.synchronize()
    return out


def test_static_scratch_entry_point_matches_the_workspace_entry_point_twice_in_a_row():
    from lyra_amd import _lib

    L = _lib.lib
    # both shapes are chunked launches (partials + arrival counters in use); the second is smaller in every respect
    shapes = [(3, 16, 4, 4096, 128, [4095, 2000, 17], 0), (2, 8, 2, 1536, 64, [1500, 700], 0)]
    rng = np.random.default_rng(5)
    for (B, N, K, S, H, pos, sw) in shapes:
        assert L.lyra_decode_attention_workspace(B, N, K, S, H, sw) > 256, "the case must use the scratch buffer"
        print(f"static scratch attention B={B} N={N} K={K} S={S} H={H}", file=sys.stderr, flush=True)
        case = U.attention_case(31 + B, B, N, K, S, H, fp8=True)
        gate = O.bf16_round((2.0 / (1.0 + np.exp(-rng.standard_normal((B, N))))).astype(np.float32))
        got = _call(case, B, N, K, S, H, pos, sw, static=True, gate=gate)
        ref = _call(case, B, N, K, S, H, pos, sw, static=False, gate=gate)
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), "static-scratch result differs from the workspace result"
        want = O.decode_attention_reference(case["q"], case["k"], case["v"], case["sinks"], H**-0.5, sw, np.array(pos), gate=gate)
        U.assert_close(U.to_np(got), want, what=f"static B={B}")
    # a launch that is not chunked never touches the array; sliding window
    B, N, K, S, H = 2, 16, 4, 512, 128
    case = U.attention_case(9, B, N, K, S, H, fp8=True)
    got = _call(case, B, N, K, S, H, [511, 100], 128, static=True)
    ref = _call(case, B, N, K, S, H, [511, 100], 128, static=False)
    assert torch.equal(got.view(torch.int16), ref.view(torch.int16))


def test_static_scratch_rejects_what_does_not_fit():
    from lyra_amd import _lib

    L = _lib.lib
    one = 256  # never dereferenced: argument and size checks answer before anything is launched
    limit = 4 << 20
    assert L.lyra_decode_attention_static(None, None, None, None, None, None, None, 1, None, None, 1, 16, 4, 4096, 128, 0.1, 0, 1, 0, None) == -1
    assert L.lyra_decode_attention_static(one, one, one, None, None, one, one, 1, None, one, 1, 16, 4, 4096, 96, 0.1, 0, 0, 0, None) == -2
    # 255 (row, kv head) pairs of 16 query heads, two chunks each: 4.3 MB of partials
    assert L.lyra_decode_attention_workspace(255, 16, 1, 8192, 128, 0) > limit
    assert L.lyra_decode_attention_static(one, one, one, None, None, one, one, 1, None, one, 255, 16, 1, 8192, 128, 0.1, 0, 0, 0, None) == -5
    assert L.lyra_decode_attention_workspace(128, 16, 1, 8192, 128, 0) <= limit
    assert b"static scratch" in L.lyra_strerror(-5)


@pytest.mark.parametrize("seed", range(16))
def test_static_scratch_entry_point_at_drawn_shapes(seed):
    """Few rows, long caches, one position per row (rows that see no key included): mostly chunked launches, whose partial
    results and counters then live in the static array; bit-identical to the workspace entry point, call after call."""
    from lyra_amd import _lib

    rng = np.random.default_rng(50000 + seed)
    pick = lambda xs: xs[int(rng.integers(0, len(xs)))]
    H, K, G = pick([64, 128]), pick([1, 2, 4, 8]), pick([1, 2, 4, 8])
    B, S, sw = int(rng.integers(1, 13)), int(rng.integers(300, 6000)), pick([0, 0, 0, 128, 700])
    pos = rng.integers(-1, S, B).tolist()
    print(f"static scratch draw {seed}: B={B} N={K * G} K={K} S={S} H={H} sw={sw} pos={pos}", file=sys.stderr, flush=True)
    assert _lib.lib.lyra_decode_attention_workspace(B, K * G, K, S, H, sw) <= 4 << 20
    case = U.attention_case(seed, B, K * G, K, S, H, fp8=True)
    ref = _call(case, B, K * G, K, S, H, pos, sw, static=False)
    got = _call(case, B, K * G, K, S, H, pos, sw, static=True)
    assert torch.equal(got.view(torch.int16), ref.view(torch.int16))
