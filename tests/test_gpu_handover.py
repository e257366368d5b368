"""The cross-workgroup hand-over (publish partial results, count arrivals, the last one to arrive reads them all) replayed
many times: the chunk merge of decode attention at small batch and the K-sliced units of the grouped matmul at one token.
Every replay must reproduce the first result bit for bit - a partial that the last workgroup read before it was visible,
or a counter that did not return to zero, would show as a different sum sooner or later."""
import sys

import numpy as np
import pytest
import torch

from tests import gpu_util as U

pytestmark = pytest.mark.gpu
REPLAYS = 300


def _replay_and_compare(launch, out: torch.Tensor, what: str):
    """Captures launch() (which writes `out`) in a HIP graph, replays it REPLAYS times keeping every result, and reports the
    first replay that differs from replay 0."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        launch()  # warm-up outside the graph: workspaces are allocated here
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        launch()
    hist = torch.empty((REPLAYS, out.numel()), dtype=torch.int16, device=out.device)
    flat = out.view(torch.int16).reshape(-1)
    for i in range(REPLAYS):
        graph.replay()
        hist[i].copy_(flat)
        if i % 50 == 49:
            torch.cuda.synchronize()  # (the program's own synchronisations between replays)
    torch.cuda.synchronize()
    differs = (hist != hist[0]).any(dim=1).cpu().numpy()
    first = int(np.argmax(differs)) if differs.any() else -1
    assert first < 0, f"{what}: replay {first} differs from replay 0 ({int(differs.sum())} of {REPLAYS} do)"


def test_chunked_attention_merge_is_reproducible_over_300_replays():
    from lyra_amd import _lib
    from lyra_amd.kernels.decode_attention import decode_attention

    B, N, K, S, H = 1, 16, 4, 4096, 128
    assert _lib.lib.lyra_decode_attention_workspace(B, N, K, S, H, 0) > 256  # chunked: partials + arrival counters
    case = U.attention_case(99, B, N, K, S, H, fp8=True)
    q, k, v, sinks = U.attention_torch_inputs(case)
    pos = torch.tensor(4095, dtype=torch.int32, device=U.dev())
    out = torch.empty_like(q)
    print("handover: chunked attention merge", file=sys.stderr, flush=True)
    _replay_and_compare(lambda: out.copy_(decode_attention(q, k, v, sinks, H**-0.5, 0, pos, implementation="pallas")), out,
                        "chunked attention")


def test_k_sliced_expert_units_are_reproducible_over_300_replays():
    from lyra_amd.kernels.decode_gemm import decode_gemm
    from lyra_amd.nn.quant import QArray

    # one token, 3 routed experts + the shared one at the lyra-medium width: 4 row blocks x 32 spans = 128 units for 256
    # workgroups, so every unit is cut into K slices that meet in the workspace
    E, C, Hd = 32, 4096, 4096
    rng = np.random.default_rng(3)
    sizes = np.zeros(E, np.int32)
    sizes[[2, 9, 20, 31]] = 1
    dev = U.dev()
    w = QArray(torch.randint(0, 0x78, (E, C, 2 * Hd), device=dev, dtype=torch.uint8).view(torch.float8_e4m3fn),
               torch.rand(E, 1, 2 * Hd, device=dev) * 0.001 + 0.0005, (C, 1))
    x = U.t_bf16(rng.standard_normal((4, C)).astype(np.float32))
    gs = torch.from_numpy(sizes).to(dev)
    out = torch.empty((4, Hd), dtype=torch.bfloat16, device=dev)
    print("handover: K-sliced expert units", file=sys.stderr, flush=True)
    _replay_and_compare(lambda: out.copy_(decode_gemm(x, w, gs, fused_swiglu=True, quant_dtype=torch.float8_e4m3fn,
                                                      implementation="pallas")), out, "K-sliced expert matmul")
    assert torch.isfinite(out.float()).all() and float(out.float().abs().max()) > 0
