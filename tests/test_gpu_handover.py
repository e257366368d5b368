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


@pytest.mark.parametrize("B,S,sw,positions", [(8, 4096, 0, "end"), (5, 700, 0, "first tiles"), (64, 1024, 128, "end")])
def test_front_step_rows_are_read_back_by_their_writer_over_300_replays(B, S, sw, positions):
    """lyra_decode_attention_qkv appends the new token's key and value rows and reads them back in the same launch, with
    nothing but the order of one wavefront's memory operations in between.  A read that overtook the stores would return the
    row's previous contents; so every replay starts from a cache whose row holds other values (a copy kernel in the graph
    restores them), and every replay's output must equal the first one's and the two-launch result."""
    from lyra_amd.kernels import decode_fused as F
    from lyra_amd.kernels.decode_attention import decode_attention
    from lyra_amd.nn.quant import QArray, quantize
    from oracle import lyra_oracle as O

    N, K, H = 16, 4, 128
    dev = U.dev()
    gen = torch.Generator(device=dev)
    gen.manual_seed(B + S)
    rng = np.random.default_rng(B)
    part = torch.randn(4, B, (N + 2 * K) * H, device=dev, generator=gen)
    qkv = F.Unsummed(part, None, 1.0)
    ones = torch.ones(H, device=dev)
    cos_t, sin_t = O.rope_tables(S, H)
    cos_t, sin_t = U.t_f32(cos_t), U.t_f32(sin_t)
    vals = np.full(B, S - 1) if positions == "end" else rng.integers(0, 128, B)
    pos = torch.from_numpy(vals.astype(np.int32)).to(dev)

    def cache():
        qa = quantize(torch.randn(B, K, S, H, device=dev, generator=gen).to(torch.bfloat16) * 3, torch.float8_e4m3fn, (1, H))
        return QArray(qa.qval, qa.scale, (1, H))

    k0, v0 = cache(), cache()  # pristine copies: the rows at `pos` hold values unrelated to the new token
    k1 = QArray(k0.qval.clone(), k0.scale.clone(), (1, H))
    v1 = QArray(v0.qval.clone(), v0.scale.clone(), (1, H))
    sinks = torch.randn(N, device=dev, generator=gen)
    # the two launches, on their own copies
    k2 = QArray(k0.qval.clone(), k0.scale.clone(), (1, H))
    v2 = QArray(v0.qval.clone(), v0.scale.clone(), (1, H))
    q = F.qkv_post(qkv, ones, ones, cos_t, sin_t, pos, k2, v2, N, K, H, 1e-5)
    want = decode_attention(q[:, :, None, :], k2, v2, sinks, H**-0.5, sw, pos, implementation="pallas").reshape(B, N * H)
    out = torch.empty_like(want)

    def launch():
        for dst, src in ((k1, k0), (v1, v0)):  # put the old rows back, so that a stale read would show
            dst.qval.view(torch.uint8).copy_(src.qval.view(torch.uint8))
            dst.scale.copy_(src.scale)
        got = F.attention_qkv(qkv, ones, ones, cos_t, sin_t, pos, k1, v1, sinks, H**-0.5, sw, N, K, H, 1e-5)
        assert got is not None
        out.copy_(got)

    print(f"handover: front step B={B} S={S} sw={sw} {positions}", file=sys.stderr, flush=True)
    _replay_and_compare(launch, out, "attention with the front step")
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
