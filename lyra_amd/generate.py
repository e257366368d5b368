"""Generation driver for decode mode (lyra/generate.py of the reference, minus tokenizer and REPL)."""
from __future__ import annotations

from dataclasses import replace

import torch

from lyra_amd.model import ModelCache, ModelConfig, ModelWeights, model_apply


def sample_token(logits: torch.Tensor, cfg: ModelConfig, generator: torch.Generator | None = None,
                 out: torch.Tensor | None = None, advance: torch.Tensor | None = None) -> torch.Tensor:
    """lyra/generate.py:46-53 applied to each row of ``logits`` [B, V]: greedy when temperature <= 0, else
    temperature scaling, top-k masking (lowest index wins ties, like lax.top_k) and a categorical draw.
    ``advance``: an int32 device scalar (the cache position) to increment by one once the tokens are chosen; the HIP
    samplers do it in the same launch."""
    # tile maxima the LM head left with these logits (model.py: `logits.tile_max`), while the tensor is as it left them
    tile_max = getattr(logits, "tile_max", None)
    tile_max = tile_max[0] if tile_max is not None and tile_max[1] == logits._version else None
    if cfg.sample_temperature <= 0:
        if logits.is_cuda and logits.dtype == torch.float32 and logits.is_contiguous() and cfg.implementation != "xla":
            from lyra_amd.kernels.decode_fused import argmax

            return argmax(logits, min(cfg.vocab_size, logits.shape[-1]), out, advance, tile_max)
        if advance is not None:
            advance += 1
        return _into(out, torch.argmax(logits, dim=-1).to(torch.int32))
    if (logits.is_cuda and logits.dtype == torch.float32 and logits.is_contiguous() and cfg.implementation != "xla"
            and 0 < cfg.sample_topk <= 8):
        # the draw is the inverse CDF over the k candidates at one uniform number per row: from the caller's torch
        # generator when one is given, else made inside the launch from the sampler's own state (no generator launches:
        # inside a captured step torch.rand costs three small kernels per token)
        from lyra_amd.kernels.decode_fused import rng_state, sample_topk

        if generator is None:
            u = rng_state(logits.device)
        else:
            u = torch.rand(logits.shape[0], device=logits.device, dtype=torch.float32, generator=generator)
        return sample_topk(logits, u, cfg.sample_topk, cfg.sample_temperature, min(cfg.vocab_size, logits.shape[-1]), out, advance,
                           tile_max)
    if advance is not None:
        advance += 1
    logits = logits.to(torch.float32) / cfg.sample_temperature
    if 0 < cfg.sample_topk < logits.shape[-1]:
        top = torch.topk(logits, cfg.sample_topk, dim=-1)
        masked = torch.full_like(logits, torch.finfo(torch.float32).min)
        logits = masked.scatter(-1, top.indices, top.values)
    probs = torch.softmax(logits, dim=-1)
    return _into(out, torch.multinomial(probs, 1, generator=generator)[:, 0].to(torch.int32))


def _into(out: torch.Tensor | None, value: torch.Tensor) -> torch.Tensor:
    if out is None:
        return value
    out.copy_(value)
    return out


def generate(tokens: torch.Tensor, model: ModelWeights, cache: ModelCache, cfg: ModelConfig,
             generator: torch.Generator | None = None) -> tuple[torch.Tensor, ModelCache]:
    """lyra/generate.py:56-61 for a batch of sequences, one new token each: tokens [B] -> next tokens [B]."""
    logits, cache = model_apply(tokens, model, cache, cfg)
    return sample_token(logits, cfg, generator), cache


class GraphedDecoder:
    """One decode step captured in a HIP graph: the per-token host work collapses to one graph launch.

    The reference jits the step (lyra/generate.py:119-125) and scans it over the tokens to draw
    (``sample_tokens``, :64-85: every drawn token is the next step's input, at the next position).  Here every kernel of
    the step is recorded once and replayed: ``tokens`` (int32, on the device) is read by the step's first kernel and
    overwritten by its last one, the sampler, which also moves the cache position on - so replays chain with no host work
    between them.  ``advance=False`` keeps the position where it is (benchmarks that time the same context again and
    again)."""

    def __init__(self, model: ModelWeights, cache: ModelCache, cfg: ModelConfig, batch: int, warmup: int = 2,
                 greedy: bool = True, advance: bool = True):
        # greedy=False: temperature / top-k sampling as configured, the uniform numbers made inside the sampler's launch
        # from its own generator state on the device (the state moves on with every replay)
        self.cfg, self.model, self.cache, self.greedy, self.advance = cfg, model, cache, greedy, advance
        dev = model.emb.device
        self.tokens = torch.zeros(batch, dtype=torch.int32, device=dev)
        self.next_tokens = self.tokens  # the sampler writes where the next step reads
        self.graph = torch.cuda.CUDAGraph()
        stream = torch.cuda.Stream(device=dev)
        stream.wait_stream(torch.cuda.current_stream(dev))
        start_pos = cache.pos.clone()
        with torch.cuda.stream(stream):
            keep = self.tokens.clone()
            for _ in range(warmup):  # allocates workspaces and warms caches outside the capture
                cache.pos.copy_(start_pos)  # (always at the caller's position: it may be the last cache row)
                self.tokens.copy_(keep)
                self._step()
            cache.pos.copy_(start_pos)
            self.tokens.copy_(keep)
            with torch.cuda.graph(self.graph, stream=stream):
                self._step()
            cache.pos.copy_(start_pos)
            self.tokens.copy_(keep)
        torch.cuda.current_stream(dev).wait_stream(stream)

    def _step(self):
        logits, _ = model_apply(self.tokens, self.model, self.cache, self.cfg, advance=False)
        self.logits = logits
        sample_token(logits, replace(self.cfg, sample_temperature=0.0) if self.greedy else self.cfg, out=self.tokens,
                     advance=self.cache.pos if self.advance else None)

    def step(self) -> torch.Tensor:
        """Run one decode step on ``self.tokens``; they are replaced by the next tokens (device, int32): greedy, or sampled."""
        self.graph.replay()
        return self.tokens

    def decode(self, n: int) -> torch.Tensor:
        """``n`` chained steps (lyra/generate.py:64-85): returns the drawn tokens [n, B]; only graph launches and one small
        copy per step are enqueued, nothing is read back in between."""
        out = torch.empty((n, self.tokens.shape[0]), dtype=torch.int32, device=self.tokens.device)
        for i in range(n):
            self.graph.replay()
            out[i].copy_(self.tokens)
        return out
