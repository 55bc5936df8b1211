"""Prefill and decode throughput of the language-model families through the
engine's step function, at layer sizes that resemble real models (random
weights, synthetic tokens): ``python bench.py --lm-bench``.

For each size a Pipizen stack (latent attention / lightning mixers, dense and
mixture-of-experts feed-forwards), a Sodonex stack (chunked sigmoid attention
with token shift and short convolutions, squared-relu experts) and a Movinex
stack (a Mamba-2 layer, full and sliding-window softmax attention, GeGLU and
sigmoid-routed experts) and a Vilulix stack (parallel layers: a matrix memory,
latent attention with a query latent, sliding-window attention with a sink
beside a gated delta rule, dense SwiGLU) run beside a Llama stack of the same
width, depth, head count and feed-forward width - the framework's plain decoder. Measured per family:

* prefill: one prompt of ``P`` tokens through ``LLMEngine.step_logits``;
* decode: ``B`` sequences at context ``P`` advancing one token per step
  (Llama: the fused decode step the scheduler replays; the others: their step
  function on a [B]-row batch).

One JSON line per (size, family); nothing here touches the default workload.
"""
from __future__ import annotations

import json
import time

import numpy as np
import torch

from ..models.configs import (ChunkAttnConfig, DeltaRuleConfig, FeedForwardConfig,
                              HybridLayerConfig, LatentAttnConfig, LightningConfig, LlamaConfig,
                              LoopConfig, Mamba2Config, MatrixMemoryConfig, MovinexConfig,
                              ParallelMixerConfig, PipizenConfig, RotaryConfig, SodonexConfig,
                              SoftmaxAttnConfig, VilulixConfig)

SIZES = {
    # name: (width, layers, heads, head_dim, rot_dim, kv_rank, ff, experts, expert_ff, top)
    "1b": (2048, 4, 16, 128, 64, 512, 5632, 16, 1408, 4),
    "7b": (4096, 4, 32, 128, 64, 512, 11008, 32, 1408, 6),
    "tiny": (64, 4, 2, 16, 8, 24, 96, 4, 32, 2),       # CPU plumbing run
}


def pipizen_stack(name: str, vocab: int = 32000) -> PipizenConfig:
    d, n, H, D, Dr, R, ff, E, eff, top = SIZES[name]
    rot = RotaryConfig(Dr, 10000.0, (8.0, 2048.0, 32.0, 1.0))
    layers = []
    for i in range(n):
        if i % 2 == 0:
            mixer = LatentAttnConfig(H, D, Dr, D, R, (D + Dr) ** -0.5, rot,
                                     None if i % 4 == 0 else i - 2)
            kind = "latent_attention"
        else:
            mixer = LightningConfig(H, D, D, tuple(0.9 + 0.099 * h / max(1, H - 1) for h in range(H)))
            kind = "lightning"
        mlp = FeedForwardConfig("dense", ff) if i % 2 == 0 else \
            FeedForwardConfig("moe", eff, E, 0, top, 4, 2, eff)
        layers.append(HybridLayerConfig(kind, mixer, mlp))
    return PipizenConfig(f"pipizen-{name}", vocab, d, 1e-6, tuple(layers))


def sodonex_stack(name: str, vocab: int = 32000, chunk: int = 768) -> SodonexConfig:
    """Every layer: grouped chunked sigmoid attention (4 query heads per
    key/value head, 4 convolution taps) and the same experts as the Pipizen
    stack's mixture layers (squared relu, no shared expert)."""
    d, n, H, D, Dr, _, _, E, eff, top = SIZES[name]
    mixer = ChunkAttnConfig(H, max(1, H // 4), D, D, 4, chunk, D ** -0.5, RotaryConfig(Dr, 10000.0))
    mlp = FeedForwardConfig("moe", eff, E, 0, top, act="relu2", router="softmax_top")
    return SodonexConfig(f"sodonex-{name}", vocab, d, 1e-6, 0.5, 1.0,
                         tuple(HybridLayerConfig("attention", mixer, mlp) for _ in range(n)))


def movinex_stack(name: str, vocab: int = 32000, window: int = 1024) -> MovinexConfig:
    """Four layers: a Mamba-2 layer (inner width 2 x width, 64 channels per
    head, state 128) with a dense GeGLU, a full-causal attention layer with
    biases and query temperature, and two sliding-window layers (keys double as
    values, rotary, soft-capping, output gate), the three attention layers with
    sigmoid-routed experts; 4 query heads per key/value head. Layers 1 - 2 are
    entered through the [x ; embedding] projection of a repeated stretch
    (one pass, so the stack stays four layer runs deep)."""
    d, n, H, D, Dr, _, ff, E, eff, top = SIZES[name]
    G = max(1, H // 4)
    mamba = Mamba2Config(max(1, 2 * d // 64), min(64, 2 * d), 128 if d >= 512 else 8, 1, 4, 1)
    full = SoftmaxAttnConfig(H, G, D, D, D ** -0.5, bias=True, q_temp=(0.1, 256))
    local = SoftmaxAttnConfig(H, G, D, D, D ** -0.5, values_from_keys=True, gate=True,
                              rot=RotaryConfig(Dr, 10000.0), softcap=30.0, window=window,
                              keep_first=4)
    moe = FeedForwardConfig("moe", eff, E, 0, top, 4, 2, router="sigmoid", group_rank=2)
    layers = [HybridLayerConfig("mamba2", mamba, FeedForwardConfig("dense", ff, act="geglu")),
              HybridLayerConfig("attention", full, moe)]
    layers += [HybridLayerConfig("attention_2", local, moe) for _ in range(max(0, n - 2))]
    return MovinexConfig(f"movinex-{name}", vocab, d, 1e-6, 1.0, tuple(layers),
                         LoopConfig(1, min(3, len(layers)), 1))


def vilulix_stack(name: str, vocab: int = 32000, window: int = 1024) -> VilulixConfig:
    """Four parallel layers, each with a dense SwiGLU beside its mixer: a matrix
    memory (the Llama stack's heads and head size for q, k and v), latent
    attention as in the Pipizen stack with a query latent of 3 x the key/value
    latent and an output gate, and twice a sliding-window attention (4 query
    heads per key/value head, rotary on half a head, zero sink) beside a gated
    delta rule (as many value heads, 4 per query/key head, 4 taps)."""
    d, n, H, D, Dr, R, ff, _, _, _ = SIZES[name]
    G = max(1, H // 4)
    mem = MatrixMemoryConfig(H, D, D, 15.0)
    lat = LatentAttnConfig(H, D, Dr, D, R, (D + Dr) ** -0.5, RotaryConfig(Dr, 10000.0, half=True),
                           q_rank=3 * R, gate=True)
    left = SoftmaxAttnConfig(H, G, D, D, D ** -0.5, rot=RotaryConfig(Dr, 10000.0, half=True),
                             window=window, qk_norm="whole", zero_sink=True)
    par = ParallelMixerConfig(left, DeltaRuleConfig(H, G, D, D, 4), 1.0, 1.0)
    mlp = FeedForwardConfig("dense", ff)
    layers = [HybridLayerConfig("mlstm", mem, mlp), HybridLayerConfig("latent_attention", lat, mlp)]
    layers += [HybridLayerConfig("parallel", par, mlp) for _ in range(max(0, n - 2))]
    return VilulixConfig(f"vilulix-{name}", vocab, d, 1e-6, 30.0, tuple(layers))


def llama_stack(name: str, vocab: int = 32000) -> LlamaConfig:
    d, n, H, D, _, _, ff, _, _, _ = SIZES[name]
    return LlamaConfig(f"llama-{name}-stack", d, n, H, max(1, H // 4), D, ff, vocab,
                       rope_theta=10000.0, max_positions=8192)


def _sync(dev):
    if dev.type == "cuda":
        torch.cuda.synchronize(dev)


def _time(fn, dev, reps: int) -> float:
    fn()
    _sync(dev)
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    _sync(dev)
    return (time.perf_counter() - t0) / reps


def bench_family(cfg, dev, *, prompt: int, batch: int, steps: int, seed: int = 0) -> dict:
    from .llm_engine import LLMEngine
    cap = -(-(prompt + steps + 8) // 64) * 64
    eng = LLMEngine(cfg, dev, seed=seed, max_seqs=batch, max_seq_len=cap, block_size=16,
                    num_blocks=batch * cap // 16 + 8, use_graphs=False)
    g = torch.Generator().manual_seed(seed)
    toks = torch.randint(0, cfg.vocab_size, (batch, prompt), generator=g).tolist()
    out = {"family": eng.family.name, "model": cfg.name, "prompt": prompt, "batch": batch}
    with torch.inference_mode():
        # prefill: each sequence's prompt as one pass (the first is the warm-up)
        seqs, times = [], []
        for b in range(batch):
            s = eng.open_sequence()
            _sync(eng.device)
            t0 = time.perf_counter()
            eng.step_logits([s], [toks[b]], [[prompt - 1]])
            _sync(eng.device)
            times.append(time.perf_counter() - t0)
            seqs.append(s)
        pre = float(np.median(times[1:])) if batch > 1 else times[0]
        out["prefill_ms"] = pre * 1e3
        out["prefill_tok_s"] = prompt / pre

        # decode: all sequences advance one token per step
        def step():
            if eng.hybrid:
                eng.step_logits(seqs, [[1]] * batch, [[0]] * batch)
                return
            from .. import ops
            max_q, max_ctx, host = eng._meta(seqs, [[1]] * batch, True, batch, ops.mpad_for(batch))
            host["mask_rows"] = np.zeros(batch, np.int32)
            d = eng._to_device(host)
            eng._forward_sample(eng._build_meta(d, max_q, max_ctx, True), d["mask_rows"])
        dt = _time(step, eng.device, steps)
        out["decode_ms"] = dt * 1e3
        out["decode_tok_s"] = batch / dt
    for s in seqs:
        eng.close_sequence(s)
    return out


def run(args) -> int:
    dev = torch.device("cuda", 0) if torch.cuda.is_available() and not args.cpu_smoke \
        else torch.device("cpu")
    sizes = [s for s in args.lm_sizes.split(",") if s]
    for name in sizes:
        fams = {"pipizen": pipizen_stack, "sodonex": sodonex_stack, "movinex": movinex_stack,
                "vilulix": vilulix_stack, "llama": llama_stack}
        for fam in [f for f in args.lm_families.split(",") if f]:
            cfg = fams[fam](name)
            if dev.type == "cpu":      # plumbing run: tiny stacks
                prompt, batch, steps = 48, 2, 2
            else:
                prompt, batch, steps = args.lm_prompt, args.lm_batch, args.lm_steps
            r = bench_family(cfg, dev, prompt=prompt, batch=batch, steps=steps, seed=args.seed)
            r["size"] = name
            r["dtype"] = "bf16"
            r["data"] = "synthetic"
            print(json.dumps(r), flush=True)
            if dev.type == "cuda":
                torch.cuda.empty_cache()
    return 0
