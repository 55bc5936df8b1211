"""Pipizen: a hybrid decoder-only language model whose config.json lists its
layers one by one. Each layer is a sequence mixer - latent (compressed-KV)
attention with a softmax sink and YaRN-scaled interleaved rotary positions, or
decayed linear ("lightning") attention with a carried per-sequence state -
followed by an optional feed-forward (dense SwiGLU, or a grouped top-k mixture
of experts with identity experts and a shared expert). Every sublayer sits
between two Dynamic-Tanh norms: x <- x + post(sublayer(pre(x))).

MI355X layout, in the manner of the Llama decoder next to it:

* activations are a flat [T, width] token batch (continuous batching: prompt
  portions and single decode tokens of different sequences in one pass); the
  sequence structure lives in the step metadata only;
* the residual stream is f32 and is updated inside the norm launch
  (``ops.dyt_add_norm``: residual += post-norm(sublayer output) and the next
  sublayer's pre-norm in one kernel);
* latent attention runs in the folded form: the per-head key up-projection is
  applied to the query (q_lat = W_uk^T q) and the value up-projection to the
  attention output, so the kernel reads only the cached latent row and the
  shared rotary key part - one key/value stream for all heads, prefill and
  decode alike; a layer with ``kv_from`` reads another layer's pages;
* the lightning state lives in f32 state slots (one per live sequence) and one
  scan kernel serves prompts and decode;
* fused projection weights: q|k|v|g of a lightning layer and gate|up of every
  feed-forward are one GEMM each; the experts' weights are stacked [E, ...] for
  the grouped expert GEMMs.

Plain GEMMs go to the vendor library through ``ops.linear`` / ``torch.bmm``;
everything around them is this repository's HIP.
"""
from __future__ import annotations

import torch

from .. import ops
from ..ops import seqmix
from ..ops.seqmix import DytParams
from .configs import PipizenConfig


def latent_prompt_layout(L: dict, m, dtype, device) -> None:
    """Padded per-head copies for the matrix-core prompt kernel (bf16): the
    query projection ``wq`` with DKp rows per head, W_uk / W_uv producing [H,
    DKp] keys and [H, DVp] values from a latent row, and W_o with DVp columns
    per head. Sizes that the kernel is built for are used as they are. ``L``
    holds ``wq`` [H (D + Dr), n], ``wuk`` [H, D, R], ``wuv_t`` [H, R, Dv] and
    ``wo``; shared by every family with latent attention layers."""
    H, D, Dr, Dv, R = m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank
    sizes = seqmix.prefill_head_sizes(D + Dr, Dv) if dtype == torch.bfloat16 else None
    if sizes is None or torch.device(device).type != "cuda":
        return
    DKp, DVp = sizes
    dev, dt = device, dtype

    def pad_rows(w, per, to):       # [H * per, n] -> [H * to, n], zero rows after each head
        if per == to:
            return w
        out = torch.zeros(H, to, w.shape[1], dtype=dt, device=dev)
        out[:, :per] = w.view(H, per, -1)
        return out.view(H * to, -1).contiguous()
    L["wq"], L["qw"] = pad_rows(L["wq"], D + Dr, DKp), DKp
    L["wuk_p"] = pad_rows(L["wuk"].reshape(H * D, R), D, DKp)
    L["wuv_p"] = pad_rows(L["wuv_t"].transpose(1, 2).reshape(H * Dv, R), Dv, DVp)
    L["wo_p"] = L["wo"] if DVp == Dv else \
        pad_rows(L["wo"].t().contiguous(), Dv, DVp).t().contiguous()
    L["prompt_sizes"] = (DKp, DVp)


def latent_mix(L: dict, m, q: torch.Tensor, z: torch.Tensor | None, pages: torch.Tensor, meta,
               eps: float, prompt_min_q: int, gate: torch.Tensor | None = None) -> torch.Tensor:
    """Latent attention of one step after its projections, for every family
    that has such layers. q [T, H * qw]: the projected queries (per head D
    unrotated then Dr rotary entries, possibly padded to ``L["qw"]``); z [T, R +
    Dr]: the projected latent and shared rotary key part, appended to ``pages``
    here (None: the pages belong to another layer and are complete). ``gate``
    [T, H Dv] multiplies the heads' outputs by sigmoid(gate) before the output
    projection. Returns the mixer's output [T, width]."""
    H, D, Dr, Dv, R = m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank
    T = q.shape[0]
    if z is not None:
        seqmix.latent_append(z, L["dkv_norm"], eps, meta.positions, L["cos_sin"], pages,
                             meta.slots, R, m.rot.dims)
    q = q.view(T, H, L["qw"])
    if "prompt_sizes" in L and meta.max_q >= prompt_min_q and meta.cu_k is not None:
        # prompt pass: per-head keys / values from the gathered latents, then
        # flash attention on the matrix cores
        DKp, DVp = L["prompt_sizes"]
        cl, kr = seqmix.latent_gather(pages, meta.block_tables, meta.cu_k, meta.total_k,
                                      meta.max_ctx, R)
        k = ops.linear(cl, L["wuk_p"]).view(-1, H, DKp)
        seqmix.latent_kfill_(k, kr, D)
        v = ops.linear(cl, L["wuv_p"]).view(-1, H, DVp)
        seqmix.rope_pairs_(q, D, m.rot.dims, meta.positions, L["cos_sin"])
        o = seqmix.latent_prefill(q, k, v, meta.cu_q, meta.cu_k, meta.positions, L["sink"],
                                  m.scale, meta.max_q)
        if gate is not None:
            seqmix.sigmoid_gate_(o.view(T, H, DVp), gate, H, Dv)
        return ops.linear(o, L["wo_p"])
    qa = torch.bmm(q[:, :, :D].transpose(0, 1), L["wuk"])            # [H, T, R]
    lat = seqmix.latent_attention(qa, q[:, :, D:D + Dr], pages, meta.cu_q, meta.ctx_lens,
                                  meta.block_tables, meta.positions, L["cos_sin"], L["sink"],
                                  m.scale, R, m.rot.dims, meta.max_ctx)
    o = torch.bmm(lat, L["wuv_t"]).transpose(0, 1).reshape(T, H * Dv)     # [T, H Dv]
    if gate is not None:
        seqmix.sigmoid_gate_(o.view(T, H, Dv), gate, H, Dv)
    return ops.linear(o, L["wo"])


class PipizenWeights:
    """Device weights in the fused layouts, from a state dict in checkpoint
    naming (``embed``, ``l<i>.norm1[.b|.alpha]``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
    ``final.norm``, ``head``)."""

    def __init__(self, cfg: PipizenConfig, sd: dict, device, dtype=torch.bfloat16,
                 max_positions: int = 8192):
        self.cfg, self.dtype, self.device = cfg, dtype, torch.device(device)
        self.max_positions = max_positions
        dev = self.device

        def W(name):            # a projection matrix in the activation dtype
            return sd[name].to(dev, dtype).contiguous()

        def F(name):            # small vectors the f32 paths read
            return sd[name].to(dev, torch.float32).contiguous()

        def norm(name):
            return DytParams(F(name), F(name + ".b"), float(sd[name + ".alpha"].float()))

        self.embed = W("embed")
        self.head = sd["head"].to(dev, torch.float32).contiguous()
        self.final_norm = norm("final.norm")
        self._tables: dict[tuple, torch.Tensor] = {}
        self.layers: list[dict] = []
        for i, lc in enumerate(cfg.layers):
            p, m = f"l{i}.", lc.mixer
            L: dict = {"norm1": norm(p + "norm1"), "norm1b": norm(p + "norm1b")}
            if lc.kind == "latent_attention":
                H, D, Dr, Dv, R = m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank
                L["wq"] = W(p + "mix.q")
                assert L["wq"].shape[0] == H * (D + Dr)
                L["qw"] = D + Dr          # per-head width of the query projection
                if m.kv_from is None:
                    L["wdkv"] = W(p + "mix.dkv")
                    L["dkv_norm"] = F(p + "mix.dkv.norm")
                    assert L["wdkv"].shape[0] == R + Dr
                # folded up-projections: [H, D, R] for the queries, [H, R, Dv]
                # for the attention output
                L["wuk"] = W(p + "mix.uk").view(H, D, R).contiguous()
                L["wuv_t"] = W(p + "mix.uv").view(H, Dv, R).transpose(1, 2).contiguous()
                L["sink"] = F(p + "mix.sink") if (p + "mix.sink") in sd else None
                L["wo"] = W(p + "mix.o")
                L["cos_sin"] = self._table(m.rot)
                self._prompt_layout(L, m)
            else:
                L["wqkvg"] = torch.cat([W(p + "mix.q"), W(p + "mix.k"), W(p + "mix.v"),
                                        W(p + "mix.g")]).contiguous()
                L["norm"] = F(p + "mix.norm")
                L["wo"] = W(p + "mix.o")
                L["decay"] = torch.tensor(m.decay, dtype=torch.float32, device=dev)
            f = lc.mlp
            if f is not None:
                L["norm2"], L["norm2b"] = norm(p + "norm2"), norm(p + "norm2b")
                if f.kind == "dense":
                    L["w_gate_up"] = torch.cat([W(p + "mlp.gate"), W(p + "mlp.up")]).contiguous()
                    L["w_down"] = W(p + "mlp.down")
                else:
                    L["router"] = F(p + "mlp.router")
                    L["correction"] = F(p + "mlp.correction") if (p + "mlp.correction") in sd else None
                    assert L["router"].shape[0] == f.experts + f.identity
                    L["e_gate_up"] = torch.stack([
                        torch.cat([W(f"{p}mlp.e{e}.gate"), W(f"{p}mlp.e{e}.up")])
                        for e in range(f.experts)]).contiguous()
                    L["e_down"] = torch.stack([W(f"{p}mlp.e{e}.down")
                                               for e in range(f.experts)]).contiguous()
                    if f.shared_ff:
                        L["s_gate_up"] = torch.cat([W(p + "mlp.shared.gate"),
                                                    W(p + "mlp.shared.up")]).contiguous()
                        L["s_down"] = W(p + "mlp.shared.down")
            self.layers.append(L)

    def _prompt_layout(self, L: dict, m) -> None:
        latent_prompt_layout(L, m, self.dtype, self.device)

    def _table(self, rot) -> torch.Tensor:
        key = (rot.dims, rot.base, rot.yarn)
        if key not in self._tables:
            self._tables[key] = seqmix.rope_table_pairs(rot.dims, self.max_positions, rot.base,
                                                        rot.yarn, self.device)
        return self._tables[key]

    @classmethod
    def random(cls, cfg: PipizenConfig, device, seed: int = 0, dtype=torch.bfloat16,
               max_positions: int = 8192) -> "PipizenWeights":
        return cls(cfg, random_state_dict(cfg, seed), device, dtype, max_positions)


def random_state_dict(cfg: PipizenConfig, seed: int = 0) -> dict:
    """Seeded random weights in checkpoint naming (bf16 matrices), scaled so
    activations stay O(1) through the stack; used by tests, smoke and bench."""
    g = torch.Generator().manual_seed(seed)
    d = cfg.d_model
    sd: dict = {}

    def mat(name, rows, cols, gain=1.0):
        sd[name] = (torch.randn(rows, cols, generator=g) * gain / cols ** 0.5).to(torch.bfloat16)

    def vec(name, n, mean=0.0, std=0.1):
        sd[name] = (mean + torch.randn(n, generator=g) * std).to(torch.bfloat16)

    def norm(name):
        vec(name, d, 1.0)
        vec(name + ".b", d, 0.0, 0.05)
        sd[name + ".alpha"] = torch.tensor(0.5 + 0.5 * torch.rand((), generator=g).item(),
                                           dtype=torch.bfloat16)

    sd["embed"] = torch.randn(cfg.vocab_size, d, generator=g).to(torch.bfloat16)
    for i, lc in enumerate(cfg.layers):
        p, m = f"l{i}.", lc.mixer
        norm(p + "norm1"); norm(p + "norm1b")
        if lc.kind == "latent_attention":
            mat(p + "mix.q", m.heads * (m.dim + m.rot_dim), d, 2.0)
            if m.kv_from is None:
                mat(p + "mix.dkv", m.kv_rank + m.rot_dim, d, 2.0)
                vec(p + "mix.dkv.norm", m.kv_rank, 1.0)
            mat(p + "mix.uk", m.heads * m.dim, m.kv_rank, 2.0)
            mat(p + "mix.uv", m.heads * m.vdim, m.kv_rank, 2.0)
            vec(p + "mix.sink", m.heads, 0.0, 1.0)
            mat(p + "mix.o", d, m.heads * m.vdim, 2.0)
        else:
            mat(p + "mix.q", m.heads * m.dim, d)
            mat(p + "mix.k", m.heads * m.dim, d)
            mat(p + "mix.v", m.heads * m.vdim, d, 2.0)
            mat(p + "mix.g", m.heads * m.vdim, d)
            vec(p + "mix.norm", m.heads * m.vdim, 1.0)
            mat(p + "mix.o", d, m.heads * m.vdim, 2.0)
        f = lc.mlp
        if f is None:
            continue
        norm(p + "norm2"); norm(p + "norm2b")
        if f.kind == "dense":
            mat(p + "mlp.gate", f.ff, d, 2.0); mat(p + "mlp.up", f.ff, d, 2.0)
            mat(p + "mlp.down", d, f.ff, 2.0)
        else:
            for e in range(f.experts):
                mat(f"{p}mlp.e{e}.gate", f.ff, d, 2.0); mat(f"{p}mlp.e{e}.up", f.ff, d, 2.0)
                mat(f"{p}mlp.e{e}.down", d, f.ff, 4.0)
            mat(p + "mlp.router", f.experts + f.identity, d, 3.0)
            vec(p + "mlp.correction", f.experts + f.identity, 0.0, 0.05)
            if f.shared_ff:
                mat(p + "mlp.shared.gate", f.shared_ff, d, 2.0)
                mat(p + "mlp.shared.up", f.shared_ff, d, 2.0)
                mat(p + "mlp.shared.down", d, f.shared_ff, 2.0)
    norm("final.norm")
    mat("head", cfg.vocab_size, d, 2.0)
    return sd


def config_to_json(cfg: PipizenConfig) -> dict:
    """The config.json of ``cfg`` (the inverse of ``pipizen_config_from_json``)."""
    layers = []
    for lc in cfg.layers:
        m = lc.mixer
        if lc.kind == "latent_attention":
            rot = {"dims": m.rot.dims, "base": m.rot.base}
            if m.rot.yarn is not None:
                rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), m.rot.yarn))
            mx = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim,
                  "kv_rank": m.kv_rank, "scale": m.scale, "rot": rot}
            if m.kv_from is not None:
                mx["kv_from"] = m.kv_from
        else:
            mx = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "decay": list(m.decay)}
        f = lc.mlp
        if f is None:
            mlp = None
        elif f.kind == "dense":
            mlp = {"kind": "dense", "ff": f.ff}
        else:
            mlp = {"kind": "moe", "expert": {"ff": f.ff},
                   "router": {"experts": f.experts, "identity": f.identity, "top": f.top,
                              "groups": {"count": f.groups, "keep": f.keep}}}
            if f.shared_ff:
                mlp["shared"] = {"ff": f.shared_ff}
        layers.append({"type": lc.kind, "mixer": mx, "mlp": mlp})
    return {"architecture": "Pipizen", "vocab": cfg.vocab_size, "width": cfg.d_model,
            "norm": {"eps": cfg.norm_eps}, "layers": layers}


class PipizenModel:
    """The step function: one pass of a flat token batch through all layers,
    reading and extending the paged latent cache and the state slots."""

    hybrid = True
    # a step whose longest feed has at least this many tokens takes the
    # matrix-core prompt path of latent attention (bf16 on the GPU); shorter
    # feeds (decode, short tails) read the latent pages directly
    prompt_min_q = 32

    def __init__(self, w: PipizenWeights):
        self.w, self.cfg = w, w.cfg

    # the cache manager sizes its storage from this
    def cache_spec(self) -> dict:
        latent, state = {}, {}
        for i, lc in enumerate(self.cfg.layers):
            m = lc.mixer
            if lc.kind == "latent_attention":
                if m.kv_from is None:
                    latent[i] = m.kv_rank + m.rot_dim
            else:
                state[i] = (m.heads, m.dim, m.vdim)
        return {"latent": latent, "state": state}

    def embed(self, tokens: torch.Tensor) -> torch.Tensor:
        return torch.nn.functional.embedding(tokens.long(), self.w.embed).float()

    def forward(self, meta, cache) -> torch.Tensor:
        """f32 logits [len(meta.logit_idx), vocab] of one step. ``meta``: the
        engine's StepMeta (tokens, positions, slots, cu_q, ctx_lens,
        block_tables, state_slots, logit_idx); ``cache``: a HybridCache."""
        w, cfg, dt = self.w, self.cfg, self.w.dtype
        x = self.embed(meta.tokens).contiguous()
        T = x.shape[0]
        h = seqmix.dyt_norm(x, w.layers[0]["norm1"], dt) if w.layers else None
        n = len(w.layers)
        for i, (lc, L) in enumerate(zip(cfg.layers, w.layers)):
            m = lc.mixer
            if lc.kind == "latent_attention":
                y = self._latent(i, m, L, h, meta, cache, T)
            else:
                y = self._lightning(i, m, L, h, meta, cache)
            nxt_layer = w.layers[i + 1]["norm1"] if i + 1 < n else None
            if lc.mlp is None:
                h = seqmix.dyt_add_norm(x, y, L["norm1b"], nxt_layer, dt)
                continue
            h = seqmix.dyt_add_norm(x, y, L["norm1b"], L["norm2"], dt)
            y = self._dense(h, L["w_gate_up"], L["w_down"]) if lc.mlp.kind == "dense" else \
                self._moe(lc.mlp, L, h)
            h = seqmix.dyt_add_norm(x, y, L["norm2b"], nxt_layer, dt)
        hf = seqmix.dyt_norm(x, w.final_norm, torch.float32, row_idx=meta.logit_idx)
        return ops.linear(hf, w.head)

    def _latent(self, i, m, L, h, meta, cache, T) -> torch.Tensor:
        src = i if m.kv_from is None else m.kv_from
        z = ops.linear(h, L["wdkv"]) if m.kv_from is None else None
        return latent_mix(L, m, ops.linear(h, L["wq"]), z, cache.latent[src], meta,
                          self.cfg.norm_eps, self.prompt_min_q)

    def _lightning(self, i, m, L, h, meta, cache) -> torch.Tensor:
        H, D, Dv = m.heads, m.dim, m.vdim
        qkvg = ops.linear(h, L["wqkvg"])
        o = seqmix.lightning_scan(qkvg, H, D, Dv, cache.state[i], meta.state_slots, meta.cu_q,
                                  meta.positions, L["decay"])
        y = seqmix.gated_rmsnorm(o, L["norm"], qkvg[:, 2 * H * D + H * Dv:], self.cfg.norm_eps,
                                 self.w.dtype)
        return ops.linear(y, L["wo"])

    @staticmethod
    def _dense(h, w_gate_up, w_down) -> torch.Tensor:
        return ops.linear(seqmix.silu_mul_any(ops.linear(h, w_gate_up)), w_down)

    def _moe(self, f, L, h) -> torch.Tensor:
        z = ops.linear(h.float(), L["router"])
        idx, wt = seqmix.moe_route(z, L["correction"], f.groups, f.keep, f.top)
        out = seqmix.moe_experts(h, idx, wt, L["e_gate_up"], L["e_down"])
        if f.shared_ff:
            out += self._dense(h, L["s_gate_up"], L["s_down"])
        return out
