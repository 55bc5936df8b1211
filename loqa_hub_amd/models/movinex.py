"""Movinex: a pre-norm decoder-only language model whose config.json lists its
layers one by one; a stretch of layers may run several times in a row with
the same weights (every run with a cache or state of its own), each pass
entered through a projection of [x ; embedding output]. A layer is

    x <- x + ls1 * mixer(norm1(x))        x <- x + ls2 * ff(norm2(x))

with RMS norms whose weights are stored around zero (x / rms(x) * (1 + w)) and
a learned per-coordinate scale on each sublayer's output. Mixers:

* ``attention``: grouped-query softmax attention, q / k / v projections with
  biases, q and k divided by their root mean square per head, a query
  temperature that grows with the logarithm of the position, full causal mask;
* ``attention_2``: no value projection (the values are the keys as projected),
  interleaved rotary positions on the first ``rot.dims`` entries of each head,
  then the per-head RMS division, scores soft-capped by a tanh, a sliding
  window that also keeps the first tokens of the sequence, and an output gate
  sigmoid(W_g h) per entry before the output projection;
* ``mamba2``: a state-space layer - one input projection laid out as z | x | B
  | C | dt, a short causal convolution with SiLU on x | B | C, the recurrence
  S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x per head (B and C
  shared by groups of heads), the gate silu(z) BEFORE a grouped RMS norm.

Feed-forwards: dense GeGLU (tanh form), or a mixture of SwiGLU experts routed
by sigmoid scores (groups of neighbouring experts rank by the sum of their two
best scores, only the best groups are eligible, weights = the plain scores).

MI355X layout, in the manner of the other decoders: a flat [T, width] token
batch (prompt portions beside decode tokens), an f32 residual stream updated
inside the norm launch, fused projection matrices (q | k | v, q | k | gate,
gate | up), K / V pages on the shared block pool and the recurrent state and
convolution tails in f32 state slots, one set per layer RUN. Plain GEMMs go to
the vendor library; everything around them is this repository's HIP
(``ops/seqmix.py``).
"""
from __future__ import annotations

import torch

from .. import ops
from ..ops import seqmix
from .configs import MovinexConfig


class MovinexWeights:
    """Device weights in the fused layouts, from a state dict in checkpoint
    naming (``embed``, ``loop.in``, ``l<i>.norm1|norm2|ls1|ls2``,
    ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``, ``head``)."""

    def __init__(self, cfg: MovinexConfig, sd: dict, device, dtype=torch.bfloat16,
                 max_positions: int = 8192):
        self.cfg, self.dtype, self.device = cfg, dtype, torch.device(device)
        self.max_positions = max_positions
        dev = self.device

        def W(name):            # a projection matrix in the activation dtype
            return sd[name].to(dev, dtype).contiguous()

        def F(name):            # small vectors the f32 paths read
            return sd[name].to(dev, torch.float32).contiguous()

        d = cfg.d_model
        self.embed = F("embed")
        if self.embed.shape != (cfg.vocab_size, d):
            raise ValueError("embed does not match vocab x width")
        self.head = F("head")
        self.final_norm = F("final.norm")
        self.loop_in = None
        if cfg.loop is not None:
            self.loop_in = W("loop.in")
            if self.loop_in.shape != (d, 2 * d):
                raise ValueError("loop.in does not match width x 2 width")
        self._tables: dict[tuple, torch.Tensor] = {}
        self.layers: list[dict] = []
        for i, lc in enumerate(cfg.layers):
            p, m = f"l{i}.", lc.mixer
            L: dict = {"norm1": F(p + "norm1"), "ls1": F(p + "ls1")}
            if lc.kind == "mamba2":
                self._mamba2(L, p, m, sd, W, F)
            else:
                self._attention(L, p, m, W)
            f = lc.mlp
            if f is not None:
                L["norm2"], L["ls2"] = F(p + "norm2"), F(p + "ls2")
                if f.kind == "dense":
                    L["w_gate_up"] = torch.cat([W(p + "mlp.gate"), W(p + "mlp.up")]).contiguous()
                    L["w_down"] = W(p + "mlp.down")
                    if L["w_gate_up"].shape != (2 * f.ff, d) or L["w_down"].shape != (d, f.ff):
                        raise ValueError(f"layer {i}: feed-forward shapes do not match the config")
                else:
                    L["router"] = F(p + "mlp.router")
                    if L["router"].shape != (f.experts, d):
                        raise ValueError(f"layer {i}: router does not match the config")
                    L["e_gate_up"] = torch.stack([
                        torch.cat([W(f"{p}mlp.e{e}.gate"), W(f"{p}mlp.e{e}.up")])
                        for e in range(f.experts)]).contiguous()
                    L["e_down"] = torch.stack([W(f"{p}mlp.e{e}.down")
                                               for e in range(f.experts)]).contiguous()
                    if L["e_gate_up"].shape != (f.experts, 2 * f.ff, d):
                        raise ValueError(f"layer {i}: expert shapes do not match the config")
            self.layers.append(L)

    def _attention(self, L: dict, p: str, m, W) -> None:
        d, dev, dt = self.cfg.d_model, self.device, self.dtype
        H, G, D, Dv = m.heads, m.kv_heads, m.dim, m.vdim
        parts = [W(p + "mix.q"), W(p + "mix.k")]
        if parts[0].shape != (H * D, d) or parts[1].shape != (G * D, d):
            raise ValueError(f"{p}: projection shapes do not match the config")
        if not m.values_from_keys:
            parts.append(W(p + "mix.v"))
            if parts[-1].shape != (G * Dv, d):
                raise ValueError(f"{p}: value projection does not match the config")
        if m.gate:
            parts.append(W(p + "mix.g"))
            if parts[-1].shape != (H * Dv, d):
                raise ValueError(f"{p}: gate projection does not match the config")
        # q | k (| v) (| gate) rows as ONE projection; zero rows pad its output
        # to a multiple of 8 columns so that its rows stay 16-byte aligned
        n = sum(w.shape[0] for w in parts)
        pad = -n % 8
        if pad:
            parts.append(torch.zeros(pad, d, dtype=dt, device=dev))
        L["w_in"] = torch.cat(parts).contiguous()
        L["b_in"] = None
        if m.bias:
            bs = [W(p + "mix.q.b"), W(p + "mix.k.b"), W(p + "mix.v.b")]
            L["b_in"] = torch.cat(bs + [torch.zeros(pad, dtype=dt, device=dev)]).contiguous()
        L["v_off"] = -1 if m.values_from_keys else (H + G) * D
        L["g_off"] = (H + G) * D + (0 if m.values_from_keys else G * Dv)
        L["wo"] = W(p + "mix.o")
        if L["wo"].shape != (d, H * Dv):
            raise ValueError(f"{p}: output projection does not match the config")
        L["cos_sin"] = self._table(m.rot) if m.rot is not None and m.rot.dims else None

    def _mamba2(self, L: dict, p: str, m, sd, W, F) -> None:
        d = self.cfg.d_model
        C = m.conv_channels
        L["w_in"] = W(p + "mix.in")
        if L["w_in"].shape != (2 * m.inner + 2 * m.groups * m.state + m.heads, d):
            raise ValueError(f"{p}: input projection does not match the config")
        conv = F(p + "mix.conv")
        if conv.shape != (C, m.taps):
            raise ValueError(f"{p}: convolution weights do not match the config")
        L["conv"] = conv.t().contiguous()                     # tap-major [taps, C]
        L["conv_b"] = F(p + "mix.conv.b")
        L["dt_bias"] = F(p + "mix.dt_bias")
        L["a_neg"] = -torch.exp(F(p + "mix.A_log"))            # the decay exponent per head
        L["skip"] = F(p + "mix.D")
        L["norm"] = F(p + "mix.norm")
        L["wo"] = W(p + "mix.o")
        if L["wo"].shape != (d, m.inner) or L["norm"].numel() != m.inner:
            raise ValueError(f"{p}: output projection does not match the config")

    def _table(self, rot) -> torch.Tensor:
        key = (rot.dims, rot.base)
        if key not in self._tables:
            self._tables[key] = seqmix.rope_table_pairs(rot.dims, self.max_positions, rot.base,
                                                        None, self.device)
        return self._tables[key]

    @classmethod
    def random(cls, cfg: MovinexConfig, device, seed: int = 0, dtype=torch.bfloat16,
               max_positions: int = 8192) -> "MovinexWeights":
        return cls(cfg, random_state_dict(cfg, seed), device, dtype, max_positions)


def random_state_dict(cfg: MovinexConfig, seed: int = 0) -> dict:
    """Seeded random weights in checkpoint naming (bf16), scaled so that
    activations stay O(1) through the stack; used by tests, smoke and bench."""
    g = torch.Generator().manual_seed(seed)
    d = cfg.d_model
    sd: dict = {}

    def mat(name, rows, cols, gain=1.0):
        sd[name] = (torch.randn(rows, cols, generator=g) * gain / cols ** 0.5).to(torch.bfloat16)

    def vec(name, n, mean=0.0, std=0.1):
        sd[name] = (mean + torch.randn(n, generator=g) * std).to(torch.bfloat16)

    sd["embed"] = torch.randn(cfg.vocab_size, d, generator=g).to(torch.bfloat16)
    if cfg.loop is not None:
        mat("loop.in", d, 2 * d, 1.4)
    for i, lc in enumerate(cfg.layers):
        p, m = f"l{i}.", lc.mixer
        vec(p + "norm1", d)
        vec(p + "ls1", d, 0.6, 0.2)
        if lc.kind == "mamba2":
            C = m.conv_channels
            mat(p + "mix.in", 2 * m.inner + 2 * m.groups * m.state + m.heads, d, 1.5)
            sd[p + "mix.conv"] = (torch.randn(C, m.taps, generator=g) * 0.5).to(torch.bfloat16)
            vec(p + "mix.conv.b", C)
            vec(p + "mix.dt_bias", m.heads, -1.0, 0.5)
            vec(p + "mix.A_log", m.heads, -0.5, 0.7)
            vec(p + "mix.D", m.heads, 1.0, 0.3)
            vec(p + "mix.norm", m.inner, 1.0)
            mat(p + "mix.o", d, m.inner, 2.0)
        else:
            H, G, D, Dv = m.heads, m.kv_heads, m.dim, m.vdim
            mat(p + "mix.q", H * D, d, 2.0)
            mat(p + "mix.k", G * D, d, 2.0)
            if m.bias:
                vec(p + "mix.q.b", H * D); vec(p + "mix.k.b", G * D); vec(p + "mix.v.b", G * Dv)
            if not m.values_from_keys:
                mat(p + "mix.v", G * Dv, d, 2.0)
            if m.gate:
                mat(p + "mix.g", H * Dv, d, 2.0)
            mat(p + "mix.o", d, H * Dv, 2.0)
        f = lc.mlp
        if f is None:
            continue
        vec(p + "norm2", d)
        vec(p + "ls2", d, 0.6, 0.2)
        if f.kind == "dense":
            mat(p + "mlp.gate", f.ff, d, 2.0); mat(p + "mlp.up", f.ff, d, 2.0)
            mat(p + "mlp.down", d, f.ff, 2.0)
        else:
            for e in range(f.experts):
                mat(f"{p}mlp.e{e}.gate", f.ff, d, 2.0); mat(f"{p}mlp.e{e}.up", f.ff, d, 2.0)
                mat(f"{p}mlp.e{e}.down", d, f.ff, 3.0)
            mat(p + "mlp.router", f.experts, d, 3.0)
    vec("final.norm", d)
    mat("head", cfg.vocab_size, d, 2.0)
    return sd


def config_to_json(cfg: MovinexConfig) -> dict:
    """The config.json of ``cfg`` (the inverse of ``movinex_config_from_json``)."""
    layers = []
    for lc in cfg.layers:
        m, f = lc.mixer, lc.mlp
        if lc.kind == "mamba2":
            mx = {"heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups,
                  "conv": m.taps, "norm_groups": m.norm_groups}
        else:
            mx = {"heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim,
                  "scale": m.scale}
            if m.rot is not None:
                mx["rot"] = {"dims": m.rot.dims, "base": m.rot.base}
            if m.q_temp is not None:
                mx["q_temp"] = {"coef": m.q_temp[0], "every": m.q_temp[1]}
            if m.softcap:
                mx["softcap"] = m.softcap
            if m.window:
                mx["mask"] = {"size": m.window, "keep_first": m.keep_first}
        if f is None:
            mlp = None
        elif f.kind == "dense":
            mlp = {"kind": "dense", "ff": f.ff}
        else:
            mlp = {"kind": "moe", "expert": {"ff": f.ff},
                   "router": {"experts": f.experts, "top": f.top,
                              "groups": {"count": f.groups, "keep": f.keep}}}
        layers.append({"type": lc.kind, "mixer": mx, "mlp": mlp})
    out = {"architecture": "Movinex", "vocab": cfg.vocab_size, "width": cfg.d_model,
           "norm": {"eps": cfg.norm_eps}, "logit_scale": cfg.logit_scale, "layers": layers}
    if cfg.loop is not None:
        out["loop"] = {"start": cfg.loop.start, "stop": cfg.loop.stop, "times": cfg.loop.times}
    return out


class MovinexModel:
    """The step function: one pass of a flat token batch through all layer
    runs, reading and extending the paged K / V cache and the state slots."""

    hybrid = True

    def __init__(self, w: MovinexWeights):
        self.w, self.cfg = w, w.cfg
        self.runs = self.cfg.runs()

    # the cache manager sizes its storage from this: one entry per layer RUN
    # (a layer of the repeated stretch holds a cache or state per pass)
    def cache_spec(self) -> dict:
        kv, state, rows = {}, {}, {}
        for r, (i, _) in enumerate(self.runs):
            lc = self.cfg.layers[i]
            m = lc.mixer
            if lc.kind == "mamba2":
                state[r] = (m.heads, m.state, m.vdim)
                if m.taps > 1:
                    rows[r] = {"tail": (m.taps - 1, m.conv_channels)}
            else:
                kv[r] = (m.kv_heads * m.dim, m.kv_heads * m.vdim)
        return {"latent": {}, "state": state, "kv_rows": kv, "rows": rows}

    def embed(self, tokens: torch.Tensor) -> torch.Tensor:
        return torch.nn.functional.embedding(tokens.long(), self.w.embed)

    def forward(self, meta, cache, trail: list | None = None) -> torch.Tensor:
        """f32 logits [len(meta.logit_idx), vocab] of one step. ``meta``: the
        engine's StepMeta; ``cache``: a HybridCache. ``trail`` collects the
        residual stream after every layer run (tests)."""
        w, cfg, dt = self.w, self.cfg, self.w.dtype
        eps = cfg.norm_eps
        x0 = self.embed(meta.tokens).contiguous()
        x = x0.clone() if cfg.loop is not None else x0
        h = None
        n = len(self.runs)
        for r, (i, first) in enumerate(self.runs):
            lc, L = cfg.layers[i], w.layers[i]
            if first:
                # a pass of the repeated stretch enters through W_in [x ; x0]
                x = ops.linear(torch.cat([x, x0], dim=1).to(dt), w.loop_in).float()
                h = None
            if h is None:
                h = seqmix.rms1p_norm(x, L["norm1"], eps, dt)
            if lc.kind == "mamba2":
                y = self._mamba2(r, lc.mixer, L, h, meta, cache)
            else:
                y = self._attention(r, lc.mixer, L, h, meta, cache)
            nxt = None
            if r + 1 < n and not self.runs[r + 1][1]:
                nxt = w.layers[self.runs[r + 1][0]]["norm1"]
            f = lc.mlp
            if f is None:
                h = seqmix.scaled_add_rms1p(x, y, L["ls1"], nxt, eps, dt)
            else:
                h = seqmix.scaled_add_rms1p(x, y, L["ls1"], L["norm2"], eps, dt)
                y = self._dense(h, L) if f.kind == "dense" else self._moe(f, L, h)
                h = seqmix.scaled_add_rms1p(x, y, L["ls2"], nxt, eps, dt)
            if trail is not None:
                trail.append(x.clone())
        hf = seqmix.rms1p_norm(x, w.final_norm, eps, torch.float32, row_idx=meta.logit_idx)
        return ops.linear(hf, w.head) * cfg.logit_scale

    def _attention(self, r, m, L, h, meta, cache) -> torch.Tensor:
        H, G, D, Dv = m.heads, m.kv_heads, m.dim, m.vdim
        u = ops.linear(h, L["w_in"], L["b_in"])
        kc, vc = cache.kv_rows[r]
        q = seqmix.qk_prep_append(u, H, G, D, Dv, L["v_off"], L["cos_sin"],
                                  m.rot.dims if L["cos_sin"] is not None else 0,
                                  self.cfg.norm_eps, m.q_temp, meta.positions, kc, vc, meta.slots,
                                  self.w.dtype)
        gate = u[:, L["g_off"]:L["g_off"] + H * Dv] if m.gate else None
        o = seqmix.window_attention(q, kc, vc, meta.cu_q, meta.ctx_lens, meta.block_tables,
                                    meta.positions, m.scale, m.softcap, m.window, m.keep_first,
                                    gate, H, G, D, Dv, meta.max_q, max_ctx=meta.max_ctx)
        return ops.linear(o, L["wo"])

    def _mamba2(self, r, m, L, h, meta, cache) -> torch.Tensor:
        Hh, P, N, inner, C = m.heads, m.vdim, m.state, m.inner, m.conv_channels
        u = ops.linear(h, L["w_in"])                  # z | x | B | C | dt
        tail = cache.rows[r]["tail"] if m.taps > 1 else \
            torch.zeros(1, 0, C, dtype=torch.float32, device=u.device)
        xbc, tok = seqmix.mamba2_prep(u, inner, C, inner + C, Hh, L["conv"], L["conv_b"],
                                      L["dt_bias"], L["a_neg"], tail, meta.state_slots, meta.cu_q,
                                      meta.positions)
        if m.taps > 1:
            # every reader of this step's tail is done: store the new rows
            seqmix.seq_state_save(None, u[:, inner:inner + C], None, tail, meta.state_slots,
                                  meta.cu_q, meta.positions)
        GN = m.groups * N
        # q = C, k = B (shared by heads // groups neighbours), v = x scaled by dt
        o = seqmix.state_scan(xbc, Hh, N, P, inner + GN, inner, 0, Hh // m.groups, cache.state[r],
                              meta.state_slots, meta.cu_q, meta.positions, tok=tok, skip=L["skip"])
        y = seqmix.gated_rmsnorm(o, L["norm"], u[:, :inner], self.cfg.norm_eps, self.w.dtype,
                                 groups=m.norm_groups, silu_first=True)
        return ops.linear(y, L["wo"])

    @staticmethod
    def _dense(h, L) -> torch.Tensor:
        return ops.linear(seqmix.act_mul_any(ops.linear(h, L["w_gate_up"]), "gelu_tanh"),
                          L["w_down"])

    @staticmethod
    def _moe(f, L, h) -> torch.Tensor:
        z = ops.linear(h.float(), L["router"])
        idx, wt = seqmix.moe_route(z, None, f.groups, f.keep, f.top, sigmoid=True,
                                   group_rank=f.group_rank)
        return seqmix.moe_experts(h, idx, wt, L["e_gate_up"], L["e_down"])
