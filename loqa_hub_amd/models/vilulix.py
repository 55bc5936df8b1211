"""Vilulix: a decoder-only language model of parallel layers whose config.json
lists its layers one by one:

    x <- x + mixer(norm1(x)) + ff(norm2(x))

with both RMS norms (weights stored around zero, x / rms(x) * (1 + w)) reading
the same x. A stretch of layers may run several times in a row with the same
weights, every run with a cache or state of its own; before each pass but the
first the embedding output is added to x. Mixers:

* ``mlstm``: a matrix memory with exponential gates. Per head a log input gate
  li = cap tanh(z_i / cap) and a log forget gate lf = logsigmoid(cap tanh(z_f /
  cap)), a running maximum m_t = max(lf + m_{t-1}, li) that starts at 0, the
  state S_t = exp(lf + m_{t-1} - m_t) S_{t-1} + exp(li - m_t) k v^T and the
  normaliser n_t likewise with k alone; the read-out S^T q / (max(|n . q|,
  exp(-m_t)) + 1e-6) is divided by its root mean square per head, weighted,
  and gated by sigmoid(W_g h);
* ``latent_attention``: causal softmax attention over a cached latent row and
  one rotary key part shared by all heads, the queries through an RMS-normed
  latent of their own, the heads' outputs times sigmoid(W_g h);
* ``parallel``: two mixers side by side on the same input, their outputs
  added with constant scales - sliding-window grouped-query softmax attention
  (q and k RMS-normed over the whole projection, rotary positions, one more
  term exp(0) in the softmax denominator) and a gated delta rule (short causal
  convolutions with SiLU on q, k, v, unit-length q and k, S <- g S; u = beta (v
  - S^T k); S <- S + k u^T; o = S^T q, a per-head RMS norm gated by silu(W_g h)).

Dense SwiGLU feed-forwards; the logits pass cap tanh(z / cap).

MI355X layout, in the manner of the other decoders: a flat [T, width] token
batch (prompt portions beside decode tokens), an f32 residual stream updated
inside the norm launch that also writes both normed inputs of the next layer,
fused projection matrices (everything that reads one input is one GEMM, the few
gate rows of the recurrences as a small f32 GEMM), latent and K / V pages on
the shared block pool, the recurrent states, running maxima and convolution
tails in f32 state slots, one set per layer RUN. The checkpoint's rotate-half
rotary layout is folded into the interleaved one the kernels read by permuting
projection rows at load time (a dot product does not see a permutation applied
to both of its sides). Plain GEMMs go to the vendor library; everything around
them is this repository's HIP (``ops/seqmix.py``).
"""
from __future__ import annotations

import torch

from .. import ops
from ..ops import seqmix
from .configs import VilulixConfig
from .pipizen import latent_mix, latent_prompt_layout


def _pairs_from_halves(dims: int, size: int) -> torch.Tensor:
    """Index vector over one head of ``size`` entries that brings the
    rotate-half layout (entry i turns with entry i + dims / 2) into the
    interleaved one (2i with 2i + 1): new[2i] = old[i], new[2i + 1] = old[i +
    dims / 2]; entries from ``dims`` on stay."""
    half = dims // 2
    idx = torch.arange(size)
    idx[0:dims:2] = torch.arange(half)
    idx[1:dims:2] = torch.arange(half) + half
    return idx


def _head_rows(heads: int, size: int, off: int, per: torch.Tensor) -> torch.Tensor:
    """Row permutation of a projection laid out head by head (``size`` rows per
    head): within every head the rows off .. off + len(per) move as ``per``."""
    idx = torch.arange(heads * size).view(heads, size).clone()
    idx[:, off:off + per.numel()] = idx[:, off:off + per.numel()][:, per]
    return idx.reshape(-1)


class VilulixWeights:
    """Device weights in the fused layouts, from a state dict in checkpoint
    naming (``embed``, ``l<i>.norm1|norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
    ``final.norm``, ``head``)."""

    def __init__(self, cfg: VilulixConfig, sd: dict, device, dtype=torch.bfloat16,
                 max_positions: int = 8192):
        self.cfg, self.dtype, self.device = cfg, dtype, torch.device(device)
        self.max_positions = max_positions
        dev = self.device

        def W(name):            # a projection matrix in the activation dtype
            return sd[name].to(dev, dtype).contiguous()

        def F(name):            # small vectors and gate rows the f32 paths read
            return sd[name].to(dev, torch.float32).contiguous()

        d = cfg.d_model
        self.embed = F("embed")
        if self.embed.shape != (cfg.vocab_size, d):
            raise ValueError("embed does not match vocab x width")
        self.head = F("head")
        self.final_norm = F("final.norm")
        self._tables: dict[tuple, torch.Tensor] = {}
        self.layers: list[dict] = []
        for i, lc in enumerate(cfg.layers):
            p, m = f"l{i}.", lc.mixer
            L: dict = {"norm1": F(p + "norm1"), "norm2": None}
            if lc.kind == "mlstm":
                self._mlstm(L, p + "mix.", m, W, F)
            elif lc.kind == "latent_attention":
                self._latent(L, p + "mix.", m, W, F)
            else:
                self._parallel(L, p + "mix.", m, W, F)
            f = lc.mlp
            if f is not None:
                L["norm2"] = F(p + "norm2")
                L["w_gate_up"] = torch.cat([W(p + "mlp.gate"), W(p + "mlp.up")]).contiguous()
                L["w_down"] = W(p + "mlp.down")
                if L["w_gate_up"].shape != (2 * f.ff, d) or L["w_down"].shape != (d, f.ff):
                    raise ValueError(f"layer {i}: feed-forward shapes do not match the config")
            self.layers.append(L)

    def _fused(self, parts: list[torch.Tensor]) -> torch.Tensor:
        """Projections of one input as ONE matrix; zero rows pad its output to
        a multiple of 8 columns so that its rows stay 16-byte aligned."""
        n = sum(w.shape[0] for w in parts)
        if -n % 8:
            parts = parts + [torch.zeros(-n % 8, parts[0].shape[1], dtype=self.dtype,
                                         device=self.device)]
        return torch.cat(parts).contiguous()

    def _mlstm(self, L: dict, p: str, m, W, F) -> None:
        d = self.cfg.d_model
        H, D, Dv = m.heads, m.dim, m.vdim
        parts = [W(p + "q"), W(p + "k"), W(p + "v"), W(p + "g")]
        if [w.shape for w in parts] != [(H * D, d)] * 2 + [(H * Dv, d)] * 2:
            raise ValueError(f"{p}: projection shapes do not match the config")
        L["w_in"] = self._fused(parts)
        L["g_off"] = 2 * H * D + H * Dv
        L["w_gates"] = torch.cat([F(p + "i"), F(p + "f")]).contiguous()        # f32 [2 H, d]
        L["i_b"], L["f_b"] = F(p + "i.b"), F(p + "f.b")
        L["norm"] = F(p + "norm")
        L["wo"] = W(p + "o")
        if L["w_gates"].shape != (2 * H, d) or L["norm"].numel() != H * Dv \
                or L["wo"].shape != (d, H * Dv):
            raise ValueError(f"{p}: gate, norm or output shapes do not match the config")

    def _latent(self, L: dict, p: str, m, W, F) -> None:
        d, dev = self.cfg.d_model, self.device
        H, D, Dr, Dv, R, Rq = m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.q_rank
        wdkv, wuq = W(p + "dkv"), W(p + "uq")
        if wdkv.shape != (R + Dr, d) or wuq.shape != (H * (D + Dr), Rq):
            raise ValueError(f"{p}: latent projection shapes do not match the config")
        if m.rot.half and m.rot.dims:
            per = _pairs_from_halves(m.rot.dims, Dr)
            wdkv = torch.cat([wdkv[:R], wdkv[R:][per.to(dev)]]).contiguous()
            wuq = wuq[_head_rows(H, D + Dr, D, per).to(dev)].contiguous()
        parts = [W(p + "dq"), wdkv, W(p + "g")]
        if parts[0].shape != (Rq, d) or parts[2].shape != (H * Dv, d):
            raise ValueError(f"{p}: query latent or gate shapes do not match the config")
        # dq | dkv | gate, each part starting on a 16-byte boundary
        pads = [torch.zeros(-w.shape[0] % 8, d, dtype=self.dtype, device=dev) for w in parts]
        L["z_off"] = Rq + pads[0].shape[0]
        L["g_off"] = L["z_off"] + R + Dr + pads[1].shape[0]
        L["w_in"] = torch.cat([t for w, z in zip(parts, pads) for t in (w, z)]).contiguous()
        L["dq_norm"], L["dkv_norm"] = F(p + "dq.norm"), F(p + "dkv.norm")
        L["wq"], L["qw"] = wuq, D + Dr
        L["wuk"] = W(p + "uk").view(H, D, R).contiguous()
        L["wuv_t"] = W(p + "uv").view(H, Dv, R).transpose(1, 2).contiguous()
        L["sink"] = None
        L["wo"] = W(p + "o")
        if L["wo"].shape != (d, H * Dv) or L["dq_norm"].numel() != Rq \
                or L["dkv_norm"].numel() != R:
            raise ValueError(f"{p}: norm or output shapes do not match the config")
        L["cos_sin"] = self._table(m.rot)
        latent_prompt_layout(L, m, self.dtype, dev)

    def _parallel(self, L: dict, p: str, m, W, F) -> None:
        d, dev = self.cfg.d_model, self.device
        a, r = m.left, m.right
        # left: windowed softmax attention
        q = p + "left."
        H, G, D, Dv = a.heads, a.kv_heads, a.dim, a.vdim
        wq, wk, wv = W(q + "q"), W(q + "k"), W(q + "v")
        qn, kn = F(q + "q.norm"), F(q + "k.norm")
        if (wq.shape, wk.shape, wv.shape) != ((H * D, d), (G * D, d), (G * Dv, d)) \
                or qn.numel() != H * D or kn.numel() != G * D:
            raise ValueError(f"{q}: projection shapes do not match the config")
        if a.rot is not None and a.rot.half and a.rot.dims:
            per = _pairs_from_halves(a.rot.dims, D)
            iq, ik = _head_rows(H, D, 0, per[:a.rot.dims]).to(dev), \
                _head_rows(G, D, 0, per[:a.rot.dims]).to(dev)
            wq, wk, qn, kn = wq[iq].contiguous(), wk[ik].contiguous(), qn[iq].contiguous(), \
                kn[ik].contiguous()
        left = self._fused([wq, wk, wv])
        L["l_q_norm"], L["l_k_norm"] = qn, kn
        L["l_v_off"] = (H + G) * D
        L["l_wo"] = W(q + "o")
        L["l_cos_sin"] = self._table(a.rot) if a.rot is not None and a.rot.dims else None
        L["l_sink"] = torch.zeros(H, dtype=torch.float32, device=dev) if a.zero_sink else None
        # right: gated delta rule
        q = p + "right."
        H, G, D, Dv = r.heads, r.kv_heads, r.dim, r.vdim
        parts = [W(q + "q"), W(q + "k"), W(q + "v"), W(q + "g")]
        if [w.shape for w in parts] != [(G * D, d)] * 2 + [(H * Dv, d)] * 2:
            raise ValueError(f"{q}: projection shapes do not match the config")
        right = self._fused(parts)
        L["r_off"] = left.shape[0]
        L["w_in"] = torch.cat([left, right]).contiguous()
        L["r_gates"] = torch.cat([F(q + "b"), F(q + "a")]).contiguous()         # f32 [2 H, d]
        conv = torch.cat([F(q + "q.conv"), F(q + "k.conv"), F(q + "v.conv")])
        if conv.shape != (r.conv_channels, r.taps) or L["r_gates"].shape != (2 * H, d):
            raise ValueError(f"{q}: convolution or gate shapes do not match the config")
        L["r_conv"] = conv.t().contiguous()                        # tap-major [taps, C]
        L["r_a_neg"] = -torch.exp(F(q + "A_log"))
        L["r_dt_bias"] = F(q + "dt_bias")
        L["r_norm"] = F(q + "norm").repeat(H).contiguous()         # shared by the heads
        L["r_wo"] = W(q + "o")
        if L["r_wo"].shape != (d, H * Dv) or L["l_wo"].shape != (d, a.heads * a.vdim) \
                or L["r_norm"].numel() != H * Dv or L["r_a_neg"].numel() != H:
            raise ValueError(f"{p}: norm or output shapes do not match the config")

    def _table(self, rot) -> torch.Tensor:
        key = (rot.dims, rot.base)
        if key not in self._tables:
            self._tables[key] = seqmix.rope_table_pairs(rot.dims, self.max_positions, rot.base,
                                                        None, self.device)
        return self._tables[key]

    @classmethod
    def random(cls, cfg: VilulixConfig, device, seed: int = 0, dtype=torch.bfloat16,
               max_positions: int = 8192) -> "VilulixWeights":
        return cls(cfg, random_state_dict(cfg, seed), device, dtype, max_positions)


def random_state_dict(cfg: VilulixConfig, seed: int = 0) -> dict:
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
    for i, lc in enumerate(cfg.layers):
        p, m = f"l{i}.", lc.mixer
        vec(p + "norm1", d)
        if lc.kind == "mlstm":
            H, D, Dv = m.heads, m.dim, m.vdim
            q = p + "mix."
            mat(q + "q", H * D, d, 2.0); mat(q + "k", H * D, d, 2.0)
            mat(q + "v", H * Dv, d, 2.0); mat(q + "g", H * Dv, d, 2.0)
            mat(q + "i", H, d, 2.0); vec(q + "i.b", H, -1.0, 1.0)
            mat(q + "f", H, d, 2.0); vec(q + "f.b", H, 3.0, 1.0)
            vec(q + "norm", H * Dv, 1.0)
            mat(q + "o", d, H * Dv, 2.0)
        elif lc.kind == "latent_attention":
            H, D, Dr, Dv, R, Rq = m.heads, m.dim, m.rot_dim, m.vdim, m.kv_rank, m.q_rank
            q = p + "mix."
            mat(q + "dq", Rq, d, 2.0); vec(q + "dq.norm", Rq, 1.0)
            mat(q + "uq", H * (D + Dr), Rq, 2.0)
            mat(q + "dkv", R + Dr, d, 2.0); vec(q + "dkv.norm", R, 1.0)
            mat(q + "uk", H * D, R, 2.0); mat(q + "uv", H * Dv, R, 2.0)
            mat(q + "g", H * Dv, d, 2.0)
            mat(q + "o", d, H * Dv, 2.0)
        else:
            a, r = m.left, m.right
            q = p + "mix.left."
            mat(q + "q", a.heads * a.dim, d, 2.0); mat(q + "k", a.kv_heads * a.dim, d, 2.0)
            mat(q + "v", a.kv_heads * a.vdim, d, 2.0)
            vec(q + "q.norm", a.heads * a.dim, 1.0); vec(q + "k.norm", a.kv_heads * a.dim, 1.0)
            mat(q + "o", d, a.heads * a.vdim, 2.0)
            q = p + "mix.right."
            GD, HV = r.kv_heads * r.dim, r.heads * r.vdim
            mat(q + "q", GD, d, 2.0); mat(q + "k", GD, d, 2.0); mat(q + "v", HV, d, 2.0)
            for n, c in (("q", GD), ("k", GD), ("v", HV)):
                sd[q + n + ".conv"] = (torch.randn(c, r.taps, generator=g) * 0.5).to(torch.bfloat16)
            mat(q + "b", r.heads, d, 2.0); mat(q + "a", r.heads, d, 2.0)
            vec(q + "A_log", r.heads, -0.5, 0.7); vec(q + "dt_bias", r.heads, -0.5, 0.5)
            vec(q + "norm", r.vdim, 1.0)
            mat(q + "g", HV, d, 2.0)
            mat(q + "o", d, HV, 2.0)
        f = lc.mlp
        if f is not None:
            vec(p + "norm2", d)
            mat(p + "mlp.gate", f.ff, d, 2.0); mat(p + "mlp.up", f.ff, d, 2.0)
            mat(p + "mlp.down", d, f.ff, 2.0)
    vec("final.norm", d)
    mat("head", cfg.vocab_size, d, 2.0)
    return sd


def config_to_json(cfg: VilulixConfig) -> dict:
    """The config.json of ``cfg`` (the inverse of ``vilulix_config_from_json``)."""
    layers = []
    for lc in cfg.layers:
        m, f = lc.mixer, lc.mlp
        if lc.kind == "mlstm":
            mx = {"heads": m.heads, "dim": m.dim, "vdim": m.vdim, "gate_cap": m.gate_cap}
        elif lc.kind == "latent_attention":
            mx = {"heads": m.heads, "dim": m.dim, "rot_dim": m.rot_dim, "vdim": m.vdim,
                  "kv_rank": m.kv_rank, "q_rank": m.q_rank, "scale": m.scale,
                  "rot": {"dims": m.rot.dims, "base": m.rot.base}}
        else:
            a, r = m.left, m.right
            mx = {"left": {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim,
                           "scale": a.scale, "mask": {"size": a.window},
                           "rot": {"dims": a.rot.dims, "base": a.rot.base}},
                  "right": {"heads": r.heads, "kv_heads": r.kv_heads, "dim": r.dim, "vdim": r.vdim,
                            "conv": r.taps},
                  "left_scale": m.left_scale, "right_scale": m.right_scale}
        layers.append({"type": lc.kind, "mixer": mx,
                       "mlp": None if f is None else {"kind": "dense", "ff": f.ff}})
    out = {"architecture": "Vilulix", "vocab": cfg.vocab_size, "width": cfg.d_model,
           "norm": {"eps": cfg.norm_eps}, "logit_softcap": cfg.logit_softcap, "layers": layers}
    if cfg.loop is not None:
        out["loop"] = {"start": cfg.loop.start, "stop": cfg.loop.stop, "times": cfg.loop.times}
    return out


class VilulixModel:
    """The step function: one pass of a flat token batch through all layer
    runs, reading and extending the paged caches and the state slots."""

    hybrid = True
    # a step whose longest feed has at least this many tokens takes the
    # matrix-core prompt path of latent attention (bf16 on the GPU)
    prompt_min_q = 32
    # a step with at least this many tokens runs the sublayers that do not
    # depend on each other on two HIP streams: the feed-forward (and the
    # attention side of a parallel mixer) beside the recurrent scan, whose few
    # long-running waves leave most of the GPU idle. Smaller steps are bound by
    # launches, and a second stream only adds events to them.
    overlap_min_tokens = 128

    def __init__(self, w: VilulixWeights):
        self.w, self.cfg = w, w.cfg
        self.runs = self.cfg.runs()
        self._side = None

    def _side_stream(self, T: int):
        """The second stream for a step of T tokens (default priority), or None."""
        if self.w.device.type != "cuda" or T < self.overlap_min_tokens:
            return None
        if self._side is None:
            from ..utils.streams import placed_stream
            self._side = placed_stream(self.w.device, "mixer")
        return self._side

    # the cache manager sizes its storage from this: one entry per layer RUN
    def cache_spec(self) -> dict:
        latent, kv, state, rows = {}, {}, {}, {}
        for r, (i, _) in enumerate(self.runs):
            lc = self.cfg.layers[i]
            m = lc.mixer
            if lc.kind == "mlstm":
                # the state's last column is the normaliser vector
                state[r] = (m.heads, m.dim, m.vdim + 1)
                rows[r] = {"m": (m.heads,)}
            elif lc.kind == "latent_attention":
                latent[r] = m.kv_rank + m.rot_dim
            else:
                a, d = m.left, m.right
                kv[r] = (a.kv_heads * a.dim, a.kv_heads * a.vdim)
                state[r] = (d.heads, d.vdim, d.dim)        # a column's rows side by side
                if d.taps > 1:
                    rows[r] = {"tail": (d.taps - 1, d.conv_channels)}
        return {"latent": latent, "state": state, "kv_rows": kv, "rows": rows}

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
        n = len(self.runs)
        side = self._side_stream(x.shape[0])
        main = torch.cuda.current_stream(x.device) if side is not None else None
        ha = hb = None
        if n:
            L = w.layers[self.runs[0][0]]
            ha, hb = seqmix.residual_rms1p(x, [], None, L["norm1"], L["norm2"], eps, dt)
        for r, (i, _) in enumerate(self.runs):
            lc, L = cfg.layers[i], w.layers[i]
            ff = None
            if lc.mlp is not None and side is not None:
                # both norms are on their way: the feed-forward goes to the
                # second stream while the mixer runs on this one. Every tensor
                # either stream reads stays referenced until the streams have
                # joined below, so neither allocator pool hands it out early.
                side.wait_stream(main)
                with torch.cuda.stream(side):
                    ff = self._dense(hb, L)
            if lc.kind == "mlstm":
                adds = [(self._mlstm(r, lc.mixer, L, ha, meta, cache, ff is not None), 1.0)]
            elif lc.kind == "latent_attention":
                adds = [(self._latent(r, lc.mixer, L, ha, meta, cache), 1.0)]
            else:
                adds = self._parallel(r, lc.mixer, L, ha, meta, cache, side)
            if lc.mlp is not None:
                adds.append((ff if ff is not None else self._dense(hb, L), 1.0))
            if side is not None:
                main.wait_stream(side)
            # the same launch adds the embedding output when the next run opens
            # a later pass of the repeated stretch, and norms for the next layer
            na = nb = extra = None
            if r + 1 < n:
                N = w.layers[self.runs[r + 1][0]]
                na, nb = N["norm1"], N["norm2"]
                extra = x0 if self.runs[r + 1][1] else None
            if trail is not None:
                seqmix.residual_rms1p(x, adds, None, None, None, eps, dt)
                trail.append(x.clone())
                adds = []
            ha, hb = seqmix.residual_rms1p(x, adds, extra, na, nb, eps, dt)
        hf = seqmix.rms1p_norm(x, w.final_norm, eps, torch.float32, row_idx=meta.logit_idx)
        z = ops.linear(hf, w.head)
        return seqmix.softcap_(z, cfg.logit_softcap) if cfg.logit_softcap > 0 else z

    def _mlstm(self, r, m, L, h, meta, cache, beside: bool = False) -> torch.Tensor:
        """``beside``: other work runs on the second stream meanwhile, so the scan
        takes the denser grid and leaves compute units to it."""
        H, D, Dv = m.heads, m.dim, m.vdim
        u = ops.linear(h, L["w_in"])                       # q | k | v | g
        gz = ops.linear(h.float(), L["w_gates"])           # f32: input | forget pre-activations
        tok, floor = seqmix.exp_gate_scan(gz, L["i_b"], L["f_b"], m.gate_cap, cache.rows[r]["m"],
                                          meta.state_slots, meta.cu_q, meta.positions)
        act = seqmix.matrix_memory_inputs(u, H, D, Dv)
        o = seqmix.state_scan(act, H, D, Dv + 1, 0, H * D, 2 * H * D, 1, cache.state[r],
                              meta.state_slots, meta.cu_q, meta.positions, tok=tok,
                              col_block=16 if beside else 0)
        y = seqmix.normalized_gated_rmsnorm(o, floor, L["norm"],
                                            u[:, L["g_off"]:L["g_off"] + H * Dv],
                                            self.cfg.norm_eps, self.w.dtype, H, Dv)
        return ops.linear(y, L["wo"])

    def _latent(self, r, m, L, h, meta, cache) -> torch.Tensor:
        H, Dv, R, Dr = m.heads, m.vdim, m.kv_rank, m.rot_dim
        eps = self.cfg.norm_eps
        u = ops.linear(h, L["w_in"])                       # dq | dkv | gate
        cq = seqmix.rms_norm_cols(u, m.q_rank, L["dq_norm"], eps, self.w.dtype)
        z = u[:, L["z_off"]:L["z_off"] + R + Dr]
        gate = u[:, L["g_off"]:L["g_off"] + H * Dv]
        return latent_mix(L, m, ops.linear(cq, L["wq"]), z, cache.latent[r], meta, eps,
                          self.prompt_min_q, gate)

    def _parallel(self, r, m, L, h, meta, cache, side=None) -> list:
        u = ops.linear(h, L["w_in"])                       # left q | k | v, right q | k | v | g
        if side is None:
            left = self._window(r, m.left, L, u, meta, cache)
        else:
            # the attention side on the second stream, beside the delta rule
            side.wait_stream(torch.cuda.current_stream(u.device))
            with torch.cuda.stream(side):
                left = self._window(r, m.left, L, u, meta, cache)
        right = self._delta(r, m.right, L, h, u[:, L["r_off"]:], meta, cache)
        return [(left, m.left_scale), (right, m.right_scale)]

    def _window(self, r, a, L, u, meta, cache) -> torch.Tensor:
        H, G, D, Dv = a.heads, a.kv_heads, a.dim, a.vdim
        kc, vc = cache.kv_rows[r]
        q = seqmix.qk_prep_append(u, H, G, D, Dv, L["l_v_off"], L["l_cos_sin"],
                                  a.rot.dims if L["l_cos_sin"] is not None else 0,
                                  self.cfg.norm_eps, None, meta.positions, kc, vc, meta.slots,
                                  self.w.dtype, L["l_q_norm"], L["l_k_norm"])
        o = seqmix.window_attention(q, kc, vc, meta.cu_q, meta.ctx_lens, meta.block_tables,
                                    meta.positions, a.scale, 0.0, a.window, 0, None, H, G, D, Dv,
                                    meta.max_q, max_ctx=meta.max_ctx, sink=L["l_sink"])
        return ops.linear(o, L["l_wo"])

    def _delta(self, r, d, L, h, u, meta, cache) -> torch.Tensor:
        H, G, D, Dv, C = d.heads, d.kv_heads, d.dim, d.vdim, d.conv_channels
        gz = ops.linear(h.float(), L["r_gates"])           # f32: beta | decay pre-activations
        tail = cache.rows[r]["tail"] if d.taps > 1 else \
            torch.zeros(1, 0, C, dtype=torch.float32, device=u.device)
        act, tok = seqmix.delta_prep(u, gz, G, D, H, Dv, L["r_conv"], tail, L["r_a_neg"],
                                     L["r_dt_bias"], meta.state_slots, meta.cu_q, meta.positions)
        if d.taps > 1:
            # every reader of this step's tail is done: store the new rows
            seqmix.seq_state_save(None, u, None, tail, meta.state_slots, meta.cu_q, meta.positions)
        o = seqmix.delta_scan(act, H, D, Dv, 0, G * D, 2 * G * D, H // G, cache.state[r],
                              meta.state_slots, meta.cu_q, meta.positions, tok)
        y = seqmix.gated_rmsnorm(o, L["r_norm"], u[:, C:C + H * Dv], self.cfg.norm_eps,
                                 self.w.dtype, groups=H, gate_act="silu")
        return ops.linear(y, L["r_wo"])

    @staticmethod
    def _dense(h, L) -> torch.Tensor:
        return ops.linear(seqmix.silu_mul_any(ops.linear(h, L["w_gate_up"])), L["w_down"])
