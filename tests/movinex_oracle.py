"""A plain, slow float64 implementation of the Movinex decoder, written from
its equations: one function per mechanism, whole sequences at once, no cache,
no batching, no code shared with ``loqa_hub_amd``. The tests compare the
framework (reference ops on the CPU, HIP kernels on the GPU) with it.

Notation: T tokens, width d, H query heads, G key/value heads, head sizes D
(queries, keys) and Dv (values); positions p = 0 .. T - 1.
"""
import math

import torch

F64 = torch.float64


# ----------------------------------------------------------------- configs
def attn(heads=4, kv_heads=2, dim=16, vdim=None, scale=None, coef=0.5, every=4):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim or dim,
         "scale": scale if scale is not None else dim ** -0.5}
    if coef is not None:
        m["q_temp"] = {"coef": coef, "every": every}
    return "attention", m


def attn2(heads=4, kv_heads=2, dim=16, scale=None, window=6, keep=2, dims=8, base=100.0, cap=5.0):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim,
         "scale": scale if scale is not None else dim ** -0.5,
         "mask": {"size": window, "keep_first": keep}, "softcap": cap}
    if dims:
        m["rot"] = {"dims": dims, "base": base}
    return "attention_2", m


def mamba(heads=4, vdim=8, state=8, groups=2, conv=4, norm_groups=2):
    return "mamba2", {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                      "norm_groups": norm_groups}


def dense_ff(ff=40):
    return {"kind": "dense", "ff": ff}


def moe_ff(experts=6, top=2, ff=16, count=3, keep=2):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}}}


def make_config(layers, width=32, vocab=50, eps=1e-5, logit_scale=0.5, loop=None):
    cfg = {"architecture": "Movinex", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "logit_scale": logit_scale,
           "layers": [{"type": t, "mixer": m, "mlp": f} for (t, m), f in layers]}
    if loop is not None:
        cfg["loop"] = dict(zip(("start", "stop", "times"), loop))
    return cfg


def make_weights(cfg, seed=0):
    """Random weights in checkpoint naming whose values are exact in bfloat16."""
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]
    sd = {}

    def put(name, t):
        sd[name] = t.to(torch.bfloat16).float()

    def mat(name, rows, cols, gain=1.0):
        put(name, torch.randn(rows, cols, generator=g) * gain / cols ** 0.5)

    def vec(name, n, mean=0.0, std=0.1):
        put(name, mean + torch.randn(n, generator=g) * std)

    put("embed", torch.randn(cfg["vocab"], d, generator=g))
    if cfg.get("loop"):
        mat("loop.in", d, 2 * d, 1.4)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        vec(p + "norm1", d, 0.0, 0.2)
        vec(p + "ls1", d, 0.7, 0.2)
        if L["type"] == "mamba2":
            inner, GN = m["heads"] * m["vdim"], m["groups"] * m["state"]
            mat(p + "mix.in", 2 * inner + 2 * GN + m["heads"], d, 1.5)
            put(p + "mix.conv", torch.randn(inner + 2 * GN, m["conv"], generator=g) * 0.5)
            vec(p + "mix.conv.b", inner + 2 * GN)
            vec(p + "mix.dt_bias", m["heads"], -0.5, 0.5)
            vec(p + "mix.A_log", m["heads"], -0.5, 0.7)
            vec(p + "mix.D", m["heads"], 1.0, 0.3)
            vec(p + "mix.norm", inner, 1.0, 0.2)
            mat(p + "mix.o", d, inner, 2.0)
        else:
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            mat(p + "mix.q", H * D, d, 2.0)
            mat(p + "mix.k", G * D, d, 2.0)
            if L["type"] == "attention":
                mat(p + "mix.v", G * Dv, d, 2.0)
                vec(p + "mix.q.b", H * D, 0.0, 0.3)
                vec(p + "mix.k.b", G * D, 0.0, 0.3)
                vec(p + "mix.v.b", G * Dv, 0.0, 0.3)
            else:
                mat(p + "mix.g", H * Dv, d, 2.0)
            mat(p + "mix.o", d, H * Dv, 2.0)
        f = L["mlp"]
        if not f:
            continue
        vec(p + "norm2", d, 0.0, 0.2)
        vec(p + "ls2", d, 0.7, 0.2)
        if f["kind"] == "dense":
            mat(p + "mlp.gate", f["ff"], d, 2.0)
            mat(p + "mlp.up", f["ff"], d, 2.0)
            mat(p + "mlp.down", d, f["ff"], 2.0)
        else:
            n = f["expert"]["ff"]
            for e in range(f["router"]["experts"]):
                mat(f"{p}mlp.e{e}.gate", n, d, 2.0)
                mat(f"{p}mlp.e{e}.up", n, d, 2.0)
                mat(f"{p}mlp.e{e}.down", d, n, 3.0)
            mat(p + "mlp.router", f["router"]["experts"], d, 4.0)
    vec("final.norm", d, 0.0, 0.2)
    mat("head", cfg["vocab"], d, 2.0)
    return sd


# -------------------------------------------------------------- mechanisms
def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z / (1.0 + torch.exp(-z))


def rotate(x, dims, base, pos=None):
    """x [T, heads, D]: entries (2i, 2i + 1), i < dims / 2, turn by p * base^(-2i / dims)."""
    T = x.shape[0]
    pos = torch.arange(T, dtype=F64) if pos is None else pos.to(F64)
    i = torch.arange(dims // 2, dtype=F64)
    ang = pos[:, None] * base ** (-2.0 * i / dims)[None, :]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    y = x.clone()
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    y[..., 0:dims:2] = a * c - b * s
    y[..., 1:dims:2] = b * c + a * s
    return y


def query_temperature(T, coef, every, pos=None):
    pos = torch.arange(T) if pos is None else pos
    return 1.0 + coef * torch.log(torch.div(pos + 1, every, rounding_mode="floor").to(F64) + 1.0)


def visible(T, window=0, keep=0):
    """[T, T] mask: row i sees column j."""
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    m = j <= i
    if window > 0:
        m = m & ((i - j < window) | (j < keep))
    return m


def softmax_attention(q, k, v, scale, mask, cap=0.0):
    """q [T, H, D], k [T, G, D], v [T, G, Dv] -> [T, H, Dv]; head h reads
    key/value head h // (H / G)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        s = q[:, h] @ k[:, g].T * scale
        if cap > 0:
            s = cap * torch.tanh(s / cap)
        s = s.masked_fill(~mask, -math.inf)
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def mixer_attention(sd, p, m, h, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ sd[p + "q"].T + sd[p + "q.b"]).view(T, H, D)
    k = (h @ sd[p + "k"].T + sd[p + "k.b"]).view(T, G, D)
    v = (h @ sd[p + "v"].T + sd[p + "v.b"]).view(T, G, Dv)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(T, qt["coef"], qt["every"])[:, None, None]
    o = softmax_attention(q, k, v, m["scale"], visible(T))
    return o.reshape(T, H * Dv) @ sd[p + "o"].T


def mixer_attention_2(sd, p, m, h, eps):
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ sd[p + "q"].T).view(T, H, D)
    k = (h @ sd[p + "k"].T).view(T, G, D)
    v = k                                           # the keys as projected are the values
    r = m.get("rot")
    if r:
        q, k = rotate(q, r["dims"], r["base"]), rotate(k, r["dims"], r["base"])
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    mk = m.get("mask") or {}
    o = softmax_attention(q, k, v, m["scale"], visible(T, mk.get("size", 0), mk.get("keep_first", 0)),
                          m.get("softcap") or 0.0)
    o = o.reshape(T, H * D) * torch.sigmoid(h @ sd[p + "g"].T)
    return o @ sd[p + "o"].T


def causal_conv(x, w, b):
    """x [T, C], w [C, taps] (last column = the current token), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F64), x])
    return torch.stack([(pad[t:t + taps].T * w).sum(-1) for t in range(T)]) + b


def mixer_mamba2(sd, p, m, h, eps):
    T = h.shape[0]
    Hh, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner, GN = Hh * P, G * N
    u = h @ sd[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * GN], u[:, 2 * inner + 2 * GN:]
    xbc = silu(causal_conv(xbc, sd[p + "conv"], sd[p + "conv.b"]))
    x = xbc[:, :inner].view(T, Hh, P)
    Bm = xbc[:, inner:inner + GN].view(T, G, N)
    Cm = xbc[:, inner + GN:].view(T, G, N)
    dt = torch.log1p(torch.exp(dt + sd[p + "dt_bias"]))
    rate = torch.exp(sd[p + "A_log"])
    y = torch.zeros(T, Hh, P, dtype=F64)
    for hh in range(Hh):
        g = hh // (Hh // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = torch.exp(-rate[hh] * dt[t, hh]) * S + dt[t, hh] * torch.outer(Bm[t, g], x[t, hh])
            y[t, hh] = S.T @ Cm[t, g] + sd[p + "D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = unit_rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * sd[p + "norm"]
    return y @ sd[p + "o"].T


def ff_dense(sd, p, h):
    return (gelu_tanh(h @ sd[p + "gate"].T) * (h @ sd[p + "up"].T)) @ sd[p + "down"].T


def route(scores, top, count, keep):
    """scores [E] -> the chosen expert indices: groups of neighbours rank by the
    sum of their two best scores, only the best ``keep`` groups are eligible."""
    E = scores.numel()
    per = E // count
    gs = scores.view(count, per).topk(min(2, per), dim=-1).values.sum(-1)
    ok = torch.zeros(count, dtype=torch.bool)
    ok[gs.topk(keep).indices] = True
    masked = scores.masked_fill(~ok.repeat_interleave(per), -math.inf)
    return masked.topk(top).indices.tolist()


def ff_moe(sd, p, f, h):
    r = f["router"]
    gr = r.get("groups") or {"count": 1, "keep": 1}
    s = torch.sigmoid(h @ sd[p + "router"].T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in route(s[t], r["top"], gr["count"], gr["keep"]):
            q = f"{p}e{e}."
            a = silu(sd[q + "gate"] @ h[t]) * (sd[q + "up"] @ h[t])
            out[t] += s[t, e] * (sd[q + "down"] @ a)
    return out


def layer_order(cfg):
    """(layer index, enters a pass of the repeated stretch) in execution order."""
    n, lp = len(cfg["layers"]), cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    mid = [(i, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return [(i, False) for i in range(lp["start"])] + mid * lp["times"] + \
        [(i, False) for i in range(lp["stop"], n)]


def forward(cfg, sd, tokens, trail=None):
    """Logits [T, vocab] of a whole sequence; ``trail`` collects the residual
    stream after every layer run."""
    sd = {k: v.to(F64) for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    x0 = sd["embed"][torch.tensor(tokens)]
    x = x0
    mixers = {"attention": mixer_attention, "attention_2": mixer_attention_2, "mamba2": mixer_mamba2}
    for i, enters in layer_order(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        if enters:
            x = torch.cat([x, x0], dim=-1) @ sd["loop.in"].T
        y = mixers[L["type"]](sd, p + "mix.", L["mixer"], norm(x, sd[p + "norm1"], eps), eps)
        x = x + y * sd[p + "ls1"]
        f = L["mlp"]
        if f:
            h = norm(x, sd[p + "norm2"], eps)
            y = ff_dense(sd, p + "mlp.", h) if f["kind"] == "dense" else ff_moe(sd, p + "mlp.", f, h)
            x = x + y * sd[p + "ls2"]
        if trail is not None:
            trail.append(x.clone())
    return norm(x, sd["final.norm"], eps) @ sd["head"].T * cfg.get("logit_scale", 1.0)
