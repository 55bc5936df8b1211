"""A plain, slow float64 implementation of the Vilulix decoder, written from
its equations: one function per mechanism, whole sequences at once, no cache,
no batching, no code shared with ``loqa_hub_amd``. The tests compare the
framework (reference ops on the CPU, HIP kernels on the GPU) with it.

Notation: T tokens, width d, H heads, G key/value (or query/key) heads, head
sizes D (queries, keys) and Dv (values); positions p = 0 .. T - 1.
"""
import math

import torch

F64 = torch.float64


# ----------------------------------------------------------------- configs
def mlstm(heads=3, dim=8, vdim=12, cap=8.0):
    return "mlstm", {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}


def latent(heads=3, dim=8, rot_dim=4, vdim=10, kv_rank=12, q_rank=14, scale=None, base=100.0):
    return "latent_attention", {
        "heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
        "q_rank": q_rank, "scale": scale if scale is not None else (dim + rot_dim) ** -0.5,
        "rot": {"dims": rot_dim, "base": base}}


def window_attn(heads=4, kv_heads=2, dim=12, vdim=10, window=6, dims=8, base=100.0, scale=None):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "scale": scale if scale is not None else dim ** -0.5, "mask": {"size": window},
            "rot": {"dims": dims, "base": base}}


def delta(heads=4, kv_heads=2, dim=8, vdim=6, conv=3):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}


def parallel(left=None, right=None, left_scale=0.8, right_scale=1.3):
    return "parallel", {"left": left or window_attn(), "right": right or delta(),
                        "left_scale": left_scale, "right_scale": right_scale}


def dense_ff(ff=40):
    return {"kind": "dense", "ff": ff}


def make_config(layers, width=32, vocab=50, eps=1e-5, softcap=10.0, loop=None):
    cfg = {"architecture": "Vilulix", "vocab": vocab, "width": width, "norm": {"eps": eps},
           "logit_softcap": softcap,
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
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        vec(p + "norm1", d, 0.0, 0.2)
        if L["type"] == "mlstm":
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            mat(p + "mix.q", H * D, d, 2.0); mat(p + "mix.k", H * D, d, 2.0)
            mat(p + "mix.v", H * Dv, d, 2.0); mat(p + "mix.g", H * Dv, d, 2.0)
            mat(p + "mix.i", H, d, 3.0); vec(p + "mix.i.b", H, -1.0, 1.0)
            mat(p + "mix.f", H, d, 3.0); vec(p + "mix.f.b", H, 3.0, 1.0)
            vec(p + "mix.norm", H * Dv, 1.0, 0.2)
            mat(p + "mix.o", d, H * Dv, 2.0)
        elif L["type"] == "latent_attention":
            H, D, Dr, Dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            R, Rq = m["kv_rank"], m["q_rank"]
            mat(p + "mix.dq", Rq, d, 2.0); vec(p + "mix.dq.norm", Rq, 1.0, 0.2)
            mat(p + "mix.uq", H * (D + Dr), Rq, 2.0)
            mat(p + "mix.dkv", R + Dr, d, 2.0); vec(p + "mix.dkv.norm", R, 1.0, 0.2)
            mat(p + "mix.uk", H * D, R, 2.0); mat(p + "mix.uv", H * Dv, R, 2.0)
            mat(p + "mix.g", H * Dv, d, 2.0)
            mat(p + "mix.o", d, H * Dv, 2.0)
        elif L["type"] == "parallel":
            a, r = m["left"], m["right"]
            q = p + "mix.left."
            H, G, D, Dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            mat(q + "q", H * D, d, 2.0); mat(q + "k", G * D, d, 2.0); mat(q + "v", G * Dv, d, 2.0)
            vec(q + "q.norm", H * D, 1.0, 0.2); vec(q + "k.norm", G * D, 1.0, 0.2)
            mat(q + "o", d, H * Dv, 2.0)
            q = p + "mix.right."
            H, G, D, Dv, K = r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"]
            mat(q + "q", G * D, d, 2.0); mat(q + "k", G * D, d, 2.0); mat(q + "v", H * Dv, d, 2.0)
            for n, c in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                put(q + n + ".conv", torch.randn(c, K, generator=g) * 0.6)
            mat(q + "b", H, d, 2.0); mat(q + "a", H, d, 2.0)
            vec(q + "A_log", H, -0.5, 0.7); vec(q + "dt_bias", H, -0.5, 0.5)
            vec(q + "norm", Dv, 1.0, 0.2)
            mat(q + "g", H * Dv, d, 2.0)
            mat(q + "o", d, H * Dv, 2.0)
        else:
            raise ValueError(L["type"])
        f = L["mlp"]
        if f is not None:
            vec(p + "norm2", d, 0.0, 0.2)
            mat(p + "mlp.gate", f["ff"], d, 2.0); mat(p + "mlp.up", f["ff"], d, 2.0)
            mat(p + "mlp.down", d, f["ff"], 2.0)
    vec("final.norm", d, 0.0, 0.2)
    mat("head", cfg["vocab"], d, 2.0)
    return sd


# -------------------------------------------------------------- mechanisms
def unit_rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """The layer norm: weight stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return unit_rms(x, eps) * w


def silu(z):
    return z * torch.sigmoid(z)


def rotate_half(x, dims, base, pos=None):
    """x [T, heads, size]: entry i of the first ``dims`` pairs with entry
    i + dims / 2; the pair turns by the angle p * base^(-2 i / dims)."""
    T = x.shape[0]
    if dims == 0:
        return x
    half = dims // 2
    p = torch.arange(T, dtype=F64) if pos is None else pos.to(F64)
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    a = p[:, None] * f[None, :]
    c, s = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def causal_conv(x, w):
    """x [T, C], w [C, taps]: y_t = sum_j w[:, j] x_{t - (taps - 1 - j)}, zeros
    before the start, no bias."""
    T, C = x.shape
    K = w.shape[1]
    xp = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x])
    y = torch.zeros_like(x)
    for j in range(K):
        y = y + xp[j:j + T] * w[:, j]
    return y


def attention(q, k, v, scale, window=0, sink=False):
    """q [T, H, D], k [T, G, D], v [T, G, Dv]; key j visible to query i when
    j <= i and (window == 0 or i - j < window). With ``sink`` the softmax
    denominator has one more term exp(0) that carries no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    i = torch.arange(T)
    vis = i[None, :] <= i[:, None]
    if window:
        vis &= (i[:, None] - i[None, :]) < window
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~vis, -math.inf)
        if sink:
            m = torch.clamp(s.max(-1, keepdim=True).values, min=0.0)
            e = torch.exp(s - m)
            p = e / (torch.exp(-m) + e.sum(-1, keepdim=True))
        else:
            p = torch.softmax(s, -1)
        out[:, h] = p @ v[:, g]
    return out


def mixer_window_attention(sd, p, m, h, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = norm_plain(h @ sd[p + "q"].T, sd[p + "q.norm"], eps).view(T, H, D)
    k = norm_plain(h @ sd[p + "k"].T, sd[p + "k.norm"], eps).view(T, G, D)
    v = (h @ sd[p + "v"].T).view(T, G, Dv)
    r = m["rot"]
    q, k = rotate_half(q, r["dims"], r["base"]), rotate_half(k, r["dims"], r["base"])
    o = attention(q, k, v, m["scale"], window=m["mask"]["size"], sink=True)
    return o.reshape(T, H * Dv) @ sd[p + "o"].T


def delta_rule(q, k, v, beta, decay):
    """Per head: S <- decay S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    q, k [T, H, D], v [T, H, Dv], beta, decay [T, H]."""
    T, H, D = q.shape
    Dv = v.shape[2]
    o = torch.zeros(T, H, Dv, dtype=F64)
    for h in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        for t in range(T):
            S = decay[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h])
            S = S + torch.outer(k[t, h], u)
            o[t, h] = S.T @ q[t, h]
    return o


def mixer_gated_delta(sd, p, m, h, eps):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ sd[p + "q"].T, sd[p + "q.conv"])).view(T, G, D)
    k = silu(causal_conv(h @ sd[p + "k"].T, sd[p + "k.conv"])).view(T, G, D)
    v = silu(causal_conv(h @ sd[p + "v"].T, sd[p + "v.conv"])).view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    rep = H // G
    q, k = q.repeat_interleave(rep, 1), k.repeat_interleave(rep, 1)
    beta = torch.sigmoid(h @ sd[p + "b"].T)
    dt = torch.nn.functional.softplus(h @ sd[p + "a"].T + sd[p + "dt_bias"])
    decay = torch.exp(-torch.exp(sd[p + "A_log"]) * dt)
    o = delta_rule(q, k, v, beta, decay)
    o = unit_rms(o, eps) * sd[p + "norm"]
    o = o.reshape(T, H * Dv) * silu(h @ sd[p + "g"].T)
    return o @ sd[p + "o"].T


def mixer_parallel(sd, p, m, h, eps):
    return m["left_scale"] * mixer_window_attention(sd, p + "mix.left.", m["left"], h, eps) + \
        m["right_scale"] * mixer_gated_delta(sd, p + "mix.right.", m["right"], h, eps)


def matrix_memory(q, k, v, li, lf):
    """Stabilised matrix memory with exponential gates. li, lf [T, H]: the log
    input and log forget gates. The running maximum starts at 0."""
    T, H, D = q.shape
    Dv = v.shape[2]
    o = torch.zeros(T, H, Dv, dtype=F64)
    for h in range(H):
        S = torch.zeros(D, Dv, dtype=F64)
        n = torch.zeros(D, dtype=F64)
        m = torch.zeros((), dtype=F64)
        for t in range(T):
            m1 = torch.maximum(lf[t, h] + m, li[t, h])
            a, b = torch.exp(lf[t, h] + m - m1), torch.exp(li[t, h] - m1)
            S = a * S + b * torch.outer(k[t, h], v[t, h])
            n = a * n + b * k[t, h]
            m = m1
            den = torch.maximum((n @ q[t, h]).abs(), torch.exp(-m)) + 1e-6
            o[t, h] = (S.T @ q[t, h]) / den
    return o


def mixer_mlstm(sd, p, m, h, eps):
    p = p + "mix."
    T = h.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ sd[p + "q"].T).view(T, H, D) * D ** -0.5
    k = (h @ sd[p + "k"].T).view(T, H, D)
    v = (h @ sd[p + "v"].T).view(T, H, Dv)
    li = cap * torch.tanh((h @ sd[p + "i"].T + sd[p + "i.b"]) / cap)
    lf = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ sd[p + "f"].T + sd[p + "f.b"]) / cap))
    o = unit_rms(matrix_memory(q, k, v, li, lf), eps).reshape(T, H * Dv)
    return (o * sd[p + "norm"] * torch.sigmoid(h @ sd[p + "g"].T)) @ sd[p + "o"].T


def mixer_latent(sd, p, m, h, eps):
    p = p + "mix."
    T = h.shape[0]
    H, D, Dr, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    r = m["rot"]
    cq = norm_plain(h @ sd[p + "dq"].T, sd[p + "dq.norm"], eps)
    q = (cq @ sd[p + "uq"].T).view(T, H, D + Dr)
    z = h @ sd[p + "dkv"].T
    c = norm_plain(z[:, :R], sd[p + "dkv.norm"], eps)
    kr = rotate_half(z[:, None, R:], r["dims"], r["base"])                 # [T, 1, Dr]
    qr = rotate_half(q[..., D:], r["dims"], r["base"])
    kk = torch.cat([(c @ sd[p + "uk"].T).view(T, H, D), kr.expand(T, H, Dr)], -1)
    qq = torch.cat([q[..., :D], qr], -1)
    v = (c @ sd[p + "uv"].T).view(T, H, Dv)
    o = attention(qq, kk, v, m["scale"]).reshape(T, H * Dv)
    return (o * torch.sigmoid(h @ sd[p + "g"].T)) @ sd[p + "o"].T


def ff_dense(sd, p, h):
    return (silu(h @ sd[p + "mlp.gate"].T) * (h @ sd[p + "mlp.up"].T)) @ sd[p + "mlp.down"].T


# ------------------------------------------------------------------ model
def layer_order(cfg):
    """(layer, first of a later pass) in execution order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    out = [(i, False) for i in range(lp["start"])]
    for t in range(lp["times"]):
        out += [(i, t > 0 and i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return out + [(i, False) for i in range(lp["stop"], n)]


MIXERS = {"mlstm": mixer_mlstm, "latent_attention": mixer_latent}


def forward(cfg, sd, tokens, trail=None):
    """f64 logits [T, vocab] of one whole sequence."""
    sd = {k: v.to(F64) for k, v in sd.items()}
    eps = cfg["norm"]["eps"]
    x0 = sd["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    for i, again in layer_order(cfg):
        L = cfg["layers"][i]
        p = f"l{i}."
        if again:
            x = x + x0
        h = norm_around_zero(x, sd[p + "norm1"], eps)
        if L["type"] == "parallel":
            y = mixer_parallel(sd, p, L["mixer"], h, eps)
        else:
            y = MIXERS[L["type"]](sd, p, L["mixer"], h, eps)
        if L["mlp"] is not None:
            y = y + ff_dense(sd, p, norm_around_zero(x, sd[p + "norm2"], eps))
        x = x + y
        if trail is not None:
            trail.append(x.clone())
    z = norm_around_zero(x, sd["final.norm"], eps) @ sd["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z
