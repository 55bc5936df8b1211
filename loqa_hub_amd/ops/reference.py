"""Plain-PyTorch fp32 reference implementations of every hot op.

These are the numerics oracle for the HIP kernels (tests compare kernel output
against them) and the CPU execution path (no GPU in the CI tier).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import numpy as np
import torch


def rmsnorm(x, w, eps, residual=None):
    if residual is not None:
        s = (x.float() + residual.float()).to(residual.dtype)
        residual.copy_(s)
        x = s
    xf = x.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(x.dtype)


def layernorm(x, w, b, eps, residual=None):
    if residual is not None:
        s = (x.float() + residual.float()).to(residual.dtype)
        residual.copy_(s)
        x = s
    y = torch.nn.functional.layer_norm(x.float(), (x.shape[-1],), w.float(), b.float(), eps)
    return y.to(x.dtype)


def gelu_tanh(z):
    """0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3)))."""
    return 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))


def act_mul(x, act: str = "silu"):
    """[gate | up] -> act(gate) * up in f32, rounded to x's dtype."""
    F = x.shape[-1] // 2
    g, u = x[..., :F].float(), x[..., F:].float()
    a = gelu_tanh(g) if act == "gelu_tanh" else torch.nn.functional.silu(g)
    return (a * u).to(x.dtype)


def silu_mul(x):
    F = x.shape[-1] // 2
    g, u = x[..., :F].float(), x[..., F:].float()
    return (torch.nn.functional.silu(g) * u).to(x.dtype)


def gelu_bias_(x, bias=None, pos=None):
    y = x.float()
    if bias is not None:
        y = y + bias.float()
    y = torch.nn.functional.gelu(y)
    if pos is not None:
        rows = y.reshape(-1, y.shape[-1]).shape[0]
        idx = torch.arange(rows, device=x.device) % pos.shape[0]
        y = (y.reshape(-1, y.shape[-1]) + pos.float()[idx]).reshape(y.shape)
    x.copy_(y.to(x.dtype))
    return x


def rope_cos_sin(head_dim: int, max_pos: int, theta: float, device=None,
                 scaling: tuple | None = None) -> torch.Tensor:
    """[max_pos, D/2, 2] f32 table of (cos, sin) for NeoX rotate-half RoPE.
    ``scaling`` = (factor, low_freq_factor, high_freq_factor, original max
    positions): Llama-3.1 frequency scaling - wavelengths longer than
    original / low are divided by ``factor``, shorter than original / high
    kept, and the band between interpolated."""
    inv = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim))
    if scaling is not None:
        factor, low, high, orig = scaling
        wavelen = 2 * math.pi / inv
        smooth = ((orig / wavelen - low) / (high - low)).clamp(0.0, 1.0)
        inv = torch.where(wavelen > orig / low, inv / factor,
                          torch.where(wavelen < orig / high, inv,
                                      (1 - smooth) * inv / factor + smooth * inv))
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    return torch.stack([ang.cos(), ang.sin()], dim=-1).float().to(device)


def apply_rope(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """x [T, H, D] (any float), cs [T, D/2, 2] -> rotated x (fp32)."""
    half = x.shape[-1] // 2
    a, b = x[..., :half].float(), x[..., half:].float()
    c, s = cs[:, None, :, 0], cs[:, None, :, 1]
    return torch.cat([a * c - b * s, b * c + a * s], dim=-1)


def rope_kv_append(qkv, positions, cos_sin, k_cache, v_cache, slots, H, Hkv, D):
    T = qkv.shape[0]
    if T == 0:
        return None
    q = qkv[:, : H * D].view(T, H, D)
    k = qkv[:, H * D:(H + Hkv) * D].view(T, Hkv, D)
    v = qkv[:, (H + Hkv) * D:(H + 2 * Hkv) * D].view(T, Hkv, D)
    if cos_sin is not None:
        cs = cos_sin[positions.long()]
        q.copy_(apply_rope(q, cs).to(q.dtype))
        k = apply_rope(k, cs).to(qkv.dtype)
    blk = k_cache.shape[2]
    sl = slots.long()
    valid = sl >= 0
    b, o = (sl // blk)[valid], (sl % blk)[valid]
    k_cache[b, :, o, :] = k[valid].to(k_cache.dtype)
    v_cache[b, :, o, :] = v[valid].to(v_cache.dtype)
    return None


def attention(q, k, v, cu_q, *, n_heads, n_kv, head_dim, causal, cu_k=None, ctx_lens=None,
              block_tables=None, scale=None, out=None):
    H, Hkv, D = n_heads, n_kv, head_dim
    scale = scale if scale is not None else 1.0 / math.sqrt(D)
    Tq = q.shape[0]
    res = torch.zeros(Tq, H * D, dtype=torch.float32, device=q.device)
    cuq = cu_q.tolist()
    G = H // Hkv
    for b in range(len(cuq) - 1):
        q0, q1 = cuq[b], cuq[b + 1]
        ql = q1 - q0
        if ql == 0:
            continue
        if block_tables is not None:
            L = int(ctx_lens[b])
            blk = k.shape[2]
            idx = torch.arange(L, device=k.device)
            bt = block_tables[b].long()[idx // blk]
            kb = k[bt, :, idx % blk, :].float()  # [L, Hkv, D]
            vb = v[bt, :, idx % blk, :].float()
        else:
            k0 = int(cu_k[b])
            k1 = k0 + int(ctx_lens[b]) if ctx_lens is not None else int(cu_k[b + 1])
            L = k1 - k0
            kb = k[k0:k1, : Hkv * D].reshape(L, Hkv, D).float()
            vb = v[k0:k1, : Hkv * D].reshape(L, Hkv, D).float()
        qb = q[q0:q1, : H * D].reshape(ql, H, D).float()
        kb = kb.repeat_interleave(G, dim=1)
        vb = vb.repeat_interleave(G, dim=1)
        s = torch.einsum("qhd,khd->hqk", qb, kb) * scale
        if causal:
            qpos = torch.arange(ql, device=q.device) + (L - ql)
            kpos = torch.arange(L, device=q.device)
            s = s.masked_fill(kpos[None, None, :] > qpos[None, :, None], float("-inf"))
        p = torch.softmax(s, dim=-1)
        p = torch.nan_to_num(p, nan=0.0)
        res[q0:q1] = torch.einsum("hqk,khd->qhd", p, vb).reshape(ql, H * D)
    r = res.to(q.dtype)
    if out is not None:
        out.copy_(r)
        return out
    return r


def masked_argmax(logits, mask=None, mask_rows=None):
    x = logits.float()
    B, V = x.shape
    if mask is not None:
        m = mask if mask_rows is None else mask[mask_rows.long()]
        bits = unpack_mask(m, V)
        x = x.masked_fill(~bits, float("-inf"))
        none = ~bits.any(dim=-1)
    else:
        none = torch.zeros(B, dtype=torch.bool, device=x.device)
    r = x.argmax(dim=-1).to(torch.int32)
    r[none] = -1
    return r


def unpack_mask(m: torch.Tensor, V: int) -> torch.Tensor:
    """int32 words [..., W] -> bool [..., V]"""
    shifts = torch.arange(32, device=m.device, dtype=torch.int32)
    bits = (m.unsqueeze(-1) >> shifts) & 1
    return bits.reshape(*m.shape[:-1], -1)[..., :V].bool()


def pack_mask(bits: torch.Tensor) -> torch.Tensor:
    """bool [..., V] -> int32 words [..., ceil(V/32)]"""
    V = bits.shape[-1]
    W = (V + 31) // 32
    pad = torch.zeros(*bits.shape[:-1], W * 32, dtype=torch.int64, device=bits.device)
    pad[..., :V] = bits.long()
    w = (pad.reshape(*bits.shape[:-1], W, 32) << torch.arange(32, device=bits.device)).sum(-1)
    w = torch.where(w >= 2**31, w - 2**32, w)
    return w.to(torch.int32)


def pcm16_to_f32_sumsq(pcm, offsets):
    f = pcm.float() / 32767.0
    off = offsets.tolist()
    ss = torch.tensor([float((f[off[i]:off[i + 1]].double() ** 2).sum()) for i in range(len(off) - 1)],
                      dtype=torch.float32)
    return f, ss


# ------------------------------------------------------------- log-mel consts
def _hz_to_mel(f):
    f = np.asarray(f, dtype=np.float64)
    f_sp = 200.0 / 3
    mels = f / f_sp
    min_log_hz = 1000.0
    min_log_mel = min_log_hz / f_sp
    logstep = np.log(6.4) / 27.0
    return np.where(f >= min_log_hz, min_log_mel + np.log(np.maximum(f, 1e-10) / min_log_hz) / logstep, mels)


def _mel_to_hz(m):
    m = np.asarray(m, dtype=np.float64)
    f_sp = 200.0 / 3
    freqs = f_sp * m
    min_log_hz = 1000.0
    min_log_mel = min_log_hz / f_sp
    logstep = np.log(6.4) / 27.0
    return np.where(m >= min_log_mel, min_log_hz * np.exp(logstep * (m - min_log_mel)), freqs)


def mel_filterbank(sr: int = 16000, n_fft: int = 400, n_mels: int = 80) -> np.ndarray:
    """Slaney-style mel filterbank (librosa defaults, as whisper uses)."""
    n_freqs = 1 + n_fft // 2
    fftfreqs = np.linspace(0, sr / 2, n_freqs)
    mel_f = _mel_to_hz(np.linspace(_hz_to_mel(0.0), _hz_to_mel(sr / 2), n_mels + 2))
    fdiff = np.diff(mel_f)
    ramps = mel_f[:, None] - fftfreqs[None, :]
    lower = -ramps[:-2] / fdiff[:-1, None]
    upper = ramps[2:] / fdiff[1:, None]
    w = np.maximum(0, np.minimum(lower, upper))
    enorm = 2.0 / (mel_f[2: n_mels + 2] - mel_f[:n_mels])
    return (w * enorm[:, None]).astype(np.float32)


@dataclass
class MelConstants:
    n_mels: int
    window: torch.Tensor      # [400]
    cos_basis: torch.Tensor   # [400, 224]
    sin_basis: torch.Tensor   # [400, 224]
    filters: torch.Tensor     # [n_mels, 201]

    @staticmethod
    def create(n_mels: int = 80) -> "MelConstants":
        n = np.arange(400)
        window = (0.5 - 0.5 * np.cos(2 * np.pi * n / 400)).astype(np.float32)  # periodic Hann
        k = np.arange(224)
        ang = 2 * np.pi * np.outer(n, k) / 400
        cosb = np.cos(ang)
        sinb = -np.sin(ang)
        cosb[:, 201:] = 0
        sinb[:, 201:] = 0
        return MelConstants(n_mels, torch.from_numpy(window), torch.from_numpy(cosb.astype(np.float32)),
                            torch.from_numpy(sinb.astype(np.float32)),
                            torch.from_numpy(mel_filterbank(n_mels=n_mels)))

    def to(self, device) -> "MelConstants":
        device = torch.device(device)
        if self.window.device == device:
            return self
        cache = self.__dict__.setdefault("_dev_cache", {})
        key = str(device)
        if key not in cache:
            cache[key] = MelConstants(self.n_mels, self.window.to(device), self.cos_basis.to(device),
                                      self.sin_basis.to(device), self.filters.to(device))
        return cache[key]


def log_mel(audio: torch.Tensor, c: MelConstants) -> torch.Tensor:
    """Whisper log-mel (whisper/audio.py semantics) in fp32: [B, n_mels, n//160]."""
    win = c.window.to(audio.device)
    st = torch.stft(audio.float(), 400, 160, window=win, return_complex=True, center=True,
                    pad_mode="reflect")
    mag = st[..., :-1].abs() ** 2
    mel = c.filters.to(audio.device) @ mag
    lg = torch.clamp(mel, min=1e-10).log10()
    mx = lg.amax(dim=(-2, -1), keepdim=True)
    lg = torch.maximum(lg, mx - 8.0)
    return (lg + 4.0) / 4.0


def im2col_k3(x, strides, B, C, L, stride):
    Lout = (L - 1) // stride + 1
    flat = x.reshape(-1)
    b = torch.arange(B, device=x.device)[:, None, None, None]
    to = torch.arange(Lout, device=x.device)[None, :, None, None]
    c = torch.arange(C, device=x.device)[None, None, :, None]
    k = torch.arange(3, device=x.device)[None, None, None, :]
    t = to * stride + k - 1
    valid = (t >= 0) & (t < L)
    idx = b * strides[0] + c * strides[1] + t.clamp(0, L - 1) * strides[2]
    vals = flat[idx.reshape(-1)].reshape(B, Lout, C, 3)
    vals = torch.where(valid.expand(B, Lout, C, 3), vals, torch.zeros((), dtype=x.dtype))
    return vals.reshape(B * Lout, 3 * C)


# ----------------------------------------------------------- decode slabs
def shuffle_weight(w):
    N, K = w.shape
    return w.reshape(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().reshape(
        N // 16, K // 32, 64, 8)


def unshuffle_weight(wp):
    T, KS = wp.shape[:2]
    return wp.reshape(T, KS, 4, 16, 8).permute(0, 3, 1, 2, 4).reshape(T * 16, KS * 32)


def skinny_gemm(x, wp, S):
    w = unshuffle_weight(wp)
    Mpad, K = x.shape
    kc = K // S
    parts = [x[:, s * kc:(s + 1) * kc].float() @ w[:, s * kc:(s + 1) * kc].float().t() for s in range(S)]
    return torch.stack(parts, 0)


def slab_rmsnorm(part, residual, w, eps, row_idx=None, write_residual=True):
    tot = part.sum(0)
    idx = row_idx.long() if row_idx is not None else torch.arange(part.shape[1], device=part.device)
    s = (tot[idx] + residual[idx].float()).to(residual.dtype)
    if write_residual:
        residual[idx] = s
    xf = s.float()
    y = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    return y.to(residual.dtype)


def slab_rope_append(part, positions, cos_sin, k_cache, v_cache, slots, H, Hkv, D, bias=None):
    tot = part.sum(0)
    if bias is not None:
        tot = tot + bias.float()
    qkv = tot.to(torch.bfloat16)
    rope_kv_append(qkv, positions, cos_sin, k_cache, v_cache, slots, H, Hkv, D)
    return qkv[:, : H * D].contiguous()


def slab_layernorm(part, residual, w, b, eps, bias=None, row_idx=None, write_residual=True):
    tot = part.sum(0)
    if bias is not None:
        tot = tot + bias.float()
    tot = tot.to(torch.bfloat16).float()
    idx = row_idx.long() if row_idx is not None else torch.arange(part.shape[1], device=part.device)
    s = (tot[idx] + residual[idx].float()).to(residual.dtype)
    if write_residual:
        residual[idx] = s
    return torch.nn.functional.layer_norm(s.float(), (s.shape[-1],), w.float(), b.float(),
                                          eps).to(residual.dtype)


def slab_bias_act(part, bias=None, act="none"):
    tot = part.sum(0)
    if bias is not None:
        tot = tot + bias.float()
    if act == "gelu":
        tot = torch.nn.functional.gelu(tot.to(torch.bfloat16).float())
    return tot.to(torch.bfloat16)


def slab_silu_mul(part):
    return silu_mul(part.sum(0).to(torch.bfloat16))


# ------------------------------------------------------------------ VITS / HiFi-GAN
def conv1d(x, w, bias=None, *, dil=1, pad=0, stride=1, pre_slope=None, act=None, res=None,
           alpha=1.0, acc=None, lens=None, Tout=None, ostride=1, ophase=0, Tq=None):
    """Reference of loqa_conv1d: x [B, Tin, Cin] (channels-last), w [Cout, Cin, K]
    (torch layout) -> y [B, Tout, Cout'] following the kernel's epilogue order.
    Returns float32 (callers round)."""
    B, Tin, Cin = x.shape
    xf = x.float()
    if pre_slope is not None:
        xf = torch.nn.functional.leaky_relu(xf, pre_slope)
    xf = xf.to(torch.bfloat16).float()  # the kernel feeds bf16 operands to the MFMA
    y = torch.nn.functional.conv1d(xf.transpose(1, 2), w.float(), None, stride=stride, padding=pad,
                                   dilation=dil).transpose(1, 2)
    if Tq is not None:
        y = y[:, :Tq]
    if bias is not None:
        y = y + bias.float()
    if act == "relu":
        y = torch.relu(y)
    elif act == "tanh":
        y = torch.tanh(y)
    elif act == "gated":
        Hh = y.shape[-1] // 2
        a, g = y[..., :Hh].to(torch.bfloat16).float(), y[..., Hh:].to(torch.bfloat16).float()
        y = torch.tanh(a) * torch.sigmoid(g)
    T_out = Tout if Tout is not None else y.shape[1] * ostride + ophase
    full = torch.zeros(B, T_out, y.shape[-1], dtype=torch.float32, device=x.device)
    q = torch.arange(y.shape[1], device=x.device)
    oi = q * ostride + ophase
    ok = (oi >= 0) & (oi < T_out)
    full[:, oi[ok]] = y[:, q[ok]]
    idx = oi[ok]
    if res is not None:
        full[:, idx] += res[:, idx].float()
    full[:, idx] *= alpha
    if acc is not None:
        full[:, idx] += acc[:, idx].float()
    if lens is not None:
        t = torch.arange(T_out, device=x.device)
        full = full * (t[None, :] < lens[:, None].to(x.device)).float()[..., None]
    return full


def conv_transpose1d(x, w, bias=None, *, stride, padding, pre_slope=None):
    """torch ConvTranspose1d on channels-last x; w [Cin, Cout, K] torch layout."""
    xf = x.float()
    if pre_slope is not None:
        xf = torch.nn.functional.leaky_relu(xf, pre_slope)
    xf = xf.to(torch.bfloat16).float()
    y = torch.nn.functional.conv_transpose1d(xf.transpose(1, 2), w.float(),
                                             None if bias is None else bias.float(),
                                             stride=stride, padding=padding)
    return y.transpose(1, 2)


def relpos_attention(qkv, emb_k, emb_v, lens, H, D, window, scale):
    B, T, _ = qkv.shape
    C = H * D
    q = qkv[..., :C].float().view(B, T, H, D).transpose(1, 2) * scale
    k = qkv[..., C:2 * C].float().view(B, T, H, D).transpose(1, 2)
    v = qkv[..., 2 * C:3 * C].float().view(B, T, H, D).transpose(1, 2)
    s = q @ k.transpose(-1, -2)
    idx = torch.arange(T, device=qkv.device)
    rel = idx[None, :] - idx[:, None]
    inwin = rel.abs() <= window
    ek = emb_k.float()
    rl = torch.einsum("bhid,rd->bhir", q, ek)  # [B,H,T,2w+1]
    ridx = (rel + window).clamp(0, 2 * window)
    s = s + torch.where(inwin, rl.gather(-1, ridx[None, None].expand(B, H, T, T)),
                        torch.zeros((), device=qkv.device))
    L = lens.to(qkv.device) if lens is not None else torch.full((B,), T, device=qkv.device)
    valid = idx[None, :] < L[:, None]
    m = valid[:, None, :, None] & valid[:, None, None, :]
    s = s.masked_fill(~m, -1e4)
    p = torch.softmax(s, -1)
    o = p @ v
    pw = torch.where(inwin, p, torch.zeros((), device=qkv.device))
    pr = torch.zeros(B, H, T, 2 * window + 1, device=qkv.device)
    pr.scatter_add_(-1, ridx[None, None].expand(B, H, T, T), pw)
    o = o + pr @ emb_v.float()
    o = o * valid[:, None, :, None]
    return o.transpose(1, 2).reshape(B, T, C)


def expand_sample(stats, cum, flen, F, noise_scale, noise=None):
    """z[b, f] = m[i(f)] + noise * exp(logs[i(f)]) * noise_scale."""
    B, T, C2 = stats.shape
    C = C2 // 2
    z = torch.zeros(B, F, C, device=stats.device)
    for b in range(B):
        n = int(flen[b])
        f = torch.arange(n, device=stats.device)
        i = torch.searchsorted(cum[b].to(stats.device), f, right=True)
        m, lg = stats[b, i, :C].float(), stats[b, i, C:].float()
        e = noise[b, :n].float() if noise is not None else torch.zeros_like(m)
        z[b, :n] = m + e * torch.exp(lg) * noise_scale
    return z


# ------------------------------------------------------------ fused decode GEMMs
def perm_rope_qkv(H, Hkv, D):
    """Row order of the fused qkv weight: per q / k head, 16-row pair tiles
    holding 8 first-half rows c0.. and their RoPE partners c0 + D/2 (the
    epilogue pairs lane l with lane l ^ 32); v rows unchanged."""
    half = D // 2
    rows = []
    for base, n in ((0, H), (H * D, Hkv)):
        for h in range(n):
            for s in range(D // 16):
                c0 = 8 * s
                rows += list(range(base + h * D + c0, base + h * D + c0 + 8))
                rows += list(range(base + h * D + half + c0, base + h * D + half + c0 + 8))
    rows += list(range((H + Hkv) * D, (H + 2 * Hkv) * D))
    return torch.tensor(rows, dtype=torch.long)


def perm_gate_up(F):
    """Row order of the fused gate|up weight: 16-row pair tiles of (8 gate, 8 up)."""
    rows = []
    for t in range(F // 8):
        rows += list(range(8 * t, 8 * t + 8)) + list(range(F + 8 * t, F + 8 * t + 8))
    return torch.tensor(rows, dtype=torch.long)


def swiglu_pairs(y):
    """silu(gate) * up of a ``perm_gate_up``-ordered product [M, 2F] (16-column
    pair tiles: 8 gate, 8 up) -> [M, F] (f32)."""
    M, F2 = y.shape
    t = y.float().view(M, F2 // 16, 2, 8)
    g, u = t[:, :, 0], t[:, :, 1]
    g = g.to(torch.bfloat16).float()
    u = u.to(torch.bfloat16).float()
    return (torch.nn.functional.silu(g) * u).reshape(M, F2 // 2)


def fused_ln_stats(rowsq_in, rowsum_in, eps, K):
    """LayerNorm (mean, 1/std) per row from per-tile partial sums [tiles, Mpad]."""
    mean = rowsum_in.float().sum(0) / K
    var = (rowsq_in.float().sum(0) / K - mean * mean).clamp_min(0.0)
    return mean, torch.rsqrt(var + eps)


def fused_row_scale(rowsq_in, eps, K):
    """RMSNorm row scale 1/rms from per-tile partial sums of squares [tiles, Mpad]."""
    tot = rowsq_in.float().sum(0)  # [Mpad]
    return torch.rsqrt(tot / K + eps)


def _fmix32(h: torch.Tensor) -> torch.Tensor:
    m = 0xFFFFFFFF
    h = h ^ (h >> 16)
    h = (h * 0x85EBCA6B) & m
    h = h ^ (h >> 13)
    h = (h * 0xC2B2AE35) & m
    return h ^ (h >> 16)


def init_uniform4(rows: int, cols: int, ld: int, row0: int, col0: int, s: int,
                  scale: float) -> torch.Tensor:
    """CPU twin of elementwise.hip ``init_uniform4_kernel``: bf16 [rows, cols],
    element (r, c) = scale * (sum_k fmix32(4 idx + k + s) / 2^32 - 2) with
    idx = (row0 + r) * ld + col0 + c (uint32 arithmetic, exact f32 sums)."""
    r = torch.arange(rows, dtype=torch.int64)[:, None] + row0
    c = torch.arange(cols, dtype=torch.int64)[None, :] + col0
    idx = (r * ld + c) & 0xFFFFFFFF
    acc = torch.zeros(rows, cols, dtype=torch.float32)
    for k in range(4):
        h = _fmix32((idx * 4 + k + s) & 0xFFFFFFFF)
        acc += (h >> 8).to(torch.float32) * (1.0 / 16777216.0)
    return ((acc - 2.0) * torch.tensor(scale, dtype=torch.float32)).to(torch.bfloat16)


# ------------------------------------------------------------ whole models
def _causal_attn(q, k, v, G: int, scale: float, q0: int = 0):
    """q [T, H, D], k / v [L, Hkv, D] (fp32); query i sits at position q0 + i."""
    k = k.repeat_interleave(G, dim=1)
    v = v.repeat_interleave(G, dim=1)
    s = torch.einsum("qhd,khd->hqk", q, k) * scale
    qpos = torch.arange(q.shape[0], device=q.device) + q0
    kpos = torch.arange(k.shape[0], device=q.device)
    s = s.masked_fill(kpos[None, None, :] > qpos[None, :, None], float("-inf"))
    return torch.einsum("hqk,khd->qhd", torch.softmax(s, dim=-1), v)


@torch.no_grad()
def llama_forward_ref(w, tokens: list[int]) -> torch.Tensor:
    """fp32 forward of a whole Llama model (``LlamaWeights``, unsharded, with
    its row-major layer copies) over one sequence at positions 0..T-1; returns
    fp32 logits [T, V]. Every weight is the model's own bf16 tensor upcast:
    the oracle of the fused bf16 decode path (tests/test_engine_gpu.py)."""
    cfg = w.cfg
    H, Hkv, D, F = w.h, w.hkv, cfg.head_dim, w.f
    dev = w.embed.device
    t = torch.tensor(tokens, dtype=torch.long, device=dev)
    T = t.numel()
    cs = w.cos_sin[:T].float()

    def rms(x, g):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + cfg.norm_eps) * g.float()
    x = w.embed[t].float()
    for L in w.layers:
        h = rms(x, L["attn_norm"])
        qkv = h @ L["wqkv"].float().t()
        q = apply_rope(qkv[:, : H * D].view(T, H, D), cs)
        k = apply_rope(qkv[:, H * D:(H + Hkv) * D].view(T, Hkv, D), cs)
        v = qkv[:, (H + Hkv) * D:].view(T, Hkv, D)
        a = _causal_attn(q, k, v, H // Hkv, 1.0 / math.sqrt(D)).reshape(T, H * D)
        x = x + a @ L["wo"].float().t()
        gu = rms(x, L["mlp_norm"]) @ L["w_gate_up"].float().t()
        x = x + (torch.nn.functional.silu(gu[:, :F]) * gu[:, F:]) @ L["w_down"].float().t()
    return rms(x, w.final_norm) @ w.lm_head.float().t()


@torch.no_grad()
def whisper_decoder_ref(w, tokens: list[int], enc: torch.Tensor) -> torch.Tensor:
    """fp32 Whisper decoder (``WhisperWeights``) over one sequence at positions
    0..T-1 with cross-attention over the encoder states ``enc`` [T_enc, d];
    returns fp32 logits [T, vocab] (tied embedding)."""
    cfg = w.cfg
    d, H, D = cfg.d_model, cfg.n_heads, cfg.head_dim
    dev = w.tok_embed.device
    t = torch.tensor(tokens, dtype=torch.long, device=dev)
    T = t.numel()
    e = enc.float()

    def ln(x, g, b):
        return torch.nn.functional.layer_norm(x, (d,), g.float(), b.float(), 1e-5)

    def lin(x, W, b):
        return x @ W.float().t() + b.float()

    def gelu(x):
        return 0.5 * x * (1.0 + torch.erf(x * 0.70710678118654752))
    x = w.tok_embed[t].float() + w.dec_pos[:T].float()
    sc = 1.0 / math.sqrt(D)
    for L in w.dec:
        qkv = lin(ln(x, L["ln1_w"], L["ln1_b"]), L["wqkv"], L["bqkv"])
        q, k, v = (qkv[:, i * d:(i + 1) * d].view(T, H, D) for i in range(3))
        x = x + lin(_causal_attn(q, k, v, 1, sc).reshape(T, d), L["wo"], L["bo"])
        q = lin(ln(x, L["lnx_w"], L["lnx_b"]), L["xq"], L["xq_b"]).view(T, H, D)
        kv = lin(e, L["xkv"], L["xkv_b"])
        Te = e.shape[0]
        k, v = kv[:, :d].view(Te, H, D), kv[:, d:].view(Te, H, D)
        p = torch.softmax(torch.einsum("qhd,khd->hqk", q, k) * sc, dim=-1)
        x = x + lin(torch.einsum("hqk,khd->qhd", p, v).reshape(T, d), L["xo"], L["xo_b"])
        x = x + lin(gelu(lin(ln(x, L["ln2_w"], L["ln2_b"]), L["fc1"], L["fc1_b"])), L["fc2"],
                    L["fc2_b"])
    return ln(x, w.dec_ln_w, w.dec_ln_b) @ w.tok_embed.float().t()


# ---------------------------------------------------------------------------
# Sequence-mixer building blocks of the hybrid decoders (models/pipizen.py):
# Dynamic-Tanh norm, interleaved rotary tables with YaRN, latent (compressed
# KV) attention with a softmax sink, decayed linear attention with a carried
# state, and a grouped top-k expert router. Everything the recurrences and the
# softmax touch is f32; ``out_dtype`` is the activation dtype of the caller.
def dyt_norm(x, w, b, alpha: float, out_dtype, row_idx=None):
    """tanh(alpha x) * w + b (no mean, no variance)."""
    if row_idx is not None:
        x = x.index_select(0, row_idx.long())
    return (torch.tanh(x.float() * alpha) * w.float() + b.float()).to(out_dtype)


def dyt_add_norm(resid, y, post, nxt, out_dtype):
    """resid (f32, in place) += dyt(y; post); returns dyt(resid; nxt) or None."""
    resid.add_(dyt_norm(y, post[0], post[1], post[2], torch.float32))
    if nxt is None:
        return None
    return dyt_norm(resid, nxt[0], nxt[1], nxt[2], out_dtype)


def rope_table_pairs(dims: int, max_pos: int, base: float, yarn: tuple | None = None,
                     device=None) -> torch.Tensor:
    """[max_pos, dims/2, 2] f32 (cos, sin) for the interleaved layout (entry 2i
    rotates with entry 2i+1). ``yarn`` = (factor, original, fast, slow): each
    frequency is a blend of itself and itself / factor, the blend ramping
    between the dimensions whose wavelength fits the original context ``fast``
    and ``slow`` times; cos and sin carry the magnitude 0.1 ln(factor) + 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    mag = 1.0
    if yarn is not None:
        factor, orig, fast, slow = (float(v) for v in yarn)

        def turn(t):   # the dimension index whose wavelength makes t turns in the original context
            return dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(base))
        lo = max(math.floor(turn(fast)), 0)
        hi = min(math.ceil(turn(slow)), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        f = f / factor * ramp + f * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * f[None, :]
    return (torch.stack([ang.cos(), ang.sin()], dim=-1) * mag).float().to(device)


def rotate_pairs(x, cs, dims: int):
    """x [T, ..., n] (any float) -> f32 copy whose first ``dims`` entries are
    rotated pairwise by cs [T, dims/2, 2]."""
    out = x.float().clone()
    u, v = out[..., 0:dims:2].clone(), out[..., 1:dims:2].clone()
    c, s = cs[..., 0], cs[..., 1]
    while c.dim() < u.dim():
        c, s = c.unsqueeze(1), s.unsqueeze(1)
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def latent_append(z, norm_w, eps: float, positions, cos_sin, cache, slots, R: int, dims: int):
    """z [T, R + Dr]: the first R entries RMS-normed (weight ``norm_w``) are
    the latent, the rest the shared rotary key part; both go to the paged
    cache [blocks, BLK, R + Dr] at ``slots`` (-1: padding row)."""
    zf = z.float()
    c = zf[:, :R]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    kr = rotate_pairs(zf[:, R:], cos_sin[positions.long()], dims)
    row = torch.cat([c, kr], dim=-1).to(cache.dtype)
    sl = slots.long()
    ok = sl >= 0
    blk = cache.shape[1]
    cache[(sl // blk)[ok], (sl % blk)[ok]] = row[ok]


def latent_attention(qa, qr, cache, cu_q, ctx_lens, block_tables, positions, cos_sin, sink,
                     scale: float, R: int, dims: int, out):
    """Causal attention of one shared key/value stream per token (the cached
    latent row): score = (qa . c + rot(qr) . k_rot) * scale, softmax whose
    denominator also holds exp(sink[h]); out[h, t] = sum_j p_j c_j.
    qa [H, T, R], qr [T, H, Dr] (unrotated), out [H, T, R]."""
    H = qa.shape[0]
    blk = cache.shape[1]
    cu = cu_q.tolist()
    qrot = rotate_pairs(qr, cos_sin[positions.long()], dims)          # [T, H, Dr] f32
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        L = int(ctx_lens[b])
        idx = torch.arange(L, device=cache.device)
        rows = cache[block_tables[b].long()[idx // blk], idx % blk].float()   # [L, R + Dr]
        s = torch.einsum("htr,lr->htl", qa[:, q0:q1].float(), rows[:, :R])
        s = (s + torch.einsum("thr,lr->htl", qrot[q0:q1], rows[:, R:])) * scale
        qpos = positions[q0:q1].long()
        s = s.masked_fill(idx[None, None, :] > qpos[None, :, None], float("-inf"))
        if sink is not None:
            s = torch.cat([s, sink.float()[:, None, None].expand(H, q1 - q0, 1)], dim=-1)
        p = torch.softmax(s, dim=-1)[..., :L]
        out[:, q0:q1] = torch.einsum("htl,lr->htr", p, rows[:, :R]).to(out.dtype)
    return out


def state_scan(act, H: int, D: int, Dv: int, q_off: int, k_off: int, v_off: int, hpg: int, state,
               state_slots, cu_q, positions, decay=None, tok=None, skip=None):
    """Linear recurrence with a carried matrix state, token by token in f32:

        S <- a S + k (c v)^T,    o = S^T q + skip_h v

    per sequence and head, with a = ``decay[h]`` (constant) or ``tok[t, h, 0]``
    (per token) and c = 1 or ``tok[t, h, 1]``. ``act`` f32 [T, W] holds the
    inputs: head h reads q at ``q_off + (h // hpg) D``, k at ``k_off + (h //
    hpg) D`` (``hpg`` neighbouring heads share one q / k group) and v at
    ``v_off + h Dv``. The state [slots, H, D, Dv] is read at the sequence's
    slot (zero when the step's first position is 0) and written back.
    Returns o f32 [T, H Dv]."""
    T = act.shape[0]
    a = act.float()
    hg = torch.arange(H, device=act.device) // hpg
    cols = torch.arange(D, device=act.device)
    q = a[:, (q_off + hg[:, None] * D + cols[None, :]).reshape(-1)].view(T, H, D)
    k = a[:, (k_off + hg[:, None] * D + cols[None, :]).reshape(-1)].view(T, H, D)
    v = a[:, v_off:v_off + H * Dv].view(T, H, Dv)
    o = torch.zeros(T, H, Dv, dtype=torch.float32, device=act.device)
    cu = cu_q.tolist()
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        slot = int(state_slots[b])
        S = torch.zeros_like(state[slot]) if int(positions[q0]) == 0 else state[slot].clone()
        for t in range(q0, q1):
            lam = decay.float()[:, None, None] if tok is None else tok[t, :, 0].float()[:, None, None]
            vt = v[t] if tok is None else v[t] * tok[t, :, 1].float()[:, None]
            S = lam * S + k[t][:, :, None] * vt[:, None, :]
            o[t] = torch.einsum("hde,hd->he", S, q[t])
            if skip is not None:
                o[t] += skip.float()[:, None] * v[t]
        state[slot] = S
    return o.view(T, H * Dv)


def lightning_scan(qkv, H: int, D: int, Dv: int, state, state_slots, cu_q, positions, decay):
    """Decayed linear attention, token by token: S <- decay_h S + k v^T,
    o = S^T q with q, k, v = silu of the [q | k | v] columns of ``qkv``. The
    state [slots, H, D, Dv] (f32) is read at the sequence's slot (zero when
    the step's first position is 0) and written back. Returns o f32 [T, H Dv]."""
    a = torch.nn.functional.silu(qkv[:, :2 * H * D + H * Dv].float())
    return state_scan(a, H, D, Dv, 0, H * D, 2 * H * D, 1, state, state_slots, cu_q, positions,
                      decay=decay)


def gated_rmsnorm(o, w, gate, eps: float, out_dtype, groups: int = 1, silu_first: bool = False,
                  gate_act: str = "sigmoid"):
    """rmsnorm(o) * w * sigmoid(gate), the row normalised as a whole (``gate_act``
    "silu": times silu(gate) instead); with ``silu_first``: rmsnorm(o *
    silu(gate)) * w (the gate before the norm). ``groups`` > 1 normalises the
    row in that many equal parts."""
    of, g = o.float(), gate.float()
    T, n = of.shape
    if silu_first:
        of = of * torch.nn.functional.silu(g)
    y = of.view(T, groups, n // groups)
    y = (y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)).view(T, n) * w.float()
    if not silu_first:
        y = y * (torch.sigmoid(g) if gate_act == "sigmoid" else torch.nn.functional.silu(g))
    return y.to(out_dtype)


def moe_route(z, correction, n_groups: int, keep: int, top: int, bias=None,
              top_softmax: bool = False, sigmoid: bool = False, group_rank: int = 1):
    """z f32 [T, E] router logits (+ ``bias`` [E]) -> (expert index int32 [T, top],
    weight f32 [T, top]). Default: scores are softmax(z); experts are chosen by
    score + correction among the ``keep`` best of ``n_groups`` equal groups of
    neighbours (a group's rank is its best choice score); the weights are the
    plain scores. ``top_softmax``: the ``top`` largest logits are chosen and the
    weights are the softmax over the chosen logits only. ``sigmoid``: the scores
    are sigmoid(z) instead of the softmax. ``group_rank`` n: a group ranks by the
    sum of its n best choice scores."""
    z = z.float() if bias is None else z.float() + bias.float()
    if top_softmax:
        best = z.topk(top, dim=-1)
        return best.indices.to(torch.int32), torch.softmax(best.values, dim=-1)
    s = torch.sigmoid(z) if sigmoid else torch.softmax(z, dim=-1)
    choice = s if correction is None else s + correction.float()
    if n_groups > 1 and keep < n_groups:
        T, E = s.shape
        per = E // n_groups
        gs = choice.view(T, n_groups, per).topk(min(max(group_rank, 1), per), dim=-1).values.sum(-1)
        kept = gs.topk(keep, dim=-1).indices
        ok = torch.zeros(T, n_groups, dtype=torch.bool, device=z.device).scatter_(1, kept, True)
        choice = choice.masked_fill(~ok.repeat_interleave(per, dim=1), float("-inf"))
    idx = choice.topk(top, dim=-1).indices
    return idx.to(torch.int32), s.gather(1, idx)


def moe_experts(h, idx, wt, w_gate_up, w_down, out_dtype, gated: bool = True):
    """Weighted sum of each token's chosen experts: expert e < E is a
    feed-forward - gated: down(silu(gate x) * (up x)) with w_gate_up [E, 2F, d]
    = gate | up rows; not gated: down(relu(up x)^2) with w_gate_up [E, F, d] -
    and w_down [E, d, F]; an index >= E is an identity expert (its output is
    h). Returns f32 [T, d]; the expert outputs are rounded to ``out_dtype``
    first, as GEMM outputs."""
    T, d = h.shape
    E = w_gate_up.shape[0]
    F = w_gate_up.shape[1] // 2 if gated else w_gate_up.shape[1]
    out = torch.zeros(T, d, dtype=torch.float32, device=h.device)
    for k in range(idx.shape[1]):
        e = idx[:, k].long()
        ident = e >= E
        out += torch.where(ident[:, None], wt[:, k:k + 1] * h.float(), torch.zeros_like(out))
        for ee in e[~ident].unique().tolist():
            rows = (e == ee).nonzero()[:, 0]
            x = h[rows].to(out_dtype)
            gu = torch.nn.functional.linear(x, w_gate_up[ee])
            if gated:
                a = (torch.nn.functional.silu(gu[:, :F].float()) * gu[:, F:].float()).to(out_dtype)
            else:
                a = torch.relu(gu.float()).pow(2).to(out_dtype)
            y = torch.nn.functional.linear(a, w_down[ee])
            out[rows] += wt[rows, k:k + 1] * y.float()
    return out


# ---------------------------------------------------------------------------
# Building blocks of decoders with per-sequence row state (models/sodonex.py):
# token shift, short causal convolutions with a carried tail, whole-projection
# RMS norm + rotate-half rotary + paged K/V append, chunked sigmoid attention
# with a per-head output gate, and a scalar-gain RMS norm on the residual step.
def rope_table_half(dims: int, max_pos: int, base: float, device=None) -> torch.Tensor:
    """[max_pos, dims/2, 2] f32 (cos, sin) for the rotate-half layout (entry i
    turns with entry i + dims/2 by position * base^(-2i/dims)); angles in f64."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / max(dims, 1))
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * f[None, :]
    return torch.stack([ang.cos(), ang.sin()], dim=-1).float().to(device)


def token_shift(x, mu, prev, state_slots, cu_q, positions, out_dtype):
    """h_t = x_t + (x_{t-1} - x_t) * mu; the row before a feed's first token
    is the sequence's saved row ``prev[slot]`` (zeros at position 0)."""
    xf = x.float()
    h = torch.empty_like(xf)
    cu = cu_q.tolist()
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        first = torch.zeros_like(xf[0]) if int(positions[q0]) == 0 else prev[int(state_slots[b])]
        before = torch.cat([first[None], xf[q0:q1 - 1]])
        h[q0:q1] = xf[q0:q1] + (before - xf[q0:q1]) * mu.float()
    return h.to(out_dtype)


def seq_state_save(x, u, prev, tail, state_slots, cu_q, positions):
    """After a step: prev[slot] = the feed's last row of x; tail[slot]
    [taps - 1, C] = the last taps - 1 rows of the projections u[:, :C] (older
    rows move up when the feed is shorter; zeros before the sequence's start)."""
    cu = cu_q.tolist()
    keep, C = tail.shape[1], tail.shape[2]
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        slot = int(state_slots[b])
        if prev is not None:
            prev[slot] = x[q1 - 1].float()
        if keep:
            old = torch.zeros_like(tail[slot]) if int(positions[q0]) == 0 else tail[slot].clone()
            rows = torch.cat([old, u[q0:q1, :C].float()])
            tail[slot] = rows[-keep:]


def conv_norm_rope_append(u, conv_w, tail, state_slots, cu_q, positions, q_norm, k_norm, eps: float,
                          cos_sin, dims: int, H: int, G: int, D: int, k_cache, v_cache, slots,
                          out_dtype):
    """u [T, >= (H + G) D]: the projected q | k rows. Causal per-channel
    convolution (weights conv_w tap-major [taps, (H + G) D], the rows before the feed from
    ``tail[slot]``), then: v = the convolved k; q and k each RMS-normed over the
    whole projection (weights q_norm / k_norm), rotated (rotate-half, the first
    ``dims`` entries of every head); k goes to its paged cache [blocks, BLK, G D]
    and v to its transposed pages [blocks, G D, BLK] at ``slots``; returns q [T, H D]."""
    T = u.shape[0]
    taps, C = conv_w.shape
    Cq = H * D
    cu = cu_q.tolist()
    y = torch.zeros(T, C, dtype=torch.float32, device=u.device)
    w = conv_w.float()
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        if taps > 1:
            old = torch.zeros_like(tail[0]) if int(positions[q0]) == 0 else \
                tail[int(state_slots[b])]
            rows = torch.cat([old.float(), u[q0:q1, :C].float()])
        else:
            rows = u[q0:q1, :C].float()
        n = q1 - q0
        for j in range(taps):
            y[q0:q1] += rows[j:j + n] * w[j]
    yq, yk = y[:, :Cq], y[:, Cq:]
    v = yk.to(v_cache.dtype)
    q = yq * torch.rsqrt(yq.pow(2).mean(-1, keepdim=True) + eps) * q_norm.float()
    k = yk * torch.rsqrt(yk.pow(2).mean(-1, keepdim=True) + eps) * k_norm.float()
    cs = cos_sin[positions[:T].long()]                          # [T, dims/2, 2]

    def turn(x, heads):
        x = x.view(T, heads, D).clone()
        half = dims // 2
        a, bb = x[..., :half].clone(), x[..., half:dims].clone()
        c, s = cs[:, None, :, 0], cs[:, None, :, 1]
        x[..., :half] = a * c - bb * s
        x[..., half:dims] = bb * c + a * s
        return x.view(T, heads * D)
    if dims:
        q, k = turn(q, H), turn(k, G)
    sl = slots[:T].long()
    ok = sl >= 0
    blk = k_cache.shape[1]
    k_cache[(sl // blk)[ok], (sl % blk)[ok]] = k.to(k_cache.dtype)[ok]
    v_cache[(sl // blk)[ok], :, (sl % blk)[ok]] = v[ok]
    return q.to(out_dtype)


def sigmoid_attention(q, k_cache, v_cache, cu_q, ctx_lens, block_tables, positions, head_bias,
                      gate, scale: float, chunk: int, H: int, G: int, D: int, out_dtype):
    """q [T, H D] against the paged k cache [blocks, BLK, G D] and the
    transposed v pages [blocks, G D, BLK]: a query at
    position p sees keys j <= p (with ``chunk`` > 0 only those of its own
    chunk, j // chunk == p // chunk); a visible key weighs
    sigmoid(q . k * scale + head_bias[h]), not normalised over keys; head h's
    output is multiplied by sigmoid(gate[t, h]). Returns [T, H D]."""
    T = q.shape[0]
    blk = k_cache.shape[1]
    rep = H // G
    cu = cu_q.tolist()
    out = torch.zeros(T, H, D, dtype=torch.float32, device=q.device)
    qf = q.float().view(T, H, D)
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        L = int(ctx_lens[b])
        idx = torch.arange(L, device=q.device)
        tab = block_tables[b].long()
        kk = k_cache[tab[idx // blk], idx % blk].float().view(L, G, D)
        vv = v_cache[tab[idx // blk], :, idx % blk].float().view(L, G, D)
        qpos = positions[q0:q1].long()
        seen = idx[None, :] <= qpos[:, None]
        if chunk > 0:
            seen &= (idx[None, :] // chunk) == (qpos[:, None] // chunk)
        for h in range(H):
            s = qf[q0:q1, h] @ kk[:, h // rep].T * scale + head_bias[h].float()
            w = torch.sigmoid(s) * seen
            out[q0:q1, h] = w @ vv[:, h // rep]
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.view(T, H * D).to(out_dtype)


def scalar_rms_add(resid, y, g: float, eps: float, mult: float, out_dtype):
    """resid (f32, in place) += mult * y / rms(y) * g; returns resid in
    ``out_dtype`` (None: nothing)."""
    yf = y.float()
    resid.add_(yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * (g * mult))
    return None if out_dtype is None else resid.to(out_dtype)


def scalar_rms_norm(x, g: float, eps: float, row_idx=None):
    """f32 rows of x / rms(x) * g (``row_idx`` gathers rows first)."""
    if row_idx is not None:
        x = x.index_select(0, row_idx.long())
    xf = x.float()
    return xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * g


# ---------------------------------------------------------------------------
# Building blocks of pre-norm decoders with softmax attention over paged K / V
# and Mamba-2 layers (models/movinex.py): RMS norm with a weight stored around
# zero fused with the layer-scaled residual step, per-head q / k preparation
# (interleaved rotary, weightless RMS norm, query temperature) with the paged
# append, softmax attention with a sliding window, kept first tokens and score
# soft-capping, and the Mamba-2 input stage (convolution, step sizes, decays).
def rms1p_norm(x, w, eps: float, out_dtype, row_idx=None):
    """x / sqrt(mean(x^2) + eps) * (1 + w) over rows (``row_idx`` gathers first)."""
    if row_idx is not None:
        x = x.index_select(0, row_idx.long())
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps) * (1.0 + w.float())).to(out_dtype)


def scaled_add_rms1p(resid, y, ls, nxt, eps: float, out_dtype):
    """resid (f32, in place) += ls * y per coordinate; returns
    rms1p_norm(resid; nxt) in ``out_dtype``, or None without ``nxt``."""
    resid.add_(y.float() * ls.float())
    return None if nxt is None else rms1p_norm(resid, nxt, eps, out_dtype)


def qk_prep_append(u, H: int, G: int, D: int, Dv: int, v_off: int, cos_sin, dims: int, eps: float,
                   q_temp, positions, k_cache, v_cache, slots, out_dtype, q_norm=None, k_norm=None):
    """u [T, >= H D + G D (+ G Dv)]: projected q | k (| v) rows. Per head: the
    first ``dims`` entries of q and k rotate pairwise (2i with 2i + 1) by the
    position's angles, then each head's q and k is divided by its root mean
    square (eps inside the root, no weight); q is multiplied by the position's
    temperature 1 + coef ln(floor((p + 1) / every) + 1) when ``q_temp`` =
    (coef, every). k goes to its pages [blocks, BLK, G D]; the value rows - the
    columns at ``v_off``, or with ``v_off`` < 0 the k columns as projected - go to
    theirs [blocks, BLK, G Dv] at ``slots`` (-1: padding row). Returns q [T, H D].
    With ``q_norm`` [H D] and ``k_norm`` [G D] the norm is another one: q and k
    are RMS-normed over their whole projection with these weights BEFORE the
    rotation, and no per-head division follows."""
    T = u.shape[0]
    uf = u.float()
    q = uf[:, :H * D].reshape(T, H, D)
    k = uf[:, H * D:(H + G) * D].reshape(T, G, D)
    v = k.reshape(T, G * D) if v_off < 0 else uf[:, v_off:v_off + G * Dv]
    pos = positions[:T].long()
    if q_norm is not None:
        q = rms_norm_cols(q.reshape(T, H * D), H * D, q_norm, eps, torch.float32).view(T, H, D)
        k = rms_norm_cols(k.reshape(T, G * D), G * D, k_norm, eps, torch.float32).view(T, G, D)
    if dims:
        cs = cos_sin[pos]
        q, k = rotate_pairs(q, cs, dims), rotate_pairs(k, cs, dims)
    if q_norm is None:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps)
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps)
    if q_temp is not None:
        coef, every = q_temp
        steps = torch.div(pos + 1, int(every), rounding_mode="floor").float()
        q = q * (1.0 + float(coef) * torch.log(steps + 1.0))[:, None, None]
    sl = slots[:T].long()
    ok = sl >= 0
    blk = k_cache.shape[1]
    k_cache[(sl // blk)[ok], (sl % blk)[ok]] = k.reshape(T, G * D).to(k_cache.dtype)[ok]
    v_cache[(sl // blk)[ok], (sl % blk)[ok]] = v.to(v_cache.dtype)[ok]
    return q.reshape(T, H * D).to(out_dtype)


def window_attention(q, k_cache, v_cache, cu_q, ctx_lens, block_tables, positions, scale: float,
                     softcap: float, window: int, keep_first: int, gate, H: int, G: int, D: int,
                     Dv: int, out_dtype, sink=None):
    """Softmax attention of q [T, H D] over paged K [blocks, BLK, G D] and V
    [blocks, BLK, G Dv]: score = q . k * scale, soft-capped to cap tanh(score /
    cap) when ``softcap`` > 0; a query at position p sees key j <= p, and with
    ``window`` > 0 only if p - j < window or j < keep_first. ``gate`` [T, H Dv]
    multiplies the output by sigmoid(gate) per entry. ``sink`` f32 [H]: the
    softmax denominator of head h also holds exp(sink[h]), a term without a
    value. Returns [T, H Dv]."""
    T = q.shape[0]
    blk = k_cache.shape[1]
    rep = H // G
    cu = cu_q.tolist()
    out = torch.zeros(T, H, Dv, dtype=torch.float32, device=q.device)
    qf = q.float().view(T, H, D)
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        L = int(ctx_lens[b])
        idx = torch.arange(L, device=q.device)
        tab = block_tables[b].long()
        kk = k_cache[tab[idx // blk], idx % blk].float().view(L, G, D)
        vv = v_cache[tab[idx // blk], idx % blk].float().view(L, G, Dv)
        qpos = positions[q0:q1].long()
        seen = idx[None, :] <= qpos[:, None]
        if window > 0:
            seen &= ((qpos[:, None] - idx[None, :]) < window) | (idx[None, :] < keep_first)
        for h in range(H):
            s = qf[q0:q1, h] @ kk[:, h // rep].T * scale
            if softcap > 0:
                s = softcap * torch.tanh(s / softcap)
            s = s.masked_fill(~seen, float("-inf"))
            if sink is not None:
                s = torch.cat([s, sink[h].float().expand(q1 - q0, 1)], dim=-1)
            out[q0:q1, h] = torch.softmax(s, dim=-1)[:, :L] @ vv[:, h // rep]
    out = out.view(T, H * Dv)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())
    return out.to(out_dtype)


def mamba2_prep(u, x_off: int, C: int, dt_off: int, Hh: int, conv_w, conv_b, dt_bias, a_neg, tail,
                state_slots, cu_q, positions):
    """The input stage of a Mamba-2 layer over a flat token batch. u [T, W]:
    the projected row; its columns x_off .. x_off + C pass a causal convolution
    per channel (weights tap-major [taps, C], the last tap is the current
    token's; rows before the feed from ``tail[slot]``, zeros before position 0),
    plus ``conv_b``, then SiLU -> f32 [T, C]. The columns dt_off .. dt_off + Hh
    give the step sizes dt = softplus(u + dt_bias) and the decays exp(a_neg dt)
    -> f32 [T, Hh, 2] = (decay, dt)."""
    T = u.shape[0]
    taps = conv_w.shape[0]
    cu = cu_q.tolist()
    xin = u[:, x_off:x_off + C].float()
    y = torch.zeros(T, C, dtype=torch.float32, device=u.device)
    w = conv_w.float()
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        if taps > 1:
            old = torch.zeros_like(tail[0]) if int(positions[q0]) == 0 else \
                tail[int(state_slots[b])]
            rows = torch.cat([old.float(), xin[q0:q1]])
        else:
            rows = xin[q0:q1]
        n = q1 - q0
        for j in range(taps):
            y[q0:q1] += rows[j:j + n] * w[j]
    y = torch.nn.functional.silu(y + conv_b.float())
    dt = torch.nn.functional.softplus(u[:, dt_off:dt_off + Hh].float() + dt_bias.float())
    return y, torch.stack([torch.exp(a_neg.float() * dt), dt], dim=-1).contiguous()


# ---------------------------------------------------------------------------
# Building blocks of decoders with parallel layers (models/vilulix.py): the
# residual step that adds several sublayer outputs at once and norms the sum
# twice, the gate scan and input stage of a stabilised matrix memory, the
# input stage and recurrence of a gated delta rule, a plain RMS norm over a
# column slice, an output gate and the soft cap of the logits.
def residual_rms1p(resid, addends, extra, w_a, w_b, eps: float, out_dtype):
    """resid (f32, in place) += sum_i scale_i * y_i (+ ``extra``, f32); returns
    (rms1p_norm(resid; w_a), rms1p_norm(resid; w_b)), None where the weight is
    None. ``addends``: up to three (tensor, scale)."""
    for y, s in addends:
        resid.add_(y.float() * float(s))
    if extra is not None:
        resid.add_(extra.float())
    return (None if w_a is None else rms1p_norm(resid, w_a, eps, out_dtype),
            None if w_b is None else rms1p_norm(resid, w_b, eps, out_dtype))


def rms_norm_cols(u, n: int, w, eps: float, out_dtype):
    """RMS norm with a plain weight over the first ``n`` columns of u [T, >= n]."""
    x = u[:, :n].float()
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def sigmoid_gate_(o, gate, H: int, Dv: int):
    """o [T, H, Dvo >= Dv] (in place): the first Dv entries of every head times
    sigmoid(gate [T, H Dv])."""
    T = o.shape[0]
    g = torch.sigmoid(gate.float()).view(T, H, Dv)
    o[:, :, :Dv] = (o[:, :, :Dv].float() * g).to(o.dtype)
    return o


def softcap_(x, cap: float):
    """x <- cap tanh(x / cap) in place (f32)."""
    return x.copy_(cap * torch.tanh(x / cap))


def exp_gate_scan(gz, i_bias, f_bias, cap: float, m_state, state_slots, cu_q, positions):
    """The gates of a stabilised exponential-gate memory over a flat token
    batch. gz f32 [T, 2 H]: pre-activations of the input gates (first H
    columns) and the forget gates. Per head: li = cap tanh((z_i + b_i) / cap),
    lf = logsigmoid(cap tanh((z_f + b_f) / cap)), running maximum m_t =
    max(lf + m_{t-1}, li) (m = 0 before position 0, else ``m_state[slot]``).
    Returns tok f32 [T, H, 2] = (exp(lf + m_{t-1} - m_t), exp(li - m_t)) and
    floor f32 [T, H] = exp(-m_t); ``m_state`` [slots, H] takes the last m."""
    T = gz.shape[0]
    H = gz.shape[1] // 2
    z = gz.float()
    li = cap * torch.tanh((z[:, :H] + i_bias.float()) / cap)
    lf = torch.nn.functional.logsigmoid(cap * torch.tanh((z[:, H:] + f_bias.float()) / cap))
    tok = torch.zeros(T, H, 2, dtype=torch.float32, device=gz.device)
    floor = torch.zeros(T, H, dtype=torch.float32, device=gz.device)
    cu = cu_q.tolist()
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        slot = int(state_slots[b])
        m = torch.zeros(H, dtype=torch.float32, device=gz.device) if int(positions[q0]) == 0 \
            else m_state[slot].clone()
        for t in range(q0, q1):
            m1 = torch.maximum(lf[t] + m, li[t])
            tok[t, :, 0] = torch.exp(lf[t] + m - m1)
            tok[t, :, 1] = torch.exp(li[t] - m1)
            floor[t] = torch.exp(-m1)
            m = m1
        m_state[slot] = m
    return tok, floor


def matrix_memory_inputs(u, H: int, D: int, Dv: int):
    """The recurrence inputs of a matrix memory from the projected rows u [T,
    >= 2 H D + H Dv] (q | k | v): f32 [T, 2 H D + H (Dv + 1)] = q D^(-1/2) | k |
    per head (v, 1) - the constant column makes the state's last column the
    normaliser vector."""
    T = u.shape[0]
    q = u[:, :H * D].float() * D ** -0.5
    k = u[:, H * D:2 * H * D].float()
    v = u[:, 2 * H * D:2 * H * D + H * Dv].float().view(T, H, Dv)
    v1 = torch.cat([v, torch.ones(T, H, 1, dtype=torch.float32, device=u.device)], dim=-1)
    return torch.cat([q, k, v1.view(T, H * (Dv + 1))], dim=1).contiguous()


def normalized_gated_rmsnorm(o, floor, w, gate, eps: float, out_dtype, H: int, Dv: int):
    """o f32 [T, H (Dv + 1)]: per head Dv values and their normaliser dot; each
    head's values are divided by max(|dot|, floor[t, h]) + 1e-6, then by their
    root mean square over the head, times w [H Dv], times sigmoid(gate)."""
    T = o.shape[0]
    oh = o.float().view(T, H, Dv + 1)
    y = oh[:, :, :Dv] / (torch.maximum(oh[:, :, Dv].abs(), floor.float()) + 1e-6)[:, :, None]
    y = y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps)
    return (y.reshape(T, H * Dv) * w.float() * torch.sigmoid(gate.float())).to(out_dtype)


def delta_prep(u, gz, G: int, D: int, H: int, Dv: int, conv_w, tail, a_neg, dt_bias, state_slots,
               cu_q, positions):
    """The input stage of a gated delta rule over a flat token batch. u [T, >=
    C], C = 2 G D + H Dv: the projected q | k | v rows pass a causal
    convolution per channel (weights tap-major [taps, C], the last tap is the
    current token's, no bias; rows before the feed from ``tail[slot]``, zeros
    before position 0) and SiLU; every q and k head becomes a unit vector x /
    sqrt(sum x^2 + 1e-6), q also times D^(-1/2) -> f32 [T, C]. gz f32 [T, 2 H]:
    the first H columns give beta = sigmoid(z), the others the decay exp(a_neg
    softplus(z + dt_bias)) -> f32 [T, H, 2] = (decay, beta)."""
    T = u.shape[0]
    taps, C = conv_w.shape
    cu = cu_q.tolist()
    xin = u[:, :C].float()
    y = torch.zeros(T, C, dtype=torch.float32, device=u.device)
    w = conv_w.float()
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        if taps > 1:
            old = torch.zeros_like(tail[0]) if int(positions[q0]) == 0 else \
                tail[int(state_slots[b])]
            rows = torch.cat([old.float(), xin[q0:q1]])
        else:
            rows = xin[q0:q1]
        n = q1 - q0
        for j in range(taps):
            y[q0:q1] += rows[j:j + n] * w[j]
    y = torch.nn.functional.silu(y)
    qk = y[:, :2 * G * D].view(T, 2 * G, D)
    qk = qk * torch.rsqrt(qk.pow(2).sum(-1, keepdim=True) + 1e-6)
    qk[:, :G] *= D ** -0.5
    act = torch.cat([qk.reshape(T, 2 * G * D), y[:, 2 * G * D:]], dim=1).contiguous()
    z = gz.float()
    beta = torch.sigmoid(z[:, :H])
    decay = torch.exp(a_neg.float() * torch.nn.functional.softplus(z[:, H:] + dt_bias.float()))
    return act, torch.stack([decay, beta], dim=-1).contiguous()


def delta_scan(act, H: int, D: int, Dv: int, q_off: int, k_off: int, v_off: int, hpg: int, state,
               state_slots, cu_q, positions, tok):
    """The gated delta rule, token by token in f32, per sequence and head:

        S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q

    with (g, beta) = ``tok[t, h]``. ``act`` f32 [T, W]: head h reads q at
    ``q_off + (h // hpg) D``, k at ``k_off + (h // hpg) D`` and v at ``v_off +
    h Dv``. The state is kept with a column's rows side by side, [slots, H, Dv,
    D]; it is read at the sequence's slot (zero when the step's first position
    is 0) and written back. Returns o f32 [T, H Dv]."""
    T = act.shape[0]
    a = act.float()
    hg = torch.arange(H, device=act.device) // hpg
    cols = torch.arange(D, device=act.device)
    q = a[:, (q_off + hg[:, None] * D + cols[None, :]).reshape(-1)].view(T, H, D)
    k = a[:, (k_off + hg[:, None] * D + cols[None, :]).reshape(-1)].view(T, H, D)
    v = a[:, v_off:v_off + H * Dv].view(T, H, Dv)
    o = torch.zeros(T, H, Dv, dtype=torch.float32, device=act.device)
    cu = cu_q.tolist()
    for b in range(len(cu) - 1):
        q0, q1 = cu[b], cu[b + 1]
        if q1 == q0:
            continue
        slot = int(state_slots[b])
        S = torch.zeros(H, D, Dv, dtype=torch.float32, device=act.device) \
            if int(positions[q0]) == 0 else state[slot].transpose(1, 2).clone()
        for t in range(q0, q1):
            S = tok[t, :, 0].float()[:, None, None] * S
            r = torch.einsum("hde,hd->he", S, k[t])
            uu = tok[t, :, 1].float()[:, None] * (v[t] - r)
            S = S + k[t][:, :, None] * uu[:, None, :]
            o[t] = torch.einsum("hde,hd->he", S, q[t])
        state[slot] = S.transpose(1, 2)
    return o.view(T, H * Dv)
