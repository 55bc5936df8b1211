"""Entry points of the sequence-mixer ops of the hybrid decoders: Dynamic-Tanh
norm, latent (compressed-KV) attention with a softmax sink over a paged latent
cache, decayed linear attention with a carried per-sequence state, and the
grouped top-k expert router with its expert feed-forward; further down the
row-state ops and sigmoid attention of the Sodonex family, and the pre-norm /
layer-scale residual step, windowed softmax attention over paged K / V and the
Mamba-2 input stage of the Movinex family (whose recurrence is ``state_scan``,
the generalised lightning scan).

As everywhere in ``ops``: GPU tensors run the HIP kernels
(``csrc/kernels/norm_dyt.hip``, ``attn_latent.hip``, ``lightning.hip``,
``moe.hip``, ``seq_rows.hip``, ``attn_sigmoid.hip``, ``norm_scalar.hip``,
``norm_rms1p.hip``, ``attn_window.hip``, ``mamba2.hip``), CPU tensors the f32
PyTorch references (the CPU test tier and the numerics oracle of the GPU
tests). Activations are bfloat16 or float32
(``_DT``); the residual stream, scores, softmax, recurrent state, router and
norm statistics are f32 in both.
"""
from __future__ import annotations

import torch

from . import reference as ref
from ._lib import check, kernels, ptr, stream_ptr

_DT = {torch.bfloat16: 0, torch.float32: 1}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"activation dtype {t.dtype} is not supported") from None


def _f32c(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.float32 or not t.is_contiguous():
        raise TypeError(f"{name} must be contiguous float32")


def _i32c(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise TypeError(f"{name} must be contiguous int32")


class DytParams:
    """One Dynamic-Tanh norm: f32 weight and bias vectors and the scalar alpha."""
    __slots__ = ("w", "b", "alpha")

    def __init__(self, w: torch.Tensor, b: torch.Tensor, alpha: float):
        self.w, self.b, self.alpha = w.float().contiguous(), b.float().contiguous(), float(alpha)

    def tup(self):
        return self.w, self.b, self.alpha


def dyt_norm(x: torch.Tensor, p: DytParams, out_dtype, row_idx: torch.Tensor | None = None
             ) -> torch.Tensor:
    """y = tanh(alpha x) * w + b over rows of x [rows, d] (f32 or an activation
    dtype); ``row_idx`` (int64) gathers rows in the same launch."""
    if not x.is_cuda:
        return ref.dyt_norm(x, p.w, p.b, p.alpha, out_dtype, row_idx)
    assert x.dim() == 2 and x.is_contiguous()
    d = x.shape[1]
    rows = x.shape[0] if row_idx is None else row_idx.numel()
    if row_idx is not None:
        assert row_idx.dtype == torch.int64 and row_idx.is_contiguous()
    assert p.w.numel() == d and p.b.numel() == d
    y = torch.empty(rows, d, dtype=out_dtype, device=x.device)
    if rows:
        check(kernels().loqa_dyt_norm(ptr(x), _dt(x), ptr(row_idx), ptr(p.w), ptr(p.b), p.alpha,
                                      ptr(y), _dt(y), rows, d, stream_ptr(x)), "dyt_norm")
    return y


def dyt_add_norm(resid: torch.Tensor, y: torch.Tensor, post: DytParams,
                 nxt: DytParams | None, out_dtype) -> torch.Tensor | None:
    """The fused residual step: resid (f32, in place) += dyt(y; post), and in
    the same launch h = dyt(resid; nxt) for the next sublayer (None: no h)."""
    if not resid.is_cuda:
        return ref.dyt_add_norm(resid, y, post.tup(), None if nxt is None else nxt.tup(), out_dtype)
    _f32c(resid, "resid")
    assert y.shape == resid.shape and y.is_contiguous()
    rows, d = resid.shape
    h = torch.empty(rows, d, dtype=out_dtype, device=resid.device) if nxt is not None else None
    if rows:
        check(kernels().loqa_dyt_add_norm(
            ptr(resid), ptr(y), _dt(y), ptr(post.w), ptr(post.b), post.alpha,
            ptr(nxt.w) if nxt else None, ptr(nxt.b) if nxt else None, nxt.alpha if nxt else 0.0,
            ptr(h), _dt(h) if h is not None else 0, rows, d, stream_ptr(resid)), "dyt_add_norm")
    return h


def rope_table_pairs(dims: int, max_pos: int, base: float, yarn: tuple | None = None,
                     device=None) -> torch.Tensor:
    """(cos, sin) table of the interleaved rotary layout, optionally YaRN-scaled
    (see :func:`reference.rope_table_pairs`); built once at load time."""
    return ref.rope_table_pairs(dims, max_pos, base, yarn, device)


def latent_append(z: torch.Tensor, norm_w: torch.Tensor, eps: float, positions: torch.Tensor,
                  cos_sin: torch.Tensor, cache: torch.Tensor, slots: torch.Tensor, R: int,
                  dims: int) -> None:
    """RMS-norm the latent part of z [T, R + Dr], rotate its rotary key part and
    store both in the paged latent cache [blocks, BLK, R + Dr] (one launch)."""
    if not z.is_cuda:
        return ref.latent_append(z, norm_w, eps, positions, cos_sin, cache, slots, R, dims)
    T, W = z.shape
    assert z.stride(1) == 1 and cache.is_contiguous() and cache.dtype == z.dtype
    assert cache.shape[2] == W and 0 < R <= W and dims % 2 == 0 and dims <= W - R
    _f32c(norm_w, "norm_w"); _f32c(cos_sin, "cos_sin"); _i32c(positions, "positions")
    _i32c(slots, "slots")
    assert norm_w.numel() == R and cos_sin.shape[1] * 2 == dims
    assert positions.numel() >= T and slots.numel() >= T
    if T:
        check(kernels().loqa_latent_append(
            ptr(z), _dt(z), z.stride(0), ptr(norm_w), eps, ptr(positions), ptr(cos_sin),
            cos_sin.shape[0], ptr(cache), cache.shape[1], cache.shape[0], ptr(slots), T, R, W - R,
            dims, stream_ptr(z)), "latent_append")


def latent_attention(qa: torch.Tensor, qr: torch.Tensor, cache: torch.Tensor, cu_q: torch.Tensor,
                     ctx_lens: torch.Tensor, block_tables: torch.Tensor, positions: torch.Tensor,
                     cos_sin: torch.Tensor, sink: torch.Tensor | None, scale: float, R: int,
                     dims: int, max_ctx: int = 0, out: torch.Tensor | None = None) -> torch.Tensor:
    """Causal attention over the paged latent cache, all heads sharing each
    cached row: score = (qa . c + rot(qr) . k_rot) * scale; softmax with
    ``sink`` [H] (f32, optional) in the denominator; out = sum_j p_j c_j.
    qa [H, T, R] (queries already folded into latent space), qr [T, H, Dr]
    (unrotated; may be a strided view), out [H, T, R]."""
    H, T, _ = qa.shape
    if out is None:
        out = torch.empty(H, T, R, dtype=qa.dtype, device=qa.device)
    if not qa.is_cuda:
        return ref.latent_attention(qa, qr, cache, cu_q, ctx_lens, block_tables, positions,
                                    cos_sin, sink, scale, R, dims, out)
    Dr = cache.shape[2] - R
    assert qa.shape[2] == R and qa.stride(2) == 1 and qr.shape == (T, H, Dr) and qr.stride(2) == 1
    assert qa.dtype == cache.dtype == qr.dtype == out.dtype and cache.is_contiguous()
    assert out.is_contiguous() and out.shape == (H, T, R)
    _i32c(cu_q, "cu_q"); _i32c(ctx_lens, "ctx_lens"); _i32c(block_tables, "block_tables")
    _i32c(positions, "positions"); _f32c(cos_sin, "cos_sin")
    if sink is not None:
        _f32c(sink, "sink")
        assert sink.numel() == H
    B = ctx_lens.numel()
    assert cu_q.numel() == B + 1 and block_tables.shape[0] == B and positions.numel() >= T
    # few query rows over a long context: split the keys over workgroups
    hg = (H + 3) // 4
    ns = 1 if T * hg >= 512 else max(1, min(32, -(-int(max_ctx) // 128), 1024 // max(1, T * hg)))
    ws = torch.empty(ns * T * H * (R + 2), dtype=torch.float32, device=qa.device) if ns > 1 else None
    if T:
        check(kernels().loqa_latent_attention(
            ptr(qa), qa.stride(1), qa.stride(0), ptr(qr), qr.stride(0), qr.stride(1), _dt(qa),
            ptr(cache), cache.shape[1], cache.shape[0], ptr(cu_q), ptr(ctx_lens), ptr(block_tables),
            block_tables.shape[1], ptr(positions), ptr(cos_sin), cos_sin.shape[0], ptr(sink),
            float(scale), B, H, T, R, Dr, dims, ptr(out), ns, ptr(ws), stream_ptr(qa)),
            "latent_attention")
    return out


PREFILL_DK = (64, 128, 192, 256)     # head sizes the matrix-core prompt kernel is built for
PREFILL_DV = (64, 128)


def prefill_head_sizes(dk: int, dv: int) -> tuple[int, int] | None:
    """The (padded) key and value head sizes of the prompt-pass kernel for a
    model's sizes, or None when it does not cover them."""
    a = next((x for x in PREFILL_DK if x >= dk), None)
    b = next((x for x in PREFILL_DV if x >= dv), None)
    return None if a is None or b is None else (a, b)


def latent_gather(cache: torch.Tensor, block_tables: torch.Tensor, cu_k: torch.Tensor,
                  total_k: int, max_ctx: int, R: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Every sequence's cached rows in position order, as contiguous latents
    [total_k, R] and rotary key parts [total_k, Dr] (bf16, GPU)."""
    assert cache.is_cuda and cache.dtype == torch.bfloat16 and cache.is_contiguous()
    _i32c(block_tables, "block_tables"); _i32c(cu_k, "cu_k")
    B, Dr = block_tables.shape[0], cache.shape[2] - R
    assert cu_k.numel() == B + 1
    cl = torch.empty(total_k, R, dtype=cache.dtype, device=cache.device)
    kr = torch.empty(total_k, Dr, dtype=cache.dtype, device=cache.device)
    check(kernels().loqa_latent_gather(ptr(cache), cache.shape[1], ptr(block_tables),
                                       block_tables.shape[1], ptr(cu_k), B, int(max_ctx), R, Dr,
                                       ptr(cl), ptr(kr), stream_ptr(cache)), "latent_gather")
    return cl, kr


def latent_kfill_(k: torch.Tensor, kr: torch.Tensor, D: int) -> None:
    """k [L, H, DK] (bf16): every head's entries D .. D + Dr take kr [L, Dr]."""
    L, H, DK = k.shape
    Dr = kr.shape[1]
    assert k.is_contiguous() and kr.is_contiguous() and kr.shape[0] == L and D + Dr <= DK
    assert k.dtype == kr.dtype == torch.bfloat16
    check(kernels().loqa_latent_kfill(ptr(k), ptr(kr), L, H, DK, D, Dr, stream_ptr(k)),
          "latent_kfill")


def rope_pairs_(x: torch.Tensor, off: int, dims: int, positions: torch.Tensor,
                cos_sin: torch.Tensor) -> None:
    """Rotate in place the interleaved pairs x[t, h, off : off + dims] (bf16)."""
    T, H, _ = x.shape
    assert x.dtype == torch.bfloat16 and x.stride(2) == 1 and off + dims <= x.shape[2]
    _i32c(positions, "positions"); _f32c(cos_sin, "cos_sin")
    assert cos_sin.shape[1] * 2 == dims and positions.numel() >= T
    check(kernels().loqa_rope_pairs(ptr(x), x.stride(0), x.stride(1), T, H, off, dims,
                                    ptr(positions), ptr(cos_sin), cos_sin.shape[0], stream_ptr(x)),
          "rope_pairs")


def latent_prefill(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_q: torch.Tensor,
                   cu_k: torch.Tensor, positions: torch.Tensor, sink: torch.Tensor | None,
                   scale: float, max_q: int) -> torch.Tensor:
    """Causal flash attention of a prompt pass on the matrix cores: q [T, H, DK]
    (rotated), k [L, H, DK], v [L, H, DV] per-head keys / values of the
    gathered contexts (``cu_k``), a query at absolute position p sees keys
    0 .. p of its sequence; ``sink`` [H] joins the softmax denominator.
    Returns [T, H * DV] (bf16)."""
    T, H, DK = q.shape
    DV = v.shape[2]
    assert q.is_cuda and q.dtype == k.dtype == v.dtype == torch.bfloat16
    assert q.stride(2) == 1 and q.stride(1) == DK and k.is_contiguous() and v.is_contiguous()
    assert k.shape[1:] == (H, DK) and v.shape[:2] == k.shape[:2]
    assert DK in PREFILL_DK and DV in PREFILL_DV
    _i32c(cu_q, "cu_q"); _i32c(cu_k, "cu_k"); _i32c(positions, "positions")
    B = cu_q.numel() - 1
    assert cu_k.numel() == B + 1
    if sink is not None:
        _f32c(sink, "sink")
    o = torch.empty(T, H * DV, dtype=q.dtype, device=q.device)
    check(kernels().loqa_latent_prefill(ptr(q), q.stride(0), ptr(k), ptr(v), ptr(o), ptr(cu_q),
                                        ptr(cu_k), ptr(positions), ptr(sink), float(scale), B, H,
                                        int(max_q), DK, DV, stream_ptr(q)), "latent_prefill")
    return o


def lightning_scan(qkv: torch.Tensor, H: int, D: int, Dv: int, state: torch.Tensor,
                   state_slots: torch.Tensor, cu_q: torch.Tensor, positions: torch.Tensor,
                   decay: torch.Tensor) -> torch.Tensor:
    """Decayed linear attention over a flat token batch: per sequence and head
    S <- decay_h S + k v^T, o = S^T q, token by token in f32, with q, k, v the
    SiLU of the first columns of ``qkv`` [T, >= 2 H D + H Dv]. ``state`` [slots,
    H, D, Dv] f32 carries S between steps (a sequence whose first position in
    this step is 0 starts from zero). Returns o f32 [T, H Dv]. Prompt portions
    and single decode tokens take the same kernel and the same order of
    operations, so the result does not depend on how a prompt was cut."""
    if not qkv.is_cuda:
        return ref.lightning_scan(qkv, H, D, Dv, state, state_slots, cu_q, positions, decay)
    T = qkv.shape[0]
    assert qkv.stride(1) == 1 and qkv.shape[1] >= 2 * H * D + H * Dv
    _f32c(state, "state"); _f32c(decay, "decay")
    assert state.shape[1:] == (H, D, Dv) and decay.numel() == H
    _i32c(state_slots, "state_slots"); _i32c(cu_q, "cu_q"); _i32c(positions, "positions")
    B = state_slots.numel()
    assert cu_q.numel() == B + 1
    if not T:
        return torch.empty(0, H * Dv, dtype=torch.float32, device=qkv.device)
    # SiLU of q | k | v once, in f32 (every column block of a head shares q and k)
    n = 2 * H * D + H * Dv
    act = torch.empty(T, n, dtype=torch.float32, device=qkv.device)
    check(kernels().loqa_lightning_prep(ptr(qkv), _dt(qkv), qkv.stride(0), T, n, ptr(act),
                                        stream_ptr(qkv)), "lightning_prep")
    return state_scan(act, H, D, Dv, 0, H * D, 2 * H * D, 1, state, state_slots, cu_q, positions,
                      decay=decay)


def state_scan(act: torch.Tensor, H: int, D: int, Dv: int, q_off: int, k_off: int, v_off: int,
               hpg: int, state: torch.Tensor, state_slots: torch.Tensor, cu_q: torch.Tensor,
               positions: torch.Tensor, decay: torch.Tensor | None = None,
               tok: torch.Tensor | None = None, skip: torch.Tensor | None = None,
               col_block: int = 0) -> torch.Tensor:
    """The linear recurrence with a carried matrix state that decayed linear
    attention and Mamba-2 layers share, per sequence and head, token by token
    in f32:  S <- a S + k (c v)^T,  o = S^T q + skip_h v,  with a = ``decay[h]``
    or per token ``tok[t, h, 0]`` and c = 1 or ``tok[t, h, 1]``. ``act`` f32
    [T, W]: head h reads q at ``q_off + (h // hpg) D``, k at ``k_off + (h // hpg)
    D`` and v at ``v_off + h Dv``. ``state`` [slots, H, D, Dv] f32 carries S
    between steps (zero when the step's first position is 0). One kernel and
    one order of operations for prompt portions and single tokens.
    ``col_block`` (8, 16 or 32; 0: chosen from the batch) sets the value columns
    per workgroup: a caller that runs other work beside the scan asks for the
    denser grid. The result does not depend on it."""
    if not act.is_cuda:
        return ref.state_scan(act, H, D, Dv, q_off, k_off, v_off, hpg, state, state_slots, cu_q,
                              positions, decay, tok, skip)
    T, W = act.shape
    _f32c(act, "act"); _f32c(state, "state")
    assert state.shape[1:] == (H, D, Dv) and hpg >= 1 and H % hpg == 0
    G = H // hpg
    assert min(q_off, k_off, v_off) >= 0 and max(q_off, k_off) + G * D <= W and v_off + H * Dv <= W
    assert (decay is None) != (tok is None)
    if decay is not None:
        _f32c(decay, "decay")
        assert decay.numel() == H
    else:
        _f32c(tok, "tok")
        assert tok.shape == (T, H, 2)
    if skip is not None:
        _f32c(skip, "skip")
        assert skip.numel() == H
    _i32c(state_slots, "state_slots"); _i32c(cu_q, "cu_q"); _i32c(positions, "positions")
    B = state_slots.numel()
    assert cu_q.numel() == B + 1 and positions.numel() >= T
    o = torch.empty(T, H * Dv, dtype=torch.float32, device=act.device)
    if T:
        check(kernels().loqa_state_scan(ptr(act), W, H, D, Dv, q_off, k_off, v_off, hpg, ptr(state),
                                        state.shape[0], ptr(state_slots), ptr(cu_q), ptr(positions),
                                        ptr(decay), ptr(tok), ptr(skip), ptr(o), B, T,
                                        int(col_block), stream_ptr(act)), "state_scan")
    return o


def gated_rmsnorm(o: torch.Tensor, w: torch.Tensor, gate: torch.Tensor, eps: float,
                  out_dtype, groups: int = 1, silu_first: bool = False,
                  gate_act: str = "sigmoid") -> torch.Tensor:
    """y = rmsnorm(o) * w * sigmoid(gate) over whole rows of o f32 [T, n]
    (``gate_act`` "silu": times silu(gate) instead), or with ``silu_first`` y =
    rmsnorm(o * silu(gate)) * w (the gate before the norm); ``groups`` > 1
    normalises a row in that many equal parts, each by its own root mean
    square. ``gate`` [T, n] may be a column slice of a wider projection."""
    assert gate_act in ("sigmoid", "silu")
    if not o.is_cuda:
        return ref.gated_rmsnorm(o, w, gate, eps, out_dtype, groups, silu_first, gate_act)
    _f32c(o, "o"); _f32c(w, "w")
    T, n = o.shape
    assert gate.shape == (T, n) and gate.stride(1) == 1 and w.numel() == n
    assert groups >= 1 and n % groups == 0
    y = torch.empty(T, n, dtype=out_dtype, device=o.device)
    if T:
        check(kernels().loqa_gated_rmsnorm(ptr(o), ptr(w), ptr(gate), _dt(gate), gate.stride(0), eps,
                                           ptr(y), _dt(y), T, n, groups,
                                           1 if silu_first else (2 if gate_act == "silu" else 0),
                                           stream_ptr(o)), "gated_rmsnorm")
    return y


_ACTS = {"silu": 0, "gelu_tanh": 1}


def act_mul_any(x: torch.Tensor, act: str = "silu") -> torch.Tensor:
    """[gate | up] -> act(gate) * up for bf16 or f32 activations; ``act`` is
    "silu" or "gelu_tanh" (0.5 z (1 + tanh(sqrt(2 / pi) (z + 0.044715 z^3))))."""
    if not x.is_cuda:
        return ref.silu_mul(x) if act == "silu" else ref.act_mul(x, act)
    assert x.dim() == 2 and x.is_contiguous() and x.shape[1] % 2 == 0
    T, F2 = x.shape
    y = torch.empty(T, F2 // 2, dtype=x.dtype, device=x.device)
    if T:
        check(kernels().loqa_act_mul_any(ptr(x), _dt(x), T, F2 // 2, _ACTS[act], ptr(y),
                                         stream_ptr(x)), "act_mul_any")
    return y


def silu_mul_any(x: torch.Tensor) -> torch.Tensor:
    """[gate | up] -> silu(gate) * up for bf16 or f32 activations."""
    return act_mul_any(x, "silu")


def moe_route(z: torch.Tensor, correction: torch.Tensor | None, n_groups: int, keep: int,
              top: int, bias: torch.Tensor | None = None, top_softmax: bool = False,
              sigmoid: bool = False, group_rank: int = 1) -> tuple[torch.Tensor, torch.Tensor]:
    """Router decisions from f32 logits z [T, E] (+ ``bias`` [E]). Default:
    softmax scores, choice by score + ``correction`` limited to the ``keep``
    best of ``n_groups`` groups of neighbouring experts, weights = the plain
    scores (not renormalised). ``top_softmax``: the ``top`` largest logits are
    chosen and weighed by the softmax over the chosen logits only. ``sigmoid``:
    the scores are sigmoid(z) instead of the softmax. ``group_rank`` n: a group
    ranks by the sum of its n best choice scores instead of its best one.
    Returns (idx int32 [T, top], weight f32 [T, top])."""
    if not z.is_cuda:
        return ref.moe_route(z, correction, n_groups, keep, top, bias, top_softmax, sigmoid,
                             group_rank)
    assert not (top_softmax and sigmoid)
    _f32c(z, "z")
    T, E = z.shape
    assert E % max(1, n_groups) == 0 and 0 < top <= E and E <= 1024
    for v, name in ((correction, "correction"), (bias, "bias")):
        if v is not None:
            _f32c(v, name)
            assert v.numel() == E
    idx = torch.empty(T, top, dtype=torch.int32, device=z.device)
    wt = torch.empty(T, top, dtype=torch.float32, device=z.device)
    if T:
        check(kernels().loqa_moe_route(ptr(z), ptr(correction), ptr(bias),
                                       1 if top_softmax else (2 if sigmoid else 0), E,
                                       max(1, n_groups), min(keep, max(1, n_groups)),
                                       max(1, group_rank), top, ptr(idx), ptr(wt), T,
                                       stream_ptr(z)), "moe_route")
    return idx, wt


def moe_experts(h: torch.Tensor, idx: torch.Tensor, wt: torch.Tensor, w_gate_up: torch.Tensor,
                w_down: torch.Tensor, gated: bool = True) -> torch.Tensor:
    """Weighted sum of every token's chosen experts, f32 [T, d]. Experts below
    E = w_gate_up.shape[0] are feed-forwards: gated (w_gate_up [E, 2F, d] with
    gate rows then up rows, SwiGLU) or not (w_gate_up [E, F, d], the square of
    relu), w_down [E, d, F]; an index >= E is an identity expert. On the GPU: a
    device-side plan (tokens grouped by expert, no host round trip), a grouped
    up GEMM with the activation as its epilogue, a grouped down GEMM, and a
    combine launch that applies the weights in f32."""
    if not h.is_cuda:
        return ref.moe_experts(h, idx, wt, w_gate_up, w_down, h.dtype, gated)
    T, d = h.shape
    E, F2, _ = w_gate_up.shape
    F = F2 // 2 if gated else F2
    top = idx.shape[1]
    assert h.is_contiguous() and w_gate_up.is_contiguous() and w_down.is_contiguous()
    assert w_gate_up.dtype == h.dtype == w_down.dtype and w_down.shape == (E, d, F)
    assert w_gate_up.shape[2] == d
    _i32c(idx, "idx"); _f32c(wt, "wt")
    dev = h.device
    P = T * top
    out = torch.empty(T, d, dtype=torch.float32, device=dev)
    if T == 0:
        return out
    # plan: offsets[E + 1] of each expert's segment, perm[P] pair ids sorted by
    # expert (identity pairs last, past offsets[E]), pos[P] = where each pair sits
    plan = torch.empty(E + 2 + 2 * P, dtype=torch.int32, device=dev)
    act = torch.empty(P, F, dtype=h.dtype, device=dev)
    y = torch.empty(P, d, dtype=h.dtype, device=dev)
    k, st = kernels(), stream_ptr(h)
    check(k.loqa_moe_plan(ptr(idx), P, E, ptr(plan), st), "moe_plan")
    check(k.loqa_moe_grouped_gemm(ptr(h), _dt(h), ptr(w_gate_up), ptr(plan), P, E, top, d, F,
                                  1 if gated else 2, ptr(act), st), "moe_up")
    check(k.loqa_moe_grouped_gemm(ptr(act), _dt(h), ptr(w_down), ptr(plan), P, E, top, F, d, 0,
                                  ptr(y), st), "moe_down")
    check(k.loqa_moe_combine(ptr(h), ptr(y), _dt(h), ptr(idx), ptr(wt), ptr(plan), T, top, E, d,
                             ptr(out), st), "moe_combine")
    return out


# ---------------------------------------------------------------------------
# Per-sequence row state (token shift, convolution tails), chunked sigmoid
# attention over paged K/V, scalar-gain RMS norm on the residual step
# (csrc/kernels/seq_rows.hip, attn_sigmoid.hip, norm_scalar.hip)
def rope_table_half(dims: int, max_pos: int, base: float, device=None) -> torch.Tensor:
    """(cos, sin) table of the rotate-half rotary layout, built once at load time."""
    return ref.rope_table_half(dims, max_pos, base, device)


def _seq_args(state_slots, cu_q, positions, T):
    _i32c(state_slots, "state_slots"); _i32c(cu_q, "cu_q"); _i32c(positions, "positions")
    B = state_slots.numel()
    assert cu_q.numel() == B + 1 and positions.numel() >= T
    return B


def token_shift(x: torch.Tensor, mu: torch.Tensor, prev: torch.Tensor, state_slots: torch.Tensor,
                cu_q: torch.Tensor, positions: torch.Tensor, out_dtype) -> torch.Tensor:
    """h_t = x_t + (x_{t-1} - x_t) * mu over a flat token batch x f32 [T, d];
    the row before a feed's first token is ``prev[slot]`` f32 [slots, d] (zeros
    when the feed starts at position 0). ``prev`` is not written here
    (:func:`seq_state_save` does, once every reader of the step is done)."""
    if not x.is_cuda:
        return ref.token_shift(x, mu, prev, state_slots, cu_q, positions, out_dtype)
    _f32c(x, "x"); _f32c(mu, "mu"); _f32c(prev, "prev")
    T, d = x.shape
    assert mu.numel() == d and prev.shape[1] == d
    B = _seq_args(state_slots, cu_q, positions, T)
    h = torch.empty(T, d, dtype=out_dtype, device=x.device)
    if T:
        check(kernels().loqa_token_shift(ptr(x), ptr(mu), ptr(prev), prev.shape[0], ptr(state_slots),
                                         ptr(cu_q), ptr(positions), B, T, d, ptr(h), _dt(h),
                                         stream_ptr(x)), "token_shift")
    return h


def seq_state_save(x: torch.Tensor | None, u: torch.Tensor, prev: torch.Tensor | None,
                   tail: torch.Tensor, state_slots: torch.Tensor, cu_q: torch.Tensor,
                   positions: torch.Tensor) -> None:
    """The step's row state: prev[slot] = the last row of each feed of x f32
    [T, d]; tail[slot] f32 [taps - 1, C] = the last taps - 1 rows of the
    projections u[:, :C] (older rows move up under a shorter feed)."""
    if not u.is_cuda:
        return ref.seq_state_save(x, u, prev, tail, state_slots, cu_q, positions)
    T = u.shape[0]
    _f32c(tail, "tail")
    keep, C = tail.shape[1], tail.shape[2]
    assert u.stride(1) == 1 and u.shape[1] >= C
    d = 0
    if prev is not None:
        _f32c(x, "x"); _f32c(prev, "prev")
        d = x.shape[1]
        assert prev.shape == (tail.shape[0], d) and x.shape[0] == T
    B = _seq_args(state_slots, cu_q, positions, T)
    if T:
        check(kernels().loqa_seq_state_save(ptr(x), d, ptr(u), _dt(u), u.stride(0), ptr(prev),
                                            ptr(tail), tail.shape[0], keep, C, ptr(state_slots),
                                            ptr(cu_q), ptr(positions), B, stream_ptr(u)),
              "seq_state_save")


def conv_norm_rope_append(u: torch.Tensor, conv_w: torch.Tensor, tail: torch.Tensor,
                          state_slots: torch.Tensor, cu_q: torch.Tensor, positions: torch.Tensor,
                          q_norm: torch.Tensor, k_norm: torch.Tensor, eps: float,
                          cos_sin: torch.Tensor, dims: int, H: int, G: int, D: int,
                          k_cache: torch.Tensor, v_cache: torch.Tensor, slots: torch.Tensor,
                          out_dtype) -> torch.Tensor:
    """One launch between the q | k projection and attention: short causal
    convolution per channel (f32 weights conv_w tap-major [taps, (H + G) D]; the
    rows before a feed come from ``tail[slot]``), v = the convolved k, RMS norm of q
    and of k over the whole projection, rotate-half rotary on the first
    ``dims`` entries of every head, k into its paged cache [blocks, BLK, G D]
    and v into its transposed pages [blocks, G D, BLK]; returns q [T, H D]."""
    if not u.is_cuda:
        return ref.conv_norm_rope_append(u, conv_w, tail, state_slots, cu_q, positions, q_norm,
                                         k_norm, eps, cos_sin, dims, H, G, D, k_cache, v_cache,
                                         slots, out_dtype)
    T = u.shape[0]
    taps, C = conv_w.shape
    assert C == (H + G) * D and u.stride(1) == 1 and u.shape[1] >= C
    _f32c(conv_w, "conv_w"); _f32c(tail, "tail"); _f32c(q_norm, "q_norm"); _f32c(k_norm, "k_norm")
    _f32c(cos_sin, "cos_sin"); _i32c(slots, "slots")
    assert tail.shape[1:] == (taps - 1, C) and q_norm.numel() == H * D and k_norm.numel() == G * D
    assert dims % 2 == 0 and dims <= D and (dims == 0 or cos_sin.shape[1] * 2 == dims)
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.shape[2] == G * D and k_cache.dtype == v_cache.dtype == out_dtype
    assert v_cache.shape == (k_cache.shape[0], G * D, k_cache.shape[1])
    assert slots.numel() >= T
    B = _seq_args(state_slots, cu_q, positions, T)
    q = torch.empty(T, H * D, dtype=out_dtype, device=u.device)
    if T:
        check(kernels().loqa_conv_norm_rope_append(
            ptr(u), _dt(u), u.stride(0), ptr(conv_w), taps, ptr(tail), tail.shape[0],
            ptr(state_slots), ptr(cu_q), ptr(positions), B, T, ptr(q_norm), ptr(k_norm), eps,
            ptr(cos_sin), cos_sin.shape[0], dims, H, G, D, ptr(k_cache), ptr(v_cache),
            k_cache.shape[1], k_cache.shape[0], ptr(slots), ptr(q), _dt(q), stream_ptr(u)),
            "conv_norm_rope_append")
    return q


SIGMOID_MFMA_D = (64, 128)        # head sizes the matrix-core form is built for


def sigmoid_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                      cu_q: torch.Tensor, ctx_lens: torch.Tensor, block_tables: torch.Tensor,
                      positions: torch.Tensor, head_bias: torch.Tensor, gate: torch.Tensor | None,
                      scale: float, chunk: int, H: int, G: int, D: int, max_q: int = 0,
                      matrix_cores: bool | None = None) -> torch.Tensor:
    """Attention without softmax over paged K [blocks, BLK, G D] and transposed
    V pages [blocks, G D, BLK]: a query at
    position p sees keys j <= p - with ``chunk`` > 0 only those of its own chunk
    (j // chunk == p // chunk, counted from the sequence's start) - and a
    visible key weighs sigmoid(q . k * scale + head_bias[h]) (f32, not
    normalised over keys). Head h's output is multiplied by sigmoid(gate[t, h])
    (``gate`` [T, H], may be a column slice). q [T, H D] -> [T, H D]. Prompt
    portions, decode tokens and mixed batches take the same launch; every
    output sums its keys in ascending position order whatever the batch."""
    if not q.is_cuda:
        return ref.sigmoid_attention(q, k_cache, v_cache, cu_q, ctx_lens, block_tables, positions,
                                     head_bias, gate, scale, chunk, H, G, D, q.dtype)
    T = q.shape[0]
    assert q.is_contiguous() and q.shape[1] == H * D and H % G == 0
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.shape[2] == G * D and k_cache.dtype == v_cache.dtype == q.dtype
    assert v_cache.shape == (k_cache.shape[0], G * D, k_cache.shape[1])
    _i32c(cu_q, "cu_q"); _i32c(ctx_lens, "ctx_lens"); _i32c(block_tables, "block_tables")
    _i32c(positions, "positions"); _f32c(head_bias, "head_bias")
    B = ctx_lens.numel()
    assert cu_q.numel() == B + 1 and block_tables.shape[0] == B and positions.numel() >= T
    assert head_bias.numel() == H
    gs = 0
    if gate is not None:
        assert gate.shape == (T, H) and gate.stride(1) == 1 and gate.dtype == q.dtype
        gs = gate.stride(0)
    o = torch.empty(T, H * D, dtype=q.dtype, device=q.device)
    if matrix_cores is None:
        matrix_cores = max_q >= 16
    mfma = bool(matrix_cores) and q.dtype == torch.bfloat16 and D in SIGMOID_MFMA_D
    if T:
        check(kernels().loqa_sigmoid_attention(
            ptr(q), _dt(q), ptr(k_cache), ptr(v_cache), k_cache.shape[1], k_cache.shape[0],
            ptr(cu_q), ptr(ctx_lens), ptr(block_tables), block_tables.shape[1], ptr(positions),
            ptr(head_bias), ptr(gate), gs, float(scale), int(chunk), B, T, H, G, D, int(max_q),
            int(mfma), ptr(o), stream_ptr(q)), "sigmoid_attention")
    return o


def scalar_rms_add(resid: torch.Tensor, y: torch.Tensor, g: float, eps: float, mult: float,
                   out_dtype=None) -> torch.Tensor | None:
    """The residual step with a norm on the sublayer's output only: resid (f32,
    in place) += mult * y / rms(y) * g with ONE gain g for all coordinates; the
    same launch returns resid in ``out_dtype`` for the next sublayer's GEMMs
    (None: nothing; float32: resid itself)."""
    if not resid.is_cuda:
        ref.scalar_rms_add(resid, y, g, eps, mult, None)
        if out_dtype is None:
            return None
        return resid if out_dtype == torch.float32 else resid.to(out_dtype)
    _f32c(resid, "resid")
    assert y.shape == resid.shape and y.is_contiguous()
    rows, d = resid.shape
    copy = out_dtype is not None and out_dtype != torch.float32
    h = torch.empty(rows, d, dtype=out_dtype, device=resid.device) if copy else None
    if rows:
        check(kernels().loqa_scalar_rms_add(ptr(resid), ptr(y), _dt(y), float(g) * float(mult),
                                            float(eps), ptr(h), rows, d, stream_ptr(resid)),
              "scalar_rms_add")
    return h if copy else (resid if out_dtype == torch.float32 else None)


def scalar_rms_norm(x: torch.Tensor, g: float, eps: float, row_idx: torch.Tensor | None = None
                    ) -> torch.Tensor:
    """f32 rows of x / rms(x) * g for x f32 [rows, d]; ``row_idx`` (int64)
    gathers rows in the same launch."""
    if not x.is_cuda:
        return ref.scalar_rms_norm(x, g, eps, row_idx)
    _f32c(x, "x")
    d = x.shape[1]
    rows = x.shape[0] if row_idx is None else row_idx.numel()
    if row_idx is not None:
        assert row_idx.dtype == torch.int64 and row_idx.is_contiguous()
    y = torch.empty(rows, d, dtype=torch.float32, device=x.device)
    if rows:
        check(kernels().loqa_scalar_rms_norm(ptr(x), ptr(row_idx), float(g), float(eps), ptr(y), rows,
                                             d, stream_ptr(x)), "scalar_rms_norm")
    return y


# ---------------------------------------------------------------------------
# Pre-norm RMS norm with a weight stored around zero and layer scale on the
# residual step, q / k preparation with paged append, softmax attention with a
# sliding window / kept first tokens / soft-capping over paged K / V, and the
# Mamba-2 input stage (csrc/kernels/norm_rms1p.hip, attn_window.hip, mamba2.hip)
def rms1p_norm(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype,
               row_idx: torch.Tensor | None = None) -> torch.Tensor:
    """y = x / sqrt(mean(x^2) + eps) * (1 + w) over rows of x f32 [rows, d];
    ``row_idx`` (int64) gathers rows in the same launch."""
    if not x.is_cuda:
        return ref.rms1p_norm(x, w, eps, out_dtype, row_idx)
    _f32c(x, "x"); _f32c(w, "w")
    d = x.shape[1]
    assert w.numel() == d
    rows = x.shape[0] if row_idx is None else row_idx.numel()
    if row_idx is not None:
        assert row_idx.dtype == torch.int64 and row_idx.is_contiguous()
    y = torch.empty(rows, d, dtype=out_dtype, device=x.device)
    if rows:
        check(kernels().loqa_rms1p_norm(ptr(x), ptr(row_idx), ptr(w), float(eps), ptr(y), _dt(y),
                                        rows, d, stream_ptr(x)), "rms1p_norm")
    return y


def scaled_add_rms1p(resid: torch.Tensor, y: torch.Tensor, ls: torch.Tensor,
                     nxt: torch.Tensor | None, eps: float, out_dtype) -> torch.Tensor | None:
    """The fused residual step of a pre-norm layer with layer scale: resid (f32,
    in place) += ls * y per coordinate, and in the same launch the next
    sublayer's input h = resid / rms(resid) * (1 + nxt) (None: no h)."""
    if not resid.is_cuda:
        return ref.scaled_add_rms1p(resid, y, ls, nxt, eps, out_dtype)
    _f32c(resid, "resid"); _f32c(ls, "ls")
    assert y.shape == resid.shape and y.is_contiguous()
    rows, d = resid.shape
    assert ls.numel() == d
    h = None
    if nxt is not None:
        _f32c(nxt, "nxt")
        assert nxt.numel() == d
        h = torch.empty(rows, d, dtype=out_dtype, device=resid.device)
    if rows:
        check(kernels().loqa_scaled_add_rms1p(ptr(resid), ptr(y), _dt(y), ptr(ls), ptr(nxt),
                                              float(eps), ptr(h), _dt(h) if h is not None else 0,
                                              rows, d, stream_ptr(resid)), "scaled_add_rms1p")
    return h


def qk_prep_append(u: torch.Tensor, H: int, G: int, D: int, Dv: int, v_off: int,
                   cos_sin: torch.Tensor | None, dims: int, eps: float, q_temp: tuple | None,
                   positions: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   slots: torch.Tensor, out_dtype, q_norm: torch.Tensor | None = None,
                   k_norm: torch.Tensor | None = None) -> torch.Tensor:
    """One launch between the fused q | k (| v) projection u [T, W] and
    attention: per head the first ``dims`` entries of q and k rotate pairwise
    (interleaved layout, table ``cos_sin`` [positions, dims / 2, 2]), then q and
    k are divided by their root mean square over the head (no weight), q is
    multiplied by the position's temperature 1 + coef ln(floor((p + 1) / every)
    + 1) (``q_temp`` = (coef, every) or None); k goes to its pages [blocks, BLK,
    G D] and the value rows - the columns at ``v_off``, or with ``v_off`` < 0
    the k columns as projected - to theirs [blocks, BLK, G Dv]. Returns q
    [T, H D]. Statistics, angles and the temperature are f32. With ``q_norm``
    [H D] and ``k_norm`` [G D] (f32) the norm is another one: q and k are
    RMS-normed over their whole projection with these weights BEFORE the
    rotation, and no per-head division follows."""
    assert (q_norm is None) == (k_norm is None)
    if not u.is_cuda:
        return ref.qk_prep_append(u, H, G, D, Dv, v_off, cos_sin, dims, eps, q_temp, positions,
                                  k_cache, v_cache, slots, out_dtype, q_norm, k_norm)
    if q_norm is not None:
        _f32c(q_norm, "q_norm"); _f32c(k_norm, "k_norm")
        assert q_norm.numel() == H * D and k_norm.numel() == G * D
    T, W = u.shape
    assert u.stride(1) == 1 and (H + G) * D <= W
    assert v_off < 0 and Dv == D or v_off >= (H + G) * D and v_off + G * Dv <= W
    assert dims % 2 == 0 and 0 <= dims <= D
    if dims:
        _f32c(cos_sin, "cos_sin")
        assert cos_sin.shape[1] * 2 == dims
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.dtype == v_cache.dtype == out_dtype == u.dtype
    assert k_cache.shape[2] == G * D and v_cache.shape == (*k_cache.shape[:2], G * Dv)
    _i32c(positions, "positions"); _i32c(slots, "slots")
    assert positions.numel() >= T and slots.numel() >= T
    coef, every = (float(q_temp[0]), int(q_temp[1])) if q_temp is not None else (0.0, 1)
    q = torch.empty(T, H * D, dtype=out_dtype, device=u.device)
    if T:
        check(kernels().loqa_qk_prep_append(
            ptr(u), _dt(u), u.stride(0), H, G, D, Dv, int(v_off), ptr(cos_sin) if dims else None,
            cos_sin.shape[0] if dims else 0, dims, float(eps), coef, every, ptr(positions),
            ptr(k_cache), ptr(v_cache), k_cache.shape[1], k_cache.shape[0], ptr(slots), ptr(q), T,
            ptr(q_norm), ptr(k_norm), stream_ptr(u)), "qk_prep_append")
    return q


WINDOW_MFMA_D = (64, 128)         # head sizes the matrix-core form is built for


def window_attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                     cu_q: torch.Tensor, ctx_lens: torch.Tensor, block_tables: torch.Tensor,
                     positions: torch.Tensor, scale: float, softcap: float, window: int,
                     keep_first: int, gate: torch.Tensor | None, H: int, G: int, D: int, Dv: int,
                     max_q: int = 0, matrix_cores: bool | None = None, max_ctx: int = 0,
                     key_splits: int | None = None, sink: torch.Tensor | None = None
                     ) -> torch.Tensor:
    """Softmax attention over paged K [blocks, BLK, G D] and V [blocks, BLK,
    G Dv] (query head h reads key/value head h // (H / G)): score = q . k *
    scale, soft-capped to cap tanh(score / cap) when ``softcap`` > 0; a query at
    position p sees key j <= p, with ``window`` > 0 only if p - j < window or
    j < keep_first (kept keys keep their own positions). ``gate`` [T, H Dv] (may
    be a column slice) multiplies the output by sigmoid(gate) per entry. q
    [T, H D] -> [T, H Dv]. Rows find their sequence through ``cu_q`` and their
    keys through the block table, so prompt portions, decode tokens and mixed
    batches are one launch. Scores, softmax and accumulators are f32. A step
    with few rows over long contexts (``max_ctx``) deals each row's keys out to
    ``key_splits`` workgroups (chosen here when None) and merges their partial
    results in a second launch. ``sink`` f32 [H]: head h's softmax denominator
    also holds exp(sink[h]), a term that carries no value."""
    if not q.is_cuda:
        return ref.window_attention(q, k_cache, v_cache, cu_q, ctx_lens, block_tables, positions,
                                    scale, softcap, window, keep_first, gate, H, G, D, Dv, q.dtype,
                                    sink)
    if sink is not None:
        _f32c(sink, "sink")
        assert sink.numel() == H
    T = q.shape[0]
    assert q.is_contiguous() and q.shape[1] == H * D and H % G == 0
    assert k_cache.is_contiguous() and v_cache.is_contiguous()
    assert k_cache.shape[2] == G * D and k_cache.dtype == v_cache.dtype == q.dtype
    assert v_cache.shape == (*k_cache.shape[:2], G * Dv)
    assert D <= 512 and Dv <= 512 and window >= 0 and keep_first >= 0 and softcap >= 0
    _i32c(cu_q, "cu_q"); _i32c(ctx_lens, "ctx_lens"); _i32c(block_tables, "block_tables")
    _i32c(positions, "positions")
    B = ctx_lens.numel()
    assert cu_q.numel() == B + 1 and block_tables.shape[0] == B and positions.numel() >= T
    gs = 0
    if gate is not None:
        assert gate.shape == (T, H * Dv) and gate.stride(1) == 1 and gate.dtype == q.dtype
        gs = gate.stride(0)
    o = torch.empty(T, H * Dv, dtype=q.dtype, device=q.device)
    if matrix_cores is None:
        matrix_cores = max_q >= 16
    mfma = bool(matrix_cores) and q.dtype == torch.bfloat16 and D in WINDOW_MFMA_D \
        and Dv in WINDOW_MFMA_D
    part = None
    if key_splits is None:
        # 64-key windows a row can have, four (one per wave) to a workgroup
        keys = max(int(max_ctx), 1) if window <= 0 else min(max(int(max_ctx), 1),
                                                           window + 64 + keep_first)
        key_splits = 1 if mfma or T * G >= 256 else \
            max(1, min(16, -(-keys // 256), 512 // max(1, T * G)))
    if key_splits > 1 and not mfma:
        part = torch.empty(T * H * key_splits * (Dv + 2), dtype=torch.float32, device=q.device)
    else:
        key_splits = 1
    if T:
        check(kernels().loqa_window_attention(
            ptr(q), _dt(q), ptr(k_cache), ptr(v_cache), k_cache.shape[1], k_cache.shape[0],
            ptr(cu_q), ptr(ctx_lens), ptr(block_tables), block_tables.shape[1], ptr(positions),
            ptr(gate), gs, float(scale), float(softcap), int(window), int(keep_first), B, T, H, G,
            D, Dv, int(max_q), int(mfma), ptr(o), int(key_splits), ptr(part), ptr(sink),
            stream_ptr(q)), "window_attention")
    return o


def mamba2_prep(u: torch.Tensor, x_off: int, C: int, dt_off: int, Hh: int, conv_w: torch.Tensor,
                conv_b: torch.Tensor, dt_bias: torch.Tensor, a_neg: torch.Tensor,
                tail: torch.Tensor, state_slots: torch.Tensor, cu_q: torch.Tensor,
                positions: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """The input stage of a Mamba-2 layer, one launch over a flat token batch:
    the columns x_off .. x_off + C of the projected rows u [T, W] pass a causal
    convolution per channel (f32 weights tap-major [taps, C], last tap = the
    current token; the rows before a feed from ``tail[slot]`` f32 [slots, taps -
    1, C], zeros before position 0) plus ``conv_b``, then SiLU -> f32 [T, C];
    the columns dt_off .. dt_off + Hh give dt = softplus(u + dt_bias) and the
    decay exp(a_neg dt) per head -> f32 [T, Hh, 2] = (decay, dt). ``tail`` is
    not written here (:func:`seq_state_save` does, after every reader)."""
    if not u.is_cuda:
        return ref.mamba2_prep(u, x_off, C, dt_off, Hh, conv_w, conv_b, dt_bias, a_neg, tail,
                               state_slots, cu_q, positions)
    T, W = u.shape
    taps = conv_w.shape[0]
    assert u.stride(1) == 1 and x_off + C <= W and dt_off + Hh <= W and conv_w.shape == (taps, C)
    for t, name, n in ((conv_w, "conv_w", taps * C), (conv_b, "conv_b", C),
                       (dt_bias, "dt_bias", Hh), (a_neg, "a_neg", Hh), (tail, "tail", None)):
        _f32c(t, name)
        assert n is None or t.numel() == n
    assert tail.shape[1:] == (taps - 1, C)
    B = _seq_args(state_slots, cu_q, positions, T)
    xbc = torch.empty(T, C, dtype=torch.float32, device=u.device)
    tok = torch.empty(T, Hh, 2, dtype=torch.float32, device=u.device)
    if T:
        check(kernels().loqa_mamba2_prep(
            ptr(u), _dt(u), u.stride(0), x_off, C, dt_off, Hh, ptr(conv_w), taps, ptr(conv_b),
            ptr(dt_bias), ptr(a_neg), ptr(tail), tail.shape[0], ptr(state_slots), ptr(cu_q),
            ptr(positions), B, T, ptr(xbc), ptr(tok), stream_ptr(u)), "mamba2_prep")
    return xbc, tok


# ---------------------------------------------------------------------------
# Parallel layers (two norms of one residual, several sublayer outputs added
# at once), the gate scan and input stage of a stabilised matrix memory, the
# gated delta rule, and small steps around latent attention and the logits
# (csrc/kernels/norm_rms1p.hip, matrix_memory.hip, delta_rule.hip)
def residual_rms1p(resid: torch.Tensor, addends: list, extra: torch.Tensor | None,
                   w_a: torch.Tensor | None, w_b: torch.Tensor | None, eps: float, out_dtype
                   ) -> tuple[torch.Tensor | None, torch.Tensor | None]:
    """The residual step of a layer whose sublayers run side by side: resid
    (f32, in place) += sum_i scale_i * y_i over up to three ``addends`` (tensor
    [rows, d] in one activation dtype, scalar scale) and ``extra`` (f32 [rows,
    d]); the same launch returns the two normed inputs of the next layer, h_a =
    resid / rms(resid) * (1 + w_a) and h_b likewise with w_b (None where the
    weight is None). Without addends it is the two norms alone."""
    if not resid.is_cuda:
        return ref.residual_rms1p(resid, addends, extra, w_a, w_b, eps, out_dtype)
    _f32c(resid, "resid")
    rows, d = resid.shape
    assert len(addends) <= 3
    ys = [None, None, None]
    sc = [0.0, 0.0, 0.0]
    ydt = 0
    for i, (y, s_) in enumerate(addends):
        assert y.shape == resid.shape and y.is_contiguous()
        assert i == 0 or y.dtype == addends[0][0].dtype
        ys[i], sc[i], ydt = y, float(s_), _dt(y)
    if extra is not None:
        _f32c(extra, "extra")
        assert extra.shape == resid.shape
    hs = []
    for w in (w_a, w_b):
        if w is None:
            hs.append(None)
            continue
        _f32c(w, "norm weight")
        assert w.numel() == d
        hs.append(torch.empty(rows, d, dtype=out_dtype, device=resid.device))
    if rows:
        check(kernels().loqa_residual_rms1p(
            ptr(resid), ptr(ys[0]), sc[0], ptr(ys[1]), sc[1], ptr(ys[2]), sc[2], ydt, ptr(extra),
            ptr(w_a), ptr(w_b), float(eps), ptr(hs[0]), ptr(hs[1]), _DT[out_dtype], rows, d,
            stream_ptr(resid)), "residual_rms1p")
    return hs[0], hs[1]


def rms_norm_cols(u: torch.Tensor, n: int, w: torch.Tensor, eps: float, out_dtype) -> torch.Tensor:
    """RMS norm with a plain weight over the first ``n`` columns of the rows of
    u [T, >= n] (a slice of a fused projection) -> [T, n]; statistics f32."""
    if not u.is_cuda:
        return ref.rms_norm_cols(u, n, w, eps, out_dtype)
    T = u.shape[0]
    assert u.stride(1) == 1 and 0 < n <= u.shape[1]
    _f32c(w, "w")
    assert w.numel() == n
    y = torch.empty(T, n, dtype=out_dtype, device=u.device)
    if T:
        check(kernels().loqa_rms_norm_cols(ptr(u), _dt(u), u.stride(0), n, ptr(w), float(eps),
                                           ptr(y), _dt(y), T, stream_ptr(u)), "rms_norm_cols")
    return y


def sigmoid_gate_(o: torch.Tensor, gate: torch.Tensor, H: int, Dv: int) -> torch.Tensor:
    """In place: the first Dv entries of every head of o [T, H, Dvo] (Dvo >= Dv:
    heads may be padded) times sigmoid(gate [T, H Dv]); ``gate`` may be a
    column slice of a wider projection."""
    if not o.is_cuda:
        return ref.sigmoid_gate_(o, gate, H, Dv)
    T, Ho, Dvo = o.shape
    assert Ho == H and Dvo >= Dv and o.is_contiguous()
    assert gate.shape == (T, H * Dv) and gate.stride(1) == 1 and gate.dtype == o.dtype
    if T:
        check(kernels().loqa_sigmoid_gate(ptr(o), _dt(o), ptr(gate), gate.stride(0), T, H, Dvo, Dv,
                                          stream_ptr(o)), "sigmoid_gate")
    return o


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap tanh(x / cap) in place over a contiguous f32 tensor."""
    if not x.is_cuda:
        return ref.softcap_(x, cap)
    _f32c(x, "x")
    assert cap > 0
    if x.numel():
        check(kernels().loqa_softcap(ptr(x), x.numel(), float(cap), stream_ptr(x)), "softcap")
    return x


def exp_gate_scan(gz: torch.Tensor, i_bias: torch.Tensor, f_bias: torch.Tensor, cap: float,
                  m_state: torch.Tensor, state_slots: torch.Tensor, cu_q: torch.Tensor,
                  positions: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """The gates of a stabilised exponential-gate memory over a flat token
    batch. gz f32 [T, 2 H]: the pre-activations of the input gates (first H
    columns) and the forget gates. Per head li = cap tanh((z_i + b_i) / cap),
    lf = logsigmoid(cap tanh((z_f + b_f) / cap)) and the running maximum m_t =
    max(lf + m_{t-1}, li), which is 0 before position 0 and otherwise carried
    in ``m_state`` [slots, H] f32 (updated here). Returns tok f32 [T, H, 2] =
    (exp(lf + m_{t-1} - m_t), exp(li - m_t)), the decay and the input scale of
    the state recurrence, and floor f32 [T, H] = exp(-m_t)."""
    if not gz.is_cuda:
        return ref.exp_gate_scan(gz, i_bias, f_bias, cap, m_state, state_slots, cu_q, positions)
    _f32c(gz, "gz"); _f32c(i_bias, "i_bias"); _f32c(f_bias, "f_bias"); _f32c(m_state, "m_state")
    T, H2 = gz.shape
    H = H2 // 2
    assert H2 == 2 * H and i_bias.numel() == H and f_bias.numel() == H and cap > 0
    assert m_state.shape[1:] == (H,)
    B = _seq_args(state_slots, cu_q, positions, T)
    tok = torch.empty(T, H, 2, dtype=torch.float32, device=gz.device)
    floor = torch.empty(T, H, dtype=torch.float32, device=gz.device)
    if T:
        check(kernels().loqa_exp_gate_scan(ptr(gz), H, ptr(i_bias), ptr(f_bias), float(cap),
                                           ptr(m_state), m_state.shape[0], ptr(state_slots),
                                           ptr(cu_q), ptr(positions), B, T, ptr(tok), ptr(floor),
                                           stream_ptr(gz)), "exp_gate_scan")
    return tok, floor


def matrix_memory_inputs(u: torch.Tensor, H: int, D: int, Dv: int) -> torch.Tensor:
    """The recurrence inputs of a matrix memory from the projected rows u [T,
    >= 2 H D + H Dv] (q | k | v): f32 [T, 2 H D + H (Dv + 1)] = q D^(-1/2) | k |
    per head (v, 1). With the constant column, :func:`state_scan` over Dv + 1
    value columns keeps the normaliser vector as the state's last column and
    returns its product with q as every head's last output."""
    if not u.is_cuda:
        return ref.matrix_memory_inputs(u, H, D, Dv)
    T = u.shape[0]
    assert u.stride(1) == 1 and u.shape[1] >= 2 * H * D + H * Dv
    act = torch.empty(T, 2 * H * D + H * (Dv + 1), dtype=torch.float32, device=u.device)
    if T:
        check(kernels().loqa_matrix_memory_inputs(ptr(u), _dt(u), u.stride(0), H, D, Dv, ptr(act),
                                                  T, stream_ptr(u)), "matrix_memory_inputs")
    return act


def normalized_gated_rmsnorm(o: torch.Tensor, floor: torch.Tensor, w: torch.Tensor,
                             gate: torch.Tensor, eps: float, out_dtype, H: int, Dv: int
                             ) -> torch.Tensor:
    """The output stage of a matrix memory. o f32 [T, H (Dv + 1)]: per head Dv
    read-out values and the normaliser's product with q; each head's values are
    divided by max(|product|, floor[t, h]) + 1e-6, then by their root mean
    square over the head, times w [H Dv], times sigmoid(gate [T, H Dv]) (may be
    a column slice). Returns [T, H Dv]."""
    if not o.is_cuda:
        return ref.normalized_gated_rmsnorm(o, floor, w, gate, eps, out_dtype, H, Dv)
    _f32c(o, "o"); _f32c(floor, "floor"); _f32c(w, "w")
    T = o.shape[0]
    assert o.shape[1] == H * (Dv + 1) and floor.shape == (T, H) and w.numel() == H * Dv
    assert gate.shape == (T, H * Dv) and gate.stride(1) == 1
    y = torch.empty(T, H * Dv, dtype=out_dtype, device=o.device)
    if T:
        check(kernels().loqa_normalized_gated_rmsnorm(
            ptr(o), ptr(floor), ptr(w), ptr(gate), _dt(gate), gate.stride(0), float(eps), ptr(y),
            _dt(y), T, H, Dv, stream_ptr(o)), "normalized_gated_rmsnorm")
    return y


def delta_prep(u: torch.Tensor, gz: torch.Tensor, G: int, D: int, H: int, Dv: int,
               conv_w: torch.Tensor, tail: torch.Tensor, a_neg: torch.Tensor,
               dt_bias: torch.Tensor, state_slots: torch.Tensor, cu_q: torch.Tensor,
               positions: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """The input stage of a gated delta rule, one launch over a flat token
    batch. The first C = 2 G D + H Dv columns of the projected rows u [T, W] (q
    | k | v) pass a causal convolution per channel (f32 weights tap-major [taps,
    C], last tap = the current token, no bias; the rows before a feed from
    ``tail[slot]`` f32 [slots, taps - 1, C], zeros before position 0) and SiLU;
    every q and k head becomes a unit vector x / sqrt(sum x^2 + 1e-6), q also
    times D^(-1/2) -> f32 [T, C]. gz f32 [T, 2 H]: the first H columns give the
    write strengths beta = sigmoid(z), the others the decays exp(a_neg
    softplus(z + dt_bias)) -> f32 [T, H, 2] = (decay, beta). ``tail`` is not
    written here (:func:`seq_state_save` does, after every reader)."""
    if not u.is_cuda:
        return ref.delta_prep(u, gz, G, D, H, Dv, conv_w, tail, a_neg, dt_bias, state_slots, cu_q,
                              positions)
    T, W = u.shape
    taps, C = conv_w.shape
    assert C == 2 * G * D + H * Dv and u.stride(1) == 1 and C <= W
    for t, name, n in ((conv_w, "conv_w", None), (tail, "tail", None), (a_neg, "a_neg", H),
                       (dt_bias, "dt_bias", H), (gz, "gz", T * 2 * H)):
        _f32c(t, name)
        assert n is None or t.numel() == n
    assert tail.shape[1:] == (taps - 1, C)
    B = _seq_args(state_slots, cu_q, positions, T)
    act = torch.empty(T, C, dtype=torch.float32, device=u.device)
    tok = torch.empty(T, H, 2, dtype=torch.float32, device=u.device)
    if T:
        check(kernels().loqa_delta_prep(
            ptr(u), _dt(u), u.stride(0), ptr(gz), G, D, H, Dv, ptr(conv_w), taps, ptr(tail),
            tail.shape[0], ptr(a_neg), ptr(dt_bias), ptr(state_slots), ptr(cu_q), ptr(positions), B,
            T, ptr(act), ptr(tok), stream_ptr(u)), "delta_prep")
    return act, tok


def delta_scan(act: torch.Tensor, H: int, D: int, Dv: int, q_off: int, k_off: int, v_off: int,
               hpg: int, state: torch.Tensor, state_slots: torch.Tensor, cu_q: torch.Tensor,
               positions: torch.Tensor, tok: torch.Tensor) -> torch.Tensor:
    """The gated delta rule with a carried matrix state, per sequence and head,
    token by token in f32:  S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;
    o = S^T q, with (g, beta) = ``tok[t, h]``. ``act`` f32 [T, W]: head h reads
    q at ``q_off + (h // hpg) D``, k at ``k_off + (h // hpg) D`` and v at
    ``v_off + h Dv``. ``state`` [slots, H, Dv, D] f32 (a column's rows side by
    side) carries S between steps (zero when the step's first position is 0).
    One kernel and one order of operations for prompt portions and single
    tokens."""
    if not act.is_cuda:
        return ref.delta_scan(act, H, D, Dv, q_off, k_off, v_off, hpg, state, state_slots, cu_q,
                              positions, tok)
    T, W = act.shape
    _f32c(act, "act"); _f32c(state, "state"); _f32c(tok, "tok")
    assert state.shape[1:] == (H, Dv, D) and hpg >= 1 and H % hpg == 0 and tok.shape == (T, H, 2)
    G = H // hpg
    assert min(q_off, k_off, v_off) >= 0 and max(q_off, k_off) + G * D <= W and v_off + H * Dv <= W
    B = _seq_args(state_slots, cu_q, positions, T)
    o = torch.empty(T, H * Dv, dtype=torch.float32, device=act.device)
    if T:
        check(kernels().loqa_delta_scan(ptr(act), W, H, D, Dv, q_off, k_off, v_off, hpg, ptr(state),
                                        state.shape[0], ptr(state_slots), ptr(cu_q), ptr(positions),
                                        ptr(tok), ptr(o), B, T, stream_ptr(act)), "delta_scan")
    return o
