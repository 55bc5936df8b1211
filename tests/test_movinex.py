"""The Movinex family through the framework (registry, weights, engine step,
hybrid cache, scheduler) against the plain float64 oracle in
``movinex_oracle.py``. Every test builds its own small configuration and
seeded weights. The same tests run on the CPU (reference ops) and, marked
``gpu``, on the HIP kernels.
"""
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import movinex_oracle as O
from loqa_hub_amd.engine.llm_engine import GenRequest, LLMEngine
from loqa_hub_amd.models.configs import movinex_config_from_json
from loqa_hub_amd.models.movinex import MovinexWeights, config_to_json, random_state_dict
from loqa_hub_amd.models.registry import family_of, lm_config_from_json
from loqa_hub_amd.ops import seqmix

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
TOL = {torch.float32: 2e-4, torch.bfloat16: 6e-2}
F64 = torch.float64


def engine(cfg_json, sd, device, dtype=torch.float32, max_tokens=256, block=16, max_seqs=4):
    cfg = lm_config_from_json(cfg_json, "t")
    w = MovinexWeights(cfg, sd, device, dtype, max_positions=max_tokens)
    return LLMEngine(cfg, device, weights=w, max_seqs=max_seqs, max_seq_len=max_tokens,
                     block_size=block, num_blocks=max_tokens // block, use_graphs=False, dtype=dtype)


def rel_err(got: torch.Tensor, want: torch.Tensor, q: float = 1.0) -> float:
    """RMS difference (mean removed per row) over the RMS of the wanted logits:
    the worst row, or the ``q`` quantile of the rows."""
    d = got.double().cpu() - want.double()
    d = d - d.mean(-1, keepdim=True)
    w = want - want.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / w.pow(2).mean().sqrt()).quantile(q))


def feed(eng, seq, toks, cuts):
    """Feed ``toks`` to one sequence in portions of ``cuts`` sizes (cycled);
    returns the logits of every position."""
    out, i, k = [], 0, 0
    while i < len(toks):
        n = min(cuts[k % len(cuts)], len(toks) - i)
        out.append(eng.step_logits([seq], [toks[i:i + n]], [list(range(n))]))
        i, k = i + n, k + 1
    return torch.cat(out)


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


# every mixer and feed-forward kind, a repeated stretch that holds a state-space
# layer and two attention kinds (so every pass needs a state and pages of its
# own), grouped and ungrouped heads, a layer without a feed-forward
FULL = [(O.mamba(), O.dense_ff()),
        (O.attn(heads=4, kv_heads=2, dim=16, vdim=8, every=5), O.moe_ff()),
        (O.mamba(heads=2, vdim=16, state=4, groups=1, conv=2, norm_groups=1), None),
        (O.attn2(heads=6, kv_heads=2, dim=8, window=7, keep=3, dims=4), O.moe_ff(9, 3, 8, 3, 1)),
        (O.attn2(heads=2, kv_heads=2, dim=24, window=20, keep=0, dims=24, cap=2.0), O.dense_ff(24))]


@pytest.fixture(scope="module")
def full_model():
    cfg = O.make_config(FULL, loop=(1, 4, 2))
    return cfg, O.make_weights(cfg, 1)


def test_registry_reads_config(full_model):
    cfg_json, _ = full_model
    cfg = lm_config_from_json(json.loads(json.dumps(cfg_json)))
    assert family_of(cfg).name == "movinex" and family_of(cfg_json).hybrid
    assert cfg.n_layers == len(FULL) and cfg.layers[2].mlp is None
    assert cfg.layers[3].mixer.window == 7 and cfg.layers[3].mixer.keep_first == 3
    assert cfg.layers[1].mixer.q_temp == (0.5, 5) and cfg.layers[1].mixer.bias
    assert cfg.layers[3].mixer.values_from_keys and cfg.layers[3].mixer.gate
    assert cfg.layers[0].mlp.act == "geglu" and cfg.layers[1].mlp.router == "sigmoid"
    assert [i for i, _ in cfg.runs()] == [0, 1, 2, 3, 1, 2, 3, 4]
    assert [f for _, f in cfg.runs()] == [False, True, False, False, True, False, False, False]
    assert config_to_json(cfg)["layers"] == json.loads(json.dumps(cfg_json))["layers"]
    assert config_to_json(cfg)["loop"] == cfg_json["loop"]
    for li, key, val in ((1, "kv_heads", 3), (3, "vdim", 9), (0, "groups", 3), (0, "norm_groups", 5)):
        bad = json.loads(json.dumps(cfg_json))
        bad["layers"][li]["mixer"][key] = val
        with pytest.raises(ValueError):
            movinex_config_from_json(bad)
    bad = json.loads(json.dumps(cfg_json))
    bad["loop"]["stop"] = 9
    with pytest.raises(ValueError):
        movinex_config_from_json(bad)
    sd = random_state_dict(cfg, 0)
    assert sd["loop.in"].shape == (32, 64) and sd["l0.mix.conv"].shape == (32 + 2 * 16, 4)
    assert "l3.mix.v" not in sd and sd["l3.mix.g"].shape == (48, 32)


# ------------------------------------------------------ each mechanism alone
def _meta(lens, starts, device):
    cu = torch.tensor([0] + lens).cumsum(0).to(torch.int32)
    pos = torch.cat([s + torch.arange(n) for n, s in zip(lens, starts)]).to(torch.int32)
    return cu.to(device), pos.to(device)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("d", [40, 256, 4100])
def test_norm_and_residual_step(device, d):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(9, d, generator=g)
    y = torch.randn(9, d, generator=g)
    ls, w1, w2 = (torch.randn(d, generator=g) * 0.3 for _ in range(3))
    eps = 1e-3
    got = seqmix.rms1p_norm(x.to(device), w1.to(device), eps, torch.float32)
    assert (got.cpu().double() - O.norm(x.double(), w1.double(), eps)).abs().max() < 1e-5
    idx = torch.tensor([7, 2], device=device)
    got = seqmix.rms1p_norm(x.to(device), w1.to(device), eps, torch.float32, row_idx=idx)
    assert (got.cpu().double() - O.norm(x[[7, 2]].double(), w1.double(), eps)).abs().max() < 1e-5
    for ydt in (torch.float32, torch.bfloat16):
        r = x.to(device).clone()
        yy = y.to(ydt)
        h = seqmix.scaled_add_rms1p(r, yy.to(device), ls.to(device), w2.to(device), eps, torch.float32)
        want = x.double() + ls.double() * yy.double()
        assert (r.cpu().double() - want).abs().max() < 1e-5
        assert (h.cpu().double() - O.norm(want, w2.double(), eps)).abs().max() < 1e-5
        r2 = x.to(device).clone()
        assert seqmix.scaled_add_rms1p(r2, yy.to(device), ls.to(device), None, eps, ydt) is None
        assert torch.equal(r2, r)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,Dv,dims,own_v,temp", [
    (4, 2, 16, 16, 8, False, None), (3, 1, 24, 8, 0, True, (0.5, 3)), (2, 2, 6, 6, 6, False, (2.0, 1)),
    (5, 5, 64, 32, 16, True, (0.25, 64)), (1, 1, 130, 130, 2, False, None)])
def test_qk_preparation_and_append(device, H, G, D, Dv, dims, own_v, temp):
    g = torch.Generator().manual_seed(1)
    T, blk, eps, base = 11, 4, 1e-4, 50.0
    W = (H + G) * D + (G * Dv if own_v else 0) + 3
    u = torch.randn(T, W, generator=g)
    pos = torch.tensor([60, 61, 62, 63, 64, 0, 1, 2, 5, 6, 7], dtype=torch.int32)
    slots = torch.tensor([9, 3, 30, 31, 12, 0, 1, 2, -1, 20, 21], dtype=torch.int32)
    table = seqmix.rope_table_pairs(dims, 80, base, None, device) if dims else None
    kc = torch.zeros(8, blk, G * D, device=device)
    vc = torch.zeros(8, blk, G * Dv, device=device)
    v_off = (H + G) * D if own_v else -1
    q = seqmix.qk_prep_append(u.to(device), H, G, D, Dv, v_off, table, dims, eps, temp,
                              pos.to(device), kc, vc, slots.to(device), torch.float32)
    ud = u.double()
    qw = ud[:, :H * D].view(T, H, D)
    kw = ud[:, H * D:(H + G) * D].view(T, G, D)
    vw = ud[:, v_off:v_off + G * Dv] if own_v else kw.reshape(T, G * D)
    if dims:
        qw, kw = O.rotate(qw, dims, base, pos), O.rotate(kw, dims, base, pos)
    qw, kw = O.unit_rms(qw, eps), O.unit_rms(kw, eps)
    if temp:
        qw = qw * O.query_temperature(T, temp[0], temp[1], pos.long())[:, None, None]
    assert (q.cpu().double() - qw.reshape(T, H * D)).abs().max() < 2e-5
    ok = slots >= 0
    rows_k = kc.view(-1, G * D).cpu().double()[slots[ok].long()]
    rows_v = vc.view(-1, G * Dv).cpu().double()[slots[ok].long()]
    assert (rows_k - kw.reshape(T, G * D)[ok]).abs().max() < 2e-5
    assert (rows_v - vw[ok]).abs().max() < 1e-6
    untouched = torch.ones(32, dtype=torch.bool)
    untouched[slots[ok].long()] = False
    assert float(kc.view(-1, G * D).cpu()[untouched].abs().max()) == 0.0


def _paged(k, v, lens, blk, device, seed=0):
    """Scatter per-sequence k / v rows into shuffled pages; returns caches and block tables."""
    nb = sum(-(-n // blk) for n in lens) + 2
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(seed)).tolist()
    kc = torch.full((nb, blk, k[0].shape[1]), 7.0)
    vc = torch.full((nb, blk, v[0].shape[1]), 7.0)
    mb = max(-(-n // blk) for n in lens)
    bt = torch.zeros(len(lens), mb, dtype=torch.int32)
    for b, n in enumerate(lens):
        for j in range(-(-n // blk)):
            page = perm.pop()
            bt[b, j] = page
            m = min(blk, n - j * blk)
            kc[page, :m] = k[b][j * blk:j * blk + m]
            vc[page, :m] = v[b][j * blk:j * blk + m]
    return kc.to(device), vc.to(device), bt.to(device)


def _attention_case(device, dtype, H, G, D, Dv, window, keep, cap, lens, feeds, gate, mfma=None,
                    spike=None, seed=2, gate_pad=(2, 5), splits=None):
    """Sequences of ``lens`` keys whose last ``feeds`` positions are this step's
    queries; compares seqmix.window_attention with the oracle. ``spike`` =
    (distance back, strength): the key that far behind each query's position
    gets a large score, so a mask that is one off shows."""
    g = torch.Generator().manual_seed(seed)
    B = len(lens)
    ks = [torch.randn(n, G * D, generator=g).to(dtype).float() for n in lens]
    vs = [torch.randn(n, G * Dv, generator=g).to(dtype).float() for n in lens]
    qs = [torch.randn(n, H * D, generator=g) for n in lens]
    if spike is not None:
        back, strength = spike
        for b, n in enumerate(lens):
            # every key is a scaled one-hot-ish direction of its position so that
            # q_i (built from key i - back) scores high against exactly that key
            for i in range(n):
                j = i - back
                if j >= 0:
                    kk = ks[b][j].view(G, D)
                    qs[b][i] = (kk.repeat_interleave(H // G, 0) * strength / D).reshape(-1)
    qs = [q.to(dtype).float() for q in qs]
    blk = 16
    kc, vc, bt = _paged(ks, vs, lens, blk, device, seed)
    starts = [n - f for n, f in zip(lens, feeds)]
    cu, pos = _meta(feeds, starts, device)
    q = torch.cat([qs[b][starts[b]:] for b in range(B)])
    g0, g1 = gate_pad                              # the gate is a column slice of a wider tensor
    gt = torch.randn(q.shape[0], H * Dv + g1, generator=g).to(dtype) if gate else None
    ctx = torch.tensor(lens, dtype=torch.int32, device=device)
    scale = 1.0 / math.sqrt(D)
    got = seqmix.window_attention(
        q.to(device, dtype), kc.to(dtype), vc.to(dtype), cu, ctx, bt, pos, scale, cap, window, keep,
        gt.to(device)[:, g0:g0 + H * Dv] if gate else None, H, G, D, Dv, max(feeds),
        matrix_cores=mfma, max_ctx=max(lens), key_splits=splits)
    want = []
    for b, n in enumerate(lens):
        o = O.softmax_attention(qs[b].double().view(n, H, D), ks[b].double().view(n, G, D),
                                vs[b].double().view(n, G, Dv), scale, O.visible(n, window, keep), cap)
        want.append(o[starts[b]:].reshape(-1, H * Dv))
    want = torch.cat(want)
    if gate:
        want = want * torch.sigmoid(gt[:, g0:g0 + H * Dv].double())
    return got.cpu().double(), want


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,G,D,Dv,window,keep,cap", [
    (4, 2, 16, 16, 0, 0, 0.0), (3, 3, 8, 24, 5, 2, 3.0), (6, 1, 64, 64, 37, 5, 20.0),
    (8, 1, 24, 8, 17, 0, 0.0), (20, 2, 32, 32, 64, 70, 1.5), (2, 2, 6, 130, 1, 1, 0.0),
    (1, 1, 260, 12, 3, 200, 0.0)])
def test_window_attention_op(device, H, G, D, Dv, window, keep, cap):
    """Prompt portions beside decode tokens of unequal sequences in shuffled
    pages, with and without an output gate."""
    for gate in (False, True):
        got, want = _attention_case(device, torch.float32, H, G, D, Dv, window, keep, cap,
                                    [150, 1, 37, 90], [150, 1, 1, 23], gate)
        assert (got - want).abs().max() < 2e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("back", [0, 1, 4, 5, 6, 63, 64, 65, 127, 128, 129, 290])
def test_window_edges_and_far_keys(device, back):
    """A key ``back`` positions behind every query carries almost all of the
    softmax weight if it is visible: windows of 5, 64 and 128 keys with 0, 2 or
    65 kept first tokens, and no window at all (a key hundreds of positions
    away), in a prompt portion and in single decoded tokens."""
    for window, keep in ((5, 0), (5, 2), (64, 65), (128, 2), (0, 0)):
        for feeds in ([300], [1]):
            got, want = _attention_case(device, torch.float32, 2, 1, 16, 16, window, keep, 0.0,
                                        [300], feeds, False, spike=(back, 40.0))
            assert (got - want).abs().max() < 2e-5, (window, keep, feeds)


def _mamba_case(device, m, cuts, dtype=torch.float32, seed=3):
    """One state-space mixer alone through the ops, fed in portions."""
    g = torch.Generator().manual_seed(seed)
    Hh, P, N, G, taps, ng = (m[k] for k in ("heads", "vdim", "state", "groups", "conv", "norm_groups"))
    inner, GN = Hh * P, G * N
    C = inner + 2 * GN
    T, eps = sum(cuts), 1e-5
    u = (torch.randn(T, 2 * inner + 2 * GN + Hh, generator=g) * 1.5).to(dtype)
    sd = {"conv": torch.randn(C, taps, generator=g) * 0.5, "conv.b": torch.randn(C, generator=g) * 0.1,
          "dt_bias": torch.randn(Hh, generator=g) * 0.5 - 0.5, "A_log": torch.randn(Hh, generator=g) * 0.7,
          "D": torch.randn(Hh, generator=g), "norm": 1.0 + 0.2 * torch.randn(inner, generator=g)}
    dev = {k: v.to(device) for k, v in sd.items()}
    state = torch.full((3, Hh, N, P), 5.0, device=device)          # dirty slots
    tail = torch.full((3, taps - 1, C), 5.0, device=device)
    slot = torch.tensor([2], dtype=torch.int32, device=device)
    conv_w = dev["conv"].t().contiguous()
    a_neg = -torch.exp(dev["A_log"])
    outs, at = [], 0
    for c in cuts:
        cu, pos = _meta([c], [at], device)
        uu = u[at:at + c].to(device)
        xbc, tok = seqmix.mamba2_prep(uu, inner, C, inner + C, Hh, conv_w, dev["conv.b"],
                                      dev["dt_bias"], a_neg, tail, slot, cu, pos)
        if taps > 1:
            seqmix.seq_state_save(None, uu[:, inner:inner + C], None, tail, slot, cu, pos)
        o = seqmix.state_scan(xbc, Hh, N, P, inner + GN, inner, 0, Hh // G, state, slot, cu, pos,
                              tok=tok, skip=dev["D"])
        outs.append(seqmix.gated_rmsnorm(o, dev["norm"], uu[:, :inner], eps, torch.float32,
                                         groups=ng, silu_first=True))
        at += c
    # the oracle's mixer with an identity input and output projection
    ud = u.double()
    sdd = {"x." + k: v.double() for k, v in sd.items()}
    sdd["x.in"] = torch.eye(ud.shape[1], dtype=F64)
    sdd["x.o"] = torch.eye(inner, dtype=F64)
    want = O.mixer_mamba2(sdd, "x.", m, ud, eps)
    assert float(state[0].min()) == 5.0 and float(state[1].max()) == 5.0
    return torch.cat(outs).cpu().double(), want


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[37], [1] * 20, [2, 1, 3, 17, 1, 13]], ids=lambda c: str(len(c)))
@pytest.mark.parametrize("m", [O.mamba()[1], O.mamba(3, 5, 3, 1, 1, 3)[1], O.mamba(8, 64, 128, 2, 3, 1)[1],
                               O.mamba(2, 12, 70, 2, 7, 4)[1]], ids=["small", "odd", "wide", "taps7"])
def test_state_space_mixer(device, m, cuts):
    got, want = _mamba_case(device, m, cuts)
    assert (got - want).abs().max() < 3e-4 * max(1.0, float(want.abs().max()))


@pytest.mark.parametrize("device", DEVICES)
def test_router_sigmoid_groups(device):
    """Groups rank by the sum of their two best scores: the first group holds
    the single best expert but loses to a group of two good ones."""
    z = torch.tensor([[3.0, -4.0, -4.0, 1.5, 1.4, -3.0, 0.1, 0.0, 0.2],
                      [0.0, 0.1, 0.2, 2.0, -5.0, -5.0, 1.0, 1.1, -1.0]])
    idx, wt = seqmix.moe_route(z.to(device), None, 3, 1, 2, sigmoid=True, group_rank=2)
    assert sorted(idx[0].tolist()) == [3, 4] and sorted(idx[1].tolist()) == [6, 7]
    for t in range(2):
        assert sorted(idx[t].tolist()) == sorted(O.route(torch.sigmoid(z[t].double()), 2, 3, 1))
        assert torch.allclose(wt[t].cpu().double(), torch.sigmoid(z[t].double())[idx[t].long().cpu()],
                              atol=1e-6)
    # by the best score alone the first group would have won
    idx1, _ = seqmix.moe_route(z.to(device), None, 3, 1, 2, sigmoid=True, group_rank=1)
    assert 0 in idx1[0].tolist()
    g = torch.Generator().manual_seed(5)
    z = torch.randn(64, 24, generator=g) * 2
    for count, keep, top in ((1, 1, 5), (24, 3, 3), (4, 2, 7), (3, 3, 1), (6, 5, 4)):
        idx, wt = seqmix.moe_route(z.to(device), None, count, keep, top, sigmoid=True, group_rank=2)
        for t in range(64):
            s = torch.sigmoid(z[t].double())
            assert sorted(idx[t].tolist()) == sorted(O.route(s, top, count, keep)), (count, t)


@pytest.mark.parametrize("device", DEVICES)
def test_geglu(device):
    g = torch.Generator().manual_seed(6)
    x = torch.randn(7, 2 * 37, generator=g) * 3
    got = seqmix.act_mul_any(x.to(device), "gelu_tanh")
    want = O.gelu_tanh(x[:, :37].double()) * x[:, 37:].double()
    assert (got.cpu().double() - want).abs().max() < 2e-6


# ------------------------------------------------------------ whole models
@pytest.mark.parametrize("device", DEVICES)
def test_residual_after_every_layer_run(device, full_model):
    cfg, sd = full_model
    toks = tokens(29, cfg["vocab"], 10)
    want = []
    O.forward(cfg, sd, toks, want)
    eng = engine(cfg, sd, device)
    max_q, max_ctx, host = eng._meta([eng.open_sequence()], [toks], decode=False)
    host["logit_idx"] = np.asarray([0], np.int64)
    meta = eng._build_meta(eng._to_device(host), max_q, max_ctx, False)
    got = []
    eng.model.forward(meta, eng.kv, got)
    assert len(got) == len(want) == 8
    for r, (a, b) in enumerate(zip(got, want)):
        assert (a.cpu().double() - b).abs().max() < 2e-4 * float(b.abs().max()), r


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_whole_prompt(device, dtype, full_model):
    cfg, sd = full_model
    toks = tokens(70, cfg["vocab"], 11)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device, dtype)
    got = eng.step_logits([eng.open_sequence()], [toks], [list(range(len(toks)))])
    if dtype == torch.float32:
        assert rel_err(got, want) < TOL[dtype]
    else:
        # single rows move under 16-bit rounding when a router score is nearly
        # tied: the typical row is what is pinned
        assert rel_err(got, want, 0.5) < TOL[dtype] and rel_err(got, want, 0.9) < 0.5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[1], [2], [3, 2, 7], [16], [17, 1, 1, 30], [5, 64]],
                         ids=lambda c: "x".join(map(str, c)))
def test_portions_and_decode(device, cuts, full_model):
    """Token-by-token decoding and portions of any size (down to two tokens,
    shorter than the convolutions, across page borders at 16 and window edges
    at 7 and 20) give the whole prompt's logits."""
    cfg, sd = full_model
    toks = tokens(53, cfg["vocab"], 12)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device)
    got = feed(eng, eng.open_sequence(), toks, cuts)
    assert rel_err(got, want) < TOL[torch.float32]


@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_and_reuse(device, full_model):
    """Four unequal requests, portions beside single tokens in one step; two
    end early and two new ones take over their pages and state slots. Every
    request's logits equal the ones it gets alone (oracle)."""
    cfg, sd = full_model
    V = cfg["vocab"]
    reqs = {n: tokens(L, V, 20 + i) for i, (n, L) in
            enumerate([("a", 41), ("b", 1), ("c", 18), ("d", 33), ("e", 25), ("f", 47)])}
    want = {n: O.forward(cfg, sd, t) for n, t in reqs.items()}
    eng = engine(cfg, sd, device, max_tokens=192, max_seqs=4)
    plan = {"a": [7, 1, 1, 16, 2, 1, 13], "b": [1], "c": [2, 15, 1], "d": [16, 16, 1],
            "e": [3, 1, 21], "f": [30, 1, 16]}
    at = {n: 0 for n in reqs}
    live, waiting, got = {}, ["a", "b", "c", "d", "e", "f"], {n: [] for n in reqs}
    steps = 0
    while waiting or live:
        while waiting and len(live) < 4:
            n = waiting.pop(0)
            live[n] = eng.open_sequence()
        names = list(live)
        feeds, wants = [], []
        for n in names:
            k = plan[n].pop(0)
            feeds.append(reqs[n][at[n]:at[n] + k])
            wants.append(list(range(k)))
            at[n] += k
        out = eng.step_logits([live[n] for n in names], feeds, wants)
        o = 0
        for n, f in zip(names, feeds):
            got[n].append(out[o:o + len(f)])
            o += len(f)
            if at[n] == len(reqs[n]):
                eng.close_sequence(live.pop(n))
        steps += 1
    assert steps > 5
    for n in reqs:
        assert rel_err(torch.cat(got[n]), want[n]) < TOL[torch.float32], n
    assert eng.kv.pool.free_blocks() == 192 // 16 and eng.kv.slots.free_slots() == 4


@pytest.mark.parametrize("device", DEVICES)
def test_slot_and_pages_reused_clean(device, full_model):
    """A pool of exactly one request's size, every state tensor and page
    overwritten with junk between requests: the next request must not see it."""
    cfg, sd = full_model
    eng = engine(cfg, sd, device, max_tokens=48, max_seqs=1)
    for i, n in enumerate([40, 48, 3, 33]):
        toks = tokens(n, cfg["vocab"], 30 + i)
        seq = eng.open_sequence()
        got = feed(eng, seq, toks, [9, 1, 2])
        eng.close_sequence(seq)
        assert rel_err(got, O.forward(cfg, sd, toks)) < TOL[torch.float32], i
        for t in eng.kv.state.values():
            t.fill_(1e3)
        for named in eng.kv.rows.values():
            for t in named.values():
                t.fill_(-1e3)
        for a, b in eng.kv.kv_rows.values():
            a.fill_(50.0), b.fill_(-50.0)
    assert eng.kv.pool.free_blocks() == 3 and eng.kv.slots.free_slots() == 1


LOOPS = {
    "none": (FULL, None), "whole": (FULL[:4], (0, 4, 3)), "once": (FULL, (2, 5, 1)),
    "one_layer": (FULL[:3], (2, 3, 4)), "empty": (FULL[:2], (1, 1, 5)),
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", list(LOOPS))
def test_repeated_stretch_variants(device, name):
    """No repetition, the whole stack repeated, a single pass, one state-space
    layer repeated four times (a state per pass), an empty stretch."""
    layers, loop = LOOPS[name]
    cfg = O.make_config(layers, width=24, vocab=40, loop=loop)
    sd = O.make_weights(cfg, 3)
    toks = tokens(31, 40, 5)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device)
    got = feed(eng, eng.open_sequence(), toks, [6, 1, 1, 9])
    assert rel_err(got, want) < TOL[torch.float32]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("window,keep", [(16, 0), (16, 16), (17, 3), (32, 1), (33, 40), (1, 0)])
def test_window_edges_in_prompts_and_decoding(device, window, keep):
    """Windows that end on, before and after page borders (16) with kept first
    tokens below, at and above a page; the sequence runs far past the window
    in portions and in single tokens."""
    cfg = O.make_config([(O.attn2(heads=2, kv_heads=1, dim=8, window=window, keep=keep, dims=4), None),
                         (O.attn2(heads=2, kv_heads=2, dim=16, window=window + 1, keep=keep, dims=0,
                                  cap=0.0), O.dense_ff(16))], width=16, vocab=30)
    sd = O.make_weights(cfg, 7)
    toks = tokens(100, 30, 8)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device, max_tokens=112)
    for cuts in ([100], [40] + [1] * 60, [15, 2, 31]):
        seq = eng.open_sequence()
        assert rel_err(feed(eng, seq, toks, cuts), want) < TOL[torch.float32], cuts
        eng.close_sequence(seq)


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(device, full_model):
    """Sequences of one, two and three tokens (shorter than every convolution
    and window), alone and side by side."""
    cfg, sd = full_model
    eng = engine(cfg, sd, device)
    seqs = [tokens(n, cfg["vocab"], 70 + n) for n in (1, 2, 3)]
    rs = [eng.open_sequence() for _ in seqs]
    got = eng.step_logits(rs, seqs, [list(range(len(s))) for s in seqs])
    want = torch.cat([O.forward(cfg, sd, s) for s in seqs])
    assert rel_err(got, want) < TOL[torch.float32]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_other_sizes(device, dtype):
    """Sizes that share no factor with the usual ones: one head, as many
    key/value heads as heads, a value size unlike the key size, one expert group,
    one expert chosen, one tap, a temperature that changes every position."""
    layers = [(O.attn(heads=1, kv_heads=1, dim=10, vdim=6, every=1, coef=1.5), O.moe_ff(5, 1, 12, 1, 1)),
              (O.mamba(heads=1, vdim=20, state=6, groups=1, conv=1, norm_groups=5), O.dense_ff(9)),
              (O.attn2(heads=3, kv_heads=3, dim=12, window=4, keep=4, dims=12, cap=0.5),
               O.moe_ff(8, 4, 4, 2, 2)),
              (O.attn(heads=9, kv_heads=1, dim=6, vdim=14, coef=None), None)]
    cfg = O.make_config(layers, width=20, vocab=33, eps=1e-3, logit_scale=2.0, loop=(0, 2, 2))
    sd = O.make_weights(cfg, 9)
    toks = tokens(45, 33, 13)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device, dtype)
    got = feed(eng, eng.open_sequence(), toks, [20, 3, 1])
    if dtype == torch.float32:
        assert rel_err(got, want) < TOL[dtype]
    else:
        assert rel_err(got, want, 0.5) < TOL[dtype] and rel_err(got, want, 0.9) < 0.5


@pytest.mark.parametrize("device", DEVICES)
def test_long_decode(device):
    """150 single-token steps over many windows and pages."""
    cfg = O.make_config([(O.mamba(heads=2, vdim=8, state=4, groups=1), None),
                         (O.attn2(heads=4, kv_heads=2, dim=8, window=9, keep=2, dims=8),
                          O.moe_ff(experts=4, top=2, ff=16, count=2, keep=1)),
                         (O.attn(heads=2, kv_heads=1, dim=8, every=16), None)],
                        width=24, vocab=60, loop=(0, 2, 2))
    sd = O.make_weights(cfg, 4)
    toks = tokens(160, 60, 6)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, device, max_tokens=160)
    got = feed(eng, eng.open_sequence(), toks, [10] + [1] * 150)
    assert rel_err(got, want) < TOL[torch.float32]


# ------------------------------------------- the engine's own entry points
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_scheduler(device, full_model):
    """Schema-less requests through ``submit_batch`` (continuous batching:
    inline prompts, chunked prompts in mixed steps, decode steps) produce the
    oracle's greedy continuation."""
    cfg, sd = full_model
    V = cfg["vocab"]
    prompts = [tokens(n, V, 40 + i) for i, n in enumerate([5, 90, 23, 70])]
    n_new = 6

    def greedy(p):
        seq = list(p)
        for _ in range(n_new):
            seq.append(int(O.forward(cfg, sd, seq)[-1].argmax()))
        return seq[len(p):]
    want = [greedy(p) for p in prompts]
    eng = engine(cfg, sd, device, max_tokens=512, max_seqs=4)
    eng.chunk_prefill = 32          # prompts longer than inline_prefill go in 32-token chunks
    eng.inline_prefill = 8
    reqs = [GenRequest(p, None, max_new_tokens=n_new) for p in prompts]
    try:
        eng.submit_batch(reqs[:2]).result(timeout=300)
        f1 = eng.submit_batch(reqs[2:3])
        f2 = eng.submit_batch(reqs[3:])
        f1.result(timeout=300), f2.result(timeout=300)
    finally:
        eng.stop()
    for r, w in zip(reqs, want):
        assert r.done and r.grammar.emitted == w
    assert eng.kv.slots.free_slots() == 4


def test_generate_entry_point(full_model):
    cfg, sd = full_model
    p = tokens(12, cfg["vocab"], 50)
    eng = engine(cfg, sd, "cpu")
    r = eng.generate([GenRequest(p, None, max_new_tokens=3)])[0]
    seq = list(p)
    for _ in range(3):
        seq.append(int(O.forward(cfg, sd, seq)[-1].argmax()))
    assert r.grammar.emitted == seq[len(p):]


def test_trace_replay_program(tmp_path, full_model):
    """The replay command on a checkpoint folder: steps on stdin, logits files
    and ``done`` lines out; a request that sits out a step goes on later."""
    from loqa_hub_amd.models.loader import write_safetensors
    cfg, sd = full_model
    model = tmp_path / "m"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(cfg))
    write_safetensors({k: v.to(torch.bfloat16) for k, v in sd.items()},
                      str(model / "model.safetensors"))
    a, b = tokens(20, cfg["vocab"], 60), tokens(9, cfg["vocab"], 61)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:11], "want": [0, 10]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:8], "want": []}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[11:], "want": [8]},
                                {"id": "b", "tokens": b[8:], "want": [0]}], "end": ["a", "b"]},
    ]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, "-m", "loqa_hub_amd.cli.trace_run", "--model", str(model),
                        "--dtype", "float32", "--out", str(out), "--max-tokens", "64",
                        "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                       capture_output=True, cwd=ROOT, timeout=300)
    assert p.returncode == 0, p.stderr
    assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == \
        ["done 0", "done 1", "done 2"]
    V = cfg["vocab"]
    wa, wb = O.forward(cfg, sd, a), O.forward(cfg, sd, b)
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V))
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V))
    assert not (out / "1.f32").exists()
    assert rel_err(g0, wa[[0, 10]]) < TOL[torch.float32]
    assert rel_err(g2, torch.stack([wa[19], wb[8]])) < TOL[torch.float32]


# ------------------------------------------- matrix-core paths (bf16, GPU only)
@pytest.mark.gpu
@pytest.mark.parametrize("H,G,D,Dv,window,keep,cap", [
    (4, 2, 64, 64, 0, 0, 0.0), (6, 2, 128, 128, 48, 5, 20.0), (8, 1, 64, 128, 70, 130, 0.0),
    (2, 2, 128, 64, 200, 0, 2.0), (16, 2, 64, 64, 1, 1, 0.0)])
def test_window_attention_matrix_cores(H, G, D, Dv, window, keep, cap):
    """The prompt-portion kernel against the oracle and against the keys-parallel
    form: long prompts whose middle key tiles are skipped, portions that start
    deep inside a sequence, single tokens beside them, an output gate."""
    for gate in (False, True):
        lens, feeds = [700, 1, 333, 90, 450], [700, 1, 70, 17, 1]
        a, want = _attention_case("cuda", torch.bfloat16, H, G, D, Dv, window, keep, cap, lens, feeds,
                                  gate, mfma=True, gate_pad=(8, 16))
        b, _ = _attention_case("cuda", torch.bfloat16, H, G, D, Dv, window, keep, cap, lens, feeds,
                               gate, mfma=False, gate_pad=(8, 16))
        scale = float(want.abs().max())
        assert (a - want).abs().max() < 0.03 * scale and (b - want).abs().max() < 0.03 * scale
        assert (a - b).abs().max() < 0.03 * scale


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("splits", [None, 2, 5, 16])
def test_window_attention_key_splits(dtype, splits):
    """Decode rows whose keys are dealt out to several workgroups and merged by
    the combine launch: long and short contexts side by side, a window with
    kept first tokens, an output gate, a far key that must be found."""
    tol = 2e-5 if dtype == torch.float32 else 0.03
    for window, keep, cap in ((0, 0, 0.0), (200, 70, 20.0)):
        got, want = _attention_case("cuda", dtype, 8, 2, 64, 64, window, keep, cap,
                                    [1500, 3, 700, 64, 65], [1, 1, 1, 1, 2], True, mfma=False,
                                    gate_pad=(8, 16), splits=splits)
        assert (got - want).abs().max() < tol * max(1.0, float(want.abs().max()))
    got, want = _attention_case("cuda", torch.float32, 2, 1, 16, 16, 0, 0, 0.0, [1500], [1], False,
                                mfma=False, spike=(1234, 40.0), splits=splits)
    assert (got - want).abs().max() < 2e-5


@pytest.mark.gpu
@pytest.mark.parametrize("back", [0, 47, 48, 49, 63, 64, 65, 300])
def test_window_edges_matrix_cores(back):
    for window, keep in ((48, 5), (64, 65), (0, 0)):
        got, want = _attention_case("cuda", torch.bfloat16, 2, 1, 64, 64, window, keep, 0.0, [400],
                                    [400], False, mfma=True, spike=(back, 60.0))
        assert (got - want).abs().max() < 0.03 * float(want.abs().max()), (window, keep)


@pytest.mark.gpu
def test_serving_sizes_bf16():
    """A model with matrix-core head sizes in bfloat16: whole prompt, portions
    and decoding agree with the oracle within 16-bit rounding."""
    layers = [(O.mamba(heads=4, vdim=32, state=16, groups=1), O.dense_ff(96)),
              (O.attn(heads=4, kv_heads=2, dim=64, every=16), O.moe_ff(6, 2, 32, 3, 2)),
              (O.attn2(heads=2, kv_heads=1, dim=128, window=24, keep=3, dims=64, cap=30.0),
               O.moe_ff(6, 2, 32, 3, 2))]
    cfg = O.make_config(layers, width=128, vocab=90, loop=(1, 3, 2))
    sd = O.make_weights(cfg, 12)
    toks = tokens(200, 90, 14)
    want = O.forward(cfg, sd, toks)
    eng = engine(cfg, sd, "cuda", torch.bfloat16, max_tokens=208)
    for cuts in ([200], [150, 30] + [1] * 20, [33, 2, 70]):
        seq = eng.open_sequence()
        got = feed(eng, seq, toks, cuts)
        eng.close_sequence(seq)
        assert rel_err(got, want, 0.5) < TOL[torch.bfloat16] and rel_err(got, want, 0.9) < 0.25, cuts
