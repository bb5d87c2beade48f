"""Nefivik in the engine against the plain oracle (tests/nefivik_oracle.py).

Every test builds its own small configuration and random (or crafted) weights
in the checkpoint's naming, runs the engine -- scheduler, page and state-slot
manager, model runner, the model's ops -- and compares with the oracle's
dense, whole-sequence float64 arithmetic.  On `cpu` the ops run their PyTorch
forms, on `cuda` (gpu marker) the gfx950 kernels, in float32 and bfloat16.
"""
from __future__ import annotations

import math

import pytest
import torch

import nefivik_oracle as O
from dynamo_exp_amd.engine.engine import EngineConfig, LLMEngine
from dynamo_exp_amd.engine.request import SamplingParams
from dynamo_exp_amd.models.config import LayeredConfig
from dynamo_exp_amd.models.nefivik import NefivikForCausalLM
from dynamo_exp_amd.ops import mixers as mx
from dynamo_exp_amd.ops import moe
from dynamo_exp_amd.ops import recurrent as rc

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
CASES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64


# ----------------------------------------------------------------- configurations
def delta(H=3, d=20):
    return {"type": "general_delta", "mixer": {"heads": H, "dim": d}}


def attn(H=6, G=3, d=20, dv=12, window=9, conv=3, rot=8, scaling=True, kv_from=None, base=100.0):
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": d ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if conv:
        m["conv"] = conv
    if rot:
        m["rot"] = {"base": base, "dims": rot}
        if scaling:
            m["rot"]["scaling"] = {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 24}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m}


def experts(E=8, top=2, ff=24, groups=(4, 2), limit=1.5):
    r = {"experts": E, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}


def layer(mix, mlp):
    return {**mix, "mlp": mlp}


def config(layers, width=72, vocab=97, side=6, eps=1e-5):
    return LayeredConfig(name="t", architecture="Nefivik", vocab_size=vocab, hidden_size=width, layers=layers,
                         rms_norm_eps=eps, token_side={"dim": side} if side else None)


def cfg_dict(cfg: LayeredConfig) -> dict:
    d = {"layers": cfg.layers, "norm": {"eps": cfg.rms_norm_eps}, "vocab": cfg.vocab_size, "width": cfg.hidden_size}
    if cfg.token_side:
        d["token_side"] = cfg.token_side
    return d


CONFIGS = {
    # both mixers, a layer that reads another's keys and values, windows and taps that differ per
    # layer, q/k width != value width, a layer without feed-forward
    "mixed": lambda: config([layer(delta(), experts()),
                             layer(attn(window=5, conv=3), experts(E=6, top=3, groups=(3, 2), ff=20)),
                             layer(delta(H=2, d=12), None),
                             layer(attn(window=9, conv=4, rot=20, kv_from=1), experts()),
                             layer(attn(H=4, G=2, d=8, dv=18, window=30, conv=2, rot=4, scaling=False), experts())]),
    # values a model may happen to make equal or one: one head, one expert per group, every group
    # kept, one choice, a window of one token, one tap, no rotation, a side input one column wide
    "ones": lambda: config([layer(attn(H=1, G=1, d=8, dv=8, window=1, conv=1, rot=0), experts(E=4, top=1, groups=(4, 4))),
                            layer(delta(H=1, d=8), experts(E=3, top=1, groups=None, ff=8)),
                            layer(attn(H=2, G=1, d=8, dv=4, window=64, conv=0, rot=8, scaling=False), experts(E=2, top=2, groups=(1, 1)))],
                           width=32, side=1),
    # nothing divides by 4 or 8 (scalar paths), no window in one layer (plain causal), no side input
    "odd": lambda: config([layer(attn(H=4, G=2, d=18, dv=7, window=0, conv=5, rot=6), experts(E=5, top=2, groups=None, ff=10)),
                           layer(delta(H=2, d=18), experts(E=5, top=2, groups=None, ff=10)),
                           layer(delta(H=1, d=34), None)], width=102, vocab=101, side=0),
    # head widths the matrix-core kernels serve (bf16 on the GPU); recurrent heads of 64 and 128
    "tiles": lambda: config([layer(attn(H=4, G=2, d=32, dv=32, window=20, rot=16), experts(ff=32)),
                             layer(delta(H=2, d=64), experts(ff=32)),
                             layer(attn(H=2, G=1, d=64, dv=64, window=70, conv=4, rot=32), experts(ff=32)),
                             layer(attn(H=2, G=1, d=64, dv=64, window=33, conv=2, rot=64, kv_from=2), None),
                             layer(delta(H=1, d=128), experts(ff=32))], width=64, side=8),
}


def weights(cfg, seed=0):
    """Random weights with a decisive router: most of a token's score mass sits on one expert, so an
    expert choice that bf16 rounding decides the other way concerns small weights only (with
    recurrent layers a wrong choice would otherwise follow the sequence through the state)."""
    sd = NefivikForCausalLM(cfg, "cpu", torch.float32).random_state(seed)
    for k in sd:
        if k.endswith("mlp.router"):
            sd[k] = (sd[k].float() * 8).bfloat16()
    return sd


def engine(cfg, sd, device, dtype, blocks=48, bs=8, graphs=False, seqs=4):
    model = NefivikForCausalLM(cfg, device, DT[dtype]).load_state(sd)
    return LLMEngine(EngineConfig(model="t", device=device, dtype=dtype, block_size=bs, num_gpu_blocks=blocks,
                                  max_model_len=blocks * bs, max_num_seqs=seqs, enable_prefix_caching=False,
                                  use_cuda_graph=graphs, graph_sizes=(1, 2, 4), async_schedule=False),
                     model_cfg=cfg, model=model)


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def close(got, want, dtype, what=""):
    """Logit rows agree: error relative to the rows' spread, after the mean is taken off.  In
    bfloat16 a minority of rows may differ more (a close expert choice decided the other way)."""
    got = got.detach().double().cpu()
    want = want.double()
    a, b = got - got.mean(-1, keepdim=True), want - want.mean(-1, keepdim=True)
    err = ((a - b) ** 2).mean(-1).sqrt() / b.pow(2).mean().sqrt()
    if dtype == "float32":
        assert float(err.max()) < 3e-4, f"{what}: error {float(err.max()):.3g} at row {int(err.argmax())}"
    else:
        assert float(err.median()) < 4e-2 and float((err > 8e-2).float().mean()) <= 0.2, \
            f"{what}: median error {float(err.median()):.3g}, max {float(err.max()):.3g}"


def run_cut(eng, rid, toks, cuts):
    """Feed `toks` in portions of the given sizes (the rest one by one); logits of all positions."""
    out, at = [], 0
    sizes = list(cuts) + [1] * (len(toks) - sum(cuts))
    for n in sizes:
        part = toks[at:at + n]
        last = at + n == len(toks)
        got = eng.forced_step([(rid, part, list(range(n)))], [rid] if last else [])
        out.append(got[rid])
        at += n
    return torch.cat(out, 0)


def step_meta(device, chunks, slots):
    """Rows of one step: chunks = [(first position, rows)] per sequence, in row order."""
    pos = torch.cat([torch.arange(p, p + n) for p, n in chunks]).to(device)
    row_seq = torch.cat([torch.full((n,), i, dtype=torch.int32) for i, (_, n) in enumerate(chunks)]).to(device)
    b = [0]
    for _, n in chunks:
        b.append(b[-1] + n)
    return pos, row_seq, torch.tensor(b, dtype=torch.int32, device=device), \
        torch.tensor(slots, dtype=torch.int32, device=device)


# ----------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,dk,dv", [(2, 16, 16), (3, 20, 20), (1, 64, 64), (2, 128, 128), (1, 34, 18), (1, 200, 40)])
def test_delta_rule_alone(device, H, dk, dv):
    """Two sequences scanned whole, then the same in steps of unequal portions (19, 2, 1, ...) with
    the slots swapped around a third sequence's garbage, against the token-by-token oracle."""
    torch.manual_seed(dk)
    T = 41
    r, k, a, w = (torch.randn(2, T, H * dk) for _ in range(4))
    v = torch.randn(2, T, H * dv)
    ab, wb = torch.randn(H * dk) * 0.5, torch.randn(H * dk)
    want = []
    for s in range(2):
        wd = torch.exp(-math.exp(-0.5) * O.sigmoid(w[s].double() + wb.double()))
        ad = O.sigmoid(a[s].double() + ab.double())
        o, S = O.delta_scan(r[s].double().view(T, H, dk), k[s].double().view(T, H, dk), v[s].double().view(T, H, dv),
                            wd.view(T, H, dk), ad.view(T, H, dk))
        want.append((o.reshape(T, H * dv), S))
    d = lambda t: t.to(device)  # noqa: E731
    state = torch.randn(5, H, dv, dk, device=device)  # garbage: position 0 must reset it
    cat = lambda t, cuts: d(torch.cat([t[s, p:p + n] for s, (p, n) in enumerate(cuts)]))  # noqa: E731
    for portions in ([(T,)], [(19, 2, 1, 1, 9, 8, 1), (3, 30, 7, 1)]):
        if len(portions) == 1:
            portions = portions * 2
        at = [0, 0]
        got = [[], []]
        it = [list(p) for p in portions]
        while any(it):
            live = [s for s in (0, 1) if it[s]]
            cuts = [(at[s], it[s].pop(0)) for s in live]
            pos, _, seq_rows, slots = step_meta(device, cuts, [3 if s == 0 else 1 for s in live])
            sel = lambda t: d(torch.cat([t[s, p:p + n] for s, (p, n) in zip(live, cuts)]))  # noqa: E731
            o = rc.delta_rule(sel(r), sel(k), sel(v), sel(a), sel(w), d(ab), d(wb), state, pos, seq_rows, slots, H, dk, dv)
            for i, (s, (p, n)) in enumerate(zip(live, cuts)):
                b0 = int(seq_rows[i])
                got[s].append(o[b0:b0 + n].cpu())
                at[s] += n
        for s in range(2):
            assert torch.allclose(torch.cat(got[s]).double(), want[s][0], atol=2e-4, rtol=1e-4)
            assert torch.allclose(state[3 if s == 0 else 1].cpu().double().transpose(1, 2), want[s][1], atol=2e-4, rtol=1e-4)
    # a decode step (row i is sequence i), one padding row that owns no slot
    pos = torch.tensor([T, T, 0], device=device)
    slots = torch.tensor([3, 1, -1], dtype=torch.int32, device=device)
    x = torch.randn(3, H * dk)
    o = rc.delta_rule(d(x), d(x), d(torch.randn(3, H * dv)), d(x), d(x), None, None, state, pos, None, slots, H, dk, dv)
    assert bool(torch.isfinite(o).all()) and float(o[2].abs().max()) == 0.0
    del cat


@pytest.mark.parametrize("device", DEVICES)
def test_delta_rule_removes_and_decays(device):
    """Crafted: with removal rate 1 and a repeated key direction the old value of that direction is
    replaced, with rate 0 it stays; the decay alone scales what a read returns."""
    H, dk, dv = 1, 16, 16
    e0 = torch.zeros(dk)
    e0[0] = 2.0
    k = torch.stack([e0, e0, e0])
    v = torch.stack([torch.full((dv,), 1.0), torch.full((dv,), 5.0), torch.zeros(dv)])
    r = torch.stack([e0, e0, e0])
    big = torch.full((3, dk), 30.0)
    pos, _, seq_rows, slots = step_meta(device, [(0, 3)], [0])
    for a_logit, w_logit, want in ((big, -big, [4.0, 20.0, 0.0]),        # a = 1, w = 1: each write replaces
                                   (-big, -big, [4.0, 24.0, 24.0]),       # a = 0, w = 1: writes add up
                                   (-big, big, [4.0, 4 * math.exp(-math.exp(-0.5)) + 20.0, None])):
        state = torch.zeros(1, H, dv, dk, device=device)
        o = rc.delta_rule(r.to(device), k.to(device), v.to(device), a_logit.to(device), w_logit.to(device), None, None,
                          state, pos, seq_rows, slots, H, dk, dv)
        for t, x in enumerate(want):
            if x is not None:
                assert abs(float(o[t, 0]) - x) < 1e-4, (t, float(o[t, 0]), x)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps,half,n_k,d,dv", [(3, 4, 2, 20, 6), (1, 0, 2, 20, 6), (5, 10, 0, 20, 6), (2, 3, 1, 20, 6),
                                               (4, 8, 2, 32, 16), (3, 16, 1, 32, 8), (2, 0, 2, 16, 24)])
def test_conv_rope_cache_alone(device, taps, half, n_k, d, dv):
    """Short convolution, rotation and cache write of two sequences, whole and in portions down to
    one row (shorter than the taps), slots reused with garbage in them, against the oracle."""
    torch.manual_seed(taps)
    n_q, T, bs = 3, 23, 4
    C = n_q * d + n_k * (d + dv)
    x = torch.randn(2, T, C + (5 if d % 8 else 8))  # (the wide shapes keep rows 16-byte aligned: the vector kernel)
    cw = torch.randn(C, taps)
    rot = {"base": 50.0, "dims": 2 * half, "scaling": {"factor": 4.0, "low": 1.0, "high": 3.0, "original": 16}}
    inv = rc.rotary_frequencies(2 * half, 50.0, rot["scaling"]) if half else None
    if half:
        assert torch.allclose(inv.double(), O.rotary_frequencies(rot), rtol=1e-6)
    want = []
    for s in range(2):
        y = O.short_conv(x[s, :, :C].double(), cw.double())
        q = O.rotate(y[:, :n_q * d].view(T, n_q, d), rot if half else None).reshape(T, -1)
        kk = O.rotate(y[:, n_q * d:(n_q + n_k) * d].view(T, n_k, d), rot if half else None).reshape(T, -1)
        want.append((q, kk, y[:, (n_q + n_k) * d:]))
    d_ = lambda t: None if t is None else t.to(device)  # noqa: E731
    tail = torch.randn(4, taps - 1, C, device=device)
    kc = torch.zeros(16 * bs, n_k * d, device=device) if n_k else None
    vc = torch.zeros(16 * bs, n_k * dv, device=device) if n_k else None
    tables = torch.randperm(16)[:12].view(2, 6)
    slot_of = lambda s, p: tables[s][p // bs] * bs + p % bs  # noqa: E731
    it = [[1, 1, 2, 9, 1, 9], [23]]
    at, got = [0, 0], [[], []]
    while any(it):
        live = [s for s in (0, 1) if it[s]]
        cuts = [(at[s], it[s].pop(0)) for s in live]
        pos, row_seq, seq_rows, slots = step_meta(device, cuts, [2 if s == 0 else 0 for s in live])
        xs = torch.cat([x[s, p:p + n] for s, (p, n) in zip(live, cuts)]).to(device)
        kvs = torch.cat([slot_of(s, torch.arange(p, p + n)) for s, (p, n) in zip(live, cuts)]).to(device)
        q = rc.conv_rope_cache(xs, d_(cw.t().contiguous()), tail, pos, kvs, row_seq, seq_rows, slots, n_q, n_k, d, dv, d_(inv), kc, vc)
        rc.conv_state_update(xs, tail, pos, seq_rows, slots)
        for i, (s, (p, n)) in enumerate(zip(live, cuts)):
            got[s].append(q[int(seq_rows[i]):int(seq_rows[i]) + n].cpu())
            at[s] += n
    for s in range(2):
        assert torch.allclose(torch.cat(got[s]).double(), want[s][0], atol=2e-5)
        if n_k:
            sl = slot_of(s, torch.arange(T)).to(device)
            assert torch.allclose(kc[sl].cpu().double(), want[s][1], atol=2e-5)
            assert torch.allclose(vc[sl].cpu().double(), want[s][2], atol=2e-5)
        if taps > 1:
            assert torch.equal(tail[2 if s == 0 else 0].cpu(), x[s, T - taps + 1:, :C])


@pytest.mark.parametrize("device", DEVICES)
def test_head_norm_gate_and_acts(device):
    torch.manual_seed(4)
    T, H, dv = 5, 3, 22
    o, w, g = torch.randn(T, H * dv) * 3, torch.randn(H * dv), torch.randn(T, H * dv + 3)
    want = O.unit_rms(o.double().view(T, H, dv), 1e-5).reshape(T, -1) * w.double() * O.sigmoid(g[:, 3:].double())
    got = rc.head_norm_gate(o.to(device), H, w.to(device), g.to(device)[:, 3:], 1e-5, torch.float32)
    assert torch.allclose(got.cpu().double(), want, atol=2e-5)
    x = torch.randn(7, 120) * 2
    xd = x.to(device)
    assert torch.allclose(mx.act_mul(xd[:, 3:40], None, "tanh").cpu().double(), torch.tanh(x[:, 3:40].double()), atol=1e-5)
    gg, uu = x[:, :60].double().clamp(max=1.5), x[:, 60:].double().clamp(-1.5, 1.5)
    want = gg * O.sigmoid(1.702 * gg) * (uu + 1)
    assert torch.allclose(mx.glu_act(xd, "swiglu_clamp", 1.5, 1.702).cpu().double(), want, atol=1e-5)
    assert float((want - x[:, :60].double() * O.sigmoid(1.702 * x[:, :60].double()) * (x[:, 60:].double() + 1)).abs().max()) > 0.1


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("W", [70, 72, 2052])
def test_gated_residual_step(device, W):
    torch.manual_seed(W)
    T, eps = 5, 1e-5
    X, c, g = torch.randn(T, W), torch.randn(T, W) * 3, torch.randn(T, W + 4) * 2
    gb, cw, nw = torch.randn(W), torch.randn(W), torch.randn(W)
    want_x = X.double() + O.rms_norm(c.double() * O.sigmoid(g[:, 4:].double() + gb.double()), cw.double(), eps)
    d = lambda t: t.to(device)  # noqa: E731
    Xd = d(X).clone()
    h, _ = mx.residual_step(Xd, c=d(c), c_w=d(cw), eps=eps, norm="rms", norm_w=d(nw), out_dtype=torch.float32,
                            c_gate=d(g)[:, 4:], c_gate_b=d(gb))
    assert torch.allclose(Xd.cpu().double(), want_x, atol=2e-5)
    assert torch.allclose(h.cpu().double(), O.rms_norm(want_x, nw.double(), eps), atol=5e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("E,top,groups", [(15, 3, (5, 2)), (8, 2, (4, 2)), (6, 1, (6, 6)), (5, 2, None), (64, 4, (8, 3))])
def test_route_softmax_groups(device, E, top, groups):
    """Softmax scores, groups ranked by their best score.  One group is made to hold the two next-best
    experts after a clear winner elsewhere: ranked by the sum of two it would win, by its best it loses."""
    torch.manual_seed(E)
    T = 40
    z = torch.randn(T, E) * 2
    if groups and groups[0] >= 3 and E // groups[0] >= 2:
        per = E // groups[0]
        z[:, :] = torch.randn(T, E) * 0.1 - 3
        z[:, 0] = 3.0            # group 0: one strong expert
        z[:, per] = 2.5          # group 1: one strong expert
        z[:, 2 * per] = 2.2      # group 2: two fairly strong experts (largest sum of two)
        z[:, 2 * per + 1] = 2.2
    r = {"experts": E, "top": top}
    gr = groups or (1, 1)
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    # the oracle's route on an identity router
    idx_w, w_w = O.route(z.double(), torch.eye(E, dtype=F64), r)
    idx, w = moe.route(z.to(device), None, top, gr[0], gr[1], score="softmax", group_score="max")
    assert torch.equal(idx.cpu().long().sort(-1).values, idx_w.sort(-1).values)
    assert torch.allclose(w.cpu().double().sort(-1).values, w_w.sort(-1).values, atol=1e-6)
    assert float(w.sum(-1).max()) <= 1.0 + 1e-5  # softmax scores of the chosen, not renormalised
    if groups and groups[0] >= 3 and groups[1] == 2 and E // groups[0] >= 2:
        assert not (idx.cpu() == 2 * (E // groups[0])).any()  # the group of the best pair lost to the two best singles


def paged(T, bs, n_blocks, width, device, dtype=torch.float32, seed=0):
    g = torch.Generator().manual_seed(seed)
    nb = -(-T // bs)
    table = torch.randperm(n_blocks, generator=g)[:nb].to(torch.int32)
    j = torch.arange(T)
    slots = table.long()[j // bs] * bs + j % bs
    return table[None].to(device), slots.to(device), torch.zeros(n_blocks * bs, width, dtype=dtype, device=device)


def dense_sigmoid_attention(q, k, v, scale, pb, size, gate):
    """Oracle: q [T, H, d], k [T, G, d], v [T, G, dv] -> [T, H, dv]."""
    T, H = q.shape[:2]
    rep = H // k.shape[1]
    s = torch.einsum("ihd,jhd->hij", q.double(), k.double().repeat_interleave(rep, 1)) * scale
    w = O.sigmoid(s + pb.double()[:, None, None]) * O.window_mask(T, size)[None]
    o = torch.einsum("hij,jhd->ihd", w, v.double().repeat_interleave(rep, 1))
    return o * O.sigmoid(gate.double())[:, :, None] if gate is not None else o


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("size", [0, 1, 6, 70])
@pytest.mark.parametrize("dims", [(4, 2, 20, 12), (3, 3, 8, 136), (4, 1, 12, 72)])
def test_row_attention_sigmoid(device, size, dims):
    """Sigmoid weights with a per-head bias and the head gate: prompt rows over a shuffled page
    table, then decode rows with the keys split in parts, against the dense oracle."""
    H, G, d, dv = dims
    T, bs = 70, 8
    torch.manual_seed(7)
    q, k, v = torch.randn(T, H, d) * 2, torch.randn(T, G, d) * 2, torch.randn(T, G, dv)
    pb, gate = torch.randn(H) - 1, torch.randn(T, H + 3)
    want = dense_sigmoid_attention(q, k, v, 0.4, pb, size, gate[:, 3:])
    table, slots, kc = paged(T, bs, 12, G * d, device)
    vc = torch.zeros(12 * bs, G * dv, device=device)
    kc[slots] = k.reshape(T, -1).to(device)
    vc[slots] = v.reshape(T, -1).to(device)
    pos = torch.arange(T, device=device)
    seq = torch.zeros(T, dtype=torch.int32, device=device)
    qd, gd = q.reshape(T, -1).to(device), gate.to(device)[:, 3:]
    mask = "window" if size else "causal"
    kw = dict(weights="sigmoid", head_bias=pb.to(device))
    got = mx.row_attention(qd, kc, vc, pos, seq, table, bs, H, 1, H // G, d, dv, 0.4, mask, size, 1, head_gate=gd, **kw)
    assert torch.allclose(got.cpu().double(), want, atol=5e-5)
    rows = torch.tensor([0, 1, 7, 8, 33, 69], device=device)
    got = mx.row_attention(qd[rows], kc, vc, pos[rows], None, table.expand(len(rows), -1).contiguous(), bs, H, 1,
                           H // G, d, dv, 0.4, mask, size, 2, head_gate=gd[rows], **kw)
    assert torch.allclose(got.cpu().double(), want[rows.cpu()], atol=5e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("size", [0, 1, 40, 129])
@pytest.mark.parametrize("dims", [(4, 2, 32, 32), (6, 2, 48, 48), (2, 2, 48, 96), (3, 1, 64, 64), (4, 4, 128, 128),
                                  (20, 1, 64, 64)])
def test_matrix_core_attention_sigmoid(size, dims):
    """The matrix-core kernels with sigmoid weights: a 263-row portion that starts at position 37 of
    a cached prefix (three tiles, the last ragged, cut inside pages and windows) beside two decode
    rows of another sequence, then decode rows alone, against the dense oracle over the bf16 values."""
    H, G, d, dv = dims
    T, bs, start = 300, 16, 37
    torch.manual_seed(5)
    q = torch.randn(T, H, d).bfloat16()
    k = (torch.randn(T, G, d) * 0.7).bfloat16()
    v = torch.randn(T, G, dv).bfloat16()
    pb = torch.randn(H) - 3
    gate = torch.randn(T, H).bfloat16()
    want = dense_sigmoid_attention(q, k, v, 0.2, pb, size, gate)
    perm = torch.randperm(40, generator=torch.Generator().manual_seed(3)).to(torch.int32)
    table = torch.stack([perm[:19], perm[19:38]]).contiguous().cuda()
    j = torch.arange(T, device="cuda")
    kc = torch.zeros(40 * bs, G * d, device="cuda", dtype=torch.bfloat16)
    vc = torch.zeros(40 * bs, G * dv, device="cuda", dtype=torch.bfloat16)
    for i in (0, 1):
        sl = table[i].long()[j // bs] * bs + j % bs
        kc[sl] = k.reshape(T, -1).cuda()
        vc[sl] = v.reshape(T, -1).cuda()
    rows = list(range(start, T)) + [5, 290]
    n_pre = T - start
    pos = torch.tensor(rows, device="cuda")
    seq = torch.tensor([0] * n_pre + [1, 1], dtype=torch.int32, device="cuda")
    tiles = torch.tensor(mx.tile_list(0, n_pre), dtype=torch.int32, device="cuda")
    qd, gd = q.reshape(T, -1).cuda()[pos], gate.cuda()[pos]
    mask = "window" if size else "causal"
    kw = dict(weights="sigmoid", head_bias=pb.cuda())
    scale_ = float(want.abs().max())
    assert mx.tile_attention_ok(qd, d, dv)
    got = mx.attention(qd, kc, vc, pos, seq, table, bs, H, 1, H // G, d, dv, 0.2, mask, size, 1, True, tiles, n_pre,
                       head_gate=gd, **kw)
    assert float((got.cpu().double() - want[rows]).abs().max()) < 1e-3 * max(1.0, scale_)
    got = mx.attention(qd, kc, vc, pos, seq, table, bs, H, 1, H // G, d, dv, 0.2, mask, size, 3, False, tiles, n_pre,
                       head_gate=gd, **kw)
    assert float((got.cpu().double() - want[rows]).abs().max()) < 2e-2 * max(1.0, scale_)
    dr = torch.tensor([0, 1, 63, 64, 65, 255, 299], device="cuda")
    got = mx.attention(q.reshape(T, -1).cuda()[dr], kc, vc, dr, None, table[:1].expand(len(dr), -1).contiguous(), bs,
                       H, 1, H // G, d, dv, 0.2, mask, size, 2, True, head_gate=gate.cuda()[dr], **kw)
    assert float((got.cpu().double() - want[dr.cpu()]).abs().max()) < 1e-3 * max(1.0, scale_)


# ----------------------------------------------------------------- crafted: one key stands out
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("size,bs", [(44, 16), (17, 8), (1, 8), (200, 8)])
def test_far_keys_window_edges(device, dtype, size, bs):
    """A cache of weak keys (weights near 0 through a negative head bias) in which one key matches
    the query strongly and carries a marked value: seen just inside the window, not just outside, at
    page borders, among hundreds, for prompt rows and decode rows alike."""
    H, G, d, dv, T = 2, 1, 32, 32, 180
    dt = DT[dtype]
    tol = 1e-4 if dtype == "float32" else 3e-2
    e0 = torch.zeros(d)
    e0[0] = 8.0
    pb = torch.full((H,), -12.0)
    table, slots, kc = paged(T, bs, 40, G * d, device, dt)
    vc = torch.zeros(40 * bs, G * dv, device=device, dtype=dt)
    for p in (T - 1, 150, bs * 9, bs * 9 + 1, 11):
        for mark in (p, p - size + 1, p - size, p - 1, 0, bs * 3 - 1, bs * 3):
            if not 0 <= mark <= p:
                continue
            K = torch.zeros(T, d)
            K[mark] = e0
            V = torch.zeros(T, dv)
            V[mark] = 1.0
            kc[slots] = K.to(device, dt)
            vc[slots] = V.to(device, dt)
            q = e0.repeat(H)[None].to(device, dt)
            seen = p - mark < size
            want = float(O.sigmoid(torch.tensor(64.0 * 0.25 - 12.0, dtype=F64))) if seen else 0.0
            pos = torch.tensor([p], device=device)
            for seq in (torch.zeros(1, dtype=torch.int32, device=device), None):  # a prompt row, a decode row
                tl = (torch.tensor([[0, 1]], dtype=torch.int32, device=device), 1) if seq is not None else (None, 0)
                got = mx.attention(q, kc, vc, pos, seq, table, bs, H, 1, H // G, d, dv, 0.25, "window", size, 1, False,
                                   *tl, weights="sigmoid", head_bias=pb.to(device))
                assert abs(float(got[0, 0, 0]) - want) < tol + 2e-3 * (1 - seen), (p, mark, seq is None, float(got[0, 0, 0]))


# ----------------------------------------------------------------- whole model
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_and_layers(device, dtype, name):
    """A whole prompt in one step: logits at every position, and (float32) the residual after
    every layer, against the oracle."""
    cfg = CONFIGS[name]()
    sd = weights(cfg, 1)
    toks = tokens(75, cfg.vocab_size, 2)
    lo = []
    want = O.forward(cfg_dict(cfg), sd, toks, lo)
    eng = engine(cfg, sd, device, dtype)
    if dtype == "float32":
        eng.model.trace_layers = []
    got = eng.forced_step([("a", toks, list(range(len(toks))))], ["a"])["a"]
    close(got, want, dtype, name)
    if dtype == "float32":
        assert len(eng.model.trace_layers) == len(cfg.layers)
        for i, (x, w) in enumerate(zip(eng.model.trace_layers, lo)):
            assert float((x.cpu().double() - w).abs().max()) < 2e-3 * float(w.abs().max()), f"layer {i}"
        eng.model.trace_layers = None
        got2 = eng.forced_step([("b", toks, list(range(len(toks))))], ["b"])["b"]  # the fused path, a reused slot
        close(got2, want, dtype, name + " fused")


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name,cuts", [("mixed", (0,)), ("mixed", (31, 2, 2, 17, 3)), ("ones", (2, 2, 2, 40)),
                                       ("odd", (50, 2)), ("tiles", (7, 64, 2)), ("tiles", (0,))])
def test_portions_and_decode(device, dtype, name, cuts):
    """Token-by-token decoding from the first token, and portions of several sizes down to two
    tokens followed by single tokens, against the whole-sequence oracle."""
    cfg = CONFIGS[name]()
    # (seeds under which no head's first read-out r.k is near zero: the unit norm per head that follows
    # would turn bf16 rounding of such a read-out into a change of sign)
    sd = weights(cfg, 4)
    toks = tokens(80, cfg.vocab_size, 5)
    want = O.forward(cfg_dict(cfg), sd, toks)
    eng = engine(cfg, sd, device, dtype)
    got = run_cut(eng, "a", toks, [c for c in cuts if c])
    close(got, want, dtype, f"{name} {cuts}")


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", ["mixed", "tiles"])
def test_mixed_batches_reuse(device, dtype, name):
    """Five unequal requests interleaved, portions beside single tokens, in a pool of pages and of
    state slots (three) that only fits them because both are given back and used again."""
    cfg = CONFIGS[name]()
    sd = weights(cfg, 5)
    lens = [70, 41, 90, 33, 58]
    reqs = {f"r{i}": tokens(n, cfg.vocab_size, 10 + i) for i, n in enumerate(lens)}
    want = {k: O.forward(cfg_dict(cfg), sd, t) for k, t in reqs.items()}
    eng = engine(cfg, sd, device, dtype, blocks=30, bs=8, seqs=3)
    plan = [[("r0", 9), ("r1", 2)], [("r0", 1), ("r1", 30), ("r2", 3)], [("r0", 40), ("r1", 1), ("r2", 1)],
            [("r0", 1), ("r1", 8), ("r2", 50)], [("r0", 19), ("r2", 1)], [("r2", 35), ("r3", 2)],
            [("r3", 31), ("r4", 2)], [("r4", 1)], [("r4", 55)]]
    at = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    for step in plan:
        entries, end = [], []
        for k, n in step:
            entries.append((k, reqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(reqs[k]):
                end.append(k)
        out = eng.forced_step(entries, end)
        for k, _ in step:
            got[k].append(out[k])
    assert eng.kv.num_free_state() == 3 and eng.kv.num_free() == 30
    for k in reqs:
        assert at[k] == len(reqs[k])
        close(torch.cat(got[k]), want[k], dtype, f"{name} {k}")


@pytest.mark.parametrize("device,dtype", CASES)
def test_long_decode_and_first_tokens(device, dtype):
    """146 consecutive decode steps after a two-token prompt: windows, taps and pages pass over
    decoded tokens; the first positions (fewer tokens than taps, than a window) are among them."""
    cfg = CONFIGS["mixed"]()
    sd = weights(cfg, 6)
    toks = tokens(148, cfg.vocab_size, 7)
    want = O.forward(cfg_dict(cfg), sd, toks)
    eng = engine(cfg, sd, device, dtype)
    got = run_cut(eng, "a", toks, (2,))
    close(got, want, dtype, "long decode")


@pytest.mark.parametrize("device,dtype", CASES)
def test_crafted_weights_show_faults(device, dtype):
    """Weights made so that faults move the logits: head biases near zero weight except for strong
    matches, a router whose second group holds the best pair but not the best expert, expert inputs
    beyond the clamp; the engine still agrees with the oracle, and the oracle's own variants with a
    window one token off or the state dropped differ visibly."""
    cfg = config([layer(delta(H=2, d=16), experts(E=6, top=2, groups=(3, 1), limit=0.5)),
                  layer(attn(H=2, G=1, d=16, dv=16, window=6, conv=3, rot=8), experts(E=6, top=2, groups=(3, 1), limit=0.5))],
                 width=48, vocab=61, side=4)
    sd = weights(cfg, 8)
    sd["l1.mix.pb"] = torch.tensor([-1.0, 0.5]).bfloat16()
    for e in range(6):
        sd[f"l0.mlp.e{e}.up"] = sd[f"l0.mlp.e{e}.up"] * 4
    toks = tokens(60, cfg.vocab_size, 9)
    want = O.forward(cfg_dict(cfg), sd, toks)
    eng = engine(cfg, sd, device, dtype)
    close(run_cut(eng, "a", toks, (13, 2, 30)), want, dtype, "crafted")
    wrong = cfg_dict(cfg)
    wrong["layers"] = [dict(L, mixer=dict(L["mixer"])) for L in wrong["layers"]]
    wrong["layers"][1]["mixer"]["mask"] = {"size": 7}
    off = O.forward(wrong, sd, toks)
    assert float((off - want).abs().max()) > 0.05 * float(want.abs().max())


# ----------------------------------------------------------------- the engine's own entry point
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation(device, dtype, graphs):
    """add_request + step(): chunked prefill, continuous batching, state slots handed out and taken
    back by the scheduler, HIP-graph decode on the GPU; greedy tokens equal the oracle's."""
    if graphs and device == "cpu":
        pytest.skip("graphs are a GPU path")
    cfg = CONFIGS["tiles" if device == "cuda" else "mixed"]()
    sd = weights(cfg, 11)
    model = NefivikForCausalLM(cfg, device, DT[dtype]).load_state(sd)
    eng = LLMEngine(EngineConfig(model="t", device=device, dtype=dtype, block_size=8, num_gpu_blocks=64,
                                 max_model_len=256, max_num_seqs=2, max_num_batched_tokens=24,
                                 use_cuda_graph=graphs, graph_sizes=(1, 2), async_schedule=False),
                    model_cfg=cfg, model=model)
    assert eng.cfg.enable_prefix_caching is False  # recurrent state cannot be served from the prefix cache
    if graphs:
        eng.warmup()
    prompts = [tokens(37, cfg.vocab_size, 20), tokens(9, cfg.vocab_size, 21), tokens(50, cfg.vocab_size, 22)]
    n_new = 12
    for i, p in enumerate(prompts):
        eng.add_request(f"g{i}", p, SamplingParams(max_tokens=n_new, ignore_eos=True))
    done = {}
    for _ in range(400):
        for r in eng.step():
            if r.finished:
                done[r.request_id] = list(r.output)
        if not eng.has_unfinished():
            break
    assert len(done) == 3 and eng.kv.num_free_state() == 2
    for i, p in enumerate(prompts):
        out = done[f"g{i}"]
        assert len(out) == n_new
        seq = list(p)
        for t in out:  # the oracle follows the engine's own path; every token on it is the oracle's best
            lg = O.forward(cfg_dict(cfg), sd, seq)[-1]
            if dtype == "float32":
                assert int(lg.argmax()) == t or float(lg.max() - lg[t]) < 1e-3, (i, len(seq))
            else:  # ... or, in bfloat16, within rounding of the best
                assert float(lg.max() - lg[t]) < 0.1 * float(lg.std()), (i, len(seq), float(lg.max() - lg[t]))
            seq.append(t)


def test_state_slots_follow_requests():
    """The KV manager hands the lowest free state slot to a request with its first pages and takes
    it back with them; a preempted request starts again from position 0 in whatever slot it gets."""
    from dynamo_exp_amd.engine.kv_manager import KVManager
    from dynamo_exp_amd.engine.request import Request

    kv = KVManager(8, 4, enable_prefix_caching=False, state_slots=2)
    a, b, c = (Request(n, [1] * 6, SamplingParams()) for n in "abc")
    assert kv.allocate_prompt(a) and kv.allocate_prompt(b)
    assert (a.state_slot, b.state_slot) == (0, 1)
    assert not kv.allocate_prompt(c) and c.state_slot is None and c.block_ids == []
    kv.free(a)
    assert a.state_slot is None and kv.ensure_slots(c, 3) and c.state_slot == 0
    kv.free(b)
    kv.free(c)
    assert kv.num_free_state() == 2 and kv.num_free() == 8
    with pytest.raises(ValueError):
        KVManager(8, 4, enable_prefix_caching=True, state_slots=2)
