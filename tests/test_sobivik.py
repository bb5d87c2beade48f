"""Sobivik in the engine against the plain oracle (tests/sobivik_oracle.py).

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

import sobivik_oracle as O
from dynamo_exp_amd.engine.engine import EngineConfig, LLMEngine
from dynamo_exp_amd.engine.request import SamplingParams
from dynamo_exp_amd.models.config import LayeredConfig, get_config
from dynamo_exp_amd.models.sobivik import SobivikForCausalLM
from dynamo_exp_amd.ops import mixers as mx
from dynamo_exp_amd.ops import recurrent as rc

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
CASES = [("cpu", "float32"), pytest.param("cuda", "float32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", marks=pytest.mark.gpu)]
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
F64 = torch.float64


# ----------------------------------------------------------------- configurations
def diff(H=4, G=2, d=12, dv=20, window=9, keep=3, lam=0.4):
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "scale": d ** -0.5, "diff": lam}
    if window:
        m["mask"] = {"size": window}
        if keep:
            m["mask"]["keep_first"] = keep
    return {"type": "attention", "mixer": m}


def ret(H=3, d=10, dv=14, decay=None):
    return {"type": "retention", "mixer": {"heads": H, "dim": d, "vdim": dv,
                                           "decay": decay or [1.0 - 2.0 ** -(2 + h) for h in range(H)]}}


def lat(H=3, d=12, dr=8, dv=10, r=24, qr=20, window=11, dims=None, scaling=True, base=100.0):
    m = {"heads": H, "dim": d, "rot_dim": dr, "vdim": dv, "kv_rank": r, "q_rank": qr, "scale": (d + dr) ** -0.5}
    if window:
        m["mask"] = {"size": window}
    dims = dr if dims is None else dims
    if dims:
        m["rot"] = {"base": base, "dims": dims}
        if scaling:
            m["rot"]["scaling"] = {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}
    return {"type": "latent_attention", "mixer": m}


def layer(mix, ff=40):
    return {**mix, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=72, vocab=97, taps=3, eps=1e-5, embed_scale=3.0, logit_scale=0.5):
    return LayeredConfig(name="t", architecture="Sobivik", vocab_size=vocab, hidden_size=width, layers=layers,
                         rms_norm_eps=eps, embedding_scale=embed_scale, logit_scale=logit_scale,
                         canon={"taps": taps} if taps else None)


def cfg_dict(cfg: LayeredConfig) -> dict:
    d = {"layers": cfg.layers, "norm": {"eps": cfg.rms_norm_eps}, "vocab": cfg.vocab_size, "width": cfg.hidden_size,
         "embedding": {"scale": cfg.embedding_scale}, "logit_scale": cfg.logit_scale}
    if cfg.canon:
        d["canon"] = cfg.canon
    return d


CONFIGS = {
    # the three mixers, windows / kept tokens / taps that differ, q/k width != value width, a layer
    # without feed-forward, partial rotation
    "mixed": lambda: config([layer(diff()), layer(ret()), layer(lat()), layer(diff(H=2, G=1, d=8, dv=6, window=5, keep=2), 0),
                             layer(ret(H=2, d=6, dv=22), 24), layer(lat(H=2, d=6, dr=12, dv=16, r=18, qr=10, window=7, dims=8))]),
    # values a model may happen to make equal or one: one head, a window of one token, one kept
    # token, one tap, no decay, scales of one, a rank of one query latent column more than a head
    "ones": lambda: config([layer(diff(H=1, G=1, d=8, dv=8, window=1, keep=1)), layer(ret(H=1, d=8, dv=8, decay=[1.0])),
                            layer(lat(H=1, d=8, dr=2, dv=8, r=8, qr=8, window=1, scaling=False)),
                            layer(diff(H=2, G=2, d=4, dv=4, window=64, keep=64))],
                           width=32, taps=1, embed_scale=1.0, logit_scale=1.0),
    # nothing divides by 4 or 8 (scalar paths), plain causal layers, no rotation, no input convolution
    "odd": lambda: config([layer(diff(H=6, G=2, d=7, dv=9, window=0, keep=0), 10), layer(ret(H=2, d=18, dv=5), 10),
                           layer(lat(H=2, d=5, dr=6, dv=7, r=9, qr=11, window=0, dims=0), 10),
                           layer(ret(H=1, d=34, dv=3), 0)], width=102, vocab=101, taps=0),
    # head widths the matrix-core kernels serve (bf16 on the GPU); retention heads of 64 and 128
    "tiles": lambda: config([layer(diff(H=2, G=1, d=64, dv=128, window=70, keep=5), 64), layer(ret(H=2, d=64, dv=64), 64),
                             layer(lat(H=4, d=32, dr=64, dv=32, r=192, qr=48, window=33, dims=64, base=1e4), 64),
                             layer(diff(H=4, G=2, d=32, dv=32, window=20, keep=20), 64),
                             layer(ret(H=1, d=128, dv=32), 0)], width=64, taps=4),
}


def weights(cfg, seed=0):
    return SobivikForCausalLM(cfg, "cpu", torch.float32).random_state(seed)


def engine(cfg, sd, device, dtype, blocks=48, bs=8, graphs=False, seqs=4):
    model = SobivikForCausalLM(cfg, device, DT[dtype]).load_state(sd)
    return LLMEngine(EngineConfig(model="t", device=device, dtype=dtype, block_size=bs, num_gpu_blocks=blocks,
                                  max_model_len=blocks * bs, max_num_seqs=seqs, enable_prefix_caching=False,
                                  use_cuda_graph=graphs, graph_sizes=(1, 2, 4), async_schedule=False),
                     model_cfg=cfg, model=model)


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def close(got, want, dtype, what=""):
    """Logit rows agree: error relative to the rows' spread, after the mean is taken off."""
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


def paged(T, bs, n_blocks, width, device, dtype, seed=3):
    """A shuffled block table for one sequence of T tokens, its slots, and an empty cache."""
    perm = torch.randperm(n_blocks, generator=torch.Generator().manual_seed(seed)).to(torch.int32)
    table = perm[: -(-T // bs)][None].contiguous().to(device)
    j = torch.arange(T, device=device)
    slots = table[0].long()[j // bs] * bs + j % bs
    return table, slots, torch.zeros(n_blocks * bs, width, device=device, dtype=dtype)


# ----------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("H,dk,dv", [(2, 16, 16), (3, 10, 14), (1, 64, 64), (2, 128, 40), (1, 34, 3), (1, 200, 70),
                                     (1, 1, 1), (2, 128, 64), (1, 32, 256), (2, 256, 32), (1, 16, 256)])
def test_retention_alone(device, dtype, H, dk, dv):
    """Two sequences scanned whole, then in steps of unequal portions (19, 2, 1, ...) in slots that hold
    garbage, then a decode step with a padding row, against the token-by-token oracle (over the
    bf16 values of the inputs where those are bf16; the scan itself is fp32 either way)."""
    torch.manual_seed(dk)
    T = 41
    dt = DT[dtype]
    q, k = torch.randn(2, T, H * dk).to(dt), torch.randn(2, T, H * dk).to(dt)
    v = torch.randn(2, T, H * dv).to(dt)
    decay = torch.tensor([1.0 - 2.0 ** -(1 + h) for h in range(H)])
    ks = dk ** -0.5
    want = [O.retention_scan(q[s].double().view(T, H, dk), k[s].double().view(T, H, dk) * ks,
                             v[s].double().view(T, H, dv), decay.double()) for s in range(2)]
    d = lambda t: t.to(device)  # noqa: E731
    state = torch.randn(5, H, dv, dk, device=device)  # garbage: position 0 must reset it
    for portions in ([(T,), (T,)], [(19, 2, 1, 1, 9, 8, 1), (3, 30, 7, 1)]):
        at, got = [0, 0], [[], []]
        it = [list(p) for p in portions]
        while any(it):
            live = [s for s in (0, 1) if it[s]]
            cuts = [(at[s], it[s].pop(0)) for s in live]
            pos, _, seq_rows, slots = step_meta(device, cuts, [3 if s == 0 else 1 for s in live])
            sel = lambda t: d(torch.cat([t[s, p:p + n] for s, (p, n) in zip(live, cuts)]))  # noqa: E731
            o = rc.retention(sel(q), sel(k), sel(v), d(decay), ks, state, pos, seq_rows, slots, H, dk, dv)
            for i, (s, (p, n)) in enumerate(zip(live, cuts)):
                b0 = int(seq_rows[i])
                got[s].append(o[b0:b0 + n].cpu())
                at[s] += n
        for s in range(2):
            assert torch.allclose(torch.cat(got[s]).double(), want[s][0].reshape(T, -1), atol=2e-4, rtol=1e-4)
            assert torch.allclose(state[3 if s == 0 else 1].cpu().double().transpose(1, 2), want[s][1], atol=2e-4,
                                  rtol=1e-4)
    pos = torch.tensor([T, T, 0], device=device)
    slots = torch.tensor([3, 1, -1], dtype=torch.int32, device=device)
    x = torch.randn(3, H * dk).to(dt)
    before = state[[0, 2, 4]].clone()
    o = rc.retention(d(x), d(x), d(torch.randn(3, H * dv).to(dt)), d(decay), ks, state, pos, None, slots, H, dk, dv)
    assert bool(torch.isfinite(o).all()) and float(o[2].abs().max()) == 0.0
    assert torch.equal(state[[0, 2, 4]], before)  # other slots are not touched


@pytest.mark.parametrize("device", DEVICES)
def test_retention_decays_and_keeps(device):
    """Crafted: one write, then reads through empty tokens: the read-out falls by the head's decay per
    token (a lost state reads 0, a decay applied at the wrong place is off by one factor)."""
    H, dk, dv, T = 2, 8, 8, 6
    decay = torch.tensor([0.5, 1.0])
    e0 = torch.zeros(dk)
    e0[0] = 2.0
    k = torch.zeros(T, H * dk)
    k[0] = e0.repeat(H)
    q = e0.repeat(H)[None].repeat(T, 1)
    v = torch.zeros(T, H * dv)
    v[0] = 3.0
    state = torch.full((2, H, dv, dk), 7.0, device=device)
    got = []
    for cuts in ([(0, 2)], [(2, 1)], [(3, 3)]):  # a portion, a single token, a portion: the state carries over
        pos, _, seq_rows, slots = step_meta(device, cuts, [1])
        p, n = cuts[0]
        got.append(rc.retention(q[p:p + n].to(device), k[p:p + n].to(device), v[p:p + n].to(device), decay.to(device),
                                1.0, state, pos, seq_rows, slots, H, dk, dv).cpu())
    o = torch.cat(got).view(T, H, dv)
    for t in range(T):
        assert abs(float(o[t, 0, 0]) - 12.0 * 0.5 ** t) < 1e-5 and abs(float(o[t, 1, 0]) - 12.0) < 1e-5


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("W,n", [(72, 1), (70, 3), (2052, 7), (8200, 4)])
def test_depth_mix_alone(device, W, n):
    """The weighted sum over planes, into a later plane of the same stack, with and without the
    norm; on chosen rows into a buffer of its own."""
    torch.manual_seed(W)
    T, eps = 6, 1e-5
    stack = torch.randn(n + 2, T, W)
    w, nw = torch.randn(n), torch.randn(W)
    want = O.depth_average([stack[j].double() for j in range(n)], w.double())
    sd = stack.to(device).clone()
    x, h = mx.depth_mix(sd, n, w.to(device), dst=sd[n], norm_w=nw.to(device), eps=eps, out_dtype=torch.float32)
    assert x.data_ptr() == sd[n].data_ptr()
    assert torch.allclose(sd[n].cpu().double(), want, atol=2e-5)
    assert torch.allclose(h.cpu().double(), O.unit_rms(want, eps) * nw.double(), atol=5e-5)
    assert torch.equal(sd[:n].cpu(), stack[:n]) and torch.equal(sd[n + 1].cpu(), stack[n + 1])
    rows = torch.tensor([4, 0, 4], device=device)
    x, h = mx.depth_mix(sd, n, w.to(device), rows=rows)
    assert h is None and torch.allclose(x.cpu().double(), want[rows.cpu()], atol=2e-5)
    # with the addend that closes the newest plane's layer: the plane is updated in the same pass
    # (all rows), or left alone while the sum uses the addend (chosen rows, one listed twice)
    c, cw = torch.randn(T, W + 4) * 3, torch.randn(W)
    last = stack[n - 1].double() + O.unit_rms(c[:, 4:].double(), eps) * cw.double()
    want = O.depth_average([stack[j].double() for j in range(n - 1)] + [last], w.double())
    x, _ = mx.depth_mix(sd, n, w.to(device), rows=rows, eps=eps, out_dtype=torch.float32, c=c.to(device)[:, 4:],
                        c_w=cw.to(device))
    assert torch.allclose(x.cpu().double(), want[rows.cpu()], atol=3e-5) and torch.equal(sd[n - 1].cpu(), stack[n - 1])
    x, h = mx.depth_mix(sd, n, w.to(device), dst=sd[n], norm_w=nw.to(device), eps=eps, out_dtype=torch.float32,
                        c=c.to(device)[:, 4:], c_w=cw.to(device))
    assert torch.allclose(sd[n - 1].cpu().double(), last, atol=2e-5) and torch.allclose(x.cpu().double(), want, atol=3e-5)
    assert torch.allclose(h.cpu().double(), O.unit_rms(want, eps) * nw.double(), atol=5e-5)


@pytest.mark.parametrize("device", DEVICES)
def test_small_ops(device):
    """Embedding scale, the norm of a column section, the silu gate after the per-head unit norm, the
    per-head sigmoid gate after the two-map combine."""
    torch.manual_seed(4)
    d = lambda t: t.to(device)  # noqa: E731
    table, ids = torch.randn(11, 36), torch.tensor([3, 10, 0])
    out = torch.zeros(3, 36, device=device)
    X = mx.embed_streams(d(ids), d(table), 1, scale=2.5, out=out)
    assert X.data_ptr() == out.data_ptr() and torch.allclose(out.cpu(), table[ids] * 2.5, atol=1e-6)
    x, w = torch.randn(5, 50) * 3, torch.randn(21)
    got = mx.section_norm(d(x)[:, 7:28], d(w), 1e-5)
    assert torch.allclose(got.cpu().double(), O.unit_rms(x[:, 7:28].double(), 1e-5) * w.double(), atol=2e-5)
    T, H, dv = 5, 3, 22
    o, g = torch.randn(T, H * dv) * 3, torch.randn(T, H * dv + 3)
    want = O.unit_rms(o.double().view(T, H, dv), 1e-5).reshape(T, -1) * O.silu(g[:, 3:].double())
    got = rc.head_norm_gate(d(o), H, None, d(g)[:, 3:], 1e-5, torch.float32, gate_act="silu")
    assert torch.allclose(got.cpu().double(), want, atol=2e-5)
    a, hg = torch.randn(T, H, 2, dv), torch.randn(T, H + 2)
    want = O.unit_rms(a[:, :, 0].double() - 0.7 * a[:, :, 1].double(), 1e-5) * 0.6 * O.sigmoid(hg[:, 2:].double())[:, :, None]
    got = mx.diff_combine(d(a), 0.7, 0.6, 1e-5, torch.float32, head_gate=d(hg)[:, 2:])
    assert torch.allclose(got.cpu().double(), want.reshape(T, -1), atol=2e-5)


def test_scaled_frequencies():
    """The blended frequencies and the factor on cosines and sines, against the oracle; the blend is
    really partial for the sizes used (some dimensions keep their frequency, some are divided)."""
    for dims, base, sc in ((8, 100.0, {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}),
                           (64, 1e4, {"factor": 8.0, "original": 512, "fast": 32.0, "slow": 1.0}), (6, 50.0, None)):
        rot = {"dims": dims, "base": base}
        if sc:
            rot["scaling"] = sc
        f, mag = rc.yarn_frequencies(dims, base, sc)
        fo, mo = O.scaled_frequencies(rot)
        assert torch.allclose(f.double(), fo, rtol=1e-6) and abs(mag - mo) < 1e-12
        plain = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
        if sc:
            ratio = fo / plain
            assert float(ratio.max()) > 0.999 and float(ratio.min()) < 1.001 / sc["factor"] and mo > 1.0


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("H,d,dr,r,dims,scaling", [(3, 12, 8, 24, 8, True), (2, 5, 6, 9, 4, False), (1, 8, 2, 8, 2, True),
                                                   (4, 32, 64, 192, 64, True), (2, 16, 16, 40, 0, False)])
def test_latent_rope_alone(device, H, d, dr, r, dims, scaling):
    """Latent norm, rotated key part and cache row, assembled query rows, for rows at scattered
    positions, one of them not cached."""
    torch.manual_seed(r)
    T, eps = 9, 1e-5
    rot = {"base": 100.0, "dims": dims}
    if scaling:
        rot["scaling"] = {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}
    inv, mag = rc.yarn_frequencies(dims, 100.0, rot.get("scaling")) if dims else (None, 1.0)
    pos = torch.tensor([0, 1, 2, 17, 18, 400, 3, 3, 1000])
    slots = torch.tensor([5, 4, 30, 2, 1, 0, -1, 9, 8])
    qa, q = torch.randn(H, T, r), torch.randn(T, H * (d + dr) + 3)
    kv, cn = torch.randn(T, r + dr + 5), torch.randn(r)
    want_c = O.unit_rms(kv[:, :r].double(), eps) * cn.double()
    want_k = O.rotate(kv[:, r:r + dr].double(), pos, rot) if dims else kv[:, r:r + dr].double()
    qr = q[:, :H * (d + dr)].double().view(T, H, d + dr)[:, :, d:]
    want_q = torch.cat([qa.double().transpose(0, 1), O.rotate(qr, pos, rot) if dims else qr], -1).reshape(T, -1)
    dv_ = lambda t: None if t is None else t.to(device)  # noqa: E731
    cache = torch.full((32, r + dr), 9.0, device=device)
    got = rc.latent_rope(dv_(qa), dv_(q), d + dr, d, dv_(kv)[:, :r + dr], r, dr, dv_(cn), eps, dv_(inv), mag, dv_(pos),
                         dv_(slots), cache)
    tol = 3e-5 * max(1.0, float(pos.max()) / 100)
    assert torch.allclose(got.cpu().double(), want_q, atol=tol)
    ok = slots >= 0
    assert torch.allclose(cache[slots[ok]].cpu().double(), torch.cat([want_c, want_k], -1)[ok], atol=tol)
    untouched = torch.ones(32, dtype=torch.bool)
    untouched[slots[ok]] = False
    assert bool((cache.cpu()[untouched] == 9.0).all())


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("taps,W", [(3, 72), (4, 64), (1, 32), (2, 102)])
def test_input_convolution_alone(device, taps, W):
    """h + conv(h) as one convolution whose last tap has weight 1 + w: two sequences in portions
    down to one row (shorter than the taps), slots reused with garbage in them."""
    torch.manual_seed(taps)
    T = 23
    x, w = torch.randn(2, T, W), torch.randn(W, taps)
    want = [O.time_conv(x[s].double(), w.double()) for s in range(2)]
    cw = w.t().contiguous().clone()
    cw[-1] += 1.0
    tail = torch.randn(4, taps - 1, W, device=device)
    it = [[1, 1, 2, 9, 1, 9], [23]]
    at, got = [0, 0], [[], []]
    while any(it):
        live = [s for s in (0, 1) if it[s]]
        cuts = [(at[s], it[s].pop(0)) for s in live]
        pos, row_seq, seq_rows, slots = step_meta(device, cuts, [2 if s == 0 else 0 for s in live])
        xs = torch.cat([x[s, p:p + n] for s, (p, n) in zip(live, cuts)]).to(device)
        y = rc.conv_rope_cache(xs, cw.to(device), tail, pos, torch.zeros_like(pos), row_seq, seq_rows, slots, 1, 0, W, 0,
                               None, None, None)
        rc.conv_state_update(xs, tail, pos, seq_rows, slots)
        for i, (s, (p, n)) in enumerate(zip(live, cuts)):
            got[s].append(y[int(seq_rows[i]):int(seq_rows[i]) + n].cpu())
            at[s] += n
    for s in range(2):
        assert torch.allclose(torch.cat(got[s]).double(), want[s], atol=2e-5)


def dense_attention(q, k, v, scale, size, keep, sink, maps=1):
    """[T, n_qh, dv]: query vector qh = head * maps + m reads key head (head // group) * maps + m."""
    T, n_qh, _ = q.shape
    n_kh, G = k.shape[1], v.shape[1]
    group = n_qh // maps // G
    pos = torch.arange(T)
    dist = pos[:, None] - pos[None, :]
    vis = dist >= 0
    if size:
        near = dist < size
        if keep:
            near = near | (pos[None, :] < keep)
        vis = vis & near
    out = torch.zeros(T, n_qh, v.shape[-1], dtype=F64)
    for qh in range(n_qh):
        head, m = qh // maps, qh % maps
        g = head // group
        sc = (q[:, qh].double() @ k[:, g * maps + m].double().T) * scale
        sc = sc.masked_fill(~vis, float("-inf"))
        if sink is not None:
            sc = torch.cat([sc, sink[qh].double().expand(T, 1)], -1)
        out[:, qh] = torch.softmax(sc, -1)[:, :T] @ v[:, g].double()
    assert n_kh == G * maps
    return out


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("size,keep", [(0, 0), (9, 0), (9, 3), (1, 1), (40, 70), (5, 12)])
@pytest.mark.parametrize("dims", [(4, 2, 12, 20, 2), (3, 1, 7, 5, 1), (6, 1, 32, 24, 1)])
def test_row_attention_keep_and_sink(device, size, keep, dims):
    """Kept first keys beside the window, and the sink in the denominator: all rows of a sequence,
    then decode rows with their keys split into parts, against the dense oracle."""
    n_qh, G, d, dv, maps = dims
    torch.manual_seed(size + keep)
    T, bs = 70, 8
    q, k, v = torch.randn(T, n_qh, d), torch.randn(T, G * maps, d), torch.randn(T, G, dv)
    sink = torch.randn(n_qh)
    table, slots, kc = paged(T, bs, 12, G * maps * d, device, torch.float32)
    vc = torch.zeros(12 * bs, G * dv, device=device)
    kc[slots] = k.reshape(T, -1).to(device)
    vc[slots] = v.reshape(T, -1).to(device)
    pos = torch.arange(T, device=device)
    seq = torch.zeros(T, dtype=torch.int32, device=device)
    mask = "window" if size else "causal"
    group = n_qh // maps // G
    for sk in (None, sink):
        want = dense_attention(q, k, v, 0.4, size, keep if size else 0, sk, maps)
        kw = dict(keep_first=keep if size else 0, sink=None if sk is None else sk.to(device))
        got = mx.row_attention(q.reshape(T, -1).to(device), kc, vc, pos, seq, table, bs, n_qh, maps, group, d, dv, 0.4,
                               mask, size, 1, **kw)
        assert torch.allclose(got.cpu().double(), want, atol=5e-5)
        rows = torch.tensor([0, 1, 7, 8, 33, 69], device=device)
        got = mx.row_attention(q.reshape(T, -1).to(device)[rows], kc, vc, pos[rows], None,
                               table.expand(len(rows), -1).contiguous(), bs, n_qh, maps, group, d, dv, 0.4, mask, size,
                               3, **kw)
        assert torch.allclose(got.cpu().double(), want[rows.cpu()], atol=5e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("size,keep", [(0, 0), (1, 1), (40, 7), (129, 70), (64, 64), (20, 200)])
@pytest.mark.parametrize("dims", [(4, 2, 32, 32, 1), (4, 1, 32, 64, 2), (4, 1, 64, 128, 2), (3, 1, 256, 192, 1),
                                  (20, 1, 256, 192, 1), (2, 2, 128, 128, 1)])
def test_matrix_core_attention_keep_and_sink(size, keep, dims):
    """The matrix-core kernels with kept first keys and a sink: a 263-row portion that starts at
    position 37 of a cached prefix (three tiles, the last ragged, cut inside pages, windows and the
    kept keys) beside two decode rows of another sequence, then decode rows alone with their keys in
    parts, against the dense oracle over the bf16 values.  K and V may be one tensor (latent rows)."""
    n_qh, G, d, dv, maps = dims
    T, bs, start = 300, 16, 37
    torch.manual_seed(5)
    shared = G == 1 and maps == 1 and d > dv  # one [latent | key part] row is key and value
    q = (torch.randn(T, n_qh, d) * (0.5 if d > 100 else 1.0)).bfloat16()
    k = (torch.randn(T, G * maps, d) * 0.7).bfloat16()
    v = k[:, :, :dv].contiguous() if shared else torch.randn(T, G, dv).bfloat16()
    sink = torch.randn(n_qh) + 1
    perm = torch.randperm(40, generator=torch.Generator().manual_seed(3)).to(torch.int32)
    table = torch.stack([perm[:19], perm[19:38]]).contiguous().cuda()
    j = torch.arange(T, device="cuda")
    kc = torch.zeros(40 * bs, G * maps * d, device="cuda", dtype=torch.bfloat16)
    vc = kc if shared else torch.zeros(40 * bs, G * dv, device="cuda", dtype=torch.bfloat16)
    for i in (0, 1):
        sl = table[i].long()[j // bs] * bs + j % bs
        kc[sl] = k.reshape(T, -1).cuda()
        if not shared:
            vc[sl] = v.reshape(T, -1).cuda()
    rows = list(range(start, T)) + [5, 290]
    n_pre = T - start
    pos = torch.tensor(rows, device="cuda")
    seq = torch.tensor([0] * n_pre + [1, 1], dtype=torch.int32, device="cuda")
    tiles = torch.tensor(mx.tile_list(0, n_pre), dtype=torch.int32, device="cuda")
    qd = q.reshape(T, -1).cuda()[pos]
    mask = "window" if size else "causal"
    group = n_qh // maps // G
    assert mx.tile_attention_ok(qd, d, dv)
    for sk in (None, sink):
        want = dense_attention(q, k, v, 0.2, size, keep if size else 0, sk, maps)
        kw = dict(keep_first=keep if size else 0, sink=None if sk is None else sk.cuda())
        scale_ = max(1.0, float(want.abs().max()))
        got = mx.attention(qd, kc, vc, pos, seq, table, bs, n_qh, maps, group, d, dv, 0.2, mask, size, 1, True, tiles,
                           n_pre, **kw)
        assert float((got.cpu().double() - want[rows]).abs().max()) < 1e-3 * scale_
        got = mx.attention(qd, kc, vc, pos, seq, table, bs, n_qh, maps, group, d, dv, 0.2, mask, size, 3, False, tiles,
                           n_pre, **kw)
        assert float((got.cpu().double() - want[rows]).abs().max()) < 2e-2 * scale_
        dr = torch.tensor([0, 1, 63, 64, 65, 255, 299], device="cuda")
        got = mx.attention(q.reshape(T, -1).cuda()[dr], kc, vc, dr, None, table[:1].expand(len(dr), -1).contiguous(),
                           bs, n_qh, maps, group, d, dv, 0.2, mask, size, 2, True, **kw)
        assert float((got.cpu().double() - want[dr.cpu()]).abs().max()) < 1e-3 * scale_


# ----------------------------------------------------------------- crafted: one key stands out
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("size,keep,bs", [(44, 5, 16), (17, 0, 8), (1, 1, 8), (200, 3, 8), (30, 70, 16)])
def test_far_keys_window_edges_sink(device, dtype, size, keep, bs):
    """A cache of empty keys in which one key matches the query strongly and carries a marked value:
    seen just inside the window, not just outside, seen again as one of the kept first keys and not
    as the next one, at page borders, among hundreds, for prompt rows and decode rows alike.  With
    a sink the empty keys (score 0 each) and exp(sink), counted once, share the rest."""
    H, G, d, dv, T = 2, 1, 32, 32, 180
    dt = DT[dtype]
    tol = 1e-4 if dtype == "float32" else 2e-2
    e0 = torch.zeros(d)
    e0[0] = 8.0
    table, slots, kc = paged(T, bs, 40, G * d, device, dt)
    vc = torch.zeros(40 * bs, G * dv, device=device, dtype=dt)
    sink = torch.tensor([math.log(50.0), math.log(7.0)])
    s_hit = 64.0 * 0.25
    for p in (T - 1, 150, bs * 9, bs * 9 + 1, 11):
        for mark in (p, p - size + 1, p - size, p - 1, 0, keep - 1, keep, bs * 3 - 1, bs * 3):
            if not 0 <= mark <= p:
                continue
            K = torch.zeros(T, d)
            K[mark] = e0
            V = torch.full((T, dv), -1.0)
            V[mark] = 1.0
            kc[slots] = K.to(device, dt)
            vc[slots] = V.to(device, dt)
            q = e0.repeat(H)[None].to(device, dt)
            seen = p - mark < size or mark < keep
            n_vis = min(p + 1, size) + min(keep, max(0, p - size + 1))  # visible keys
            pos = torch.tensor([p], device=device)
            for sk in (None, sink):
                for seq in (torch.zeros(1, dtype=torch.int32, device=device), None):  # a prompt row, a decode row
                    tl = (torch.tensor([[0, 1]], dtype=torch.int32, device=device), 1) if seq is not None else (None, 0)
                    got = mx.attention(q, kc, vc, pos, seq, table, bs, H, 1, H // G, d, dv, 0.25, "window", size, 1,
                                       False, *tl, keep_first=keep, sink=None if sk is None else sk.to(device))
                    for h in range(H):
                        extra = float(sk[h].exp()) if sk is not None else 0.0
                        hit = math.exp(s_hit) if seen else 0.0
                        rest = n_vis - (1 if seen else 0)
                        want = (hit - rest) / (hit + rest + extra)
                        assert abs(float(got[0, h, 0]) - want) < tol, (p, mark, h, sk is None, seq is None,
                                                                       float(got[0, h, 0]), want)


# ----------------------------------------------------------------- whole model
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_and_layers(device, dtype, name):
    """A whole prompt in one step: logits at every position, and (float32) what goes on after every
    layer, against the oracle."""
    cfg = CONFIGS[name]()
    sd = weights(cfg, 1)
    toks = tokens(75, cfg.vocab_size, 2)
    want, after = O.forward(cfg_dict(cfg), sd, toks)
    eng = engine(cfg, sd, device, dtype)
    if dtype == "float32":
        eng.model.trace_layers = []
    got = eng.forced_step([("a", toks, list(range(len(toks))))], ["a"])["a"]
    close(got, want, dtype, name)
    if dtype == "float32":
        assert len(eng.model.trace_layers) == len(cfg.layers)
        for i, (x, w) in enumerate(zip(eng.model.trace_layers, after)):
            assert float((x.cpu().double() - w).abs().max()) < 2e-3 * float(w.abs().max()), f"layer {i}"


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name,cuts", [("mixed", (0,)), ("mixed", (31, 2, 2, 17, 3)), ("ones", (2, 2, 2, 40)),
                                       ("odd", (50, 2)), ("tiles", (7, 64, 2)), ("tiles", (0,))])
def test_portions_and_decode(device, dtype, name, cuts):
    """Token-by-token decoding from the first token, and portions of several sizes down to two
    tokens followed by single tokens, against the whole-sequence oracle."""
    cfg = CONFIGS[name]()
    sd = weights(cfg, 4)
    toks = tokens(80, cfg.vocab_size, 5)
    want, _ = O.forward(cfg_dict(cfg), sd, toks)
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
    want = {k: O.forward(cfg_dict(cfg), sd, t)[0] for k, t in reqs.items()}
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
    """146 consecutive decode steps after a two-token prompt: windows, kept tokens, taps and pages
    pass over decoded tokens; the first positions (fewer tokens than taps, than a window, than the
    kept ones) are among them."""
    cfg = CONFIGS["mixed"]()
    sd = weights(cfg, 6)
    toks = tokens(148, cfg.vocab_size, 7)
    want, _ = O.forward(cfg_dict(cfg), sd, toks)
    eng = engine(cfg, sd, device, dtype)
    got = run_cut(eng, "a", toks, (2,))
    close(got, want, dtype, "long decode")


@pytest.mark.parametrize("device,dtype", CASES)
def test_crafted_weights_show_faults(device, dtype):
    """Weights made so that faults move the logits: large sinks and depth weights spread over all
    planes; the engine agrees with the oracle, and the oracle's own variants -- a window one token
    off, one kept token fewer, no sink, no depth average, a decay slightly off -- differ visibly."""
    cfg = config([layer(diff(H=2, G=1, d=16, dv=16, window=6, keep=4)), layer(ret(H=2, d=16, dv=16, decay=[0.9, 0.99])),
                  layer(lat(H=2, d=16, dr=8, dv=16, r=16, qr=16, window=6))], width=48, vocab=61)
    sd = weights(cfg, 8)
    sd["l2.mix.sink"] = torch.tensor([2.0, 3.0]).bfloat16()
    for i in range(3):
        sd[f"l{i}.dwa"] = (torch.ones(i + 2) / (i + 2) + torch.arange(i + 2) * 0.1).bfloat16()
    toks = tokens(60, cfg.vocab_size, 9)
    want, _ = O.forward(cfg_dict(cfg), sd, toks)
    eng = engine(cfg, sd, device, dtype)
    close(run_cut(eng, "a", toks, (13, 2, 30)), want, dtype, "crafted")

    def variant(change):
        c = cfg_dict(cfg)
        c["layers"] = [dict(L, mixer=dict(L["mixer"], mask=dict(L["mixer"].get("mask") or {}))) for L in c["layers"]]
        s2 = dict(sd)
        change(c, s2)
        return O.forward(c, s2, toks)[0]

    def differs(off):
        return float((off - want).abs().max()) > 0.02 * float(want.abs().max())

    assert differs(variant(lambda c, s: c["layers"][0]["mixer"]["mask"].update(size=7)))
    assert differs(variant(lambda c, s: c["layers"][0]["mixer"]["mask"].update(keep_first=3)))
    assert differs(variant(lambda c, s: c["layers"][2]["mixer"]["mask"].update(size=5)))
    assert differs(variant(lambda c, s: s.pop("l2.mix.sink")))
    assert differs(variant(lambda c, s: s.pop("l1.dwa")))
    assert differs(variant(lambda c, s: c["layers"][1]["mixer"].update(decay=[0.8, 0.99])))


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
    model = SobivikForCausalLM(cfg, device, DT[dtype]).load_state(sd)
    eng = LLMEngine(EngineConfig(model="t", device=device, dtype=dtype, block_size=8, num_gpu_blocks=64,
                                 max_model_len=256, max_num_seqs=2, max_num_batched_tokens=24,
                                 use_cuda_graph=graphs, graph_sizes=(1, 2), async_schedule=False),
                    model_cfg=cfg, model=model)
    assert eng.cfg.enable_prefix_caching is False  # per-sequence state cannot be served from the prefix cache
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
            lg = O.forward(cfg_dict(cfg), sd, seq)[0][-1]
            if dtype == "float32":
                assert int(lg.argmax()) == t or float(lg.max() - lg[t]) < 1e-3, (i, len(seq))
            else:  # ... or, in bfloat16, within rounding of the best
                assert float(lg.max() - lg[t]) < 0.1 * float(lg.std()), (i, len(seq), float(lg.max() - lg[t]))
            seq.append(t)


@pytest.mark.parametrize("device,dtype", CASES)
def test_trace_replay_command(tmp_path, monkeypatch, capsys, device, dtype):
    """The replay command on a checkpoint directory: the class follows config.json, a portion beside
    a shorter one, a decode token beside a portion, a step in which nothing is wanted, a slot and
    pages used again; logits files against the oracle."""
    import io
    import json
    import sys

    import numpy as np
    from safetensors.torch import save_file

    from dynamo_exp_amd.cli import trace_run

    cfg = CONFIGS["mixed"]()
    sd = weights(cfg, 21)
    model_dir, out = tmp_path / "m", tmp_path / "out"
    cfg.write_hf_config(str(model_dir))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(model_dir / "model.safetensors"))
    a, b = tokens(40, cfg.vocab_size, 31), tokens(9, cfg.vocab_size, 32)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:25], "want": [0, 24]},
                                     {"id": "b", "tokens": b[:2], "want": [1]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[25:26], "want": [0]},
                                     {"id": "b", "tokens": b[2:], "want": [0, 6]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[26:], "want": []}], "end": ["a"]},
             {"step": 3, "entries": [{"id": "c", "tokens": b, "want": [8]}], "end": ["c"]}]
    monkeypatch.setattr(sys, "stdin", io.StringIO("\n".join(json.dumps(st) for st in steps) + "\n"))
    rc_ = trace_run.main(["--model", str(model_dir), "--dtype", dtype, "--out", str(out), "--max-tokens", "128",
                          "--device", device])
    assert rc_ == 0
    assert [ln for ln in capsys.readouterr().out.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    assert not (out / "2.f32").exists()
    wa, wb = O.forward(cfg_dict(cfg), sd, a)[0], O.forward(cfg_dict(cfg), sd, b)[0]
    got = {i: torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, cfg.vocab_size)) for i in (0, 1, 3)}
    close(got[0], torch.cat([wa[[0, 24]], wb[[1]]]), dtype, "step 0")
    close(got[1], torch.cat([wa[[25]], wb[[2, 8]]]), dtype, "step 1")
    close(got[3], wb[[8]], dtype, "step 3")


def test_config_round_trip(tmp_path):
    """config.json keys -> LayeredConfig -> config.json; the preset builds and counts its weights."""
    cfg = CONFIGS["mixed"]()
    cfg.write_hf_config(str(tmp_path))
    back = get_config(str(tmp_path))
    assert back.architecture == "Sobivik" and back.layers == cfg.layers and back.canon == cfg.canon
    assert back.embedding_scale == cfg.embedding_scale and back.logit_scale == cfg.logit_scale
    tiny = get_config("sobivik-tiny")
    sd = SobivikForCausalLM(tiny, "cpu", torch.float32).random_state(0)
    assert sum(v.numel() for v in sd.values()) == tiny.num_params()
    from dynamo_exp_amd.models.registry import build_model, supports_dtype

    assert supports_dtype("Sobivik", "float32") and supports_dtype("Sobivik", "bfloat16")
    assert isinstance(build_model(back, "cpu", dtype="float32"), SobivikForCausalLM)
    with pytest.raises(ValueError):
        SobivikForCausalLM(config([{"type": "general_delta", "mixer": {"heads": 1, "dim": 8}, "mlp": None}]), "cpu",
                           torch.float32)
