"""`bench.py --layered`: the layer-listed models (Bekulix, Bolinex, Nefivik, Sobivik)
beside the closest existing model (Llama; for Nefivik also Bolinex, for Sobivik
also Bekulix, the closest layer-listed ones) at equal layer sizes, random weights.
`--layered-family` picks which family runs (default: Bekulix and Bolinex).

Two parts, both on one GPU:
  * engine throughput through the engine's own entry point (add_request +
    step: scheduler, paged caches, HIP graphs for decode, greedy sampling):
    one prefill step of `prefill_seqs` x `isl` tokens, then decode of
    `decode_seqs` streams at context `isl` for `osl` tokens;
  * the attention kernels alone at the layer's head shape: matrix-core
    prefill kernels in TFLOP/s (causal FLOPs 4 d L^2 / 2 per head), decode
    kernels in TB/s of cache bytes read -- each kernel's distance from its
    roofline, Bekulix's next to Llama's.
"""
from __future__ import annotations

import math
import sys
import time

import torch

from .. import ops
from ..engine.engine import EngineConfig, LLMEngine
from ..engine.request import SamplingParams
from ..models.config import ModelConfig, _bekulix_preset, _bolinex_preset, _nefivik_preset, _sobivik_preset
from ..ops import mixers as mx
from ..ops import moe
from ..ops import recurrent as rc

# layer sizes of real models (width, ff, heads, kv heads, head dim), a few layers each
SIZES = {
    "1b-shapes": dict(W=2048, ff=8192, H=16, G=4, d=128, layers=8, vocab=32000),
    "8b-shapes": dict(W=4096, ff=14336, H=32, G=8, d=128, layers=8, vocab=128256),
}


def _configs(s: dict):
    bek = _bekulix_preset(f"bekulix {s['W']}", s["W"], s["ff"], s["layers"], s["H"], s["G"], s["d"], 256, 1024, 2048,
                          vocab=s["vocab"])
    lla = ModelConfig(name=f"llama {s['W']}", vocab_size=s["vocab"], hidden_size=s["W"], intermediate_size=s["ff"],
                      num_hidden_layers=s["layers"], num_attention_heads=s["H"], num_key_value_heads=s["G"],
                      head_dim=s["d"], max_position_embeddings=8192, bos_token_id=1, eos_token_id=[2])
    return bek, lla


def _bolinex_config(s: dict):
    """Bolinex at the size's layer shapes: window 1024, every second feed-forward 8 experts of a
    quarter of the dense width (two chosen, in two of four groups) plus a shared one."""
    return _bolinex_preset(f"bolinex {s['W']}", s["W"], s["ff"], s["layers"], s["H"], s["G"], s["d"], 1024, experts=8,
                           top=2, expert_ff=s["ff"] // 4, shared_ff=s["ff"] // 4, groups=(4, 2), side=256,
                           vocab=s["vocab"])


def _nefivik_config(s: dict):
    """Nefivik at the size's layer shapes: three generalized-delta-rule layers, then a windowed
    (1024) sigmoid-attention layer with 4-tap convolutions, twice; the second attention layer
    reads the first one's keys and values; every feed-forward routes 2 of 8 experts of a quarter
    of the dense width (two of four groups kept); token input of 256 columns."""
    return _nefivik_preset(f"nefivik {s['W']}", s["W"], s["layers"], s["H"], s["G"], s["d"], 1024, experts=8, top=2,
                           expert_ff=s["ff"] // 4, groups=(4, 2), side=256, vocab=s["vocab"], conv=4, attn_every=4)


def _sobivik_config(s: dict):
    """Sobivik at the size's layer shapes: differential attention (window 1024 that keeps the
    first 64 tokens; half the heads at twice the value width), retention and latent attention
    (rank 192 + 64 rotated columns, window 1024, sink) in turn, 4-tap input convolutions, dense
    feed-forwards, the depth average after every layer."""
    return _sobivik_preset(f"sobivik {s['W']}", s["W"], s["ff"], s["layers"], s["H"], s["G"], s["d"], 192,
                           s["W"] // 4, 64, 1024, 64, vocab=s["vocab"])


def _timed(fn, iters=10, warm=2) -> float:
    for _ in range(warm):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        fn()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) / iters * 1e3  # us


def engine_throughput(mcfg, dev, isl: int, osl: int, prefill_seqs: int, decode_seqs: int, seed: int = 0) -> dict:
    """Prefill and decode tokens/s of one model through LLMEngine."""
    out = {}
    g = torch.Generator().manual_seed(seed)
    for phase, B in (("prefill", prefill_seqs), ("decode", decode_seqs)):
        print(f"[layered] {mcfg.name}: {phase}", file=sys.stderr, flush=True)
        eng = LLMEngine(EngineConfig(model=mcfg.name, device=str(dev), block_size=64, max_model_len=isl + osl + 64,
                                     max_num_seqs=B, max_num_batched_tokens=max(8192, prefill_seqs * isl),
                                     chunked_prefill=False, max_prefill_streak=1 << 30, enable_prefix_caching=False,
                                     num_gpu_blocks=B * (-(-(isl + osl + 64) // 64)) + 8, graph_sizes=(B,),
                                     async_schedule=False, seed=seed), model_cfg=mcfg)
        eng.warmup()
        best = None
        for rep in range(3):  # first repetition warms the GEMM library at these sizes
            first = {}
            for i in range(B):
                p = torch.randint(3, mcfg.vocab_size, (isl,), generator=g).tolist()
                eng.add_request(f"{phase}{rep}_{i}", p, SamplingParams(max_tokens=osl if phase == "decode" else 1,
                                                                        ignore_eos=True),
                                on_output=lambda r, t, lp, fin: first.setdefault(r.request_id, True))
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            while len(first) < B:
                eng.step()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            while eng.has_unfinished():
                eng.step()
            torch.cuda.synchronize()
            t2 = time.perf_counter()
            v = B * isl / (t1 - t0) if phase == "prefill" else B * (osl - 1) / (t2 - t1)
            if rep:
                best = max(best or 0.0, v)
        out[f"{phase}_tok_s"] = round(best, 1)
        del eng
        torch.cuda.empty_cache()
    return out


def attention_kernels(s: dict, L: int, B: int) -> dict:
    """The attention kernels alone at head shape (H, G, d): one prompt of L
    tokens (prefill) and B streams at context L (decode)."""
    H, G, d, bs = s["H"], s["G"], s["d"], 64
    dev, dt = "cuda", torch.bfloat16
    res = {}
    flops = 4 * d * H * L * (L + 1) / 2
    nb = L // bs + 1
    # ---- prefill
    q = torch.randn(L, H * d, device=dev, dtype=dt)
    pos = torch.arange(L, device=dev)
    seq = torch.zeros(L, dtype=torch.int32, device=dev)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(1, nb)
    kc = torch.randn(nb * bs, G * d, device=dev, dtype=dt)
    vc = torch.randn_like(kc)
    tiles = torch.tensor(mx.tile_list(0, L), dtype=torch.int32, device=dev)
    us = _timed(lambda: mx.attention(q, kc, vc, pos, seq, bt, bs, H, 1, H // G, d, d, d ** -0.5, "causal", 0, 1, False,
                                     tiles, L))
    res["bekulix_prefill_causal"] = {"us": round(us, 1), "TFLOPs": round(flops / us / 1e6, 1)}
    for mask, size in (("window", 1024), ("chunk", 2048)):
        j = torch.arange(L)
        lo = mx.first_visible(j, mask, size)
        fl = 4 * d * H * float((j - lo + 1).sum())
        us = _timed(lambda: mx.attention(q, kc, vc, pos, seq, bt, bs, H, 1, H // G, d, d, d ** -0.5, mask, size, 1,
                                         False, tiles, L))
        res[f"bekulix_prefill_{mask}{size}"] = {"us": round(us, 1), "TFLOPs": round(fl / us / 1e6, 1)}
    kl = torch.randn(nb, G, bs, d, device=dev, dtype=dt)
    vl = torch.randn_like(kl)
    ql = q.view(L, H, d)
    cu = torch.tensor([0, L], dtype=torch.int32, device=dev)
    ctx = torch.tensor([L], dtype=torch.int32, device=dev)
    work = torch.tensor(ops.prefill_work_list([L], [L], H, G), dtype=torch.int32, device=dev)
    out = torch.empty_like(ql)
    us = _timed(lambda: ops.prefill_attention(ql, kl, vl, bt, cu, ctx, d ** -0.5, out, work=work))
    res["llama_prefill_causal"] = {"us": round(us, 1), "TFLOPs": round(flops / us / 1e6, 1)}
    # ---- decode
    nbb = B * nb
    byts = B * L * G * d * 2 * 2
    bt = torch.randperm(nbb, device=dev).to(torch.int32).view(B, nb)
    kc = torch.randn(nbb * bs, G * d, device=dev, dtype=dt)
    vc = torch.randn_like(kc)
    q = torch.randn(B, H * d, device=dev, dtype=dt)
    pos = torch.full((B,), L - 1, device=dev)
    parts = mx.row_attention_parts(B, G, L, mx.GROUP_TARGET_WAVES)
    us = _timed(lambda: mx.attention(q, kc, vc, pos, None, bt, bs, H, 1, H // G, d, d, d ** -0.5, "causal", 0, parts))
    res["bekulix_decode"] = {"us": round(us, 1), "TB/s": round(byts / us / 1e6, 2), "parts": parts}
    kl = torch.randn(nbb, G, bs, d, device=dev, dtype=dt)
    vl = torch.randn_like(kl)
    ql = q.view(B, H, d)
    ctx = torch.full((B,), L, dtype=torch.int32, device=dev)
    out = torch.empty_like(ql)
    mp = ops.decode_num_parts(B, G, L)
    ws = ops.decode_workspace(B, H, d, mp, dev)
    us = _timed(lambda: ops.decode_attention(ql, kl, vl, bt, ctx, d ** -0.5, out, mp, workspace=ws))
    res["llama_decode"] = {"us": round(us, 1), "TB/s": round(byts / us / 1e6, 2), "parts": mp}
    return res


def rowwise_kernels(s: dict, T: int) -> dict:
    """The memory-bound row kernels alone at T rows, in TB/s of the bytes each
    has to move: residual step + norm, gated activation, head prep + cache write,
    each beside Llama's counterpart."""
    W, ff, H, G, d = s["W"], s["ff"], s["H"], s["G"], s["d"]
    dev, dt, S, bs = "cuda", torch.bfloat16, 4, 64
    res = {}

    def put(name, us, byts):
        res[name] = {"us": round(us, 1), "TB/s": round(byts / us / 1e6, 2)}

    X = torch.randn(T, S, W, device=dev)
    y = torch.randn(T, W, device=dev, dtype=dt)
    mixw = torch.eye(S, device=dev) + 0.01
    ones = torch.ones(S, device=dev)
    nw = torch.ones(W, device=dev)
    put("bekulix_stream_step", _timed(lambda: mx.stream_step(X, y, mixw, ones, ones, nw, 1e-6, dt)),
        T * W * (2 * S * 4 + 2 + 2))  # streams read + written (fp32), y in, normed row out
    h = torch.randn(T, W, device=dev, dtype=dt)
    r = torch.randn(T, W, device=dev, dtype=dt)
    w16 = torch.ones(W, device=dev, dtype=dt)
    put("llama_add_rmsnorm", _timed(lambda: ops.add_rmsnorm(h, r, w16, 1e-6)), T * W * 2 * 4)
    gu = torch.randn(T, 2 * ff, device=dev, dtype=dt)
    put("bekulix_glu_act", _timed(lambda: mx.glu_act(gu, "relu")), T * ff * 2 * 3)
    put("llama_silu_and_mul", _timed(lambda: ops.silu_and_mul(gu)), T * ff * 2 * 3)
    nb = T // bs + 1
    p = torch.randn(T, (H + G) * d, device=dev, dtype=dt)
    pos = torch.arange(T, device=dev)
    kc = torch.zeros(nb * bs, G * d, device=dev, dtype=dt)
    vc = torch.zeros_like(kc)
    qn = torch.ones(d, device=dev)
    put("bekulix_headprep_cache", _timed(lambda: mx.headprep_cache(p, pos, pos, H, G, d, H * d, qn, qn, 1e-6, (0.1, 4096),
                                                                   kc, vc, v_mode=1)),
        T * d * 2 * (2 * H + 3 * G))  # q read + written, k read, K and V rows written
    qkv = torch.randn(T, (H + 2 * G) * d, device=dev, dtype=dt)
    from ..ops import reference as ref
    cs = ref.rope_cos_sin(d, T + 1, 500000.0, None).to(dev)
    kl = torch.zeros(nb, G, bs, d, device=dev, dtype=dt)
    vl = torch.zeros_like(kl)
    put("llama_rope_cache", _timed(lambda: ops.rope_cache(qkv, pos, cs, pos, kl, vl, H, G, d, bs)),
        T * d * 2 * (2 * H + 4 * G))
    return res


def bolinex_kernels(s: dict, L: int, B: int, T: int) -> dict:
    """Bolinex's kernels alone, each beside its counterpart: window attention with the score
    cap and the distance penalty against the same kernels without them (prefill in TFLOP/s of
    the visible scores, decode in TB/s of the window's cache bytes); the residual step with a
    layer norm against Llama's add + RMS norm; the gate product; routing, plan and the grouped
    GEMMs of one routed feed-forward against one dense GEMM pair of the same FLOPs."""
    H, G, d, W, ff, bs = s["H"], s["G"], s["d"], s["W"], s["ff"], 64
    dev, dt, win = "cuda", torch.bfloat16, 1024
    res = {}
    nb = L // bs + 1
    q = torch.randn(L, H * d, device=dev, dtype=dt)
    pos = torch.arange(L, device=dev)
    seq = torch.zeros(L, dtype=torch.int32, device=dev)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(1, nb)
    kc = torch.randn(nb * bs, G * d, device=dev, dtype=dt)
    vc = torch.randn_like(kc)
    tiles = torch.tensor(mx.tile_list(0, L), dtype=torch.int32, device=dev)
    r1 = torch.rand(H, device=dev)
    r2 = torch.rand(H, device=dev) + 0.1
    j = torch.arange(L)
    fl = 4 * d * H * float((j - mx.first_visible(j, "window", win) + 1).sum())
    for name, kw in (("plain", {}), ("cap", dict(softcap=30.0)), ("cap_penalty", dict(softcap=30.0, dist_bias=(r1, r2)))):
        us = _timed(lambda: mx.attention(q, kc, vc, pos, seq, bt, bs, H, 1, H // G, d, d, d ** -0.5, "window", win, 1,
                                         False, tiles, L, **kw))
        res[f"prefill_window{win}_{name}"] = {"us": round(us, 1), "TFLOPs": round(fl / us / 1e6, 1)}
    nbb = B * nb
    byts = B * min(L, win) * G * d * 2 * 2
    btd = torch.randperm(nbb, device=dev).to(torch.int32).view(B, nb)
    kcd = torch.randn(nbb * bs, G * d, device=dev, dtype=dt)
    vcd = torch.randn_like(kcd)
    qd = torch.randn(B, H * d, device=dev, dtype=dt)
    posd = torch.full((B,), L - 1, device=dev)
    parts = mx.row_attention_parts(B, G, win, mx.GROUP_TARGET_WAVES)
    for name, kw in (("plain", {}), ("cap_penalty", dict(softcap=30.0, dist_bias=(r1, r2)))):
        us = _timed(lambda: mx.attention(qd, kcd, vcd, posd, None, btd, bs, H, 1, H // G, d, d, d ** -0.5, "window", win,
                                         parts, **kw))
        res[f"decode_window{win}_{name}"] = {"us": round(us, 1), "TB/s": round(byts / us / 1e6, 2), "parts": parts}

    def put(name, us, byts=None, flops=None):
        res[name] = {"us": round(us, 1)}
        if byts:
            res[name]["TB/s"] = round(byts / us / 1e6, 2)
        if flops:
            res[name]["TFLOPs"] = round(flops / us / 1e6, 1)

    X = torch.randn(T, W, device=dev)
    a, b, c = (torch.randn(T, W, device=dev, dtype=dt) for _ in range(3))
    nw = torch.ones(W, device=dev)
    put("residual_step_two_addends_layernorm",
        _timed(lambda: mx.residual_step(X, a, b, eps=1e-5, norm="layer", norm_w=nw, norm_b=nw, out_dtype=dt)),
        T * W * (4 + 4 + 2 + 2 + 2))
    put("residual_step_unit_rms_addend_layernorm",
        _timed(lambda: mx.residual_step(X, c=c, c_w=nw, eps=1e-5, norm="layer", norm_w=nw, norm_b=nw, out_dtype=dt)),
        T * W * (4 + 4 + 2 + 2))
    r = torch.randn(T, W, device=dev, dtype=dt)
    w16 = torch.ones(W, device=dev, dtype=dt)
    put("llama_add_rmsnorm", _timed(lambda: ops.add_rmsnorm(a, r, w16, 1e-6)), T * W * 2 * 4)
    p = torch.randn(T, 2 * H * d, device=dev, dtype=dt)
    put("act_mul_sigmoid_gate", _timed(lambda: mx.act_mul(p[:, H * d:], p[:, :H * d], "sigmoid")), T * H * d * 2 * 3)
    u = torch.randn(T, ff, device=dev, dtype=dt)
    put("act_mul_relu2", _timed(lambda: mx.act_mul(u, None, "relu2")), T * ff * 2 * 2)
    gu = torch.randn(T, 2 * ff, device=dev, dtype=dt)
    put("llama_silu_and_mul", _timed(lambda: ops.silu_and_mul(gu)), T * ff * 2 * 3)
    # one routed feed-forward: E experts of width ff / 4, two per token
    E, top, fe = 8, 2, ff // 4
    for rows, tag in ((T, "prefill"), (B, "decode")):
        h = torch.randn(rows, W, device=dev, dtype=dt)
        z = torch.randn(rows, E, device=dev)
        corr = torch.zeros(E, device=dev)
        put(f"moe_route_{tag}", _timed(lambda: moe.route(z, corr, top, 4, 2)))
        idx, wgt = moe.route(z, corr, top, 4, 2)
        put(f"moe_plan_{tag}", _timed(lambda: moe.plan(idx, E)))
        order, offsets = moe.plan(idx, E)
        wgu = torch.randn(E, 2 * fe, W, device=dev, dtype=dt) * W ** -0.5
        wdn = torch.randn(E, W, fe, device=dev, dtype=dt) * fe ** -0.5
        f1, f2 = 2.0 * rows * top * W * 2 * fe, 2.0 * rows * top * fe * W
        # decode: the weights of the experts in use are what has to move
        used = int((offsets[1:] > offsets[:-1]).sum())
        wb1, wb2 = used * 2 * fe * W * 2, used * W * fe * 2
        put(f"grouped_gemm_gate_up_{tag}", _timed(lambda: moe.grouped_gemm(h, wgu, order, offsets, top, True, False)),
            wb1 if tag == "decode" else None, f1)
        act = torch.randn(rows * top, fe, device=dev, dtype=dt)
        put(f"grouped_gemm_down_{tag}", _timed(lambda: moe.grouped_gemm(act, wdn, order, offsets, top, False, True)),
            wb2 if tag == "decode" else None, f2)
        # the library's dense GEMMs of the same FLOPs (rows * top rows against one expert's weights)
        hd = torch.randn(rows * top, W, device=dev, dtype=dt)
        put(f"dense_gemm_gate_up_{tag}", _timed(lambda: torch.matmul(hd, wgu[0].t())),
            2 * fe * W * 2 if tag == "decode" else None, f1)
        put(f"dense_gemm_down_{tag}", _timed(lambda: torch.matmul(act, wdn[0].t())),
            W * fe * 2 if tag == "decode" else None, f2)
        y = torch.randn(rows * top, W, device=dev, dtype=dt)
        sh = torch.randn(rows, W, device=dev, dtype=dt)
        put(f"moe_combine_{tag}", _timed(lambda: moe.combine(y, wgt, sh)), rows * W * 2 * (top + 2))
    return res


def nefivik_kernels(s: dict, L: int, B: int, T: int) -> dict:
    """Nefivik's kernels alone, each beside its counterpart where there is one: the delta-rule
    scan over 4 prompts of L / 2 tokens (tokens/s, and the bytes of its inputs and outputs) and
    over B decode rows (TB/s of the state read and written); convolution + rotation + cache
    write against Llama's rope_cache; sigmoid-weight window attention against the same kernels
    with softmax; the gated residual step against Llama's add + RMS norm; the clamped gated
    unit against silu_and_mul; the softmax router."""
    H, G, d, W, ff, bs = s["H"], s["G"], s["d"], s["W"], s["ff"], 64
    dev, dt, win = "cuda", torch.bfloat16, 1024
    res = {}

    def put(name, us, byts=None, flops=None, **kw):
        res[name] = {"us": round(us, 1), **kw}
        if byts:
            res[name]["TB/s"] = round(byts / us / 1e6, 2)
        if flops:
            res[name]["TFLOPs"] = round(flops / us / 1e6, 1)

    # ---- delta rule: prompts, then decode rows
    n = H * d
    for tag, n_seq, rows in (("prefill", 4, L // 2), ("decode", B, 1)):
        Tn = n_seq * rows
        p = torch.randn(Tn, 5 * n, device=dev, dtype=dt)
        wl = torch.randn(Tn, n, device=dev, dtype=dt)
        ab, wb = torch.zeros(n, device=dev), torch.zeros(n, device=dev)
        state = torch.zeros(n_seq, H, d, d, device=dev)
        pos = (torch.arange(rows, device=dev) + 1).repeat(n_seq)
        seq_rows = torch.arange(0, Tn + 1, rows, dtype=torch.int32, device=dev) if rows > 1 else None
        slots = torch.arange(n_seq, dtype=torch.int32, device=dev)
        us = _timed(lambda: rc.delta_rule(p[:, :n], p[:, n:2 * n], p[:, 2 * n:3 * n], p[:, 3 * n:4 * n], wl, ab, wb, state,
                                          pos, seq_rows, slots, H, d, d))
        io = Tn * n * (5 * 2 + 4)  # five bf16 inputs, fp32 output
        st = n_seq * H * d * d * 4 * 2  # state read and written
        put(f"delta_rule_{tag}", us, io + st, 2.0 * 4 * Tn * H * d * d, tok_per_s=round(Tn / us * 1e6),
            state_TBs=round(st / us / 1e6, 2))
        o = torch.randn(Tn, n, device=dev)
        hw = torch.ones(n, device=dev)
        put(f"head_norm_gate_{tag}", _timed(lambda: rc.head_norm_gate(o, H, hw, p[:, 4 * n:5 * n], 1e-5, dt)),
            Tn * n * (4 + 2 + 2))
    # ---- convolution + rotation + cache write
    taps, C = 4, (H + 2 * G) * d
    x = torch.randn(T, C, device=dev, dtype=dt)
    cw = torch.randn(taps, C, device=dev)
    tail = torch.zeros(1, taps - 1, C, device=dev, dtype=dt)
    nbt = T // bs + 1
    kc = torch.zeros(nbt * bs, G * d, device=dev, dtype=dt)
    vc = torch.zeros_like(kc)
    posT = torch.arange(T, device=dev)
    rs = torch.zeros(T, dtype=torch.int32, device=dev)
    sr = torch.tensor([0, T], dtype=torch.int32, device=dev)
    s0 = torch.zeros(1, dtype=torch.int32, device=dev)
    inv = rc.rotary_frequencies(d // 2, 500000.0, None).to(dev)
    put("conv_rope_cache", _timed(lambda: rc.conv_rope_cache(x, cw, tail, posT, posT, rs, sr, s0, H, G, d, d, inv, kc, vc)),
        T * d * 2 * (2 * H + 4 * G))
    qkv = torch.randn(T, C, device=dev, dtype=dt)
    from ..ops import reference as ref
    cs = ref.rope_cos_sin(d, T + 1, 500000.0, None).to(dev)
    kl = torch.zeros(nbt, G, bs, d, device=dev, dtype=dt)
    vl = torch.zeros_like(kl)
    put("llama_rope_cache", _timed(lambda: ops.rope_cache(qkv, posT, cs, posT, kl, vl, H, G, d, bs)),
        T * d * 2 * (2 * H + 4 * G))
    # ---- window attention: sigmoid weights + head bias + head gate against softmax
    nb = L // bs + 1
    q = torch.randn(L, H * d, device=dev, dtype=dt)
    pos = torch.arange(L, device=dev)
    seq = torch.zeros(L, dtype=torch.int32, device=dev)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(1, nb)
    kc = torch.randn(nb * bs, G * d, device=dev, dtype=dt)
    vc = torch.randn_like(kc)
    tiles = torch.tensor(mx.tile_list(0, L), dtype=torch.int32, device=dev)
    pb = torch.randn(H, device=dev) - 3
    gate = torch.randn(L, H, device=dev, dtype=dt)
    j = torch.arange(L)
    fl = 4 * d * H * float((j - mx.first_visible(j, "window", win) + 1).sum())
    for name, kw in (("softmax", {}), ("sigmoid_gate", dict(weights="sigmoid", head_bias=pb, head_gate=gate))):
        us = _timed(lambda: mx.attention(q, kc, vc, pos, seq, bt, bs, H, 1, H // G, d, d, d ** -0.5, "window", win, 1,
                                         False, tiles, L, **kw))
        put(f"prefill_window{win}_{name}", us, None, fl)
    nbb = B * nb
    byts = B * min(L, win) * G * d * 2 * 2
    btd = torch.randperm(nbb, device=dev).to(torch.int32).view(B, nb)
    kcd = torch.randn(nbb * bs, G * d, device=dev, dtype=dt)
    vcd = torch.randn_like(kcd)
    qd = torch.randn(B, H * d, device=dev, dtype=dt)
    posd = torch.full((B,), L - 1, device=dev)
    parts = mx.row_attention_parts(B, G, win, mx.GROUP_TARGET_WAVES)
    for name, kw in (("softmax", {}), ("sigmoid_gate", dict(weights="sigmoid", head_bias=pb, head_gate=gate[:B]))):
        us = _timed(lambda: mx.attention(qd, kcd, vcd, posd, None, btd, bs, H, 1, H // G, d, d, d ** -0.5, "window", win,
                                         parts, **kw))
        put(f"decode_window{win}_{name}", us, byts, parts=parts)
    # ---- row kernels
    X = torch.randn(T, W, device=dev)
    c, g = torch.randn(T, W, device=dev, dtype=dt), torch.randn(T, W, device=dev, dtype=dt)
    nw = torch.ones(W, device=dev)
    put("residual_step_gated_unit_rms_addend_rmsnorm",
        _timed(lambda: mx.residual_step(X, c=c, c_w=nw, eps=1e-5, norm="rms", norm_w=nw, out_dtype=dt, c_gate=g,
                                        c_gate_b=nw)), T * W * (4 + 4 + 2 + 2 + 2))
    a, r = torch.randn(T, W, device=dev, dtype=dt), torch.randn(T, W, device=dev, dtype=dt)
    w16 = torch.ones(W, device=dev, dtype=dt)
    put("llama_add_rmsnorm", _timed(lambda: ops.add_rmsnorm(a, r, w16, 1e-6)), T * W * 2 * 4)
    fe = ff // 4
    gu = torch.randn(2 * T, 2 * fe, device=dev, dtype=dt)
    put("glu_act_swiglu_clamp", _timed(lambda: mx.glu_act(gu, "swiglu_clamp", 7.0, 1.702)), 2 * T * fe * 2 * 3)
    put("llama_silu_and_mul", _timed(lambda: ops.silu_and_mul(gu)), 2 * T * fe * 2 * 3)
    z = torch.randn(T, 8, device=dev)
    put("moe_route_softmax", _timed(lambda: moe.route(z, None, 2, 4, 2, score="softmax", group_score="max")))
    return res


def sobivik_kernels(s: dict, L: int, B: int, T: int) -> dict:
    """Sobivik's kernels alone, each beside its counterpart: the retention scan beside the
    delta-rule scan (4 prompts of L / 2 tokens; B decode rows); window attention with kept first
    keys (two maps) and with a sink over one shared latent head, beside the same kernels without
    either; the depth average (with the closing addend and the next norm) beside the residual
    step; the input convolution and the latent / rotary preparation beside Nefivik's convolution +
    rotation + cache write; the per-head norm with a silu gate beside the sigmoid one."""
    H, G, d, W, bs = s["H"], s["G"], s["d"], s["W"], 64
    dev, dt, win, keep = "cuda", torch.bfloat16, 1024, 64
    res = {}

    def put(name, us, byts=None, flops=None, **kw):
        res[name] = {"us": round(us, 1), **kw}
        if byts:
            res[name]["TB/s"] = round(byts / us / 1e6, 2)
        if flops:
            res[name]["TFLOPs"] = round(flops / us / 1e6, 1)

    # ---- the two scans: prompts, then decode rows
    n = H * d
    for tag, n_seq, rows in (("prefill", 4, L // 2), ("decode", B, 1)):
        Tn = n_seq * rows
        p = torch.randn(Tn, 5 * n, device=dev, dtype=dt)
        state = torch.zeros(n_seq, H, d, d, device=dev)
        pos = (torch.arange(rows, device=dev) + 1).repeat(n_seq)
        seq_rows = torch.arange(0, Tn + 1, rows, dtype=torch.int32, device=dev) if rows > 1 else None
        slots = torch.arange(n_seq, dtype=torch.int32, device=dev)
        decay = torch.full((H,), 0.97, device=dev)
        st = n_seq * H * d * d * 4 * 2  # state read and written
        us = _timed(lambda: rc.retention(p[:, :n], p[:, n:2 * n], p[:, 2 * n:3 * n], decay, d ** -0.5, state, pos,
                                         seq_rows, slots, H, d, d))
        put(f"retention_{tag}", us, Tn * n * (3 * 2 + 4) + st, 2.0 * 2 * Tn * H * d * d, tok_per_s=round(Tn / us * 1e6),
            state_TBs=round(st / us / 1e6, 2))
        wl = torch.randn(Tn, n, device=dev, dtype=dt)
        zb = torch.zeros(n, device=dev)
        us = _timed(lambda: rc.delta_rule(p[:, :n], p[:, n:2 * n], p[:, 2 * n:3 * n], p[:, 3 * n:4 * n], wl, zb, zb, state,
                                          pos, seq_rows, slots, H, d, d))
        put(f"nefivik_delta_rule_{tag}", us, Tn * n * (5 * 2 + 4) + st, 2.0 * 4 * Tn * H * d * d,
            tok_per_s=round(Tn / us * 1e6), state_TBs=round(st / us / 1e6, 2))
        o = torch.randn(Tn, n, device=dev)
        for act in ("silu", "sigmoid"):
            put(f"head_norm_gate_{act}_{tag}",
                _timed(lambda: rc.head_norm_gate(o, H, None, p[:, 4 * n:5 * n], 1e-5, dt, gate_act=act)), Tn * n * (4 + 2 + 2))
    # ---- attention: (name, query vectors, maps, group, d, dv, shared K/V row, extras)
    Hd, Gd = H // 2, max(1, G // 2)
    shapes = [("diff", 2 * Hd, 2, Hd // Gd, d, 2 * d, False, dict(keep_first=keep)),
              ("latent", H, 1, H, 256, 192, True, dict(sink=torch.randn(H, device=dev)))]
    nb = L // bs + 1
    pos = torch.arange(L, device=dev)
    seq = torch.zeros(L, dtype=torch.int32, device=dev)
    bt = torch.arange(nb, dtype=torch.int32, device=dev).view(1, nb)
    tiles = torch.tensor(mx.tile_list(0, L), dtype=torch.int32, device=dev)
    j = torch.arange(L)
    vis = (j - mx.first_visible(j, "window", win) + 1)
    nbb = B * nb
    btd = torch.randperm(nbb, device=dev).to(torch.int32).view(B, nb)
    posd = torch.full((B,), L - 1, device=dev)
    for name, n_qh, maps, group, dd, dv, shared, extra in shapes:
        n_kh, n_vh = n_qh // group, n_qh // maps // group
        q = torch.randn(L, n_qh * dd, device=dev, dtype=dt)
        kc = torch.randn(nb * bs, n_kh * dd, device=dev, dtype=dt)
        vc = kc if shared else torch.randn(nb * bs, n_vh * dv, device=dev, dtype=dt)
        sc = dd ** -0.5
        for tag, kw in (("plain", {}), ("keep" if "keep_first" in extra else "sink", extra)):
            seen = vis + (torch.minimum(torch.tensor(keep), mx.first_visible(j, "window", win)) if "keep_first" in kw else 0)
            fl = 2.0 * (dd + dv) * n_qh * float(seen.sum())
            us = _timed(lambda: mx.attention(q, kc, vc, pos, seq, bt, bs, n_qh, maps, group, dd, dv, sc, "window", win, 1,
                                             maps == 2, tiles, L, **kw))
            put(f"{name}_prefill_window{win}_{tag}", us, None, fl)
        kcd = torch.randn(nbb * bs, n_kh * dd, device=dev, dtype=dt)
        vcd = kcd if shared else torch.randn(nbb * bs, n_vh * dv, device=dev, dtype=dt)
        qd = torch.randn(B, n_qh * dd, device=dev, dtype=dt)
        parts = mx.row_attention_parts(B, n_kh * (-(-group // 32)), win, mx.GROUP_TARGET_WAVES)
        for tag, kw in (("plain", {}), ("keep" if "keep_first" in extra else "sink", extra)):
            rows_read = min(L, win) + (keep if "keep_first" in kw else 0)
            byts = B * rows_read * (n_kh * dd + (0 if shared else n_vh * dv)) * 2
            us = _timed(lambda: mx.attention(qd, kcd, vcd, posd, None, btd, bs, n_qh, maps, group, dd, dv, sc, "window",
                                             win, parts, maps == 2, **kw))
            put(f"{name}_decode_window{win}_{tag}", us, byts, parts=parts)
    # ---- depth average (5 planes, closing addend, next norm) beside the residual step (addend, next norm)
    planes = 5
    stack = torch.randn(planes + 1, T, W, device=dev)
    wts = torch.full((planes,), 1.0 / planes, device=dev)
    c = torch.randn(T, W, device=dev, dtype=dt)
    nw = torch.ones(W, device=dev)
    put(f"depth_mix_{planes}_planes_addend_rmsnorm",
        _timed(lambda: mx.depth_mix(stack, planes, wts, dst=stack[planes], norm_w=nw, eps=1e-5, out_dtype=dt, c=c, c_w=nw)),
        T * W * (4 * planes + 4 + 4 + 2 + 2 + 2))  # planes read, newest written back, sum written, addend (twice), norm out
    X = torch.randn(T, W, device=dev)
    put("residual_step_unit_rms_addend_rmsnorm",
        _timed(lambda: mx.residual_step(X, c=c, c_w=nw, eps=1e-5, norm="rms", norm_w=nw, out_dtype=dt)),
        T * W * (4 + 4 + 2 + 2))
    # ---- input convolution (all W channels) and latent / rotary preparation beside Nefivik's convolution + rotation
    taps = 4
    x = torch.randn(T, W, device=dev, dtype=dt)
    cw = torch.randn(taps, W, device=dev)
    tail = torch.zeros(1, taps - 1, W, device=dev, dtype=dt)
    posT = torch.arange(T, device=dev)
    rs = torch.zeros(T, dtype=torch.int32, device=dev)
    sr = torch.tensor([0, T], dtype=torch.int32, device=dev)
    s0 = torch.zeros(1, dtype=torch.int32, device=dev)
    put("input_conv", _timed(lambda: rc.conv_rope_cache(x, cw, tail, posT, posT, rs, sr, s0, 1, 0, W, 0, None, None, None)),
        T * W * 2 * 2)
    C = (H + 2 * G) * d
    xq = torch.randn(T, C, device=dev, dtype=dt)
    cwq = torch.randn(taps, C, device=dev)
    tailq = torch.zeros(1, taps - 1, C, device=dev, dtype=dt)
    nbt = T // bs + 1
    kcn = torch.zeros(nbt * bs, G * d, device=dev, dtype=dt)
    vcn = torch.zeros_like(kcn)
    inv = rc.rotary_frequencies(d // 2, 500000.0, None).to(dev)
    put("nefivik_conv_rope_cache",
        _timed(lambda: rc.conv_rope_cache(xq, cwq, tailq, posT, posT, rs, sr, s0, H, G, d, d, inv, kcn, vcn)),
        T * d * 2 * (2 * H + 4 * G))
    r, dr = 192, 64
    qa = torch.randn(H, T, r, device=dev, dtype=dt)
    qp = torch.randn(T, H * (d + dr), device=dev, dtype=dt)
    kv = torch.randn(T, r + dr, device=dev, dtype=dt)
    cn = torch.ones(r, device=dev)
    fr, mag = rc.yarn_frequencies(dr, 10000.0, {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0})
    cache = torch.zeros(nbt * bs, r + dr, device=dev, dtype=dt)
    put("latent_rope", _timed(lambda: rc.latent_rope(qa, qp, d + dr, d, kv, r, dr, cn, 1e-5, fr.to(dev), mag, posT, posT,
                                                      cache)), T * 2 * (2 * H * (r + dr) + 2 * (r + dr)))
    sn = torch.randn(T, W // 4 + r + dr, device=dev, dtype=dt)
    qn = torch.ones(W // 4, device=dev)
    put("section_norm", _timed(lambda: mx.section_norm(sn[:, :W // 4], qn, 1e-5)), T * (W // 4) * 2 * 2)
    return res


def run_layered_compare(args, dev) -> dict:
    isl, osl = min(args.isl, 2048), min(args.osl, 64)
    fam = getattr(args, "layered_family", "all")
    sizes = {}
    for name, s in SIZES.items():
        bek, lla = _configs(s)
        row = {"layers": s["layers"], "isl": isl, "osl": osl, "prefill_seqs": 4, "decode_seqs": 64}
        if fam in ("all", "bekulix"):
            row["bekulix"] = engine_throughput(bek, dev, isl, osl, 4, 64, args.seed)
        if fam in ("all", "bolinex"):
            row["bolinex"] = engine_throughput(_bolinex_config(s), dev, isl, osl, 4, 64, args.seed)
            row["bolinex_kernels"] = bolinex_kernels(s, 4096, 64, 8192)
        if fam == "sobivik":
            row["sobivik"] = engine_throughput(_sobivik_config(s), dev, isl, osl, 4, 64, args.seed)
            row["sobivik_kernels"] = sobivik_kernels(s, 4096, 64, 8192)
            row["bekulix"] = engine_throughput(bek, dev, isl, osl, 4, 64, args.seed)
        if fam == "nefivik":
            row["nefivik"] = engine_throughput(_nefivik_config(s), dev, isl, osl, 4, 64, args.seed)
            row["nefivik_kernels"] = nefivik_kernels(s, 4096, 64, 8192)
            row["bolinex"] = engine_throughput(_bolinex_config(s), dev, isl, osl, 4, 64, args.seed)
        row["llama"] = engine_throughput(lla, dev, isl, osl, 4, 64, args.seed)
        if fam in ("nefivik", "sobivik"):
            sizes[name] = row
            continue
        row["attention_kernels"] = attention_kernels(s, 4096, 64)
        if fam in ("all", "bekulix"):
            row["rowwise_kernels"] = rowwise_kernels(s, 8192)
        sizes[name] = row
    return {"metric": "layer-listed models (Bekulix, Bolinex, Nefivik, Sobivik) beside Llama at equal layer sizes: engine prefill / "
                      "decode tokens/s and kernels alone", "unit": "tokens/s", "n_gpus": 1, "dtype": "bf16",
            "family": fam, "data": "synthetic (random-token prompts, random-init weights)", "sizes": sizes}
