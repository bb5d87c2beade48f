"""Plain, slow oracle of the Nefivik design for the tests: one function per
mechanism, whole sequences, dense [T, T] score matrices, token-by-token
recurrences, float64 throughout.  It shares nothing with the engine's model,
ops or kernels; it consumes a config dict (the keys of a checkpoint's
config.json) and a name -> tensor dict in the checkpoint's naming.

Notation: T tokens of one sequence at positions 0 .. T-1; x [T, width] the
residual; h the normed sublayer input; weights stored [out, in], applied as
h @ W^T.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return unit_rms(x, eps) * w


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


# ----------------------------------------------------------------- recurrent mixer
def delta_decay(h, w1, w2, w0):
    """Per key channel decay in (exp(-e^-0.5), 1): exp(-e^-0.5 * sigmoid(w2 tanh(w1 h) + w0))."""
    return torch.exp(-math.exp(-0.5) * sigmoid(torch.tanh(h @ w1.T) @ w2.T + w0))


def delta_scan(r, k, v, w, a):
    """The generalized delta rule over one sequence from a zero state.
    r, k, w, a [T, H, dk]; v [T, H, dv].  Per head, with u the unit key,
        S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,   o_t = S_t^T r_t.
    Returns o [T, H, dv] and the final state [H, dk, dv]."""
    T, H, dk = k.shape
    dv = v.shape[-1]
    S = torch.zeros(H, dk, dv, dtype=F)
    out = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        u = k[t] / torch.sqrt((k[t] * k[t]).sum(-1, keepdim=True) + 1e-6)
        uS = torch.einsum("hi,hij->hj", u, S)
        S = w[t][:, :, None] * S - (a[t] * u)[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hi,hij->hj", r[t], S)
    return out, S


def general_delta(h, W, p, m, eps):
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    r = (h @ W[p + "r"].T).view(T, H, d)
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, d)
    w = delta_decay(h, W[p + "w1"], W[p + "w2"], W[p + "w0"]).view(T, H, d)
    a = sigmoid(h @ W[p + "a"].T + W[p + "a.b"]).view(T, H, d)
    o, _ = delta_scan(r, k, v, w, a)
    o = unit_rms(o, eps).reshape(T, H * d) * W[p + "norm"] * sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


# ----------------------------------------------------------------- attention mixer
def short_conv(u, w):
    """Causal depthwise convolution over time: y_t = sum_j w[:, j] u_(t - taps + 1 + j)."""
    T, C = u.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=F), u], 0)
    y = torch.zeros(T, C, dtype=F)
    for j in range(taps):
        y = y + pad[j:j + T] * w[:, j]
    return y


def rotary_frequencies(rot):
    """f_i = base^(-2i/dims), i < dims/2, rescaled band by band when `scaling` is given."""
    dims = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
    sc = rot.get("scaling")
    if sc:
        fac, low, high, orig = sc["factor"], sc["low"], sc["high"], sc["original"]
        out = []
        for fi in f.tolist():
            wl = 2.0 * math.pi / fi
            if wl < orig / high:
                out.append(fi)
            elif wl > orig / low:
                out.append(fi / fac)
            else:
                s = (orig / wl - low) / (high - low)
                out.append((1.0 - s) * fi / fac + s * fi)
        f = torch.tensor(out, dtype=F)
    return f


def rotate(x, rot):
    """x [T, heads, d]: the first rot.dims columns of every head rotated pairwise (i, i + dims/2)."""
    if not rot or not rot.get("dims"):
        return x
    T = x.shape[0]
    dims = rot["dims"]
    half = dims // 2
    ang = torch.arange(T, dtype=F)[:, None] * rotary_frequencies(rot)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = x[..., :half], x[..., half:dims]
    return torch.cat([a * c - b * s, b * c + a * s, x[..., dims:]], -1)


def window_mask(T, size):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if size:
        m &= (i - j) < size
    return m


def attention_keys_values(h, W, p, m):
    """The layer's cached keys (convolved, rotated) and values (convolved)."""
    T = h.shape[0]
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = h @ W[p + "k"].T
    v = h @ W[p + "v"].T
    if m.get("conv"):
        k, v = short_conv(k, W[p + "k.conv"]), short_conv(v, W[p + "v.conv"])
    return rotate(k.view(T, G, d), m.get("rot")), v.view(T, G, dv)


def attention(h, W, p, m, kv):
    """Sigmoid attention: visible keys weigh sigmoid(q.k * scale + pb_h), not normalised."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ W[p + "q"].T
    if m.get("conv"):
        q = short_conv(q, W[p + "q.conv"])
    q = rotate(q.view(T, H, d), m.get("rot"))
    k, v = kv
    rep = H // G
    k, v = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
    s = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    wts = sigmoid(s + W[p + "pb"][:, None, None])
    wts = wts * window_mask(T, (m.get("mask") or {}).get("size"))[None]
    o = torch.einsum("hij,jhd->ihd", wts, v)
    o = o * sigmoid(h @ W[p + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ W[p + "o"].T


# ----------------------------------------------------------------- feed-forward
def route(h, Wr, r, gaps=None):
    """(chosen experts [T, top], their weights): softmax scores; groups ranked by
    their best score; the top scores among the kept groups; weights are the scores.
    gaps collects, per token, how far the weakest choice (expert or group) is ahead
    of the strongest one not chosen."""
    s = torch.softmax(h @ Wr.T, -1)
    T, E = s.shape
    c = s.clone()
    gr = r.get("groups")
    if gr and gr["count"] > 1:
        per = E // gr["count"]
        gs = s.view(T, gr["count"], per).max(-1).values
        kept = torch.zeros(T, gr["count"], dtype=torch.bool)
        kept.scatter_(1, gs.topk(gr["keep"], -1).indices, True)
        c = c.masked_fill(~kept.repeat_interleave(per, 1), -1.0)
        if gaps is not None and gr["keep"] < gr["count"]:
            g2 = gs.topk(gr["keep"] + 1, -1).values
            gaps.append(g2[:, -2] - g2[:, -1])
    idx = c.topk(r["top"], -1).indices
    if gaps is not None and r["top"] < E:
        c2 = c.topk(r["top"] + 1, -1).values
        gaps.append(torch.where(c2[:, -1] >= 0, c2[:, -2] - c2[:, -1], torch.ones(T, dtype=F)))
    return idx, s.gather(1, idx)


def expert(h, Wg, Wu, Wd, limit):
    g = (h @ Wg.T).clamp(max=limit)
    u = (h @ Wu.T).clamp(-limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1.0)) @ Wd.T


def moe(h, W, p, mlp, gaps=None):
    idx, wts = route(h, W[p + "router"], mlp["router"], gaps)
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wts[t]):
            q = f"{p}e{e}."
            out[t] += w * expert(h[t:t + 1], W[q + "gate"], W[q + "up"], W[q + "down"], mlp["expert"]["limit"])[0]
    return out


# ----------------------------------------------------------------- the model
def token_input(x, e, W, p, eps):
    y = (gelu_tanh(x @ W[p + "gate"].T) * e) @ W[p + "proj"].T
    return unit_rms(y, eps) * W[p + "norm"]


def forward(cfg: dict, W: dict, toks: list[int], layers_out: list | None = None, gaps: list | None = None):
    """Logits [T, vocab] of one sequence; layers_out collects the residual after every layer,
    gaps the margins of every routing decision ([T] each)."""
    W = {k: v.to(F) if v.is_floating_point() else v for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    side = (cfg.get("token_side") or {}).get("dim", 0)
    toks = torch.as_tensor(toks, dtype=torch.long)
    x = W["embed"][toks]
    kvs = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = rms_norm(x, W[p + "norm1"], eps)
        if L["type"] == "general_delta":
            y = general_delta(h, W, p + "mix.", m, eps)
        elif L["type"] == "attention":
            if m.get("kv_from") is None:
                kvs[i] = attention_keys_values(h, W, p + "mix.", m)
            y = attention(h, W, p + "mix.", m, kvs[i if m.get("kv_from") is None else m["kv_from"]])
        else:
            raise ValueError(L["type"])
        y = y * sigmoid(h @ W[p + "rg1"].T + W[p + "rg1.b"])
        x = x + rms_norm(y, W[p + "norm1b"], eps)
        if L.get("mlp"):
            h = rms_norm(x, W[p + "norm2"], eps)
            y = moe(h, W, p + "mlp.", L["mlp"], gaps)
            y = y * sigmoid(h @ W[p + "rg2"].T + W[p + "rg2.b"])
            x = x + rms_norm(y, W[p + "norm2b"], eps)
        if side:
            x = x + token_input(x, W["side.embed"][toks][:, i * side:(i + 1) * side], W, p + "side.", eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T
