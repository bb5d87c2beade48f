"""Plain, slow oracle of the Sobivik design for the tests: one function per
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


def sigmoid(z):
    return 1.0 / (1.0 + torch.exp(-z))


def silu(z):
    return z * sigmoid(z)


# ----------------------------------------------------------------- around the sublayers
def time_conv(h, w):
    """h + conv(h): per channel c, y_t = h_t + sum_j w[c, j] h_(t - taps + 1 + j), zeros before t = 0."""
    T = h.shape[0]
    taps = w.shape[1]
    y = h.clone()
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                y[t] += w[:, j] * h[s]
    return y


def depth_average(xs, w):
    """sum_j w[j] xs[j] over every result so far (xs[0] the embedding output)."""
    assert len(xs) == w.numel()
    return sum(w[j] * xs[j] for j in range(len(xs)))


def dense_ff(h, gate, up, down):
    return (silu(h @ gate.T) * (h @ up.T)) @ down.T


# ----------------------------------------------------------------- retention
def retention_scan(q, k, v, decay):
    """q, k [T, H, d], v [T, H, dv], decay [H]:  S_t = decay S_(t-1) + k_t v_t^T,  o_t = S_t^T q_t."""
    T, H, d = q.shape
    S = torch.zeros(H, d, v.shape[-1], dtype=F)
    out = torch.zeros(T, H, v.shape[-1], dtype=F)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hi,hij->hj", q[t], S)
    return out, S


def retention(h, p, m, eps):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ p["q"].T).view(T, H, d)
    k = (h @ p["k"].T).view(T, H, d) * d ** -0.5
    v = (h @ p["v"].T).view(T, H, dv)
    o, _ = retention_scan(q, k, v, torch.tensor(m["decay"], dtype=F))
    o = unit_rms(o, eps).reshape(T, H * dv) * silu(h @ p["g"].T)
    return o @ p["o"].T


# ----------------------------------------------------------------- rotary positions
def scaled_frequencies(rot):
    """f_i = base^(-2i/dims), blended towards f_i / factor over the band of
    dimensions between the ones whose wavelengths fit `fast` and `slow` times
    into the original length; and the factor on cos and sin."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def dim_of(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=F), 0.1 * math.log(factor) + 1.0


def rotate(x, pos, rot):
    """x [T, ..., n]: the first rot.dims columns rotated, column i with i + dims/2."""
    f, mag = scaled_frequencies(rot)
    half = f.numel()
    ang = pos.to(F)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = (torch.cos(ang) * mag).view(shape), (torch.sin(ang) * mag).view(shape)
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], -1)


# ----------------------------------------------------------------- latent attention
def latent_attention(h, p, m, eps):
    T = h.shape[0]
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = unit_rms(h @ p["dq"].T, eps) * p["dq.norm"]
    q = (cq @ p["uq"].T).view(T, H, d + dr)
    kv = h @ p["dkv"].T
    c = unit_rms(kv[:, :r], eps) * p["dkv.norm"]
    kr = kv[:, r:]
    rot = m.get("rot")
    q_rot, k_rot = q[..., d:], kr
    if rot:
        q_rot, k_rot = rotate(q_rot, pos, rot), rotate(kr, pos, rot)
    kn = (c @ p["uk"].T).view(T, H, d)
    val = (c @ p["uv"].T).view(T, H, dv)
    sc = (torch.einsum("ihd,jhd->hij", q[..., :d], kn) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * m["scale"]
    dist = pos[:, None] - pos[None, :]
    vis = dist >= 0
    size = (m.get("mask") or {}).get("size")
    if size:
        vis = vis & (dist < size)
    sc = sc.masked_fill(~vis[None], float("-inf"))
    sink = p.get("sink")
    if sink is not None:
        sc = torch.cat([sc, sink.view(H, 1, 1).expand(H, T, 1)], -1)
    w = torch.softmax(sc, -1)[..., :T]
    o = torch.einsum("hij,jhd->ihd", w, val).reshape(T, H * dv)
    return (o * sigmoid(h @ p["g"].T)) @ p["o"].T


# ----------------------------------------------------------------- differential attention
def diff_attention(h, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ p["q"].T).view(T, H, 2, d)
    k = (h @ p["k"].T).view(T, G, 2, d)
    v = (h @ p["v"].T).view(T, G, dv)
    pos = torch.arange(T)
    dist = pos[:, None] - pos[None, :]
    vis = dist >= 0
    mask = m.get("mask") or {}
    if mask.get("size"):
        near = dist < mask["size"]
        if mask.get("keep_first"):
            near = near | (pos[None, :] < mask["keep_first"])
        vis = vis & near
    lam = math.exp(float((p["lq1"] * p["lk1"]).sum())) - math.exp(float((p["lq2"] * p["lk2"]).sum())) + m["diff"]
    out = torch.zeros(T, H, dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        a = []
        for mp in range(2):
            sc = (q[:, hh, mp] @ k[:, g, mp].T) * m["scale"]
            a.append(torch.softmax(sc.masked_fill(~vis, float("-inf")), -1) @ v[:, g])
        out[:, hh] = unit_rms(a[0] - lam * a[1], eps) * (1.0 - m["diff"])
    out = out * sigmoid(h @ p["g"].T)[:, :, None]
    return out.reshape(T, H * dv) @ p["o"].T


MIXERS = {"retention": retention, "latent_attention": latent_attention, "attention": diff_attention}


# ----------------------------------------------------------------- the model
def forward(cfg: dict, sd: dict, tokens, upto: int | None = None):
    """Logits [T, vocab] of one sequence, and what goes on after every layer."""
    sd = {k: v.to(F) for k, v in sd.items()}
    eps = float(cfg["norm"]["eps"])
    x = sd["embed"][torch.as_tensor(tokens)] * float(cfg["embedding"]["scale"])
    xs, after = [x], []
    for i, L in enumerate(cfg["layers"][:upto]):
        pre = f"l{i}."
        p = {k[len(pre) + 4:]: v for k, v in sd.items() if k.startswith(pre + "mix.")}
        h = unit_rms(x, eps) * sd[pre + "norm1"]
        if pre + "canon1" in sd:
            h = time_conv(h, sd[pre + "canon1"])
        x = x + unit_rms(MIXERS[L["type"]](h, p, L["mixer"], eps), eps) * sd[pre + "norm1b"]
        if L.get("mlp"):
            h = unit_rms(x, eps) * sd[pre + "norm2"]
            y = dense_ff(h, sd[pre + "mlp.gate"], sd[pre + "mlp.up"], sd[pre + "mlp.down"])
            x = x + unit_rms(y, eps) * sd[pre + "norm2b"]
        xs.append(x)
        if pre + "dwa" in sd:
            x = depth_average(xs, sd[pre + "dwa"])
        after.append(x)
    x = unit_rms(x, eps) * sd["final.norm"]
    return (x @ sd["head"].T) * float(cfg.get("logit_scale", 1.0)), after
