"""Ops with per-sequence state: the generalized delta rule (a running matrix
per head), retention (a running matrix with a fixed decay per head), short
causal convolutions over time fused with rotary positions and the paged cache
write, the query / key preparation of latent attention with a rotated key
part, and the per-head unit-RMS + gate that follows a recurrent mixer.

State lives in slots: state tensors are [slots, ...], the engine's KV manager
hands a slot to every live request, and a step names the slot of each of its
sequences (`state_slots` [n_seq] int32, -1: a padding row that touches
nothing).  A step's rows are grouped by sequence: `seq_rows` [n_seq + 1] int32
holds the first row of every sequence (None: row i is sequence i, a decode
step); within a sequence rows are consecutive positions.  A sequence whose
first row of the step is at position 0 starts from zero state, whatever its
slot held before, so slots need no clearing when they change hands.

GPU tensors run the gfx950 kernels of ``_C_mixers`` (csrc/mixers/recurrent.hip);
CPU tensors run the PyTorch forms below.  Decays, removal rates, unit keys and
the state are fp32 in every dtype.
"""
from __future__ import annotations

import math

import torch

from .mixers import _f32, _fp32_param, _m, _ptr, _stream


def _seq_bounds(seq_rows: torch.Tensor | None, n_seq: int) -> list[int]:
    return list(range(n_seq + 1)) if seq_rows is None else seq_rows.tolist()


def _check_step(positions, seq_rows, state_slots):
    if positions.dtype != torch.int64 or state_slots.dtype != torch.int32 or \
            (seq_rows is not None and (seq_rows.dtype != torch.int32 or seq_rows.numel() != state_slots.numel() + 1)):
        raise TypeError("int64 positions, int32 state_slots [n_seq] and seq_rows [n_seq + 1]")


# ----------------------------------------------------------------- rotary frequencies
def rotary_frequencies(dims: int, base: float, scaling: dict | None = None) -> torch.Tensor:
    """f_i = base^(-2 i / dims), i < dims / 2 (fp32, computed in float64).  With
    scaling = {factor, low, high, original}: a frequency whose wavelength
    l = 2 pi / f is below original / high stays, one above original / low is
    divided by factor, and between the two it is (1 - s) f / factor + s f with
    s = (original / l - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            fac, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wl = 2.0 * math.pi / f
            if wl > orig / low:
                f = f / fac
            elif wl >= orig / high:
                s = (orig / wl - low) / (high - low)
                f = (1.0 - s) * f / fac + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64).to(torch.float32)


def yarn_frequencies(dims: int, base: float, scaling: dict | None = None) -> tuple[torch.Tensor, float]:
    """(f [dims / 2] fp32, mag): f_i = base^(-2 i / dims), and with scaling =
    {factor, original, fast, slow} (YaRN) the blend
        f_i / factor * ramp_i + f_i * (1 - ramp_i),   ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
    between the dimensions lo = max(floor(dim(fast)), 0) and hi = min(ceil(dim(slow)), dims - 1), where
    dim(t) = dims * ln(original / (2 pi t)) / (2 ln base) is the dimension whose wavelength fits t
    times into the original length; mag = 0.1 ln(factor) + 1 multiplies cosines and sines
    (1 without scaling).  Computed in float64."""
    f = [float(base) ** (-2.0 * i / dims) for i in range(dims // 2)]
    mag = 1.0
    if scaling:
        fac, orig = float(scaling["factor"]), float(scaling["original"])

        def dim_of(turns: float) -> float:
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(float(base)))

        lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
        hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
        for i in range(dims // 2):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / fac * ramp + f[i] * (1.0 - ramp)
        mag = 0.1 * math.log(fac) + 1.0
    return torch.tensor(f, dtype=torch.float64).to(torch.float32), mag


def latent_rope(qa: torch.Tensor, q: torch.Tensor, q_head: int, q_off: int, kv: torch.Tensor, r: int, dr: int,
                norm_w: torch.Tensor, eps: float, inv_freq: torch.Tensor | None, mag: float,
                positions: torch.Tensor, kv_slots: torch.Tensor, cache: torch.Tensor) -> torch.Tensor:
    """Query / key preparation of latent attention with a rotated key part.
    Per token row t: the latent kv[t, :r] is RMS-normed (weight norm_w) into
    cache[slot, :r]; the key part kv[t, r:r + dr], shared by all heads and not
    normed, is rotated into cache[slot, r:]; and head h's query is assembled
    as [qa[h, t] (r) | rotate(q[t, h * q_head + q_off : + dr])] -- qa [H, T, r]
    is the head's unrotated query part already times the head's key
    up-projection.  Returns q' [T, H * (r + dr)].  Rotation: the first
    2 len(inv_freq) columns of a part, column i paired with i + len(inv_freq),
    by the angle position * inv_freq[i], cosines and sines times mag; the rest
    pass unchanged.  Rows with slot < 0 cache nothing."""
    H, T, _ = qa.shape
    half = 0 if inv_freq is None else inv_freq.numel()
    _fp32_param(norm_w, "norm_w")
    _fp32_param(inv_freq, "inv_freq")
    Wc = r + dr
    if qa.shape != (H, T, r) or not qa.is_contiguous() or kv.shape[0] != T or kv.shape[1] < Wc or kv.stride(1) != 1 or \
            q.shape[0] != T or q.stride(1) != 1 or q.shape[1] < (H - 1) * q_head + q_off + dr or 2 * half > dr or \
            q_off + dr > q_head or norm_w.numel() != r:
        raise ValueError("latent_rope: sections do not fit the rows")
    if cache.shape[-1] != Wc or not cache.is_contiguous() or any(t.dtype != qa.dtype for t in (q, kv, cache)):
        raise ValueError("latent_rope: cache rows are [latent | rotated key] of the activation dtype")
    if not qa.is_cuda:
        def rot(x):  # [T, ..., dr]
            if not half:
                return x
            ang = positions.to(torch.float32)[:, None] * inv_freq[None, :]
            shape = [T] + [1] * (x.dim() - 2) + [half]
            c, s_ = (torch.cos(ang) * mag).view(shape), (torch.sin(ang) * mag).view(shape)
            a_, b_ = x[..., :half], x[..., half:2 * half]
            return torch.cat([a_ * c - b_ * s_, b_ * c + a_ * s_, x[..., 2 * half:]], -1)

        kvf = kv.float()
        c = kvf[:, :r]
        c = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps) * norm_w
        row = torch.cat([c, rot(kvf[:, r:Wc])], -1).to(cache.dtype)
        ok = kv_slots >= 0
        cache[kv_slots[ok]] = row[ok]
        qr = torch.stack([q[:, h * q_head + q_off:h * q_head + q_off + dr] for h in range(H)], 1).float()
        out = torch.cat([qa.transpose(0, 1).float(), rot(qr)], -1).to(qa.dtype)
        return out.reshape(T, H * Wc)
    if positions.dtype != torch.int64 or kv_slots.dtype != torch.int64:
        raise TypeError("latent_rope: int64 positions and kv_slots")
    out = torch.empty((T, H * Wc), dtype=qa.dtype, device=qa.device)
    _m().latent_rope(out.data_ptr(), qa.data_ptr(), q.data_ptr(), q.stride(0), q_head, q_off, kv.data_ptr(),
                     kv.stride(0), norm_w.data_ptr(), float(eps), _ptr(inv_freq), half, float(mag),
                     positions.data_ptr(), kv_slots.data_ptr(), cache.data_ptr(), T, H, r, dr, _f32(qa), _stream())
    return out


# ----------------------------------------------------------------- short convolution + rotary + cache write
def conv_rope_cache(x: torch.Tensor, conv_w: torch.Tensor, conv_state: torch.Tensor, positions: torch.Tensor,
                    kv_slots: torch.Tensor, row_seq: torch.Tensor | None, seq_rows: torch.Tensor | None,
                    state_slots: torch.Tensor, n_q: int, n_k: int, d: int, dv: int, inv_freq: torch.Tensor | None,
                    kc: torch.Tensor | None, vc: torch.Tensor | None) -> torch.Tensor:
    """Per row of a fused projection x = [q (n_q d) | k (n_k d) | v (n_k dv) | ...]:
    every channel c of the C = n_q d + n_k (d + dv) leading columns is
    convolved over time, y_t = sum_j conv_w[j, c] u_(t - taps + 1 + j) (conv_w
    [taps, C] fp32, tap-major: the transpose of a checkpoint's [C, taps]), where u
    at a position before the step's first row of the sequence comes from
    conv_state [slots, taps - 1, C] (the last taps - 1 projected rows the
    sequence had before this step) and is zero before position 0.  Then the
    first 2 len(inv_freq) columns of every q and k head are rotated by the
    angles position * inv_freq, column i paired with column i + len(inv_freq).
    Returns q [T, n_q d]; k and v go to the paged caches kc [slots, n_k d],
    vc [slots, n_k dv] at kv_slots (rows with slot < 0 cache nothing; n_k = 0:
    no caches, a layer that reads another layer's).  conv_state is not changed
    (conv_state_update does that, after this)."""
    T = x.shape[0]
    taps, C = conv_w.shape
    n_seq = state_slots.numel()
    _fp32_param(conv_w, "conv_w")
    _fp32_param(inv_freq, "inv_freq")
    _check_step(positions, seq_rows, state_slots)
    half = 0 if inv_freq is None else inv_freq.numel()
    if C != n_q * d + n_k * (d + dv) or x.shape[1] < C or x.stride(1) != 1 or 2 * half > d or taps < 1:
        raise ValueError("conv_rope_cache: sections do not fit the row")
    if conv_state.shape[1:] != (taps - 1, C) or conv_state.dtype != x.dtype or not conv_state.is_contiguous():
        raise ValueError("conv_rope_cache: conv_state is [slots, taps - 1, C] of x's dtype")
    if n_k and (kc.shape[-1] != n_k * d or vc.shape[-1] != n_k * dv or kc.dtype != x.dtype or vc.dtype != x.dtype or
                not kc.is_contiguous() or not vc.is_contiguous()):
        raise ValueError("conv_rope_cache: cache row widths / dtype do not match the sections")
    if not x.is_cuda:
        y = torch.zeros((T, C), dtype=torch.float32)
        b = _seq_bounds(seq_rows, n_seq)
        for s in range(n_seq):
            r0, r1 = b[s], b[s + 1]
            sl = int(state_slots[s])
            if sl < 0 or r1 <= r0:
                continue
            p0 = int(positions[r0])
            hist = conv_state[sl].float().clone()  # positions p0 - taps + 1 .. p0 - 1
            for m in range(taps - 1):
                if p0 - (taps - 1) + m < 0:
                    hist[m] = 0.0
            u = torch.cat([hist, x[r0:r1, :C].float()], 0)
            for j in range(taps):
                y[r0:r1] += u[j:j + r1 - r0] * conv_w[j]
        qk = y[:, : (n_q + n_k) * d].reshape(T, n_q + n_k, d)
        if half:
            ang = positions.to(torch.float32)[:, None] * inv_freq[None, :]
            c, s_ = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
            a_, b_ = qk[..., :half].clone(), qk[..., half:2 * half].clone()
            qk[..., :half] = a_ * c - b_ * s_
            qk[..., half:2 * half] = b_ * c + a_ * s_
        qk = qk.reshape(T, (n_q + n_k) * d)
        if n_k:
            ok = kv_slots >= 0
            kc[kv_slots[ok]] = qk[ok, n_q * d:].to(kc.dtype)
            vc[kv_slots[ok]] = y[ok, (n_q + n_k) * d:].to(vc.dtype)
        return qk[:, : n_q * d].to(x.dtype).contiguous()
    if kv_slots.dtype != torch.int64 or (row_seq is not None and row_seq.dtype != torch.int32) or \
            ((row_seq is None) != (seq_rows is None)):
        raise TypeError("conv_rope_cache: int64 kv_slots, int32 row_seq together with seq_rows")
    q = torch.empty((T, n_q * d), dtype=x.dtype, device=x.device)
    _m().conv_rope_cache(q.data_ptr(), x.data_ptr(), x.stride(0), conv_w.data_ptr(), taps, conv_state.data_ptr(),
                         conv_state.shape[0], positions.data_ptr(), kv_slots.data_ptr(), _ptr(row_seq), _ptr(seq_rows),
                         state_slots.data_ptr(), n_seq, T, n_q, n_k, d, dv, _ptr(inv_freq), half, _ptr(kc), _ptr(vc),
                         _f32(x), _stream())
    return q


def conv_state_update(x: torch.Tensor, conv_state: torch.Tensor, positions: torch.Tensor,
                      seq_rows: torch.Tensor | None, state_slots: torch.Tensor) -> None:
    """After a step: conv_state [slots, taps - 1, C] of every sequence of the
    step becomes the last taps - 1 projected rows (the leading C columns of x)
    up to and including this step's; a step shorter than taps - 1 rows shifts
    the older ones down.  Entries that lie before position 0 are zero."""
    n_seq = state_slots.numel()
    m, C = conv_state.shape[1:]
    _check_step(positions, seq_rows, state_slots)
    if x.shape[1] < C or x.stride(1) != 1 or conv_state.dtype != x.dtype or not conv_state.is_contiguous():
        raise ValueError("conv_state_update: x covers the state's channels, in its dtype")
    if m == 0:
        return
    if not x.is_cuda:
        b = _seq_bounds(seq_rows, n_seq)
        for s in range(n_seq):
            r0, r1 = b[s], b[s + 1]
            sl = int(state_slots[s])
            if sl < 0 or r1 <= r0:
                continue
            p0 = int(positions[r0])
            old = conv_state[sl].clone()
            for i in range(m):
                if p0 - m + i < 0:
                    old[i] = 0
            conv_state[sl] = torch.cat([old, x[r0:r1, :C]], 0)[-m:]
        return
    _m().conv_state_update(conv_state.data_ptr(), conv_state.shape[0], x.data_ptr(), x.stride(0),
                           positions.data_ptr(), _ptr(seq_rows), state_slots.data_ptr(), n_seq, x.shape[0], C, m + 1,
                           _f32(x), _stream())


# ----------------------------------------------------------------- generalized delta rule
DELTA_DECAY_SCALE = math.exp(-0.5)


def delta_rule(r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a: torch.Tensor, w: torch.Tensor,
               a_bias: torch.Tensor | None, w_bias: torch.Tensor | None, state: torch.Tensor, positions: torch.Tensor,
               seq_rows: torch.Tensor | None, state_slots: torch.Tensor, n_heads: int, dk: int, dv: int,
               decay_scale: float = DELTA_DECAY_SCALE, key_eps: float = 1e-6) -> torch.Tensor:
    """The generalized delta rule over the rows of a step, per sequence and head
    from the sequence's state S [dk, dv] (fp32; stored column by column,
    state [slots, H, dv, dk] with state[s, h, j, i] = S[i, j], so that the
    kernel's threads, which own columns, read and write contiguous runs;
    updated in place):
        decay   w_t = exp(-decay_scale * sigmoid(w + w_bias))       per key channel
        removal a_t = sigmoid(a + a_bias)                           per key channel
        unit key u_t = k_t / sqrt(sum(k_t^2) + key_eps)
        S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T      (both terms read S_(t-1))
        o_t = S_t^T r_t
    r, k, a, w [T, H dk] and v [T, H dv] are column sections (contiguous rows,
    any row stride) of projection outputs.  Returns o [T, H dv] fp32.
    Everything but reading the inputs is fp32."""
    T = r.shape[0]
    n_seq = state_slots.numel()
    _fp32_param(a_bias, "a_bias")
    _fp32_param(w_bias, "w_bias")
    _check_step(positions, seq_rows, state_slots)
    for t, wd in ((r, dk), (k, dk), (a, dk), (w, dk), (v, dv)):
        if t.shape != (T, n_heads * wd) or t.stride(1) != 1 or t.dtype != r.dtype:
            raise ValueError("delta_rule: r, k, a, w [T, H dk] and v [T, H dv] with contiguous rows, one dtype")
    if state.shape[1:] != (n_heads, dv, dk) or state.dtype != torch.float32 or not state.is_contiguous():
        raise ValueError("delta_rule: state is contiguous float32 [slots, H, dv, dk]")
    if not r.is_cuda:
        out = torch.zeros((T, n_heads, dv), dtype=torch.float32)
        H = n_heads
        rf, kf, vf = r.float().view(T, H, dk), k.float().view(T, H, dk), v.float().view(T, H, dv)
        wf = torch.exp(-decay_scale * torch.sigmoid(w.float() + (w_bias if w_bias is not None else 0.0))).view(T, H, dk)
        af = torch.sigmoid(a.float() + (a_bias if a_bias is not None else 0.0)).view(T, H, dk)
        uf = kf * torch.rsqrt((kf * kf).sum(-1, keepdim=True) + key_eps)
        b = _seq_bounds(seq_rows, n_seq)
        for s in range(n_seq):
            r0, r1 = b[s], b[s + 1]
            sl = int(state_slots[s])
            if sl < 0 or r1 <= r0:
                continue
            S = state[sl].transpose(1, 2).clone() if int(positions[r0]) > 0 else \
                torch.zeros((H, dk, dv), dtype=torch.float32)
            for t in range(r0, r1):
                uS = torch.einsum("hi,hij->hj", uf[t], S)
                S = wf[t][:, :, None] * S - (af[t] * uf[t])[:, :, None] * uS[:, None, :] + \
                    kf[t][:, :, None] * vf[t][:, None, :]
                out[t] = torch.einsum("hi,hij->hj", rf[t], S)
            state[sl] = S.transpose(1, 2)
        return out.view(T, H * dv)
    out = torch.empty((T, n_heads * dv), dtype=torch.float32, device=r.device)
    # unit key, decay and removal rate * unit key of every row, formed by a pass of its own in front of the scan
    prep = torch.empty((T, n_heads, 3, dk), dtype=torch.float32, device=r.device)
    _m().delta_rule(out.data_ptr(), state.data_ptr(), state.shape[0], prep.data_ptr(), r.data_ptr(), r.stride(0), k.data_ptr(),
                    k.stride(0), v.data_ptr(), v.stride(0), a.data_ptr(), a.stride(0), w.data_ptr(), w.stride(0),
                    _ptr(a_bias), _ptr(w_bias), float(decay_scale), float(key_eps), positions.data_ptr(),
                    _ptr(seq_rows), state_slots.data_ptr(), n_seq, T, n_heads, dk, dv, _f32(r), _stream())
    return out


def retention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, k_scale: float,
              state: torch.Tensor, positions: torch.Tensor, seq_rows: torch.Tensor | None, state_slots: torch.Tensor,
              n_heads: int, dk: int, dv: int) -> torch.Tensor:
    """Retention (linear attention with a fixed decay per head, no softmax and
    no denominator) over the rows of a step, per sequence and head from the
    sequence's state S [dk, dv] (fp32; stored column by column, state
    [slots, H, dv, dk] with state[s, h, j, i] = S[i, j]; updated in place):
        S_t = decay[h] S_(t-1) + (k_scale k_t) v_t^T,     o_t = S_t^T q_t.
    q, k [T, H dk] and v [T, H dv] are column sections (contiguous rows, any
    row stride) of projection outputs; decay fp32 [H].  Returns o [T, H dv]
    fp32.  Everything but reading the inputs is fp32."""
    T = q.shape[0]
    n_seq = state_slots.numel()
    _fp32_param(decay, "decay")
    _check_step(positions, seq_rows, state_slots)
    for t, wd in ((q, dk), (k, dk), (v, dv)):
        if t.shape != (T, n_heads * wd) or t.stride(1) != 1 or t.dtype != q.dtype:
            raise ValueError("retention: q, k [T, H dk] and v [T, H dv] with contiguous rows, one dtype")
    if state.shape[1:] != (n_heads, dv, dk) or state.dtype != torch.float32 or not state.is_contiguous() or \
            decay.numel() != n_heads:
        raise ValueError("retention: state is contiguous float32 [slots, H, dv, dk], decay [H]")
    if not q.is_cuda:
        H = n_heads
        out = torch.zeros((T, H, dv), dtype=torch.float32)
        qf, kf, vf = q.float().view(T, H, dk), k.float().view(T, H, dk) * k_scale, v.float().view(T, H, dv)
        b = _seq_bounds(seq_rows, n_seq)
        for s in range(n_seq):
            r0, r1 = b[s], b[s + 1]
            sl = int(state_slots[s])
            if sl < 0 or r1 <= r0:
                continue
            S = state[sl].transpose(1, 2).clone() if int(positions[r0]) > 0 else \
                torch.zeros((H, dk, dv), dtype=torch.float32)
            for t in range(r0, r1):
                S = decay[:, None, None] * S + kf[t][:, :, None] * vf[t][:, None, :]
                out[t] = torch.einsum("hi,hij->hj", qf[t], S)
            state[sl] = S.transpose(1, 2)
        return out.view(T, H * dv)
    out = torch.empty((T, n_heads * dv), dtype=torch.float32, device=q.device)
    _m().retention(out.data_ptr(), state.data_ptr(), state.shape[0], q.data_ptr(), q.stride(0), k.data_ptr(),
                   k.stride(0), v.data_ptr(), v.stride(0), decay.data_ptr(), float(k_scale), positions.data_ptr(),
                   _ptr(seq_rows), state_slots.data_ptr(), n_seq, T, n_heads, dk, dv, _f32(q), _stream())
    return out


GATE_ACTS = {"sigmoid": 0, "silu": 1}


def head_norm_gate(o: torch.Tensor, n_heads: int, weight: torch.Tensor | None, gate: torch.Tensor | None, eps: float,
                   out_dtype: torch.dtype, gate_act: str = "sigmoid") -> torch.Tensor:
    """o [T, H dv] fp32 -> every head divided by its root mean square
    (sqrt(mean(o_h^2) + eps)), times weight [H dv] (fp32), times act(gate)
    (gate [T, H dv], a column section of the activation dtype; gate_act
    'sigmoid', or 'silu': z sigmoid(z)), in out_dtype."""
    if gate_act not in GATE_ACTS:
        raise ValueError(f"unknown gate activation {gate_act!r}")
    T, W = o.shape
    if o.dtype != torch.float32 or not o.is_contiguous() or W % n_heads:
        raise TypeError("head_norm_gate: o is contiguous float32 [T, H dv]")
    _fp32_param(weight, "weight")
    if gate is not None and (gate.shape != o.shape or gate.stride(1) != 1 or gate.dtype != out_dtype):
        raise ValueError("head_norm_gate: gate [T, H dv] of the output dtype with contiguous rows")
    if not o.is_cuda:
        oh = o.view(T, n_heads, W // n_heads)
        y = (oh * torch.rsqrt((oh * oh).mean(-1, keepdim=True) + eps)).reshape(T, W)
        if weight is not None:
            y = y * weight
        if gate is not None:
            g = gate.float()
            y = y * (torch.sigmoid(g) if gate_act == "sigmoid" else g * torch.sigmoid(g))
        return y.to(out_dtype)
    out = torch.empty((T, W), dtype=out_dtype, device=o.device)
    _m().head_norm_gate(out.data_ptr(), o.data_ptr(), _ptr(weight), _ptr(gate), gate.stride(0) if gate is not None else 0,
                        T, n_heads, W // n_heads, float(eps), GATE_ACTS[gate_act], int(out_dtype == torch.float32),
                        _stream())
    return out
