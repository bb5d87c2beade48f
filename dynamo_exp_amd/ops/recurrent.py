"""Ops with per-sequence state: the generalized delta rule (a running matrix
per head), short causal convolutions over time fused with rotary positions and
the paged cache write, and the per-head unit-RMS + gate that follows a
recurrent mixer.

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


def head_norm_gate(o: torch.Tensor, n_heads: int, weight: torch.Tensor | None, gate: torch.Tensor | None, eps: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """o [T, H dv] fp32 -> every head divided by its root mean square
    (sqrt(mean(o_h^2) + eps)), times weight [H dv] (fp32), times sigmoid(gate)
    (gate [T, H dv], a column section of the activation dtype), in out_dtype."""
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
            y = y * torch.sigmoid(gate.float())
        return y.to(out_dtype)
    out = torch.empty((T, W), dtype=out_dtype, device=o.device)
    _m().head_norm_gate(out.data_ptr(), o.data_ptr(), _ptr(weight), _ptr(gate), gate.stride(0) if gate is not None else 0,
                        T, n_heads, W // n_heads, float(eps), int(out_dtype == torch.float32), _stream())
    return out
