"""Ops of the layer-listed (hybrid) models: multi-stream residual steps, gated
feed-forward activations, per-head q/k preparation fused with the paged cache
write, masked paged attention over rows of mixed sequences, and the two-map
(differential) combine.

GPU tensors run the gfx950 kernels of ``_C_mixers`` (csrc/mixers); CPU tensors
run the PyTorch forms below (CPU CI of the engine).  A GPU call never falls
back.  Every op works on bf16 or fp32 activations; residual streams, norms,
scores and softmax weights are fp32 in both.

Layouts:
  * residual streams X [T, S, W] fp32, updated in place
  * paged caches, token-major: K [num_blocks * block_size, Wk], V likewise
    [.., Wv]; slot = block * block_size + offset
  * rows of one step: positions [T] int64, slots [T] int64 (-1: not cached),
    seq [T] int32 -> row of block_tables (None: row i is sequence i)
"""
from __future__ import annotations

import math

import torch

from .. import _native

MASKS = {"causal": 0, "window": 1, "chunk": 2}
ACTS = {"relu": 0, "silu": 1, "gelu_tanh": 2, "sigmoid": 3, "relu2": 4, "tanh": 5, "swiglu_clamp": 6}
WEIGHTS = {"softmax": 0, "sigmoid": 1}
NORMS = {None: 0, "rms": 1, "layer": 2}
MAX_STREAMS = 8
# row attention: aim for this many waves per launch, never split a row's keys
# into parts shorter than ROW_MIN_PART
ROW_TARGET_WAVES = 2048
ROW_MIN_PART = 128
# grouped decode kernel: one wave per workgroup, four workgroups resident per CU (LDS), so
# about 1024 waves fill the chip once; more parts only add merge work
GROUP_TARGET_WAVES = 1024


def _m():
    return _native.mixers()


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _f32(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return 1
    if t.dtype == torch.bfloat16:
        return 0
    raise TypeError(f"activations must be bfloat16 or float32, got {t.dtype}")


def _ptr(t: torch.Tensor | None) -> int:
    return 0 if t is None else t.data_ptr()


def _fp32_param(t: torch.Tensor | None, name: str):
    if t is not None and (t.dtype != torch.float32 or not t.is_contiguous()):
        raise TypeError(f"{name}: expected a contiguous float32 tensor")


# ----------------------------------------------------------------- residual streams
def embed_streams(ids: torch.Tensor, table: torch.Tensor, n_streams: int, pos_table: torch.Tensor | None = None,
                  positions: torch.Tensor | None = None, scale: float = 1.0,
                  out: torch.Tensor | None = None) -> torch.Tensor:
    """X [T, S, W] fp32 with every stream equal to table[ids] * scale, plus the
    learned position vector pos_table[positions] when a table of them is given
    (product and sum are formed in fp32).  out: a contiguous fp32 tensor of
    T * S * W elements to fill instead of a new one."""
    T = ids.shape[0]
    V, W = table.shape
    if pos_table is not None and (positions is None or pos_table.shape[1] != W or pos_table.dtype != table.dtype):
        raise ValueError("embed_streams: position table of the embedding's width and dtype, with positions")
    if not table.is_cuda:
        x = table[ids].float() * scale
        if pos_table is not None:
            x = x + pos_table[positions].float()
        x = x[:, None, :].repeat(1, n_streams, 1).contiguous()
        if out is None:
            return x
        out.view(T, n_streams, W).copy_(x)
        return out.view(T, n_streams, W)
    if out is not None and (out.dtype != torch.float32 or not out.is_contiguous() or out.numel() != T * n_streams * W):
        raise TypeError("embed_streams: out is contiguous float32 with T * S * W elements")
    X = out.view(T, n_streams, W) if out is not None else \
        torch.empty((T, n_streams, W), dtype=torch.float32, device=table.device)
    ids = ids if ids.dtype == torch.int64 else ids.long()
    if pos_table is not None and (positions.dtype != torch.int64 or not pos_table.is_contiguous()):
        raise TypeError("embed_streams: int64 positions, contiguous position table")
    _m().embed_streams(X.data_ptr(), table.data_ptr(), ids.data_ptr(), T, n_streams, W, V, _ptr(pos_table),
                       _ptr(positions) if pos_table is not None else 0,
                       pos_table.shape[0] if pos_table is not None else 0, float(scale), _f32(table), _stream())
    return X


def gather_rows(table: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """table[ids] in the table's dtype (rows outside the table read as zeros)."""
    if not table.is_cuda:
        return table[ids]
    T, (V, W) = ids.shape[0], table.shape
    out = torch.empty((T, W), dtype=table.dtype, device=table.device)
    ids = ids if ids.dtype == torch.int64 else ids.long()
    _m().gather_rows(out.data_ptr(), table.data_ptr(), ids.data_ptr(), T, W, V, _f32(table), _stream())
    return out


def residual_step(X: torch.Tensor, a: torch.Tensor | None = None, b: torch.Tensor | None = None,
                  c: torch.Tensor | None = None, c_w: torch.Tensor | None = None, eps: float = 1e-6,
                  norm: str | None = None, norm_w: torch.Tensor | None = None, norm_b: torch.Tensor | None = None,
                  out_dtype: torch.dtype = torch.bfloat16, want_cast: bool = False,
                  c_gate: torch.Tensor | None = None, c_gate_b: torch.Tensor | None = None):
    """One step of a single fp32 residual X [T, W], in place:
        X <- X + a + b + c / sqrt(mean(c^2) + eps) * c_w        (each addend optional)
    with c_gate [T, W] (a column section, of the activation dtype) c is first
    multiplied by sigmoid(c_gate + c_gate_b), in fp32: a sublayer result gated
    element by element before it is normed into the residual;
    then, returned as (normed, cast):
        normed = norm(X) in out_dtype: 'rms'  X / sqrt(mean(X^2) + eps) * norm_w,
                                       'layer' (X - mean) / sqrt(var + eps) * norm_w + norm_b, None: nothing;
        cast   = X in out_dtype when want_cast.
    Sums, means and variances are fp32.  a and b are the outputs of sublayers that
    read the same normed input (a parallel block); c is an addend that enters
    with unit RMS and a learned per-column weight."""
    T, W = X.shape
    if X.dtype != torch.float32 or not X.is_contiguous():
        raise TypeError("the residual must be contiguous float32")
    if norm not in NORMS or (norm and norm_w is None) or (norm == "layer" and norm_b is None) or \
            (c is not None and c_w is None):
        raise ValueError("residual_step: bad norm / weights")
    if c_gate is not None and c is None:
        raise ValueError("residual_step: a gate needs the addend c")
    for t, n in ((c_w, "c_w"), (norm_w, "norm_w"), (norm_b, "norm_b"), (c_gate_b, "c_gate_b")):
        _fp32_param(t, n)
    for t in (a, b, c, c_gate):
        if t is not None and (t.shape != X.shape or t.stride(-1) != 1 or t.dtype != out_dtype):
            raise TypeError("residual_step: addends [T, W] with contiguous rows, of the activation dtype")
    if not X.is_cuda:
        for t in (a, b):
            if t is not None:
                X += t.float()
        if c is not None:
            cf = c.float()
            if c_gate is not None:
                cf = cf * torch.sigmoid(c_gate.float() + (c_gate_b if c_gate_b is not None else 0.0))
            X += cf * torch.rsqrt((cf * cf).mean(-1, keepdim=True) + eps) * c_w
        h = None
        if norm == "rms":
            h = (X * torch.rsqrt((X * X).mean(-1, keepdim=True) + eps) * norm_w).to(out_dtype)
        elif norm == "layer":
            mu = X.mean(-1, keepdim=True)
            var = ((X - mu) ** 2).mean(-1, keepdim=True)
            h = ((X - mu) * torch.rsqrt(var + eps) * norm_w + norm_b).to(out_dtype)
        return h, (X.to(out_dtype) if want_cast else None)
    h = torch.empty((T, W), dtype=out_dtype, device=X.device) if norm else None
    xc = torch.empty((T, W), dtype=out_dtype, device=X.device) if want_cast else None
    _m().residual_step(X.data_ptr(), _ptr(a), a.stride(0) if a is not None else 0, _ptr(b),
                       b.stride(0) if b is not None else 0, _ptr(c), c.stride(0) if c is not None else 0, _ptr(c_w),
                       _ptr(c_gate), c_gate.stride(0) if c_gate is not None else 0, _ptr(c_gate_b), float(eps), NORMS[norm], _ptr(norm_w), _ptr(norm_b), _ptr(h), _ptr(xc), T, W,
                       int(out_dtype == torch.float32), _stream())
    return h, xc


def stream_step(X: torch.Tensor, y: torch.Tensor | None, mix: torch.Tensor | None, gain: torch.Tensor | None,
                rin: torch.Tensor | None, norm_w: torch.Tensor | None, eps: float,
                out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor | None:
    """One residual step over S streams, in place on X [T, S, W] (fp32):
    with y [T, W]:  X_t <- sum_s mix[s, t] X_s + gain[t] y   (all t from the old X);
    with rin [S]:   returns norm(sum_s rin[s] X_s) * norm_w  (norm_w None: the plain sum).
    S = 1 with mix = gain = rin = 1 is the ordinary pre-norm residual."""
    T, S, W = X.shape
    if X.dtype != torch.float32 or not X.is_contiguous():
        raise TypeError("residual streams must be contiguous float32")
    if S > MAX_STREAMS:
        raise ValueError(f"{S} residual streams (kernel limit {MAX_STREAMS})")
    for t, n in ((mix, "mix"), (gain, "gain"), (rin, "rin"), (norm_w, "norm_w")):
        _fp32_param(t, n)
    if not X.is_cuda:
        if y is not None:
            X.copy_(torch.einsum("st,nsw->ntw", mix, X) + gain[None, :, None] * y.float()[:, None, :])
        if rin is None:
            return None
        u = torch.einsum("s,nsw->nw", rin, X)
        if norm_w is not None:
            u = u * torch.rsqrt((u * u).mean(-1, keepdim=True) + eps) * norm_w
        return u.to(out_dtype)
    out = torch.empty((T, W), dtype=out_dtype, device=X.device) if rin is not None else None
    if y is not None:
        if y.dtype != out_dtype and out is not None:
            raise TypeError("y and the output share one activation dtype")
        if y.stride(-1) != 1:
            raise ValueError("y: last dim must be contiguous")
    f32 = _f32(y) if y is not None else int(out_dtype == torch.float32)
    _m().stream_step(X.data_ptr(), _ptr(y), y.stride(0) if y is not None else 0, _ptr(mix), _ptr(gain), _ptr(rin),
                     _ptr(norm_w), float(eps), _ptr(out), W, T, S, W, f32, _stream())
    return out


def section_norm(x: torch.Tensor, weight: torch.Tensor | None, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * weight over a column section x [T, n] of
    wider rows (contiguous rows, any row stride), e.g. a low-rank latent inside
    a fused projection's output; fp32 sums, result [T, n] in x's dtype."""
    T, n = x.shape
    _fp32_param(weight, "weight")
    if x.stride(1) != 1 or (weight is not None and weight.numel() != n):
        raise ValueError("section_norm: rows contiguous, one weight per column")
    if not x.is_cuda:
        xf = x.float()
        y = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps)
        return (y * weight if weight is not None else y).to(x.dtype)
    out = torch.empty((T, n), dtype=x.dtype, device=x.device)
    _m().section_norm(out.data_ptr(), x.data_ptr(), x.stride(0), _ptr(weight), T, n, float(eps), _f32(x), _stream())
    return out


def depth_mix(stack: torch.Tensor, n: int, weights: torch.Tensor, dst: torch.Tensor | None = None,
              rows: torch.Tensor | None = None, norm_w: torch.Tensor | None = None, eps: float = 1e-6,
              out_dtype: torch.dtype = torch.bfloat16, c: torch.Tensor | None = None,
              c_w: torch.Tensor | None = None):
    """A weighted sum over depth: stack [>= n, T, W] fp32 holds one [T, W]
    plane per layer result (plane 0 the embedding output);
        x[r] = sum_{j < n} weights[j] * stack[j, rows[r]]        (rows None: every row)
    in fp32, summed in the order j = 0, 1, ....  x is written to dst (fp32
    [len(rows) or T, W]; a later plane of the stack is the usual choice, so the
    next layer updates it in place into its own result) and returned together
    with norm(x) = x / sqrt(mean(x^2) + eps) * norm_w in out_dtype (None without
    norm_w).  With c [T, W] (the last sublayer's output, of out_dtype) the newest
    plane first takes its closing addend, stack[n - 1] += c / sqrt(mean(c^2) +
    eps) * c_w: the residual step that ends a layer, in the same pass.  With
    `rows` the plane itself is left as it was (only the sum uses the addend)."""
    if stack.dim() != 3 or stack.dtype != torch.float32 or not stack.is_contiguous() or not 1 <= n <= stack.shape[0]:
        raise TypeError("depth_mix: stack is contiguous float32 [planes, T, W] with n <= planes")
    _, T, W = stack.shape
    _fp32_param(weights, "weights")
    _fp32_param(norm_w, "norm_w")
    _fp32_param(c_w, "c_w")
    if weights.numel() != n or (norm_w is not None and norm_w.numel() != W):
        raise ValueError("depth_mix: one weight per plane, one norm weight per column")
    if c is not None and (c_w is None or c_w.numel() != W or c.shape != (T, W) or c.stride(1) != 1 or
                          c.dtype != out_dtype):
        raise ValueError("depth_mix: the addend is [T, W] of the activation dtype with a weight per column")
    R = T if rows is None else rows.numel()
    if dst is None:
        dst = torch.empty((R, W), dtype=torch.float32, device=stack.device)
    if dst.shape != (R, W) or dst.dtype != torch.float32 or not dst.is_contiguous():
        raise TypeError("depth_mix: dst is contiguous float32 [rows, W]")
    if not stack.is_cuda:
        last = stack[n - 1]
        if c is not None:
            cf = c.float()
            last = last + cf * torch.rsqrt((cf * cf).mean(-1, keepdim=True) + eps) * c_w
            if rows is None:
                stack[n - 1] = last
        planes = [stack[j] for j in range(n - 1)] + [last]
        x = torch.zeros((R, W), dtype=torch.float32)
        for j in range(n):
            x += weights[j] * (planes[j] if rows is None else planes[j][rows.long()])
        dst.copy_(x)
        h = None
        if norm_w is not None:
            h = (x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * norm_w).to(out_dtype)
        return dst, h
    if rows is not None and (rows.dtype != torch.int64 or not rows.is_contiguous()):
        raise TypeError("depth_mix: rows must be contiguous int64")
    h = torch.empty((R, W), dtype=out_dtype, device=stack.device) if norm_w is not None else None
    _m().depth_mix(dst.data_ptr(), stack.data_ptr(), T * W, n, weights.data_ptr(), _ptr(rows), R, float(eps),
                   _ptr(norm_w), _ptr(h), _ptr(c), c.stride(0) if c is not None else 0, _ptr(c_w), W,
                   int(out_dtype == torch.float32), _stream())
    return dst, h


# ----------------------------------------------------------------- feed-forward
def _act(z: torch.Tensor, act: str) -> torch.Tensor:
    if act == "relu":
        return torch.relu(z)
    if act == "silu":
        return z * torch.sigmoid(z)
    if act == "sigmoid":
        return torch.sigmoid(z)
    if act == "relu2":
        return torch.relu(z) ** 2
    if act == "tanh":
        return torch.tanh(z)
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def glu_act(gu: torch.Tensor, act: str = "relu", limit: float = 0.0, alpha: float = 1.0) -> torch.Tensor:
    """[T, 2F] = [gate | up] -> act(gate) * up, [T, F] (act_mul on the two halves)."""
    F = gu.shape[1] // 2
    return act_mul(gu[:, :F], gu[:, F:], act, limit, alpha)


def act_mul(gate: torch.Tensor, up: torch.Tensor | None = None, act: str = "silu", limit: float = 0.0,
            alpha: float = 1.0) -> torch.Tensor:
    """act(gate) * up, [T, F] (up None: the activation alone).  gate and up may
    be column sections of wider tensors (contiguous rows, any row stride), e.g.
    a gate that is part of a fused projection's output.
    'swiglu_clamp' is the clamped gated unit: with g = min(gate, limit) and
    u = clamp(up, -limit, limit) the result is g * sigmoid(alpha * g) * (u + 1)."""
    T, F = gate.shape
    if act not in ACTS:
        raise ValueError(f"unknown activation {act!r}")
    if gate.stride(1) != 1 or (up is not None and (up.shape != gate.shape or up.stride(1) != 1 or
                                                   up.dtype != gate.dtype)):
        raise ValueError("act_mul: [T, F] sections with contiguous rows and one dtype")
    if act == "swiglu_clamp" and (up is None or not limit > 0):
        raise ValueError("act_mul: the clamped gated unit needs `up` and a positive limit")
    if not gate.is_cuda:
        if act == "swiglu_clamp":
            g, u = gate.float().clamp(max=limit), up.float().clamp(-limit, limit)
            return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(gate.dtype)
        o = _act(gate.float(), act)
        return (o * up.float() if up is not None else o).to(gate.dtype)
    out = torch.empty((T, F), dtype=gate.dtype, device=gate.device)
    _m().act_mul(out.data_ptr(), gate.data_ptr(), gate.stride(0), _ptr(up), up.stride(0) if up is not None else 0, T, F,
                 F, ACTS[act], float(limit), float(alpha), _f32(gate), _stream())
    return out


# ----------------------------------------------------------------- q/k preparation + cache write
def headprep_cache(x: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor, n_q: int, n_k: int, d: int,
                   k_off: int, q_w: torch.Tensor | None, k_w: torch.Tensor | None, eps: float,
                   temp: tuple[float, float] | None, kc: torch.Tensor, vc: torch.Tensor | None, v_mode: int = 0,
                   v_off: int = 0, v_w: int = 0, v_first: torch.Tensor | None = None, v_lambda: float = 0.0) -> None:
    """Per row of the fused projection output x = [q | k | v] (in place):
    q heads: unit RMS times q_w (when given) and the position gain
    1 + coef * ln(floor((p + 1) / every) + 1) (temp = (coef, every));
    k heads at column k_off: unit RMS times k_w (when given) into the K cache;
    v_mode 0: no V cache; 1: the k columns as projected are the value;
    2: the v_w columns at v_off are.  With v_first [T, v_w] (v_mode 2; the same
    tokens' values of an earlier layer, a column section of any row stride) the
    cached value is (1 - v_lambda) v + v_lambda v_first, formed in fp32.
    Rows with slot < 0 cache nothing."""
    T = x.shape[0]
    coef, every = (float(temp[0]), float(temp[1])) if temp else (0.0, 1.0)
    _fp32_param(q_w, "q_w")
    _fp32_param(k_w, "k_w")
    if x.stride(-1) != 1 or kc.dtype != x.dtype or not kc.is_contiguous():
        raise ValueError("headprep_cache: x rows contiguous, caches contiguous and of x's dtype")
    k_wd = n_k * d
    if kc.shape[-1] != k_wd or (v_mode == 1 and vc.shape[-1] != k_wd) or (v_mode == 2 and vc.shape[-1] != v_w):
        raise ValueError("headprep_cache: cache row widths do not match the sections")
    if max(n_q * d, k_off + k_wd, (v_off + v_w) if v_mode == 2 else 0) > x.shape[1]:
        raise ValueError("headprep_cache: sections exceed the row")
    if v_first is not None and (v_mode != 2 or v_first.shape != (T, v_w) or v_first.stride(1) != 1 or
                                v_first.dtype != x.dtype):
        raise ValueError("headprep_cache: v_first is [T, v_w] of x's dtype, with v_mode 2")
    if not x.is_cuda:
        xf = x.float()
        if q_w is not None or coef != 0.0:
            q = xf[:, : n_q * d].reshape(T, n_q, d)
            if q_w is not None:
                q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * q_w
            if coef != 0.0:
                k_ = torch.floor((positions.double() + 1.0) / every).float()
                q = q * (1.0 + coef * torch.log(k_ + 1.0))[:, None, None]
            x[:, : n_q * d] = q.reshape(T, n_q * d).to(x.dtype)
        ok = slots >= 0
        sl = slots[ok]
        k = xf[ok, k_off:k_off + k_wd]
        if v_mode == 1:
            vc[sl] = x[ok, k_off:k_off + k_wd]
        if k_w is not None:
            kh = k.reshape(-1, n_k, d)
            k = (kh * torch.rsqrt((kh * kh).mean(-1, keepdim=True) + eps) * k_w).reshape(-1, k_wd)
        kc[sl] = k.to(kc.dtype)
        if v_mode == 2:
            v = x[ok, v_off:v_off + v_w]
            if v_first is not None:
                v = ((1.0 - v_lambda) * v.float() + v_lambda * v_first[ok].float()).to(x.dtype)
            vc[sl] = v
        return
    if positions.dtype != torch.int64 or slots.dtype != torch.int64:
        raise TypeError("positions and slots must be int64")
    _m().headprep_cache(x.data_ptr(), x.stride(0), positions.data_ptr(), slots.data_ptr(), T, n_q, n_k, d, k_off,
                        _ptr(q_w), _ptr(k_w), float(eps), coef, every, kc.data_ptr(), _ptr(vc) if v_mode else 0,
                        v_mode, v_off, v_w, _ptr(v_first), v_first.stride(0) if v_first is not None else 0,
                        float(v_lambda), _f32(x), _stream())


# ----------------------------------------------------------------- attention
def row_attention_parts(rows: int, n_qh: int, max_visible: int, target: int = ROW_TARGET_WAVES) -> int:
    """Key partitions per row so a launch has about `target` waves (n_qh: the
    independent units per row -- query heads for the row kernel, K heads for
    the grouped decode kernel, whose target is GROUP_TARGET_WAVES)."""
    if rows <= 0:
        return 1
    want = -(-target // (rows * n_qh))
    return max(1, min(want, max_visible // ROW_MIN_PART))


def first_visible(p: torch.Tensor, mask: str, size: int) -> torch.Tensor:
    if mask == "window":
        return (p - size + 1).clamp_min(0)
    if mask == "chunk":
        return torch.div(p, size, rounding_mode="floor") * size
    return torch.zeros_like(p)


TILE_ROWS = 128  # rows of one sequence per tile_attention workgroup


def tile_list(row0: int, n: int) -> list[tuple[int, int]]:
    """(first row, row count) tiles of a prompt chunk of n rows starting at stream row row0."""
    return [(row0 + t, min(TILE_ROWS, n - t)) for t in range(0, n, TILE_ROWS)]


def tile_attention_ok(q: torch.Tensor, d: int, dv: int) -> bool:
    """Whether the matrix-core prefill kernel serves these rows (bf16 on the
    GPU, head widths it is instantiated for); otherwise row_attention does."""
    return q.is_cuda and q.dtype == torch.bfloat16 and bool(_m().tile_attention_ok(d, dv))


def attention(q: torch.Tensor, kc: torch.Tensor, vc: torch.Tensor, positions: torch.Tensor,
              seq: torch.Tensor | None, block_tables: torch.Tensor, block_size: int, n_qh: int, maps: int,
              group: int, d: int, dv: int, scale: float, mask: str = "causal", size: int = 0, parts: int = 1,
              out_f32: bool = False, tiles: torch.Tensor | None = None, n_tile_rows: int = 0, softcap: float = 0.0,
              dist_bias: tuple[torch.Tensor, torch.Tensor] | None = None, weights: str = "softmax",
              head_bias: torch.Tensor | None = None, head_gate: torch.Tensor | None = None, keep_first: int = 0,
              sink: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of one step's rows: the first n_tile_rows rows (prompt chunks,
    cut into `tiles` [n, 2] = first row, row count) on the matrix-core prefill
    kernel where it applies, all other rows (decode tokens; every row when it
    does not apply) on the row kernel.  Same arguments and result as
    row_attention."""
    T = q.shape[0]
    if not tile_attention_ok(q, d, dv) or not scale > 0:  # the matrix-core kernels fold a positive scale
        return row_attention(q, kc, vc, positions, seq, block_tables, block_size, n_qh, maps, group, d, dv, scale,
                             mask, size, parts, out_f32, softcap, dist_bias, weights, head_bias, head_gate, keep_first,
                             sink)
    _check_score_terms(softcap, dist_bias, n_qh)
    _check_weight_terms(weights, head_bias, head_gate, q, n_qh, maps)
    _check_mask_terms(mask, keep_first, sink, weights, n_qh)
    if tiles is None:
        n_tile_rows = 0
    if kc.dtype != q.dtype or vc.dtype != q.dtype or not kc.is_contiguous() or not vc.is_contiguous() or \
            q.stride(1) != 1 or (seq is not None and seq.dtype != torch.int32) or positions.dtype != torch.int64 or \
            block_tables.dtype != torch.int32 or block_tables.stride(1) != 1:
        raise TypeError("attention: bf16 caches, int32 seq / block_tables / tiles, int64 positions")
    if n_qh % maps or (n_qh // maps) % group or mask not in MASKS or (mask != "causal" and size < 1):
        raise ValueError("attention: bad head counts or mask")
    if q.shape[1] < n_qh * d or kc.shape[-1] < n_qh // group * d or vc.shape[-1] < n_qh // maps // group * dv:
        raise ValueError("attention: widths do not cover the heads")
    if seq is None and block_tables.shape[0] < T:
        raise ValueError("attention: fewer block-table rows than rows")
    odt = torch.float32 if out_f32 else q.dtype
    out = torch.empty((T, n_qh, dv), dtype=odt, device=q.device)
    common = (block_tables.data_ptr(), block_tables.stride(0), block_size)
    heads = (n_qh, maps, group, d, dv, kc.shape[-1], vc.shape[-1], float(scale), MASKS[mask], int(size),
             float(softcap), _ptr(dist_bias[0]) if dist_bias else 0, _ptr(dist_bias[1]) if dist_bias else 0,
             WEIGHTS[weights], _ptr(head_bias))
    gs = head_gate.stride(0) if head_gate is not None else 0
    if n_tile_rows:
        if seq is None or tiles.dtype != torch.int32 or not tiles.is_contiguous():
            raise TypeError("attention: prompt-chunk rows need seq and int32 tiles")
        _m().tile_attention(out.data_ptr(), q.data_ptr(), q.stride(0), kc.data_ptr(), vc.data_ptr(),
                            positions.data_ptr(), seq.data_ptr(), *common, tiles.data_ptr(), tiles.shape[0], *heads,
                            _ptr(head_gate), gs, int(keep_first), _ptr(sink), int(out_f32), _stream())
    n_dec = T - n_tile_rows
    if n_dec:  # decode rows: the heads of a K/V group share one wave's key tiles
        r0 = n_tile_rows
        ws = torch.empty((n_dec, n_qh, parts, 2 + dv), dtype=torch.float32, device=q.device)
        _m().group_decode(out[r0:].data_ptr(), ws.data_ptr(), q[r0:].data_ptr(), q.stride(0), kc.data_ptr(),
                          vc.data_ptr(), positions[r0:].data_ptr(), _ptr(seq[r0:] if seq is not None else None),
                          *common, n_dec, *heads, _ptr(head_gate[r0:]) if head_gate is not None else 0, gs,
                          int(keep_first), _ptr(sink), parts, int(out_f32), _stream())
    return out


def _check_score_terms(softcap: float, dist_bias, n_qh: int) -> None:
    if softcap < 0:
        raise ValueError("softcap must be positive (0: none)")
    if dist_bias is not None:
        for t in dist_bias:
            _fp32_param(t, "dist_bias")
            if t.numel() != n_qh:
                raise ValueError("dist_bias: one (r1, r2) pair per query vector")


def _check_mask_terms(mask: str, keep_first: int, sink, weights: str, n_qh: int) -> None:
    if keep_first < 0 or (keep_first and mask != "window"):
        raise ValueError("keep_first: a count of first keys that a window mask keeps visible")
    _fp32_param(sink, "sink")
    if sink is not None and (sink.numel() != n_qh or weights != "softmax"):
        raise ValueError("sink: one number per query vector, with softmax weights")


def _check_weight_terms(weights: str, head_bias, head_gate, q: torch.Tensor, n_qh: int, maps: int) -> None:
    if weights not in WEIGHTS:
        raise ValueError(f"unknown attention weights {weights!r}")
    _fp32_param(head_bias, "head_bias")
    if head_bias is not None and head_bias.numel() != n_qh:
        raise ValueError("head_bias: one number per query vector")
    if head_gate is not None and (head_gate.shape != (q.shape[0], n_qh // maps) or head_gate.stride(1) != 1 or
                                  head_gate.dtype != q.dtype):
        raise ValueError("head_gate: [T, heads] of q's dtype with contiguous rows")


def row_attention(q: torch.Tensor, kc: torch.Tensor, vc: torch.Tensor, positions: torch.Tensor,
                  seq: torch.Tensor | None, block_tables: torch.Tensor, block_size: int, n_qh: int, maps: int,
                  group: int, d: int, dv: int, scale: float, mask: str = "causal", size: int = 0, parts: int = 1,
                  out_f32: bool = False, softcap: float = 0.0,
                  dist_bias: tuple[torch.Tensor, torch.Tensor] | None = None, weights: str = "softmax",
                  head_bias: torch.Tensor | None = None, head_gate: torch.Tensor | None = None, keep_first: int = 0,
                  sink: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of T rows over their sequences' paged caches.
    q [T, >= n_qh * d] (n_qh = heads * maps query vectors per row); returns
    [T, n_qh, dv].  Query vector qh reads K head (qh // maps // group) * maps +
    qh % maps and V head qh // maps // group.  The score of query position i
    and key position j is s = q . k * scale; with softcap > 0 then
    s <- softcap * tanh(s / softcap); with dist_bias = (r1, r2), fp32 [n_qh]
    each, then s <- s - r1[qh] * ln(1 + r2[qh] * (i - j)); with head_bias
    (fp32 [n_qh]) then s <- s + head_bias[qh].  weights 'softmax': the visible
    keys' weights are softmax(s); 'sigmoid': every visible key weighs
    sigmoid(s), not normalised over the keys.  With head_gate [T, heads]
    (logits, a column section) head h's result is multiplied by
    sigmoid(head_gate[:, h]).  Masks: 'causal' j <= i; 'window' also
    i - j < size, or j < keep_first (the sequence's first keep_first keys stay
    visible at their true positions); 'chunk' floor(j / size) = floor(i / size).
    With sink (fp32 [n_qh]) the softmax denominator also holds exp(sink[qh]):
    a key without a value, neither scaled nor masked, counted once."""
    T = q.shape[0]
    _check_score_terms(softcap, dist_bias, n_qh)
    _check_weight_terms(weights, head_bias, head_gate, q, n_qh, maps)
    _check_mask_terms(mask, keep_first, sink, weights, n_qh)
    if mask not in MASKS:
        raise ValueError(f"unknown mask {mask!r}")
    if mask != "causal" and size < 1:
        raise ValueError("window / chunk masks need a size >= 1")
    if n_qh % maps or (n_qh // maps) % group:
        raise ValueError("head counts do not divide")
    n_kh = n_qh // maps // group * maps
    Wk, Wv = kc.shape[-1], vc.shape[-1]
    if Wk < n_kh * d or Wv < n_qh // maps // group * dv or q.shape[1] < n_qh * d:
        raise ValueError("row_attention: widths do not cover the heads")
    odt = torch.float32 if (out_f32 or q.dtype == torch.float32) else q.dtype
    if not q.is_cuda:
        out = torch.empty((T, n_qh, dv), dtype=torch.float32)
        sq = seq.long() if seq is not None else torch.arange(T)
        qf = q[:, : n_qh * d].float().reshape(T, n_qh, d)
        heads = torch.arange(n_qh) // maps
        kh = heads // group * maps + torch.arange(n_qh) % maps
        vh = heads // group
        for s in sq.unique().tolist():
            rows = (sq == s).nonzero().flatten()
            p = positions[rows].long()
            n = int(p.max()) + 1
            j = torch.arange(n)
            sl = block_tables[s].long()[j // block_size] * block_size + j % block_size
            K = kc[sl].float()[:, : n_kh * d].reshape(n, n_kh, d)[:, kh]  # [n, n_qh, d]
            V = vc[sl].float()[:, : (n_qh // maps // group) * dv].reshape(n, -1, dv)[:, vh]
            sc = torch.einsum("ihd,jhd->hij", qf[rows], K) * scale
            if softcap:
                sc = softcap * torch.tanh(sc / softcap)
            if dist_bias is not None:
                dist = (p[:, None] - j[None, :]).clamp_min(0).float()
                sc = sc - dist_bias[0][:, None, None] * torch.log1p(dist_bias[1][:, None, None] * dist[None])
            if head_bias is not None:
                sc = sc + head_bias[:, None, None]
            near = j[None, :] >= first_visible(p, mask, size)[:, None]
            if keep_first:
                near = near | (j[None, :] < keep_first)
            vis = (j[None, :] <= p[:, None]) & near
            sc = sc.masked_fill(~vis[None], float("-inf"))
            if weights == "softmax" and sink is not None:
                sc = torch.cat([sc, sink.view(n_qh, 1, 1).expand(n_qh, sc.shape[1], 1)], -1)
                wt = torch.softmax(sc, -1)[..., :n]
            else:
                wt = torch.softmax(sc, -1) if weights == "softmax" else torch.sigmoid(sc)
            out[rows] = torch.einsum("hij,jhd->ihd", wt, V)
        if head_gate is not None:
            out = out * torch.sigmoid(head_gate.float()).repeat_interleave(maps, 1)[:, :, None]
        return out.to(odt)
    if kc.dtype != q.dtype or vc.dtype != q.dtype or not kc.is_contiguous() or not vc.is_contiguous():
        raise TypeError("row_attention: caches contiguous and of q's dtype")
    if q.stride(1) != 1 or positions.dtype != torch.int64 or block_tables.dtype != torch.int32 or \
            (seq is not None and seq.dtype != torch.int32) or block_tables.stride(1) != 1:
        raise TypeError("row_attention: q rows contiguous, positions int64, seq / block_tables int32")
    if seq is None and block_tables.shape[0] < T:
        raise ValueError("row_attention: fewer block-table rows than rows")
    out = torch.empty((T, n_qh, dv), dtype=odt, device=q.device)
    ws = torch.empty((T, n_qh, parts, 2 + dv), dtype=torch.float32, device=q.device) if parts > 1 else None
    _m().row_attention(out.data_ptr(), _ptr(ws), q.data_ptr(), q.stride(0), kc.data_ptr(), vc.data_ptr(),
                       positions.data_ptr(), _ptr(seq), block_tables.data_ptr(), block_tables.stride(0), block_size,
                       T, n_qh, maps, group, d, dv, Wk, Wv, float(scale), MASKS[mask], int(size), float(softcap),
                       _ptr(dist_bias[0]) if dist_bias else 0, _ptr(dist_bias[1]) if dist_bias else 0,
                       WEIGHTS[weights], _ptr(head_bias), _ptr(head_gate),
                       head_gate.stride(0) if head_gate is not None else 0, int(keep_first), _ptr(sink), parts, _f32(q),
                       int(odt == torch.float32), _stream())
    return out


def diff_combine(a: torch.Tensor, lam: float, post: float, eps: float, out_dtype: torch.dtype,
                 head_gate: torch.Tensor | None = None) -> torch.Tensor:
    """a [T, H, 2, dv] fp32 (two maps' outputs) -> [T, H * dv]:
    unit_rms_over_dv(a1 - lam * a2) * post; with head_gate [T, H] (logits, a
    column section of out_dtype) head h is then multiplied by
    sigmoid(head_gate[:, h]) -- after the unit norm, which would cancel a gate
    applied to the maps."""
    T, H, two, dv = a.shape
    if two != 2 or a.dtype != torch.float32 or not a.is_contiguous():
        raise TypeError("diff_combine: a must be contiguous float32 [T, H, 2, dv]")
    if head_gate is not None and (head_gate.shape != (T, H) or head_gate.stride(1) != 1 or
                                  head_gate.dtype != out_dtype):
        raise ValueError("diff_combine: head_gate is [T, H] of the output dtype with contiguous rows")
    if not a.is_cuda:
        o = a[:, :, 0] - lam * a[:, :, 1]
        o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps) * post
        if head_gate is not None:
            o = o * torch.sigmoid(head_gate.float())[:, :, None]
        return o.reshape(T, H * dv).to(out_dtype)
    out = torch.empty((T, H * dv), dtype=out_dtype, device=a.device)
    _m().diff_combine(out.data_ptr(), a.data_ptr(), T * H, dv, float(lam), float(post), float(eps), _ptr(head_gate),
                      head_gate.stride(0) if head_gate is not None else 0, H, int(out_dtype == torch.float32),
                      _stream())
    return out
