"""Mixture-of-experts ops: routing, the per-step expert plan, grouped GEMMs over
the tokens of each expert, and the weighted combine.

GPU tensors run the gfx950 kernels of ``_C_mixers`` (csrc/mixers/moe.hip);
CPU tensors run the PyTorch forms below.  Nothing here reads a result back to
the host: expert counts stay on the device, so a step can be captured in a
HIP graph.

A step of T tokens that each use `top` experts has R = T * top slots; slot
t * top + k is token t's k-th choice.  `plan` sorts the slots by expert
(stable): `order` [R] lists slots expert by expert, `offsets` [E + 1] bounds
each expert's run of `order`.  Grouped GEMMs work on rows in that sorted
order.
"""
from __future__ import annotations

import torch

from .. import _native
from .mixers import _f32, _fp32_param, _ptr, _stream

ROUTER_SCORES = {"sigmoid": 0, "softmax": 1}
GROUP_SCORES = {"top2": 0, "max": 1}
GLU_BLOCK = 32  # rows per gate / up block of weights interleaved for the fused SwiGLU epilogue


def _m():
    return _native.mixers()


def route(z: torch.Tensor, correction: torch.Tensor | None, top: int, n_groups: int = 1, keep_groups: int = 1,
          score: str = "sigmoid", group_score: str = "top2") -> tuple[torch.Tensor, torch.Tensor]:
    """Expert choice per token from router logits z [T, E] (fp32).
    s = sigmoid(z), or softmax(z) over all experts (`score`); the choice score
    is s + correction (correction None: s); experts form n_groups equal groups
    of neighbours, a group's score is the sum of its two largest choice scores
    (of its one score when groups hold a single expert; group_score 'top2') or
    its largest ('max'), and only experts of the keep_groups best groups compete;
    the `top` largest choice scores among those win.  Returns (idx [T, top]
    int32, w [T, top] fp32) with w = s of the chosen (no correction, not
    renormalised), best choice first; ties go to the lower index."""
    T, E = z.shape
    if z.dtype != torch.float32 or not z.is_contiguous():
        raise TypeError("route: router logits are contiguous float32")
    _fp32_param(correction, "correction")
    if score not in ROUTER_SCORES or group_score not in GROUP_SCORES:
        raise ValueError(f"unknown router score {score!r} / group score {group_score!r}")
    if n_groups < 1 or E % n_groups or not 1 <= keep_groups <= n_groups or top < 1 or \
            top > keep_groups * (E // n_groups):
        raise ValueError("route: groups must divide the experts and hold at least `top` in those kept")
    if not z.is_cuda:
        s = torch.sigmoid(z) if score == "sigmoid" else torch.softmax(z, -1)
        c = s + correction if correction is not None else s.clone()
        if n_groups > 1:
            per = E // n_groups
            gs = c.view(T, n_groups, per).topk(min(2 if group_score == "top2" else 1, per), -1).values.sum(-1)
            kept = torch.zeros(T, n_groups, dtype=torch.bool)
            kept.scatter_(1, gs.topk(keep_groups, -1).indices, True)
            c = c.masked_fill(~kept[:, :, None].expand(T, n_groups, per).reshape(T, E), float("-inf"))
        idx = c.topk(top, -1).indices
        return idx.to(torch.int32), s.gather(1, idx)
    idx = torch.empty((T, top), dtype=torch.int32, device=z.device)
    w = torch.empty((T, top), dtype=torch.float32, device=z.device)
    _m().moe_route(idx.data_ptr(), w.data_ptr(), z.data_ptr(), _ptr(correction), T, E, top, n_groups, keep_groups,
                   ROUTER_SCORES[score], GROUP_SCORES[group_score], _stream())
    return idx, w


def plan(idx: torch.Tensor, n_experts: int) -> tuple[torch.Tensor, torch.Tensor]:
    """(order [R] int32, offsets [E + 1] int32) of a step's choices idx [T, top]:
    the slots sorted by expert, stable within an expert."""
    T, top = idx.shape
    R = T * top
    if idx.dtype != torch.int32 or not idx.is_contiguous():
        raise TypeError("plan: idx is contiguous int32")
    if not idx.is_cuda:
        flat = idx.reshape(-1).long()
        order = torch.sort(flat, stable=True).indices.to(torch.int32)
        counts = torch.bincount(flat, minlength=n_experts)
        offsets = torch.zeros(n_experts + 1, dtype=torch.int32)
        offsets[1:] = counts.cumsum(0)
        return order, offsets
    order = torch.empty(R, dtype=torch.int32, device=idx.device)
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=idx.device)
    _m().moe_plan(order.data_ptr(), offsets.data_ptr(), idx.data_ptr(), R, n_experts, _stream())
    return order, offsets


def tile_gemm_ok(a: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the 256 x 256-tile matrix-core GEMM (csrc/kernels/gemm256.hip, grouped
    mode) takes a [rows, K] against w [E, N, K]; the 64 x 64-tile kernel of
    csrc/mixers/moe.hip takes everything else."""
    E, N, K = w.shape
    return (a.is_cuda and a.dtype == torch.bfloat16 and N % 256 == 0 and K % 128 == 0 and a.stride(0) % 8 == 0
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and N * K < 2 ** 31
            and a.shape[0] * a.stride(0) < 2 ** 31)


def interleave_glu(w: torch.Tensor) -> torch.Tensor:
    """[E, 2F, K] = per expert [gate | up] rows -> blocks of GLU_BLOCK gate rows followed by
    their GLU_BLOCK up rows, the layout of the fused SwiGLU epilogue (F % GLU_BLOCK == 0)."""
    E, F2, K = w.shape
    F = F2 // 2
    if F % GLU_BLOCK:
        raise ValueError("interleave_glu: the expert width must be a multiple of the block")
    g, u = w[:, :F].view(E, F // GLU_BLOCK, GLU_BLOCK, K), w[:, F:].view(E, F // GLU_BLOCK, GLU_BLOCK, K)
    return torch.stack([g, u], 2).reshape(E, F2, K).contiguous()


def grouped_gemm(a: torch.Tensor, w: torch.Tensor, order: torch.Tensor, offsets: torch.Tensor, top: int,
                 gather: bool, scatter: bool, glu: bool = False) -> torch.Tensor:
    """Per expert e, the rows r of its run offsets[e] .. offsets[e + 1] times
    w[e]^T  (w [E, N, K], stored [out, in]).  Row r reads a[order[r] // top]
    when `gather` (a holds one row per token) and a[r] otherwise (a is already
    in sorted order); it is written to out[order[r]] when `scatter` (slot
    order) and to out[r] otherwise.  Products accumulate in fp32.
    `glu`: w holds gate and up rows interleaved (interleave_glu) and the result
    is silu(gate) * up, [R, N / 2], formed in the GEMM's epilogue; only where
    tile_gemm_ok (the caller keeps plain [gate | up] weights otherwise)."""
    E, N, K = w.shape
    R = order.shape[0]
    if a.dtype != w.dtype or a.shape[1] != K or a.stride(1) != 1 or not w.is_contiguous():
        raise TypeError("grouped_gemm: a [rows, K] and w [E, N, K] of one dtype, contiguous rows")
    if (not gather and a.shape[0] != R) or (gather and a.shape[0] * top != R):
        raise ValueError("grouped_gemm: row count does not fit the plan")
    if not a.is_cuda:
        if glu:
            raise ValueError("grouped_gemm: the fused SwiGLU epilogue is a GPU path")
        out = torch.empty((R, N), dtype=a.dtype)
        o = order.long()
        off = offsets.tolist()
        for e in range(E):
            r = torch.arange(off[e], off[e + 1])
            if r.numel():
                src = a[o[r] // top] if gather else a[r]
                out[o[r] if scatter else r] = (src.float() @ w[e].float().t()).to(a.dtype)
        return out
    if order.dtype != torch.int32 or offsets.dtype != torch.int32 or offsets.numel() != E + 1:
        raise TypeError("grouped_gemm: int32 order and offsets [E + 1]")
    if glu and not tile_gemm_ok(a, w):
        raise ValueError("grouped_gemm: the fused SwiGLU epilogue needs tile_gemm_ok operands")
    out = torch.empty((R, N // 2 if glu else N), dtype=a.dtype, device=a.device)
    if tile_gemm_ok(a, w):
        _native.kernels().gemm256_grouped(out.data_ptr(), out.stride(0), a.data_ptr(), a.stride(0), a.shape[0],
                                          w.data_ptr(), order.data_ptr(), offsets.data_ptr(), R, E, N, K, top,
                                          int(gather), int(scatter), int(glu), 8, _stream())
        return out
    _m().grouped_gemm(out.data_ptr(), a.data_ptr(), a.stride(0), w.data_ptr(), order.data_ptr(), offsets.data_ptr(),
                      R, E, N, K, top, int(gather), int(scatter), _f32(a), _stream())
    return out


def combine(y: torch.Tensor, w: torch.Tensor, shared: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = sum_k w[t, k] * y[t * top + k] (+ shared[t]); y [T * top, W] in
    slot order, w [T, top] fp32; the sum is fp32, in the order of k."""
    T, top = w.shape
    W = y.shape[1]
    if y.shape[0] != T * top or not y.is_contiguous() or w.dtype != torch.float32 or not w.is_contiguous():
        raise TypeError("combine: y [T * top, W] contiguous, w [T, top] float32")
    if shared is not None and (shared.shape != (T, W) or shared.dtype != y.dtype or shared.stride(1) != 1):
        raise TypeError("combine: shared [T, W] of y's dtype")
    if not y.is_cuda:
        out = (y.view(T, top, W).float() * w[:, :, None]).sum(1)
        if shared is not None:
            out = out + shared.float()
        return out.to(y.dtype)
    out = torch.empty((T, W), dtype=y.dtype, device=y.device)
    _m().moe_combine(out.data_ptr(), y.data_ptr(), w.data_ptr(), _ptr(shared),
                     shared.stride(0) if shared is not None else 0, T, top, W, _f32(y), _stream())
    return out
