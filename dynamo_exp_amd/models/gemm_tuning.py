"""Decode-size GEMM selection shared by model classes: per batch size M and
projection shape, hipBLASLt against the launch configurations of the
hand-written small-M GEMMs (csrc/kernels/skinny_gemm.hip, dstream_gemm.hip),
timed over a model's own per-layer weights in turn (together they exceed the
Infinity Cache, so every call streams its weights from HBM as in a real step).
LlamaForCausalLM.tune_gemms follows the same procedure with its fused-partial
and SwiGLU variants on top; this is the plain form for models whose
projections all end in a stored [M, N] result.
"""
from __future__ import annotations

import os

import torch

from .. import ops


def _timed(fn, reps: int) -> float:
    fn()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    ev0.record()
    for _ in range(reps):
        fn()
    ev1.record()
    ev1.synchronize()
    return ev0.elapsed_time(ev1) * 1e3 / reps


@torch.no_grad()
def tune_small_m(groups: list[list[torch.Tensor]], sizes, plan: dict, tuned: set, min_gain: float = 0.03,
                 reps: int = 2) -> list[dict]:
    """groups: per projection, the bf16 weights [N, K] of all layers that have
    it.  Fills plan[(M, N, K)] = config where a hand kernel beats the library by
    min_gain, after a numerics check on the first and the last layer's weights.
    Returns the timings."""
    report = []
    if os.environ.get("DX_SKINNY", "1") == "0":
        return report
    for M in sorted(set(int(m) for m in sizes)):
        if not 1 <= M <= ops.SKINNY_MAX_M:
            continue
        for ws in groups:
            N, K = ws[0].shape
            key = (M, N, K)
            if key in tuned or ws[0].dtype != torch.bfloat16 or not ws[0].is_cuda:
                continue
            tuned.add(key)
            cfgs = [c for c in ops.skinny_configs(M, N, K) + ops.dstream_tune_configs(M, N, K)
                    if c[0] == ops.DSTREAM or not ((M <= 32 and c[1] == 64) or (c[0] == 128 and M <= 32))]
            row = {"key": key, "lib_us": None, "best_us": None, "cfg": None, "adopted": False}
            if cfgs:
                x = torch.randn(M, K, device=ws[0].device, dtype=torch.bfloat16)
                lib = _timed(lambda: [torch.matmul(x, w.t()) for w in ws], reps) / len(ws)
                best = None
                for cfg in cfgs:
                    try:
                        t = _timed(lambda: [ops.skinny_linear(x, w, cfg) for w in ws], reps) / len(ws)
                    except ValueError:  # a launch configuration that does not divide this N or K
                        continue
                    if best is None or t < best[0]:
                        best = (t, cfg)
                row.update(lib_us=round(lib, 2), best_us=round(best[0], 2) if best else None,
                           cfg=best[1] if best else None)
                if best is not None and best[0] < lib * (1 - min_gain):
                    for w in (ws[0], ws[-1]):
                        want = torch.matmul(x, w.t()).float()
                        got = ops.skinny_linear(x, w, best[1]).float()
                        err = ((got - want).abs().max() / want.abs().max().clamp_min(1e-6)).item()
                        if not err < 2e-2:
                            raise RuntimeError(f"small-M GEMM {best[1]} at {key}: relative error {err:.3g}")
                    plan[key] = best[1]
                    row["adopted"] = True
            report.append(row)
    return report


def planned_mm(plan: dict, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """x @ w.T on the kernel the plan holds for (M, N, K), else on the library."""
    M = x.shape[0]
    if plan and M <= ops.SKINNY_MAX_M:
        cfg = plan.get((M, w.shape[0], w.shape[1]))
        if cfg is not None and x.data_ptr() % 16 == 0 and x.stride(1) == 1 and x.stride(0) % 8 == 0:
            return ops.skinny_linear(x, w, cfg)
    return torch.matmul(x, w.t())
