"""Sobivik: a layer-listed hybrid decoder for the MI355X engine: differential
attention (a window that keeps a sequence's first tokens), retention (linear
attention with a fixed decay per head) and latent attention (low-rank queries
and keys/values, a rotated key part shared by all heads, a window and a
softmax sink), under sandwich norms with one scalar weight each, a short
causal convolution over time on every mixer's input, and a learned average
over the results of all earlier layers after every layer.

Per layer i, T rows of one engine step (prompt chunks and decode tokens of
different sequences; state per sequence in the slot the engine assigned).
The results of all layers live in one fp32 stack [layers + 1, T, W]; plane 0
is the embedding output and plane i + 1 starts as layer i's input (the depth
average of planes 0 .. i) and is updated in place into layer i's result:

  x, h = depth_mix(planes 0..i, dwa of layer i-1)          HIP  weighted sum over depth + rms(x) g1: one pass
  h    = h + conv(h)                                       HIP  conv_rope_cache (taps over time; tail state per slot)
  attention (differential)
    p  = h @ [Wq | Wk | Wv | Wg]^T                         hipBLASLt, one fused projection
         headprep_cache: K (two maps per head), V -> pages HIP
    a  = attention(q, K, V; maps = 2, window + kept first) HIP  tile kernel (prompt chunks) / grouped decode / row kernel
    ym = diff_combine(a1 - lambda a2, head gate) @ Wo^T    HIP  unit RMS, (1 - diff), sigmoid(g_h) per head
  retention
    p  = h @ [Wq | Wk | Wv | Wg]^T
    o  = retention(q, k d^-1/2, v; S)                      HIP  S <- decay_h S + k v^T, o = S^T q, fp32, token by token
    ym = head_norm_gate(o, silu(g)) @ Wo^T                 HIP
  latent_attention
    p  = h @ [Wdq | Wdkv | Wg]^T
    q  = section_norm(p_dq) @ Wuq^T                        HIP + hipBLASLt
    qa = q_unrotated @ Wuk (per head)                      batched GEMM: the key up-projection folded into the query
    q' = latent_rope(qa, q_rot; latent, key part -> pages) HIP  latent norm, rotary (scaled frequencies), cache row
                                                                [latent | rotated key], query rows [qa | rotated]
    a  = attention(q', C, C; one shared head, window, sink)
    ym = (a @ Wuv (per head) * sigmoid(p_g)) @ Wo^T        batched GEMM + HIP act_mul
  all
    x += rms(ym) g1b; h2 = rms(x) g2                       HIP  residual_step
    yf = ff(h2)                                            hipBLASLt + HIP glu_act (silu)
    x += rms(yf) g2b                                       joined with the next layer's depth_mix (or the final one,
                                                           on the chosen rows)

Norms, the residual and its depth average, scores and weights, decays and the
retention state, positions and angles are fp32; projections, the convolution
and activations are bf16 (dtype=bfloat16) or everything is fp32
(dtype=float32).
"""
from __future__ import annotations

import glob
import math
import os

import torch

from ..ops import mixers as mx
from ..ops import recurrent as rc
from .config import LayeredConfig
from .gemm_tuning import planned_mm, tune_small_m
from .llama import AttnMeta, TPGroup

MIXERS = ("attention", "retention", "latent_attention")
IN_PAD = 64  # fused in-projections that end in a narrow section (a gate per head) are padded with zero
#              rows to a multiple of this, the GEMM kernels' column tile


class SobivikForCausalLM:
    #: the runner builds per-row sequence ids and one block table over all rows of a step
    unified_rows = True
    #: the runner allocates per-sequence state (alloc_state) and names every sequence's slot
    state_slots = True

    def __init__(self, cfg: LayeredConfig, device: torch.device | str = "cuda", dtype=torch.bfloat16,
                 tp: TPGroup | None = None):
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.tp = tp or TPGroup()
        if self.tp.size != 1:
            raise ValueError("Sobivik runs on one GPU per engine (tensor parallel size 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"unsupported dtype {dtype}")
        if cfg.loop or cfg.streams:
            raise ValueError("Sobivik has neither a layer loop nor parallel residual streams")
        for i, L in enumerate(cfg.layers):
            m = L["mixer"]
            if L["type"] not in MIXERS:
                raise ValueError(f"unknown mixer type {L['type']!r}")
            if L.get("mlp") and L["mlp"].get("kind") != "dense":
                raise ValueError(f"unknown feed-forward kind {L['mlp'].get('kind')!r}")
            if L["type"] == "attention" and m["heads"] % m["kv_heads"]:
                raise ValueError(f"layer {i}: {m['heads']} heads over {m['kv_heads']} key/value heads")
            if L["type"] == "retention" and len(m["decay"]) != m["heads"]:
                raise ValueError(f"layer {i}: {len(m['decay'])} decays for {m['heads']} heads")
            if L["type"] == "latent_attention" and m.get("rot") and int(m["rot"]["dims"]) > m["rot_dim"]:
                raise ValueError(f"layer {i}: {m['rot']['dims']} rotated dimensions in a part of {m['rot_dim']}")
        self.taps = int((cfg.canon or {}).get("taps", 0))
        self.layers: list[dict] = []
        self.embed = self.head = self.final_w = None
        self.fp8 = False
        self.kv_scales = (1.0, 1.0)
        self.kv_amax = None
        self.layer_hook = None
        self.gemm_plan: dict = {}
        self.gemm_tuned: set = set()
        # debugging: when a list, forward() appends what goes on to the next layer after every layer
        self.trace_layers: list | None = None
        # per layer, the index of its convolution tail and of its retention matrix in the state list
        self._state_index: list[tuple[int | None, int | None]] = []
        self.state_shapes()

    # ------------------------------------------------------------------ engine hooks (no-ops here)
    def enable_fused_mlp(self) -> bool:
        return False

    def fold_norms(self) -> bool:
        return False

    #: dense projections of a layer, by the name of their weight
    LINEARS = ("w_in", "w_uq", "w_o", "w_gu", "w_down")

    def tune_gemms(self, sizes, **kw) -> list:
        """Decode batch sizes: the hand-written small-M GEMMs where they beat the
        library (bf16 on the GPU; models/gemm_tuning.py)."""
        if self.device.type != "cuda" or self.dtype != torch.bfloat16 or not self.layers:
            return []
        groups: dict = {}  # layers of different mixers have projections of different shapes
        for n in self.LINEARS:
            for L in self.layers:
                if L.get(n) is not None:
                    groups.setdefault((n, tuple(L[n].shape)), []).append(L[n])
        return tune_small_m(list(groups.values()), sizes, self.gemm_plan, self.gemm_tuned, **kw)

    def _mm(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        return planned_mm(self.gemm_plan, x, w)

    def tune_prefill_gemms(self, max_tokens, **kw) -> list:
        return []

    def quantize_fp8(self):
        raise ValueError("fp8 linears are not available for Sobivik")

    @torch.no_grad()
    def warmup_linears(self, tokens: int) -> None:
        seen = set()
        for L in self.layers:
            for name in self.LINEARS:
                w = L.get(name)
                if w is None or tuple(w.shape) in seen:
                    continue
                seen.add(tuple(w.shape))
                torch.matmul(torch.zeros(tokens, w.shape[1], device=self.device, dtype=self.dtype), w.t())

    def weight_bytes(self) -> int:
        ts = [t for L in self.layers for t in L.values() if isinstance(t, torch.Tensor)]
        ts += [t for t in (self.embed, self.head) if t is not None]
        return sum(t.numel() * t.element_size() for t in ts)

    # ------------------------------------------------------------------ paged caches and state slots
    def cache_widths(self) -> list[tuple[int, int] | None]:
        """(K row width, V row width) of every layer's paged cache: two key
        maps and one value per key/value head (differential attention), one
        [latent | rotated key] row that is key and value (V width 0), or none
        (retention)."""
        out = []
        for L in self.cfg.layers:
            m = L["mixer"]
            if L["type"] == "attention":
                out.append((m["kv_heads"] * 2 * m["dim"], m["kv_heads"] * m["vdim"]))
            elif L["type"] == "latent_attention":
                out.append((m["kv_rank"] + m["rot_dim"], 0))
            else:
                out.append(None)
        return out

    def kv_bytes_per_block(self, block_size: int, dtype: torch.dtype) -> int:
        es = torch.empty((), dtype=dtype).element_size()
        return sum((w[0] + w[1]) * block_size * es for w in self.cache_widths() if w)

    def alloc_kv_caches(self, num_blocks: int, block_size: int, dtype: torch.dtype) -> list[tuple]:
        """One (K, V) pair per layer, token-major [num_blocks * block_size,
        width], indexed by the engine's one block table; a latent layer's pair
        is the same tensor twice, a retention layer's an empty one.  Windowed
        layers keep every page of a live sequence; the mask alone bounds what
        is read."""
        if dtype != self.dtype:
            raise ValueError(f"the cache holds the model's activation dtype {self.dtype}, not {dtype}")
        out: list[tuple] = []
        for w in self.cache_widths():
            if not w:
                e = torch.empty((0, 0), dtype=dtype, device=self.device)
                out.append((e, e))
                continue
            k = torch.zeros((num_blocks * block_size, w[0]), dtype=dtype, device=self.device)
            v = torch.zeros((num_blocks * block_size, w[1]), dtype=dtype, device=self.device) if w[1] else k
            out.append((k, v))
        return out

    def state_shapes(self) -> list[tuple[tuple, torch.dtype]]:
        """Shape (without the slot dimension) and dtype of every per-sequence
        state tensor: per layer the last taps - 1 normed inputs in front of the
        input convolution, and per retention layer the running matrix of every
        head (fp32, stored column by column)."""
        out, index = [], []
        W = self.cfg.hidden_size
        for L in self.cfg.layers:
            m = L["mixer"]
            ci = ri = None
            if self.taps:
                ci = len(out)
                out.append(((max(0, self.taps - 1), W), self.dtype))
            if L["type"] == "retention":
                ri = len(out)
                out.append(((m["heads"], m["vdim"], m["dim"]), torch.float32))
            index.append((ci, ri))
        self._state_index = index
        return out

    def state_bytes_per_slot(self) -> int:
        return sum(math.prod(s) * torch.empty((), dtype=dt).element_size() for s, dt in self.state_shapes())

    def alloc_state(self, num_slots: int) -> list[torch.Tensor]:
        return [torch.zeros((num_slots, *s), dtype=dt, device=self.device) for s, dt in self.state_shapes()]

    # ------------------------------------------------------------------ weights
    def random_state(self, seed: int = 0) -> dict[str, torch.Tensor]:
        """Random weights in the checkpoint's naming and dtypes (bf16), scaled
        so activations stay O(1)."""
        cfg = self.cfg
        g = torch.Generator().manual_seed(seed)
        W = cfg.hidden_size

        def rnd(*shape, std):
            return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

        def num(mean, std):
            return (mean + torch.randn((), generator=g) * std).to(torch.bfloat16)

        sd = {"embed": rnd(cfg.vocab_size, W, std=1.0 / max(cfg.embedding_scale, 1e-6)), "final.norm": num(1.0, 0.1),
              "head": rnd(cfg.vocab_size, W, std=W ** -0.5)}
        for i, L in enumerate(cfg.layers):
            m, p, q = L["mixer"], f"l{i}.mix.", f"l{i}."
            for n in ("norm1", "norm2"):
                sd[q + n] = num(1.0, 0.1)
            for n in ("norm1b", "norm2b"):
                sd[q + n] = num(0.5, 0.1)
            if self.taps:
                sd[q + "canon1"] = rnd(W, self.taps, std=0.5 * self.taps ** -0.5)
            sd[q + "dwa"] = (torch.cat([torch.zeros(i + 1), torch.ones(1)]) +
                             torch.randn(i + 2, generator=g) * 0.1).to(torch.bfloat16)
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            if L["type"] == "retention":
                for n, rows in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
                    sd[p + n] = rnd(rows, W, std=W ** -0.5)
            elif L["type"] == "latent_attention":
                r, qr, dr = m["kv_rank"], m["q_rank"], m["rot_dim"]
                sd[p + "dq"], sd[p + "dq.norm"] = rnd(qr, W, std=W ** -0.5), 1 + rnd(qr, std=0.1)
                sd[p + "uq"] = rnd(H * (d + dr), qr, std=qr ** -0.5)
                sd[p + "dkv"], sd[p + "dkv.norm"] = rnd(r + dr, W, std=W ** -0.5), 1 + rnd(r, std=0.1)
                sd[p + "uk"], sd[p + "uv"] = rnd(H * d, r, std=r ** -0.5), rnd(H * dv, r, std=r ** -0.5)
                sd[p + "sink"] = rnd(H, std=1.0)
                sd[p + "g"] = rnd(H * dv, W, std=W ** -0.5)
            else:
                G = m["kv_heads"]
                for n, rows in (("q", H * 2 * d), ("k", G * 2 * d), ("v", G * dv), ("g", H)):
                    sd[p + n] = rnd(rows, W, std=W ** -0.5)
                for n in ("lq1", "lk1", "lq2", "lk2"):
                    sd[p + n] = rnd(d, std=0.1)
            sd[p + "o"] = rnd(W, H * dv, std=(H * dv) ** -0.5)
            if L.get("mlp"):
                F = L["mlp"]["ff"]
                sd[q + "mlp.gate"], sd[q + "mlp.up"] = rnd(F, W, std=W ** -0.5), rnd(F, W, std=W ** -0.5)
                sd[q + "mlp.down"] = rnd(W, F, std=F ** -0.5)
        return sd

    def random_init(self, seed: int = 0) -> "SobivikForCausalLM":
        return self.load_state(self.random_state(seed))

    def load_safetensors(self, path: str) -> "SobivikForCausalLM":
        from safetensors import safe_open

        files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
        if not files:
            raise FileNotFoundError(f"no safetensors in {path}")
        tensors = {}
        for f in files:
            with safe_open(f, framework="pt", device="cpu") as sf:
                for k in sf.keys():
                    tensors[k] = sf.get_tensor(k)
        return self.load_state(tensors)

    def load_state(self, sd: dict[str, torch.Tensor]) -> "SobivikForCausalLM":
        """Build the run-time weights from a checkpoint-named state dict: fused
        projection matrices in the activation dtype; norm weights (a scalar
        spread over the columns), convolution taps, decays, sinks, depth
        weights and rotary frequencies in fp32."""
        cfg, dev, dt = self.cfg, self.device, self.dtype
        W = cfg.hidden_size

        def act(*names, pad: int = 0):  # (fused) projection weight; pad: zero rows up to a multiple of it
            t = torch.cat([sd[n] for n in names], 0) if len(names) > 1 else sd[names[0]]
            if pad and t.shape[0] % pad:
                t = torch.cat([t, t.new_zeros((pad - t.shape[0] % pad, t.shape[1]))], 0)
            return t.to(dev, dt).contiguous()

        def f32(t):
            return t.to(dev, torch.float32).contiguous()

        def spread(name):  # a norm with one weight for all columns, as the per-column weight the kernels take
            return torch.full((W,), float(sd[name].float()), dtype=torch.float32, device=dev)

        self.layers = []
        for i, L in enumerate(cfg.layers):
            m, p, q = L["mixer"], f"l{i}.mix.", f"l{i}."
            mlp = L.get("mlp")
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            out = dict(m=m, type=L["type"], mlp=mlp, norm1=spread(q + "norm1"), norm1b=spread(q + "norm1b"),
                       w_o=act(p + "o"))
            if self.taps and q + "canon1" in sd:
                # tap-major [taps, W]; h + conv(h) is one convolution whose last tap (the token itself) has weight 1 + w
                cw = sd[q + "canon1"].float().t().contiguous()
                cw[-1] += 1.0
                out["canon_w"] = f32(cw)
            elif self.taps:
                raise KeyError(f"{q}canon1: the config gives convolution taps but the layer has no weights")
            dwa = sd.get(q + "dwa")
            # without depth weights what goes on is the layer's own result
            out["dwa"] = f32(dwa) if dwa is not None else \
                f32(torch.cat([torch.zeros(i + 1), torch.ones(1)]))
            if out["dwa"].numel() != i + 2:
                raise ValueError(f"{q}dwa: {out['dwa'].numel()} weights for {i + 2} results")
            if L["type"] == "retention":
                out.update(w_in=act(p + "q", p + "k", p + "v", p + "g"),
                           decay=torch.tensor([float(x) for x in m["decay"]], dtype=torch.float32, device=dev))
            elif L["type"] == "latent_attention":
                r = m["kv_rank"]
                rot = m.get("rot")
                freq, mag = rc.yarn_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling")) \
                    if rot and rot.get("dims") else (None, 1.0)
                sink = sd.get(p + "sink")
                if sd[p + "dkv"].shape[0] != r + m["rot_dim"] or sd[p + "uq"].shape[0] != H * (d + m["rot_dim"]):
                    raise ValueError(f"{p}: projection rows do not fit kv_rank, rot_dim, heads and dim")
                out.update(w_in=act(p + "dq", p + "dkv", p + "g"), qn=f32(sd[p + "dq.norm"]), w_uq=act(p + "uq"),
                           qr=int(sd[p + "dq"].shape[0]),  # the query latent's width is the tensor's
                           cn=f32(sd[p + "dkv.norm"]), sink=f32(sink) if sink is not None else None,
                           uk=sd[p + "uk"].to(dev, dt).view(H, d, r).contiguous(),
                           uv=sd[p + "uv"].to(dev, dt).view(H, dv, r).transpose(1, 2).contiguous(),
                           inv_freq=freq.to(dev) if freq is not None else None, mag=mag)
            else:
                lam = math.exp(float((sd[p + "lq1"].double() * sd[p + "lk1"].double()).sum())) \
                    - math.exp(float((sd[p + "lq2"].double() * sd[p + "lk2"].double()).sum())) + float(m["diff"])
                out.update(w_in=act(p + "q", p + "k", p + "v", p + "g", pad=IN_PAD), lam=lam)
            if mlp:
                out.update(norm2=spread(q + "norm2"), norm2b=spread(q + "norm2b"),
                           w_gu=act(q + "mlp.gate", q + "mlp.up"), w_down=act(q + "mlp.down"))
            self.layers.append(out)
        self.embed = act("embed")
        self.head = act("head")
        self.final_w = spread("final.norm")
        self.one = torch.ones(1, dtype=torch.float32, device=dev)
        return self

    # ------------------------------------------------------------------ forward
    def _parts(self, rows: int, n_qh: int, group: int, visible: int, meta: AttnMeta) -> int:
        """Key partitions of the step's decode rows (rows that are no prompt-chunk tiles)."""
        vis = meta.max_ctx if meta.max_ctx else self.cfg.max_position_embeddings
        if visible:
            vis = min(vis, visible)
        grouped = self.dtype == torch.bfloat16 and self.device.type == "cuda"
        if meta.is_prefill and grouped:
            rows -= meta.num_prefill_tokens
        units = n_qh if not grouped else max(1, n_qh // group) * (-(-group // 32))
        return mx.row_attention_parts(max(rows, 1), units, vis,
                                      mx.GROUP_TARGET_WAVES if grouped else mx.ROW_TARGET_WAVES)

    @staticmethod
    def _mask(m: dict) -> tuple[str, int, int]:
        mask = m.get("mask") or {}
        size = int(mask.get("size") or 0)
        return ("window", size, int(mask.get("keep_first") or 0)) if size else ("causal", 0, 0)

    def _diff_attention(self, L: dict, h: torch.Tensor, meta: AttnMeta, kc, vc, seq, tables, bs: int):
        m, T = L["m"], h.shape[0]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        nq, nk = H * 2 * d, G * 2 * d
        p = self._mm(h, L["w_in"])  # [q (two maps per head) | k (two maps per key head) | v | g (one per head)]
        mx.headprep_cache(p, meta.positions, meta.slot_mapping, 2 * H, 2 * G, d, nq, None, None, self.cfg.rms_norm_eps,
                          None, kc, vc, v_mode=2, v_off=nq + nk, v_w=G * dv)
        mask, size, keep = self._mask(m)
        tl = (meta.row_tiles, meta.num_prefill_tokens) if meta.is_prefill else (None, 0)
        a = mx.attention(p, kc, vc, meta.positions, seq, tables, bs, 2 * H, 2, H // G, d, dv, m["scale"], mask, size,
                         self._parts(T, 2 * H, H // G, size + keep if size else 0, meta), True, *tl, keep_first=keep)
        g0 = nq + nk + G * dv
        o = mx.diff_combine(a.view(T, H, 2, dv), L["lam"], 1.0 - float(m["diff"]), self.cfg.rms_norm_eps, self.dtype,
                            head_gate=p[:, g0:g0 + H])
        return self._mm(o, L["w_o"])

    def _retention(self, L: dict, h: torch.Tensor, meta: AttnMeta, state: torch.Tensor):
        m = L["m"]
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        n, nv = H * d, H * dv
        p = self._mm(h, L["w_in"])  # [q | k | v | g]
        o = rc.retention(p[:, :n], p[:, n:2 * n], p[:, 2 * n:2 * n + nv], L["decay"], d ** -0.5, state, meta.positions,
                         meta.seq_rows, meta.state_slots, H, d, dv)
        o = rc.head_norm_gate(o, H, None, p[:, 2 * n + nv:2 * n + 2 * nv], self.cfg.rms_norm_eps, self.dtype,
                              gate_act="silu")
        return self._mm(o, L["w_o"])

    def _latent_attention(self, L: dict, h: torch.Tensor, meta: AttnMeta, cache, seq, tables, bs: int):
        m, T = L["m"], h.shape[0]
        H, d, dr, dv, r, qr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], L["qr"]
        eps = self.cfg.rms_norm_eps
        p = self._mm(h, L["w_in"])  # [query latent (q_rank) | key/value latent (kv_rank) | key part (rot_dim) | g]
        q = self._mm(mx.section_norm(p[:, :qr], L["qn"], eps), L["w_uq"])  # per head [dim unrotated | rot_dim]
        # fold the key up-projection into the query: the cached latent is the one key/value head of every query head
        qa = torch.bmm(q.view(T, H, d + dr)[:, :, :d].transpose(0, 1), L["uk"])
        ql = rc.latent_rope(qa, q, d + dr, d, p[:, qr:qr + r + dr], r, dr, L["cn"], eps, L["inv_freq"], L["mag"],
                            meta.positions, meta.slot_mapping, cache)
        mask, size, _ = self._mask(m)
        tl = (meta.row_tiles, meta.num_prefill_tokens) if meta.is_prefill else (None, 0)
        a = mx.attention(ql, cache, cache, meta.positions, seq, tables, bs, H, 1, H, r + dr, r, m["scale"], mask, size,
                         self._parts(T, H, H, size, meta), False, *tl, sink=L["sink"])
        o = torch.bmm(a.view(T, H, r).transpose(0, 1), L["uv"]).transpose(0, 1).reshape(T, H * dv)
        g0 = qr + r + dr
        return self._mm(mx.act_mul(p[:, g0:g0 + H * dv], o, "sigmoid"), L["w_o"])

    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, kv_caches: list[tuple]) -> torch.Tensor:
        """Final-normed hidden rows at meta.logits_idx (or all rows)."""
        cfg, eps, dt = self.cfg, self.cfg.rms_norm_eps, self.dtype
        if meta.state is None or meta.state_slots is None:
            raise ValueError("Sobivik needs the step's state slots (a runner with state support)")
        T, W, n = input_ids.shape[0], cfg.hidden_size, len(self.layers)
        # plane j: the result of layer j - 1 (plane 0: the embedding output); plane i + 1 first holds layer i's input
        stack = torch.empty((n + 1, T, W), dtype=torch.float32, device=self.embed.device)
        mx.embed_streams(input_ids, self.embed, 1, scale=cfg.embedding_scale, out=stack[0])
        if meta.is_prefill:  # rows of several sequences: per-row sequence ids + one table
            seq, tables = meta.row_seq, meta.row_tables
        else:  # decode: row i is sequence i
            seq, tables = None, meta.block_tables
        bs = meta.block_size
        rs = dict(eps=eps, out_dtype=dt)
        pick = meta.logits_idx
        if n == 0:
            X = stack[0] if pick is None else stack[0].index_select(0, pick)
            return mx.residual_step(X, norm="rms", norm_w=self.final_w, **rs)[0]
        X, h = mx.depth_mix(stack, 1, self.one, dst=stack[1], norm_w=self.layers[0]["norm1"], **rs)
        for i, L in enumerate(self.layers):
            ci, ri = self._state_index[i]
            if ci is not None:
                cstate = meta.state[ci]
                hc = rc.conv_rope_cache(h, L["canon_w"], cstate, meta.positions, meta.slot_mapping,
                                        meta.row_seq if meta.is_prefill else None, meta.seq_rows, meta.state_slots,
                                        1, 0, W, 0, None, None, None)
                rc.conv_state_update(h, cstate, meta.positions, meta.seq_rows, meta.state_slots)
                h = hc
            kc, vc = kv_caches[i]
            if L["type"] == "attention":
                y = self._diff_attention(L, h, meta, kc, vc, seq, tables, bs)
            elif L["type"] == "retention":
                y = self._retention(L, h, meta, meta.state[ri])
            else:
                y = self._latent_attention(L, h, meta, kc, seq, tables, bs)
            if self.layer_hook is not None and meta.is_prefill:
                self.layer_hook(i)
            if L["mlp"]:
                h2, _ = mx.residual_step(X, c=y, c_w=L["norm1b"], norm="rms", norm_w=L["norm2"], **rs)
                pend = dict(c=self._mm(mx.glu_act(self._mm(h2, L["w_gu"]), "silu"), L["w_down"]), c_w=L["norm2b"])
            else:
                pend = dict(c=y, c_w=L["norm1b"])
            # the addend that closes the layer joins plane i + 1, the layer's result, in the pass that
            # forms what goes on: the average over planes 0 .. i + 1 (and the next layer's norm)
            if self.trace_layers is not None:
                mx.residual_step(X, **pend, **rs)
                pend = {}
                self.trace_layers.append(mx.depth_mix(stack, i + 2, L["dwa"])[0])
            if i + 1 < n:
                X, h = mx.depth_mix(stack, i + 2, L["dwa"], dst=stack[i + 2], norm_w=self.layers[i + 1]["norm1"],
                                    **pend, **rs)
        if pick is not None and pick.numel() == 0:
            return torch.empty((0, W), device=stack.device, dtype=dt)
        # the last average and the final norm, on the chosen rows only
        return mx.depth_mix(stack, n + 1, self.layers[-1]["dwa"], rows=pick, norm_w=self.final_w, **pend, **rs)[1]

    def compute_logits(self, hidden: torch.Tensor, fp32: bool = False) -> torch.Tensor:
        """Logits of final-normed rows, times the model's logit scale; fp32:
        the products of the bf16 operands accumulated and returned in fp32
        (scoring), in vocabulary slices so no fp32 copy of the head persists."""
        ls = float(self.cfg.logit_scale)
        if not fp32 or hidden.dtype == torch.float32:
            out = torch.matmul(hidden, self.head.t())
            return out.mul_(ls) if ls != 1.0 else out
        hf = hidden.float()
        V = self.head.shape[0]
        out = torch.empty((hidden.shape[0], V), dtype=torch.float32, device=hidden.device)
        for v0 in range(0, V, 16384):
            torch.matmul(hf, self.head[v0:v0 + 16384].float().t(), out=out[:, v0:v0 + 16384])
        return out.mul_(ls) if ls != 1.0 else out

    def sample_sharded(self, *a, **kw):
        raise RuntimeError("vocab-sharded sampling needs tensor parallelism, which Sobivik does not use")
