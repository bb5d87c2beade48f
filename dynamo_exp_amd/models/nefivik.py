"""Nefivik: a layer-listed hybrid decoder for the MI355X engine: recurrent
(generalized delta rule) and windowed sigmoid-attention mixers under sandwich
norms with gated residuals, routed experts, and a per-layer token input.

A checkpoint lists its layers.  Every sublayer is normed before and after,
and its result is gated element by element from its own input:
x <- x + rms(sub(h) * sigmoid(h Wrg^T + b)) * w_after,  h = rms(x) * w_before.
Per layer, T rows of one engine step (prompt chunks and decode tokens of
different sequences; state per sequence in the slot the engine assigned):

  general_delta
    p  = h @ [Wr | Wk | Wv | Wg | Wa | Wrg1 | Ww1]^T     hipBLASLt, one fused projection
    wl = tanh(p_w1) @ Ww2^T                              HIP act_mul + hipBLASLt
    o  = delta_rule(r, k, v, a, wl; S)                   HIP  decay, removal rate, unit key and the
                                                              running matrix S in fp32, token by token
    ym = head_norm_gate(o, w, g) @ Wo^T                  HIP + hipBLASLt
  attention
    p  = h @ [Wq | Wk | Wv | Wrg1 | Wg]^T                hipBLASLt (a layer that reads another layer's
                                                              keys and values has no Wk, Wv)
    q  = conv_rope_cache(p; conv state)                  HIP  short causal convolution over time, partial
                                                              rotary positions, K / V into the paged caches
    a  = attention(q, K, V, sigmoid weights)             HIP  weight sigmoid(q.k scale + b_h) per visible key of
                                                              the window, no normalisation, head gate in the epilogue
    ym = a @ Wo^T
  both
    X += rms(ym * sigmoid(p_rg1 + b)) w1b; h2 = rms(X) w2     HIP residual_step (gate, unit RMS, sum, next norm: one pass)
    yf = combine(experts(h2))                                  HIP route -> plan -> grouped GEMMs -> weighted sum
    X += rms(yf * sigmoid(h2 Wrg2^T + b)) w2b; xa = cast(X)    HIP residual_step
    y  = (gelu(xa @ Wsg^T) * e_tok) @ Wsp^T                    per-layer token input
    X += unit_rms(y) * ws; h = rms(X) w1'                      HIP residual_step: the next layer's norm in the same pass

Norms, the residual, scores and weights, router, decays and the recurrent
state are fp32; projections and activations are bf16 (dtype=bfloat16) or
everything is fp32 (dtype=float32).
"""
from __future__ import annotations

import glob
import math
import os

import torch

from ..ops import mixers as mx
from ..ops import moe
from ..ops import recurrent as rc
from .config import LayeredConfig
from .gemm_tuning import planned_mm, tune_small_m
from .llama import AttnMeta, TPGroup

MIXERS = ("general_delta", "attention")
EXPERT_ALPHA = 1.702  # the experts' gate is g * sigmoid(EXPERT_ALPHA * g)
IN_PAD = 64  # fused in-projections end in narrow sections (a gate per head, the decay's inner width): their
#              row count is padded with zero rows to a multiple of this, the GEMM kernels' column tile


class NefivikForCausalLM:
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
            raise ValueError("Nefivik runs on one GPU per engine (tensor parallel size 1)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"unsupported dtype {dtype}")
        if cfg.loop or cfg.streams:
            raise ValueError("Nefivik has neither a layer loop nor parallel residual streams")
        for i, L in enumerate(cfg.layers):
            m = L["mixer"]
            if L["type"] not in MIXERS:
                raise ValueError(f"unknown mixer type {L['type']!r}")
            if L.get("mlp") and L["mlp"].get("kind") != "moe":
                raise ValueError(f"unknown feed-forward kind {L['mlp'].get('kind')!r}")
            if L["type"] != "attention":
                continue
            if m["heads"] % m["kv_heads"]:
                raise ValueError(f"layer {i}: {m['heads']} heads over {m['kv_heads']} key/value heads")
            j = m.get("kv_from")
            if j is not None:
                src = cfg.layers[j] if 0 <= j < i else None
                if src is None or src["type"] != "attention" or src["mixer"].get("kv_from") is not None:
                    raise ValueError(f"layer {i}: kv_from {j} is no earlier attention layer with keys of its own")
                if any(src["mixer"][k] != m[k] for k in ("kv_heads", "dim", "vdim")):
                    raise ValueError(f"layer {i}: key/value sizes differ from layer {j}'s")
        self.side_dim = int((cfg.token_side or {}).get("dim", 0))
        self.layers: list[dict] = []
        self.embed = self.head = self.side_embed = self.final_w = None
        self.fp8 = False
        self.kv_scales = (1.0, 1.0)
        self.kv_amax = None
        self.layer_hook = None
        self.gemm_plan: dict = {}
        self.gemm_tuned: set = set()
        # debugging: when a list, forward() appends the residual after every layer
        self.trace_layers: list | None = None

    # ------------------------------------------------------------------ engine hooks (no-ops here)
    def enable_fused_mlp(self) -> bool:
        return False

    def fold_norms(self) -> bool:
        return False

    #: dense projections of a layer, by the name of their weight
    LINEARS = ("w_in", "w_w2", "w_o", "w_rg2", "side_gate", "side_proj")

    def tune_gemms(self, sizes, **kw) -> list:
        """Decode batch sizes: the hand-written small-M GEMMs where they beat the
        library (bf16 on the GPU; models/gemm_tuning.py)."""
        if self.device.type != "cuda" or self.dtype != torch.bfloat16 or not self.layers:
            return []
        groups: dict = {}  # layers of different mixers have in-projections of different shapes
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
        raise ValueError("fp8 linears are not available for Nefivik")

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
        ts += [t for t in (self.embed, self.head, self.side_embed) if t is not None]
        return sum(t.numel() * t.element_size() for t in ts)

    # ------------------------------------------------------------------ paged caches and state slots
    def cache_widths(self) -> list[tuple[int, int] | None]:
        """(K row width, V row width) of every layer that caches keys and values of its own."""
        return [(L["mixer"]["kv_heads"] * L["mixer"]["dim"], L["mixer"]["kv_heads"] * L["mixer"]["vdim"])
                if L["type"] == "attention" and L["mixer"].get("kv_from") is None else None for L in self.cfg.layers]

    def kv_bytes_per_block(self, block_size: int, dtype: torch.dtype) -> int:
        es = torch.empty((), dtype=dtype).element_size()
        return sum((w[0] + w[1]) * block_size * es for w in self.cache_widths() if w)

    def alloc_kv_caches(self, num_blocks: int, block_size: int, dtype: torch.dtype) -> list[tuple]:
        """One (K, V) pair per layer, token-major [num_blocks * block_size,
        width], indexed by the engine's one block table.  A layer that reads
        another layer's keys and values gets that layer's pair; recurrent layers
        an empty one.  Windowed layers keep every page of a live sequence; the
        mask alone bounds what is read."""
        if dtype != self.dtype:
            raise ValueError(f"the cache holds the model's activation dtype {self.dtype}, not {dtype}")
        out: list[tuple] = []
        for L, w in zip(self.cfg.layers, self.cache_widths()):
            if w:
                out.append((torch.zeros((num_blocks * block_size, w[0]), dtype=dtype, device=self.device),
                            torch.zeros((num_blocks * block_size, w[1]), dtype=dtype, device=self.device)))
            elif L["type"] == "attention":
                out.append(out[L["mixer"]["kv_from"]])
            else:
                e = torch.empty((0, 0), dtype=dtype, device=self.device)
                out.append((e, e))
        return out

    def _conv_channels(self, m: dict) -> int:
        own = m.get("kv_from") is None
        return m["heads"] * m["dim"] + (m["kv_heads"] * (m["dim"] + m["vdim"]) if own else 0)

    def state_shapes(self) -> list[tuple[tuple, torch.dtype]]:
        """Per layer, shape (without the slot dimension) and dtype of its
        per-sequence state: the running matrix of every head (fp32), or the
        last taps - 1 projected rows in front of the short convolution."""
        out = []
        for L in self.cfg.layers:
            m = L["mixer"]
            if L["type"] == "general_delta":
                out.append(((m["heads"], m["dim"], m["dim"]), torch.float32))
            else:
                out.append(((max(0, int(m.get("conv") or 1) - 1), self._conv_channels(m)), self.dtype))
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
        W, sdim = cfg.hidden_size, self.side_dim

        def rnd(*shape, std):
            return (torch.randn(*shape, generator=g) * std).to(torch.bfloat16)

        sd = {"embed": rnd(cfg.vocab_size, W, std=1.0), "final.norm": 1 + rnd(W, std=0.1),
              "head": rnd(cfg.vocab_size, W, std=W ** -0.5)}
        if sdim:
            sd["side.embed"] = rnd(cfg.vocab_size, sdim * len(cfg.layers), std=1.0)
        for i, L in enumerate(cfg.layers):
            m, p, q = L["mixer"], f"l{i}.mix.", f"l{i}."
            for n in ("norm1", "norm2"):
                sd[q + n] = 1 + rnd(W, std=0.1)
            for n in ("norm1b", "norm2b"):
                sd[q + n] = 0.5 + rnd(W, std=0.1)
            for n in ("rg1", "rg2"):
                sd[q + n], sd[q + n + ".b"] = rnd(W, W, std=W ** -0.5), rnd(W, std=0.5)
            H, d = m["heads"], m["dim"]
            if L["type"] == "general_delta":
                lo = int(m.get("decay_rank") or max(8, d // 4))
                for n in ("r", "k", "v", "g", "a"):
                    sd[p + n] = rnd(H * d, W, std=W ** -0.5)
                sd[p + "a.b"], sd[p + "w0"] = rnd(H * d, std=0.5), rnd(H * d, std=1.0)
                sd[p + "w1"], sd[p + "w2"] = rnd(lo, W, std=W ** -0.5), rnd(H * d, lo, std=lo ** -0.5)
                sd[p + "norm"] = 1 + rnd(H * d, std=0.1)
                sd[p + "o"] = rnd(W, H * d, std=(H * d) ** -0.5)
            else:
                G, dv, taps = m["kv_heads"], m["vdim"], int(m.get("conv") or 0)
                own = m.get("kv_from") is None
                sd[p + "q"] = rnd(H * d, W, std=W ** -0.5)
                if own:
                    sd[p + "k"], sd[p + "v"] = rnd(G * d, W, std=W ** -0.5), rnd(G * dv, W, std=W ** -0.5)
                if taps:
                    for n, c in (("q", H * d), ("k", G * d), ("v", G * dv)):
                        if own or n == "q":
                            sd[p + n + ".conv"] = rnd(c, taps, std=taps ** -0.5)
                sd[p + "pb"] = rnd(H, std=1.0) - 2.0
                sd[p + "g"] = rnd(H, W, std=W ** -0.5)
                sd[p + "o"] = rnd(W, H * dv, std=(H * dv) ** -0.5)
            mlp = L.get("mlp")
            if mlp:
                E, F = mlp["router"]["experts"], mlp["expert"]["ff"]
                for e in range(E):
                    sd[f"{q}mlp.e{e}.gate"], sd[f"{q}mlp.e{e}.up"] = rnd(F, W, std=W ** -0.5), rnd(F, W, std=W ** -0.5)
                    sd[f"{q}mlp.e{e}.down"] = rnd(W, F, std=F ** -0.5)
                sd[q + "mlp.router"] = rnd(E, W, std=2.0 * W ** -0.5)
            if sdim:
                sd[q + "side.gate"] = rnd(sdim, W, std=W ** -0.5)
                sd[q + "side.proj"] = rnd(W, sdim, std=sdim ** -0.5)
                sd[q + "side.norm"] = rnd(W, std=0.3)
        return sd

    def random_init(self, seed: int = 0) -> "NefivikForCausalLM":
        return self.load_state(self.random_state(seed))

    def load_safetensors(self, path: str) -> "NefivikForCausalLM":
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

    def load_state(self, sd: dict[str, torch.Tensor]) -> "NefivikForCausalLM":
        """Build the run-time weights from a checkpoint-named state dict: fused
        projection matrices in the activation dtype; norms, biases, the router,
        convolution taps and rotary frequencies in fp32."""
        cfg, dev, dt = self.cfg, self.device, self.dtype

        def act(*names, pad: int = 0):  # (fused) projection weight; pad: zero rows up to a multiple of it
            t = torch.cat([sd[n] for n in names], 0) if len(names) > 1 else sd[names[0]]
            if pad and t.shape[0] % pad:
                t = torch.cat([t, t.new_zeros((pad - t.shape[0] % pad, t.shape[1]))], 0)
            return t.to(dev, dt).contiguous()

        def f32(t):
            return t.to(dev, torch.float32).contiguous()

        self.layers = []
        for i, L in enumerate(cfg.layers):
            m, p, q = L["mixer"], f"l{i}.mix.", f"l{i}."
            mlp = L.get("mlp")
            out = dict(m=m, type=L["type"], mlp=mlp, norm1=f32(sd[q + "norm1"]), norm1b=f32(sd[q + "norm1b"]),
                       rg1_b=f32(sd[q + "rg1.b"]), w_o=act(p + "o"))
            if L["type"] == "general_delta":
                out.update(w_in=act(p + "r", p + "k", p + "v", p + "g", p + "a", q + "rg1", p + "w1", pad=IN_PAD),
                           w_w2=act(p + "w2"), a_b=f32(sd[p + "a.b"]), w0=f32(sd[p + "w0"]), hnorm=f32(sd[p + "norm"]),
                           lora=sd[p + "w1"].shape[0])
            else:
                own = m.get("kv_from") is None
                names = [p + "q"] + ([p + "k", p + "v"] if own else [])
                out.update(w_in=act(*names, q + "rg1", p + "g", pad=IN_PAD), pb=f32(sd[p + "pb"]), own=own)
                taps = int(m.get("conv") or 0)
                # tap-major [taps, C]: a run of neighbouring channels shares one load in the kernel
                out["conv_w"] = f32(torch.cat([sd[n + ".conv"] for n in names], 0).t()) if taps else \
                    torch.ones((1, self._conv_channels(m)), dtype=torch.float32, device=dev)
                rot = m.get("rot")
                out["inv_freq"] = rc.rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling")).to(dev) \
                    if rot and rot.get("dims") else None
            if mlp:
                E = mlp["router"]["experts"]
                w = f"l{i}.mlp."
                out.update(norm2=f32(sd[q + "norm2"]), norm2b=f32(sd[q + "norm2b"]), w_rg2=act(q + "rg2"),
                           rg2_b=f32(sd[q + "rg2.b"]), router=f32(sd[w + "router"]),
                           w_egu=torch.stack([torch.cat([sd[f"{w}e{e}.gate"], sd[f"{w}e{e}.up"]], 0)
                                              for e in range(E)]).to(dev, dt).contiguous(),
                           w_edown=torch.stack([sd[f"{w}e{e}.down"] for e in range(E)]).to(dev, dt).contiguous())
            if self.side_dim:
                out.update(side_gate=act(q + "side.gate"), side_proj=act(q + "side.proj"),
                           side_w=f32(sd[q + "side.norm"]))
            self.layers.append(out)
        self.embed = act("embed")
        self.head = act("head")
        self.side_embed = act("side.embed") if self.side_dim else None
        self.final_w = f32(sd["final.norm"])
        return self

    # ------------------------------------------------------------------ forward
    def _parts(self, rows: int, H: int, group: int, size: int, meta: AttnMeta) -> int:
        """Key partitions of the step's decode rows (rows that are no prompt-chunk tiles)."""
        vis = meta.max_ctx if meta.max_ctx else self.cfg.max_position_embeddings
        if size:
            vis = min(vis, size)
        if meta.is_prefill:
            rows -= meta.num_prefill_tokens if self.dtype == torch.bfloat16 and self.device.type == "cuda" else 0
        units = H if self.dtype != torch.bfloat16 else max(1, H // group) * (-(-group // 32))
        grouped = self.dtype == torch.bfloat16 and self.device.type == "cuda"
        return mx.row_attention_parts(max(rows, 1), units, vis,
                                      mx.GROUP_TARGET_WAVES if grouped else mx.ROW_TARGET_WAVES)

    def _delta(self, L: dict, h: torch.Tensor, meta: AttnMeta, state: torch.Tensor):
        m, W = L["m"], self.cfg.hidden_size
        H, d = m["heads"], m["dim"]
        n = H * d
        p = self._mm(h, L["w_in"])  # [r | k | v | g | a | rg1 | w1]
        wl = self._mm(mx.act_mul(p[:, 5 * n + W:5 * n + W + L["lora"]], None, "tanh"), L["w_w2"])
        o = rc.delta_rule(p[:, :n], p[:, n:2 * n], p[:, 2 * n:3 * n], p[:, 4 * n:5 * n], wl, L["a_b"], L["w0"], state,
                          meta.positions, meta.seq_rows, meta.state_slots, H, d, d)
        o = rc.head_norm_gate(o, H, L["hnorm"], p[:, 3 * n:4 * n], self.cfg.rms_norm_eps, self.dtype)
        return self._mm(o, L["w_o"]), p[:, 5 * n:5 * n + W]

    def _attend(self, L: dict, h: torch.Tensor, meta: AttnMeta, kc, vc, cstate, seq, tables, bs: int):
        m, T, W = L["m"], h.shape[0], self.cfg.hidden_size
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        p = self._mm(h, L["w_in"])  # [q | k | v | rg1 | g]  (k, v only with keys of its own)
        C = L["conv_w"].shape[1]
        q = rc.conv_rope_cache(p, L["conv_w"], cstate, meta.positions, meta.slot_mapping,
                               meta.row_seq if meta.is_prefill else None, meta.seq_rows, meta.state_slots, H,
                               G if L["own"] else 0, d, dv, L["inv_freq"], kc if L["own"] else None,
                               vc if L["own"] else None)
        rc.conv_state_update(p, cstate, meta.positions, meta.seq_rows, meta.state_slots)
        size = int((m.get("mask") or {}).get("size") or 0)
        tl = (meta.row_tiles, meta.num_prefill_tokens) if meta.is_prefill else (None, 0)
        a = mx.attention(q, kc, vc, meta.positions, seq, tables, bs, H, 1, H // G, d, dv, m["scale"],
                         "window" if size else "causal", size, self._parts(T, H, H // G, size, meta), False, *tl,
                         weights="sigmoid", head_bias=L["pb"], head_gate=p[:, C + W:C + W + H])
        return self._mm(a.view(T, H * dv), L["w_o"]), p[:, C:C + W]

    def _ff(self, L: dict, h: torch.Tensor) -> torch.Tensor:
        mlp = L["mlp"]
        r = mlp["router"]
        gr = r.get("groups") or {"count": 1, "keep": 1}
        z = torch.matmul(h.float(), L["router"].t())
        idx, w = moe.route(z, None, r["top"], gr["count"], gr["keep"], score="softmax", group_score="max")
        order, offsets = moe.plan(idx, r["experts"])
        gu = moe.grouped_gemm(h, L["w_egu"], order, offsets, r["top"], gather=True, scatter=False)
        act = mx.glu_act(gu, "swiglu_clamp", float(mlp["expert"]["limit"]), EXPERT_ALPHA)
        y = moe.grouped_gemm(act, L["w_edown"], order, offsets, r["top"], gather=False, scatter=True)
        return moe.combine(y, w, None)

    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, kv_caches: list[tuple]) -> torch.Tensor:
        """Final-normed hidden rows at meta.logits_idx (or all rows)."""
        cfg, eps, dt = self.cfg, self.cfg.rms_norm_eps, self.dtype
        if meta.state is None or meta.state_slots is None:
            raise ValueError("Nefivik needs the step's state slots (a runner with state support)")
        X = mx.embed_streams(input_ids, self.embed, 1)
        X = X.view(X.shape[0], X.shape[2])
        if meta.is_prefill:  # rows of several sequences: per-row sequence ids + one table
            seq, tables = meta.row_seq, meta.row_tables
        else:  # decode: row i is sequence i
            seq, tables = None, meta.block_tables
        bs = meta.block_size
        side = mx.gather_rows(self.side_embed, input_ids) if self.side_dim else None
        n = len(self.layers)
        rs = dict(eps=eps, out_dtype=dt)
        h, _ = mx.residual_step(X, norm="rms", norm_w=self.layers[0]["norm1"], **rs)
        pend = None  # the addend that closes the layer: joined with the next norm
        for i, L in enumerate(self.layers):
            kc, vc = kv_caches[i]
            if L["type"] == "general_delta":
                y, gate = self._delta(L, h, meta, meta.state[i])
            else:
                y, gate = self._attend(L, h, meta, kc, vc, meta.state[i], seq, tables, bs)
            if self.layer_hook is not None and meta.is_prefill:
                self.layer_hook(i)
            pend = dict(c=y, c_gate=gate, c_gate_b=L["rg1_b"], c_w=L["norm1b"])
            if L["mlp"]:
                h2, _ = mx.residual_step(X, norm="rms", norm_w=L["norm2"], **pend, **rs)
                pend = dict(c=self._ff(L, h2), c_gate=self._mm(h2, L["w_rg2"]), c_gate_b=L["rg2_b"], c_w=L["norm2b"])
            if self.side_dim:
                _, xa = mx.residual_step(X, want_cast=dt != torch.float32, **pend, **rs)
                xa = X if xa is None else xa
                sd_ = self.side_dim
                g = mx.act_mul(self._mm(xa, L["side_gate"]), side[:, i * sd_:(i + 1) * sd_], "gelu_tanh")
                pend = dict(c=self._mm(g, L["side_proj"]), c_w=L["side_w"])
            last = i + 1 == n
            if self.trace_layers is not None:
                mx.residual_step(X, **pend, **rs)
                self.trace_layers.append(X.clone())
                pend = None
            if not last:
                h, _ = mx.residual_step(X, norm="rms", norm_w=self.layers[i + 1]["norm1"], **(pend or {}), **rs)
        pick = meta.logits_idx
        if pick is not None:
            if pick.numel() == 0:
                return torch.empty((0, cfg.hidden_size), device=X.device, dtype=dt)
            X = X.index_select(0, pick)
            if pend:  # the last addend joins the residual on the chosen rows only
                pend = {k: (v.index_select(0, pick) if k in ("c", "c_gate") and v is not None else v)
                        for k, v in pend.items()}
        return mx.residual_step(X, norm="rms", norm_w=self.final_w, **(pend or {}), **rs)[0]

    def compute_logits(self, hidden: torch.Tensor, fp32: bool = False) -> torch.Tensor:
        """Logits of final-normed rows; fp32: the products of the bf16 operands
        accumulated and returned in fp32 (scoring), in vocabulary slices so no
        fp32 copy of the head persists."""
        if not fp32 or hidden.dtype == torch.float32:
            return torch.matmul(hidden, self.head.t())
        hf = hidden.float()
        V = self.head.shape[0]
        out = torch.empty((hidden.shape[0], V), dtype=torch.float32, device=hidden.device)
        for v0 in range(0, V, 16384):
            torch.matmul(hf, self.head[v0:v0 + 16384].float().t(), out=out[:, v0:v0 + 16384])
        return out

    def sample_sharded(self, *a, **kw):
        raise RuntimeError("vocab-sharded sampling needs tensor parallelism, which Nefivik does not use")
