"""Model configurations (Llama family) and presets.

Presets cover the BASELINE.json configs: Llama-3-8B, Llama-3-70B and
DeepSeek-R1-Distill-Llama-8B (Llama-3.1-8B architecture), plus tiny test
models.  ``ModelConfig.from_hf_dir`` reads a HuggingFace ``config.json`` so a
local checkpoint directory (config + tokenizer, optional safetensors) works.
"""
from __future__ import annotations

import dataclasses
import json
import os
from dataclasses import dataclass, field

LLAMA3_ROPE_SCALING = {
    "rope_type": "llama3",
    "factor": 8.0,
    "low_freq_factor": 1.0,
    "high_freq_factor": 4.0,
    "original_max_position_embeddings": 8192,
}


@dataclass
class ModelConfig:
    name: str = "llama"
    architecture: str = "LlamaForCausalLM"
    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: int = 128
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    rope_scaling: dict | None = None
    max_position_embeddings: int = 8192
    tie_word_embeddings: bool = False
    bos_token_id: int = 128000
    eos_token_id: list[int] = field(default_factory=lambda: [128001, 128009])
    # multimodal (LLaVA): CLIP vision tower + projector config, image placeholder id
    vision: dict | None = None
    image_token_id: int | None = None

    @property
    def q_size(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def num_params(self) -> int:
        h, f, v, L = self.hidden_size, self.intermediate_size, self.vocab_size, self.num_hidden_layers
        per_layer = h * (self.q_size + 2 * self.kv_size) + self.q_size * h + 3 * h * f + 2 * h
        return L * per_layer + v * h * (1 if self.tie_word_embeddings else 2) + h

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return self.num_hidden_layers * 2 * self.kv_size * dtype_bytes

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @classmethod
    def from_dict(cls, d: dict) -> "ModelConfig":
        names = {f.name for f in dataclasses.fields(cls)}
        return cls(**{k: v for k, v in d.items() if k in names})

    @classmethod
    def from_hf_dir(cls, path: str) -> "ModelConfig":
        with open(os.path.join(path, "config.json")) as f:
            c = json.load(f)
        vision = image_tok = None
        if "text_config" in c:  # LLaVA-style composite config
            vc = c.get("vision_config") or {}
            vision = dict(CLIP_L_336)
            vision.update({k: vc[k] for k in ("image_size", "patch_size", "hidden_size", "num_hidden_layers",
                                               "num_attention_heads", "intermediate_size", "layer_norm_eps")
                           if k in vc})
            vision["feature_layer"] = c.get("vision_feature_layer", -2)
            image_tok = c.get("image_token_index", 32000)
            c = {**c["text_config"], "architectures": c.get("architectures")}
            c.setdefault("vocab_size", 32064)
        heads = c["num_attention_heads"]
        eos = c.get("eos_token_id", 2)
        cfg = cls(
            name=os.path.basename(os.path.normpath(path)),
            architecture=(c.get("architectures") or ["LlamaForCausalLM"])[0],
            vocab_size=c["vocab_size"],
            hidden_size=c["hidden_size"],
            intermediate_size=c["intermediate_size"],
            num_hidden_layers=c["num_hidden_layers"],
            num_attention_heads=heads,
            num_key_value_heads=c.get("num_key_value_heads", heads),
            head_dim=c.get("head_dim", c["hidden_size"] // heads),
            rms_norm_eps=c.get("rms_norm_eps", 1e-5),
            rope_theta=c.get("rope_theta", 10000.0),
            rope_scaling=c.get("rope_scaling"),
            max_position_embeddings=c.get("max_position_embeddings", 8192),
            tie_word_embeddings=c.get("tie_word_embeddings", False),
            bos_token_id=c.get("bos_token_id", 1) or 1,
            eos_token_id=eos if isinstance(eos, list) else [eos],
            vision=vision,
            image_token_id=image_tok,
        )
        return cfg

    def write_hf_config(self, path: str) -> None:
        os.makedirs(path, exist_ok=True)
        d = {
            "architectures": [self.architecture],
            "model_type": "llama",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "intermediate_size": self.intermediate_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": self.rope_scaling,
            "max_position_embeddings": self.max_position_embeddings,
            "tie_word_embeddings": self.tie_word_embeddings,
            "bos_token_id": self.bos_token_id,
            "eos_token_id": self.eos_token_id,
            "torch_dtype": "bfloat16",
        }
        with open(os.path.join(path, "config.json"), "w") as f:
            json.dump(d, f, indent=2)


@dataclass
class LayeredConfig:
    """A model given as an explicit list of layers (config.json key `layers`),
    each naming its mixer type, the mixer's sizes and constants, and its
    feed-forward (or none), with an optional `loop` that repeats a span of
    layers with shared weights and per-pass caches, and optional parallel
    residual streams.  Every size and constant comes from the file; the
    engine-facing fields below mirror ModelConfig's."""

    name: str = "layered"
    architecture: str = "Bekulix"
    vocab_size: int = 0
    hidden_size: int = 0
    layers: list = field(default_factory=list)  # [{"type", "mixer": {...}, "mlp": {...} | None}]
    loop: dict | None = None  # {"start", "stop", "times"}
    rms_norm_eps: float = 1e-6
    streams: int | None = None  # parallel residual streams (None: one plain residual)
    token_side: dict | None = None  # {"dim"}: per-layer token input (a slice of a second embedding per layer)
    learned_positions: bool = False  # a learned vector per position is added to the embedding
    embedding_scale: float = 1.0  # the embedding row is multiplied by this
    logit_scale: float = 1.0  # the logits are multiplied by this
    canon: dict | None = None  # {"taps"}: a short causal convolution over time on every mixer's input
    max_position_embeddings: int = 1 << 20
    tie_word_embeddings: bool = False
    bos_token_id: int = 0
    eos_token_id: list[int] = field(default_factory=list)
    vision: dict | None = None
    image_token_id: int | None = None

    def layer_runs(self) -> list[int]:
        """Layer index of every layer run, in execution order."""
        n = len(self.layers)
        lp = self.loop
        if not lp:
            return list(range(n))
        a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
        if not (0 <= a <= b <= n and times >= 0):
            raise ValueError(f"bad loop {lp!r} for {n} layers")
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layer_runs())

    def num_params(self) -> int:
        W = self.hidden_size
        n = 2 * self.vocab_size * W + W
        if self.architecture == "Bolinex":
            return n + self._bolinex_params()
        if self.architecture == "Nefivik":
            return n + self._nefivik_params()
        if self.architecture == "Sobivik":
            return n - W + 1 + self._sobivik_params()
        for L in self.layers:
            m, t = L["mixer"], L["type"]
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            if t == "latent_attention":
                r = m["kv_rank"]
                n += H * d * W + r * W + H * d * r + H * dv * r + W * H * dv
            elif t == "attention":
                n += (H + m["kv_heads"]) * d * W + W * H * dv
            else:
                n += (2 * H * d + 2 * m["kv_heads"] * d + m["kv_heads"] * dv) * W + W * H * dv
            if L.get("mlp"):
                n += 3 * W * L["mlp"]["ff"]
        return n

    def _bolinex_params(self) -> int:
        W = self.hidden_size
        n = W  # norm biases ride with the weights: final bias
        if self.learned_positions:
            n += self.max_position_embeddings * W
        side = (self.token_side or {}).get("dim", 0)
        n += self.vocab_size * side * len(self.layers)
        for L in self.layers:
            m = L["mixer"]
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            n += 2 * W + (H * d + G * d + G * dv + H * dv) * W + W * H * dv + 2 * H + 1
            mlp = L.get("mlp")
            if mlp and mlp["kind"] == "dense":
                n += 2 * W * mlp["ff"]
            elif mlp:
                E = mlp["router"]["experts"]
                n += E * 3 * W * mlp["expert"]["ff"] + E * W + E
                if mlp.get("shared"):
                    n += 3 * W * mlp["shared"]["ff"]
            n += 2 * W * side + (W if side else 0)
        return n

    def _nefivik_params(self) -> int:
        W = self.hidden_size
        side = (self.token_side or {}).get("dim", 0)
        n = self.vocab_size * side * len(self.layers)
        for L in self.layers:
            m = L["mixer"]
            H, d = m["heads"], m["dim"]
            n += 2 * W + W * W + W  # sandwich norms and the gate of the mixer's result
            if L["type"] == "general_delta":
                lo = int(m.get("decay_rank") or max(8, d // 4))
                n += 6 * H * d * W + 3 * H * d + lo * (W + H * d)
            else:
                G, dv, taps = m["kv_heads"], m["vdim"], int(m.get("conv") or 0)
                own = (G * d + G * dv) if m.get("kv_from") is None else 0
                n += (H * d + own) * (W + taps) + H * (W + 1) + W * H * dv
            mlp = L.get("mlp")
            if mlp:
                E = mlp["router"]["experts"]
                n += 2 * W + W * W + W + E * 3 * W * mlp["expert"]["ff"] + E * W
            n += 2 * W * side + (W if side else 0)
        return n

    def _sobivik_params(self) -> int:
        W = self.hidden_size
        taps = int((self.canon or {}).get("taps", 0))
        n = 0
        for i, L in enumerate(self.layers):
            m = L["mixer"]
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            n += 4 + W * taps + i + 2  # scalar norms, input convolution, depth weights
            if L["type"] == "retention":
                n += (2 * H * d + 2 * H * dv) * W + W * H * dv
            elif L["type"] == "latent_attention":
                r, qr, dr = m["kv_rank"], m["q_rank"], m["rot_dim"]
                n += qr * (W + 1) + H * (d + dr) * qr + (r + dr) * W + r + H * (d + dv) * r + H + 2 * H * dv * W
            else:
                G = m["kv_heads"]
                n += (2 * H * d + 2 * G * d + G * dv + H) * W + 4 * d + W * H * dv
            if L.get("mlp"):
                n += 3 * W * L["mlp"]["ff"]
        return n

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @classmethod
    def from_dict(cls, c: dict, name: str = "layered") -> "LayeredConfig":
        """From the checkpoint's config.json."""
        maxpos = c.get("max_positions", c.get("max_position_embeddings"))
        return cls(name=name, architecture=c["architecture"], vocab_size=int(c["vocab"]), hidden_size=int(c["width"]),
                   layers=list(c["layers"]), loop=c.get("loop"), rms_norm_eps=float(c["norm"]["eps"]),
                   streams=c.get("streams"), token_side=c.get("token_side"),
                   learned_positions="max_positions" in c,
                   embedding_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                   logit_scale=float(c.get("logit_scale", 1.0)), canon=c.get("canon"),
                   max_position_embeddings=int(maxpos) if maxpos else 1 << 20,
                   eos_token_id=list(c.get("eos_token_id", [])))

    def write_hf_config(self, path: str) -> None:
        os.makedirs(path, exist_ok=True)
        d = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
             "layers": self.layers, "norm": {"eps": self.rms_norm_eps}}
        if self.loop:
            d["loop"] = self.loop
        if self.streams:
            d["streams"] = self.streams
        if self.token_side:
            d["token_side"] = self.token_side
        if self.learned_positions:
            d["max_positions"] = self.max_position_embeddings
        if self.embedding_scale != 1.0:
            d["embedding"] = {"scale": self.embedding_scale}
        if self.logit_scale != 1.0:
            d["logit_scale"] = self.logit_scale
        if self.canon:
            d["canon"] = self.canon
        with open(os.path.join(path, "config.json"), "w") as f:
            json.dump(d, f, indent=1)


# config.json `architecture` values served by LayeredConfig
LAYERED_ARCHITECTURES = ("Bekulix", "Bolinex", "Nefivik", "Sobivik")


def _bekulix_preset(name, W, ff, n_layers, heads, kv_heads, d, rank, window, chunk, vocab=32000, streams=4):
    """A Bekulix stack at a real model's layer sizes: latent (windowed), plain
    and differential (chunked) attention layers in turn."""
    att = {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": d,
                                          "scale": d ** -0.5, "q_temp": {"coef": 0.1, "every": 4096}},
           "mlp": {"kind": "dense", "ff": ff}}
    lat = {"type": "latent_attention", "mixer": {"heads": heads, "dim": d, "vdim": d, "kv_rank": rank,
                                                 "scale": d ** -0.5, "mask": {"size": window}},
           "mlp": {"kind": "dense", "ff": ff}}
    dif = {"type": "attention_2", "mixer": {"heads": heads // 2, "kv_heads": max(1, kv_heads // 2), "dim": d,
                                            "vdim": 2 * d, "scale": d ** -0.5, "diff": 0.8, "mask": {"size": chunk}},
           "mlp": {"kind": "dense", "ff": ff}}
    cyc = [att, lat, att, dif]
    return LayeredConfig(name=name, vocab_size=vocab, hidden_size=W, layers=[dict(cyc[i % 4]) for i in range(n_layers)],
                         streams=streams)


def _bolinex_preset(name, W, ff, n_layers, heads, kv_heads, d, window, experts=0, top=2, expert_ff=0, shared_ff=0,
                    groups=(1, 1), side=0, vocab=32000, max_positions=8192, softcap=30.0):
    """A Bolinex stack at a real model's layer sizes: windowed grouped-query
    attention with a tanh score cap, a distance penalty, value mixing and an
    output gate, in parallel with a dense (relu squared) feed-forward or, on
    every second layer when `experts` > 0, a routed mixture of experts."""
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": d, "scale": d ** -0.5, "softcap": softcap,
             "mask": {"size": window}, "v_mix": True}
    dense = {"kind": "dense", "ff": ff}
    moe = {"kind": "moe", "expert": {"ff": expert_ff}, "shared": {"ff": shared_ff} if shared_ff else None,
           "router": {"experts": experts, "top": top, "groups": {"count": groups[0], "keep": groups[1]}}}
    layers = [{"type": "attention", "mixer": dict(mixer), "mlp": dict(moe if experts and i % 2 else dense)}
              for i in range(n_layers)]
    return LayeredConfig(name=name, architecture="Bolinex", vocab_size=vocab, hidden_size=W, layers=layers,
                         rms_norm_eps=1e-5, token_side={"dim": side} if side else None, learned_positions=True,
                         max_position_embeddings=max_positions)


def _nefivik_preset(name, W, n_layers, heads, kv_heads, d, window, experts, top, expert_ff, groups=(1, 1), side=0,
                    vocab=32000, conv=4, rot_dims=None, attn_every=3, limit=7.0):
    """A Nefivik stack at a real model's layer sizes: generalized-delta-rule
    layers with every `attn_every`-th layer a windowed sigmoid-attention layer
    (short convolutions, partial rotary positions, head gate); every second
    attention layer reads the previous attention layer's keys and values; all
    feed-forwards are routed experts."""
    rot_dims = rot_dims or d // 2
    delta = {"type": "general_delta", "mixer": {"heads": heads, "dim": d}}
    attn = {"heads": heads, "kv_heads": kv_heads, "dim": d, "vdim": d, "scale": d ** -0.5, "conv": conv,
            "mask": {"size": window},
            "rot": {"base": 500000.0, "dims": rot_dims,
                    "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
    mlp = {"kind": "moe", "expert": {"ff": expert_ff, "limit": limit},
           "router": {"experts": experts, "top": top, "groups": {"count": groups[0], "keep": groups[1]}}}
    layers, src = [], None
    for i in range(n_layers):
        if (i + 1) % attn_every:
            layers.append({**delta, "mixer": dict(delta["mixer"]), "mlp": dict(mlp)})
            continue
        mixer = dict(attn)
        if src is not None:
            mixer["kv_from"], src = src, None
        else:
            src = i
        layers.append({"type": "attention", "mixer": mixer, "mlp": dict(mlp)})
    return LayeredConfig(name=name, architecture="Nefivik", vocab_size=vocab, hidden_size=W, layers=layers,
                         rms_norm_eps=1e-5, token_side={"dim": side} if side else None)


def _sobivik_preset(name, W, ff, n_layers, heads, kv_heads, d, rank, q_rank, rot_dim, window, keep, vocab=32000,
                    taps=4):
    """A Sobivik stack at a real model's layer sizes: differential attention
    (a window that keeps the first tokens), retention and latent attention
    (rotated key part, window, sink) layers in turn, all with a dense gated
    feed-forward, the input convolution and the depth average."""
    dif = {"type": "attention", "mixer": {"heads": heads // 2, "kv_heads": max(1, kv_heads // 2), "dim": d,
                                          "vdim": 2 * d, "scale": d ** -0.5, "diff": 0.3,
                                          "mask": {"size": window, "keep_first": keep}}}
    ret = {"type": "retention", "mixer": {"heads": heads, "dim": d, "vdim": d,
                                          "decay": [1.0 - 2.0 ** (-5 - 3 * h / max(1, heads - 1)) for h in range(heads)]}}
    lat = {"type": "latent_attention", "mixer": {
        "heads": heads, "dim": d, "rot_dim": rot_dim, "vdim": d, "kv_rank": rank, "q_rank": q_rank,
        "scale": (d + rot_dim) ** -0.5, "mask": {"size": window},
        "rot": {"base": 10000.0, "dims": rot_dim, "scaling": {"factor": 4.0, "original": 4096, "fast": 32.0, "slow": 1.0}}}}
    cyc = [dif, ret, lat]
    layers = [{**cyc[i % 3], "mixer": dict(cyc[i % 3]["mixer"]), "mlp": {"kind": "dense", "ff": ff}}
              for i in range(n_layers)]
    return LayeredConfig(name=name, architecture="Sobivik", vocab_size=vocab, hidden_size=W, layers=layers,
                         rms_norm_eps=1e-5, embedding_scale=float(W) ** 0.5, logit_scale=0.25, canon={"taps": taps})


# CLIP ViT-L/14 at 336 px, the LLaVA-1.5 vision tower; features from the
# second-to-last layer, CLS dropped, projected by a 2-layer GELU MLP
CLIP_L_336 = {
    "image_size": 336, "patch_size": 14, "hidden_size": 1024, "num_hidden_layers": 24, "num_attention_heads": 16,
    "intermediate_size": 4096, "layer_norm_eps": 1e-5, "feature_layer": -2,
}

PRESETS: dict[str, ModelConfig] = {
    "llama3-8b": ModelConfig(name="Llama-3-8B", rope_theta=500000.0, rope_scaling=None, max_position_embeddings=8192),
    "llama3.1-8b": ModelConfig(name="Llama-3.1-8B", rope_scaling=dict(LLAMA3_ROPE_SCALING), max_position_embeddings=131072),
    "deepseek-r1-distill-llama-8b": ModelConfig(
        name="DeepSeek-R1-Distill-Llama-8B", rope_scaling=dict(LLAMA3_ROPE_SCALING), max_position_embeddings=131072,
        eos_token_id=[128001],
    ),
    "llama3-70b": ModelConfig(
        name="Llama-3-70B", hidden_size=8192, intermediate_size=28672, num_hidden_layers=80, num_attention_heads=64,
        num_key_value_heads=8, rope_scaling=None, max_position_embeddings=8192,
    ),
    "llama3.1-70b": ModelConfig(
        name="Llama-3.1-70B", hidden_size=8192, intermediate_size=28672, num_hidden_layers=80, num_attention_heads=64,
        num_key_value_heads=8, rope_scaling=dict(LLAMA3_ROPE_SCALING), max_position_embeddings=131072,
    ),
    "llama2-7b": ModelConfig(
        name="Llama-2-7B", vocab_size=32000, intermediate_size=11008, num_key_value_heads=32, rope_theta=10000.0,
        max_position_embeddings=4096, bos_token_id=1, eos_token_id=[2],
    ),
    "llava-1.5-7b": ModelConfig(
        name="llava-1.5-7b", architecture="LlavaForConditionalGeneration", vocab_size=32064, intermediate_size=11008,
        num_key_value_heads=32, rope_theta=10000.0, max_position_embeddings=4096, bos_token_id=1, eos_token_id=[2],
        vision=dict(CLIP_L_336), image_token_id=32000,
    ),
    # tiny models for CI / smoke (GQA 4 like Llama-3; head_dim 128 as the kernels require)
    "tiny": ModelConfig(
        name="tiny-llama", vocab_size=512, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
        num_attention_heads=4, num_key_value_heads=1, head_dim=128, max_position_embeddings=4096,
        bos_token_id=1, eos_token_id=[2],
    ),
    "tiny-llava": ModelConfig(
        name="tiny-llava", architecture="LlavaForConditionalGeneration", vocab_size=512, hidden_size=256,
        intermediate_size=512, num_hidden_layers=2, num_attention_heads=4, num_key_value_heads=1, head_dim=128,
        max_position_embeddings=4096, bos_token_id=1, eos_token_id=[2], image_token_id=500,
        vision={"image_size": 56, "patch_size": 14, "hidden_size": 64, "num_hidden_layers": 3, "num_attention_heads": 4,
                "intermediate_size": 128, "layer_norm_eps": 1e-5, "feature_layer": -2},
    ),
    "small": ModelConfig(
        name="small-llama", vocab_size=32000, hidden_size=1024, intermediate_size=2816, num_hidden_layers=4,
        num_attention_heads=8, num_key_value_heads=2, head_dim=128, max_position_embeddings=8192,
        bos_token_id=1, eos_token_id=[2],
    ),
}


PRESETS["bekulix-tiny"] = _bekulix_preset("bekulix-tiny", 256, 512, 4, 4, 2, 64, 64, 48, 96, vocab=512)
# Llama-3-8B's layer sizes (width 4096, ff 14336, 32 x 128 heads, 8 KV heads), 8 layers
PRESETS["bekulix-8b-shapes"] = _bekulix_preset("bekulix-8b-shapes", 4096, 14336, 8, 32, 8, 128, 512, 1024, 2048,
                                               vocab=128256)


PRESETS["bolinex-tiny"] = _bolinex_preset("bolinex-tiny", 256, 512, 4, 4, 2, 64, 96, experts=8, top=2, expert_ff=128,
                                          shared_ff=128, groups=(4, 2), side=32, vocab=512, max_positions=4096)
# Llama-3-8B's layer sizes, 8 layers, every second feed-forward 16 experts of a quarter of the dense width
PRESETS["bolinex-8b-shapes"] = _bolinex_preset("bolinex-8b-shapes", 4096, 14336, 8, 32, 8, 128, 1024, experts=16,
                                               top=2, expert_ff=3584, shared_ff=3584, groups=(4, 2), side=256,
                                               vocab=128256)


PRESETS["nefivik-tiny"] = _nefivik_preset("nefivik-tiny", 192, 6, 3, 1, 32, 48, experts=8, top=2, expert_ff=64,
                                          groups=(4, 2), side=16, vocab=512, conv=4, rot_dims=16, limit=3.0)
# Llama-3-8B's layer sizes (width 4096, 32 x 128 heads, 8 KV heads), 9 layers; 16 experts of a quarter
# of the dense width, 2 chosen
PRESETS["nefivik-8b-shapes"] = _nefivik_preset("nefivik-8b-shapes", 4096, 9, 32, 8, 128, 1024, experts=16, top=2,
                                               expert_ff=3584, groups=(4, 2), side=256, vocab=128256)


PRESETS["sobivik-tiny"] = _sobivik_preset("sobivik-tiny", 192, 384, 6, 4, 2, 32, 64, 48, 32, 40, 6, vocab=512, taps=3)
# Llama-3-8B's layer sizes (width 4096, ff 14336, 32 x 128 heads, 8 KV heads), 9 layers; latent rank 192 + 64 rotated
PRESETS["sobivik-8b-shapes"] = _sobivik_preset("sobivik-8b-shapes", 4096, 14336, 9, 32, 8, 128, 192, 1536, 64, 1024,
                                               64, vocab=128256)


def get_config(name_or_path: str) -> ModelConfig:
    """A preset, an HF directory, or `<preset>@<layers>`: the preset's
    architecture truncated to its first <layers> decoder layers (one-GPU
    rehearsals of a big model's TP / transfer mechanics at its real layer
    shapes; never a throughput number for the full model)."""
    if "@" in name_or_path and not os.path.isdir(name_or_path):
        base, n = name_or_path.rsplit("@", 1)
        cfg = get_config(base)
        layers = int(n)
        if not 1 <= layers <= cfg.num_hidden_layers:
            raise ValueError(f"{name_or_path!r}: layer count must be 1..{cfg.num_hidden_layers}")
        return dataclasses.replace(cfg, num_hidden_layers=layers,
                                   name=f"{cfg.name} ({layers} of {cfg.num_hidden_layers} layers)")
    if name_or_path in PRESETS:
        return dataclasses.replace(PRESETS[name_or_path])
    if os.path.isdir(name_or_path) and os.path.exists(os.path.join(name_or_path, "config.json")):
        with open(os.path.join(name_or_path, "config.json")) as f:
            raw = json.load(f)
        if raw.get("architecture") in LAYERED_ARCHITECTURES:  # the model class follows the file
            return LayeredConfig.from_dict(raw, name=os.path.basename(os.path.normpath(name_or_path)))
        return ModelConfig.from_hf_dir(name_or_path)
    key = name_or_path.lower().replace("meta-llama/", "").replace("meta-", "")
    for k in PRESETS:
        if k.replace(".", "").replace("-", "") in key.replace(".", "").replace("-", "").replace("_", ""):
            return dataclasses.replace(PRESETS[k])
    raise ValueError(f"unknown model {name_or_path!r}; presets: {sorted(PRESETS)}")
