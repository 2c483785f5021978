"""Configuration: model presets, parallel layout, engine settings, feature flags.

Precedence: explicit arguments / CLI > BFLY_* environment > YAML/JSON file >
preset. The reference only states "Use feature flags for incompatible changes during
transition" (/root/reference/CLAUDE.md:81); the flag registry lives in utils/flags.py.
"""
from __future__ import annotations

import dataclasses
import json
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Optional


@dataclass
class ModelConfig:
    name: str
    arch: str                       # "llama" | "gpt2" | "mixtral" | "nesizen" | "zinesun" | "lizizen" | "gevipel"
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    max_position: int = 8192
    rope_theta: float = 500000.0
    rope_scaling: Optional[dict] = None
    norm_eps: float = 1e-5
    norm: str = "rms"               # "rms" | "layer"
    act: str = "silu"               # "silu" (SwiGLU) | "gelu" (plain MLP)
    pos_emb: str = "rope"           # "rope" | "learned"
    bias: bool = False              # linear biases (GPT-2)
    tie_embeddings: bool = False
    num_experts: int = 0            # > 0: MoE FFN
    experts_per_token: int = 0
    init_std: float = 0.02
    # heterogeneous stacks (arch "nesizen"): one normalised spec per layer (layer_spec below);
    # the flat fields above then hold the largest value over the layers (workspace sizing)
    layer_specs: Optional[list] = None
    residual_streams: int = 1       # > 1: hyper-connections (parallel residual streams)
    embed_scale: float = 1.0        # the embedding rows are multiplied by this
    conv_taps: int = 0              # > 1: causal per-channel convolution over time on a mixer's input
    # layer indices in the order they run, when a span of layers repeats with the same weights
    # (every run has its own cache and state); None: each layer once, in order
    layer_runs: Optional[list] = None
    residual_mult: float = 1.0      # a sublayer's (normed) output is multiplied by this before the residual sum
    loop_start: int = -1            # >= 0: first layer of the repeated span (the embedding output re-enters
                                    # the residual before every repetition of it but the first)

    # ---- derived quantities ------------------------------------------------------------
    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def padded_vocab(self, multiple: int = 256) -> int:
        return (self.vocab_size + multiple - 1) // multiple * multiple

    def layer_params(self) -> int:
        if self.layer_specs:
            return sum(layer_spec_params(self.hidden_size, sp) for sp in self.layer_specs) // len(self.layer_specs)
        h, f = self.hidden_size, self.intermediate_size
        attn = h * (self.q_size + 2 * self.kv_size) + self.q_size * h
        mlp = (3 if self.act == "silu" else 2) * h * f
        if self.is_moe:
            mlp = mlp * self.num_experts + h * self.num_experts
        norms = 2 * h * (2 if self.norm == "layer" else 1)
        b = 0
        if self.bias:
            b = self.q_size + 2 * self.kv_size + h + f + h
        return attn + mlp + norms + b

    def param_count(self) -> int:
        emb = self.vocab_size * self.hidden_size
        head = 0 if self.tie_embeddings else emb
        pos = self.max_position * self.hidden_size if self.pos_emb == "learned" else 0
        final = self.hidden_size * (2 if self.norm == "layer" else 1)
        return emb + head + pos + final + self.num_layers * self.layer_params()

    def active_params_per_token(self) -> int:
        if not self.is_moe:
            return self.param_count()
        h, f = self.hidden_size, self.intermediate_size
        dense_mlp = 3 * h * f
        per_layer = self.layer_params() - dense_mlp * self.num_experts + dense_mlp * self.experts_per_token
        return self.param_count() - self.num_layers * (self.layer_params() - per_layer)

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        if self.layer_specs:
            # a latent-attention layer caches its latent twice (key rows and transposed value
            # rows) and the shared rotated key part once
            runs = [self.layer_specs[i] for i in (self.layer_runs or range(len(self.layer_specs)))]
            return sum(sp["kv_heads"] * (sp["dim"] + sp["vdim"]) * dtype_bytes for sp in runs
                       if sp["type"] == "attention" and sp["kv_from"] is None) + \
                sum((2 * sp["kv_rank"] + sp["rot_dim"]) * dtype_bytes for sp in runs
                    if sp["type"] == "latent_attention") + \
                sum(sp["kv_heads"] * (sp["maps"] * sp["dim"] + sp["vdim"]) * dtype_bytes for sp in runs
                    if sp["type"] in ("biased_attention", "diff_attention", "sloped_attention"))
        return 2 * self.num_layers * self.kv_size * dtype_bytes

    # ---- (de)serialisation -------------------------------------------------------------
    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @classmethod
    def from_dict(cls, d: dict) -> "ModelConfig":
        names = {f.name for f in dataclasses.fields(cls)}
        return cls(**{k: v for k, v in d.items() if k in names})

    @classmethod
    def from_preset(cls, name: str, **overrides) -> "ModelConfig":
        if name not in PRESETS:
            raise KeyError(f"unknown model preset {name!r}; known: {sorted(PRESETS)}")
        d = dict(PRESETS[name])
        d.update(overrides)
        return cls(name=name, **d)

    @classmethod
    def from_nesizen(cls, js: dict, name: str = "nesizen") -> "ModelConfig":
        """Map a Nesizen config.json ("architecture": "Nesizen") to ModelConfig. Every size and
        every per-layer constant is taken from the file; layers may differ from one another."""
        specs = [layer_spec(i, L) for i, L in enumerate(js["layers"])]
        for sp in specs:
            j = sp["kv_from"]
            if j is not None:
                o = specs[j] if 0 <= j < sp["index"] else None
                if o is None or o["type"] != "attention" or o["kv_from"] is not None:
                    raise ValueError(f"layer {sp['index']}: kv_from must name an earlier attention layer with its own keys")
                if (o["kv_heads"], o["dim"], o["vdim"]) != (sp["kv_heads"], sp["dim"], sp["vdim"]):
                    raise ValueError(f"layer {sp['index']}: key/value shape differs from layer {j}")
        mx = lambda key: max([sp.get(key) or 0 for sp in specs] + [0])  # noqa: E731
        moe = [sp["ffn"] for sp in specs if sp["ffn"] and sp["ffn"]["kind"] == "moe"]
        return cls(name=name, arch="nesizen", vocab_size=int(js["vocab"]), hidden_size=int(js["width"]),
                   intermediate_size=max([sp["ffn"]["ff"] for sp in specs if sp["ffn"]] + [0]),
                   num_layers=len(specs), num_heads=mx("heads"), num_kv_heads=max(mx("kv_heads"), 1),
                   head_dim=max(mx("dim"), mx("vdim")), max_position=1 << 30, norm_eps=float(js["norm"]["eps"]),
                   norm="rms", act="relu2", pos_emb="rope", tie_embeddings=False,
                   num_experts=max([m["experts"] for m in moe] + [0]),
                   experts_per_token=max([m["top"] for m in moe] + [0]),
                   layer_specs=specs, residual_streams=int(js.get("streams", 1)))

    @classmethod
    def from_zinesun(cls, js: dict, name: str = "zinesun") -> "ModelConfig":
        """Map a Zinesun config.json ("architecture": "Zinesun") to ModelConfig: latent-attention
        layers with dense or routed feed-forwards, post-sublayer layer norms, a causal convolution
        on every mixer's input and a learned average over the outputs of all earlier layers. Every
        size and per-layer constant is taken from the file."""
        specs = [layer_spec(i, L) for i, L in enumerate(js["layers"])]
        mx = lambda key: max([sp.get(key) or 0 for sp in specs] + [0])  # noqa: E731
        moe = [sp["ffn"] for sp in specs if sp["ffn"] and sp["ffn"]["kind"] == "moe"]
        taps = int((js.get("canon") or {}).get("taps", 0))
        if taps < 0:
            raise ValueError("canon.taps must be >= 0")
        return cls(name=name, arch="zinesun", vocab_size=int(js["vocab"]), hidden_size=int(js["width"]),
                   intermediate_size=max([sp["ffn"]["ff"] for sp in specs if sp["ffn"]] + [0]),
                   num_layers=len(specs), num_heads=mx("heads"), num_kv_heads=1,
                   head_dim=max(mx("kv_rank") + mx("rot_dim"), mx("dim") + mx("rot_dim"), mx("vdim")),
                   max_position=1 << 30, norm_eps=float(js["norm"]["eps"]),
                   norm="layer", act="xielu", pos_emb="rope", tie_embeddings=True,
                   num_experts=max([m["experts"] for m in moe] + [0]),
                   experts_per_token=max([m["top"] for m in moe] + [0]),
                   layer_specs=specs, embed_scale=float((js.get("embedding") or {}).get("scale", 1.0)),
                   conv_taps=taps)

    @classmethod
    def from_lizizen(cls, js: dict, name: str = "lizizen") -> "ModelConfig":
        """Map a Lizizen config.json ("architecture": "Lizizen") to ModelConfig: parallel layers (mixer
        and feed-forward read two norms of the same residual) with a token shift on the mixer's
        input, softmax attention with a distance bias and a sink ("attention") or differential
        attention over chunks ("attention_2"), clamped-GLU feed-forwards with biases, and a span of
        layers that may run several times with the same weights ("loop"). Every size and per-layer
        constant is taken from the file."""
        kinds = {"attention": "biased_attention", "attention_2": "diff_attention"}
        specs = []
        for i, L in enumerate(js["layers"]):
            if L["type"] not in kinds:
                raise ValueError(f"layer {i}: Lizizen has no mixer {L['type']!r}")
            specs.append(layer_spec(i, {**L, "type": kinds[L["type"]]}))
        n = len(specs)
        runs = list(range(n))
        lp = js.get("loop")
        if lp:
            a, b, times = int(lp["start"]), int(lp["stop"]), int(lp.get("times", 1))
            if not (0 <= a <= b <= n) or times < 1:
                raise ValueError("loop: need 0 <= start <= stop <= layers and times >= 1")
            runs = list(range(a)) + list(range(a, b)) * times + list(range(b, n))
        mx = lambda key: max([sp.get(key) or 0 for sp in specs] + [0])  # noqa: E731
        return cls(name=name, arch="lizizen", vocab_size=int(js["vocab"]), hidden_size=int(js["width"]),
                   intermediate_size=max([sp["ffn"]["ff"] for sp in specs if sp["ffn"]] + [0]),
                   num_layers=n, num_heads=max([sp["heads"] * sp["maps"] for sp in specs] + [0]),
                   num_kv_heads=max(max([sp["kv_heads"] * sp["maps"] for sp in specs] + [0]), 1),
                   head_dim=max(mx("dim"), mx("vdim")), max_position=1 << 30, norm_eps=float(js["norm"]["eps"]),
                   norm="rms", act="glu_clamp", pos_emb="rope", tie_embeddings=False, bias=True,
                   layer_specs=specs, layer_runs=runs)

    @classmethod
    def from_gevipel(cls, js: dict, name: str = "gevipel") -> "ModelConfig":
        """Map a Gevipel config.json ("architecture": "Gevipel") to ModelConfig: layers with a layer
        norm before and after every sublayer and a constant factor on the normed sublayer output,
        three mixers (sliding-window attention with a linear distance bias whose values are the keys,
        "attention"; the gated delta rule with short convolutions, "delta"; causal latent attention
        with a sink, "latent_attention"), routed squared-ReLU experts chosen with a score correction,
        a scaled embedding, and a span of layers that may run several times with the same weights
        ("loop"), the embedding output re-entering before every repetition. Every size and per-layer
        constant is taken from the file."""
        kinds = {"attention": "sloped_attention", "delta": "delta", "latent_attention": "latent_attention"}
        specs = []
        for i, L in enumerate(js["layers"]):
            if L["type"] not in kinds:
                raise ValueError(f"layer {i}: Gevipel has no mixer {L['type']!r}")
            sp = layer_spec(i, {**L, "type": kinds[L["type"]]})
            if sp["ffn"]:
                if sp["ffn"]["kind"] != "moe":
                    raise ValueError(f"layer {i}: Gevipel has no feed-forward {sp['ffn']['kind']!r}")
                sp["ffn"]["glu"] = False          # experts are W_down relu(W_up h)^2
            specs.append(sp)
        n = len(specs)
        runs, start = list(range(n)), -1
        lp = js.get("loop")
        if lp:
            a, b, times = int(lp["start"]), int(lp["stop"]), int(lp.get("times", 1))
            if not (0 <= a <= b <= n) or times < 0:
                raise ValueError("loop: need 0 <= start <= stop <= layers and times >= 0")
            runs = list(range(a)) + list(range(a, b)) * times + list(range(b, n))      # (times 0: the span is left out)
            start = a if (b > a and times > 0) else -1
        mx = lambda key: max([sp.get(key) or 0 for sp in specs] + [0])  # noqa: E731
        moe = [sp["ffn"] for sp in specs if sp["ffn"]]
        return cls(name=name, arch="gevipel", vocab_size=int(js["vocab"]), hidden_size=int(js["width"]),
                   intermediate_size=max([m["ff"] for m in moe] + [0]),
                   num_layers=n, num_heads=mx("heads"), num_kv_heads=max(mx("kv_heads"), 1),
                   head_dim=max(mx("dim") + mx("rot_dim"), mx("kv_rank") + mx("rot_dim"), mx("vdim")),
                   max_position=1 << 30, norm_eps=float(js["norm"]["eps"]),
                   norm="layer", act="relu2", pos_emb="rope", tie_embeddings=False,
                   num_experts=max([m["experts"] for m in moe] + [0]),
                   experts_per_token=max([m["top"] for m in moe] + [0]),
                   layer_specs=specs, layer_runs=runs, loop_start=start,
                   embed_scale=float((js.get("embedding") or {}).get("scale", 1.0)),
                   residual_mult=float(js.get("residual_mult", 1.0)))

    @classmethod
    def from_model_dir(cls, path, name: Optional[str] = None) -> "ModelConfig":
        """config.json of a model folder -> ModelConfig; the "architecture" / "model_type" key
        chooses the family."""
        js = json.loads((Path(path) / "config.json").read_text())
        name = name or Path(path).name
        family = str(js.get("architecture", "")).lower()
        if family == "nesizen":
            return cls.from_nesizen(js, name=name)
        if family == "zinesun":
            return cls.from_zinesun(js, name=name)
        if family == "lizizen":
            return cls.from_lizizen(js, name=name)
        if family == "gevipel":
            return cls.from_gevipel(js, name=name)
        return cls.from_hf(js, name=name)

    @classmethod
    def from_hf(cls, hf: dict, name: str = "hf") -> "ModelConfig":
        """Map a HuggingFace config.json (Llama / Mistral / Mixtral / GPT-2) to ModelConfig."""
        mt = hf.get("model_type", "llama")
        if mt == "gpt2":
            h = hf["n_embd"]
            return cls(name=name, arch="gpt2", vocab_size=hf["vocab_size"], hidden_size=h,
                       intermediate_size=hf.get("n_inner") or 4 * h, num_layers=hf["n_layer"],
                       num_heads=hf["n_head"], num_kv_heads=hf["n_head"], head_dim=h // hf["n_head"],
                       max_position=hf["n_positions"], norm="layer", act="gelu", pos_emb="learned",
                       bias=True, tie_embeddings=True, norm_eps=hf.get("layer_norm_epsilon", 1e-5))
        h = hf["hidden_size"]
        nh = hf["num_attention_heads"]
        arch = "mixtral" if mt == "mixtral" else "llama"
        # rope: older configs carry rope_theta / rope_scaling at top level, newer ones a
        # "rope_parameters" dict; llama3-style frequency scaling is normalised to our keys
        rp = dict(hf.get("rope_parameters") or {})
        theta = rp.get("rope_theta", hf.get("rope_theta", 10000.0))
        scaling = hf.get("rope_scaling") or (rp if rp.get("rope_type", "default") != "default" else None)
        if scaling:
            kind = scaling.get("rope_type", scaling.get("type"))
            scaling = {"type": kind, **{k: v for k, v in scaling.items() if k not in ("rope_type", "type", "rope_theta")}}
        return cls(name=name, arch=arch, vocab_size=hf["vocab_size"], hidden_size=h,
                   intermediate_size=hf["intermediate_size"], num_layers=hf["num_hidden_layers"],
                   num_heads=nh, num_kv_heads=hf.get("num_key_value_heads", nh),
                   head_dim=hf.get("head_dim", h // nh),
                   max_position=hf.get("max_position_embeddings", 8192),
                   rope_theta=theta, rope_scaling=scaling,
                   norm_eps=hf.get("rms_norm_eps", 1e-5),
                   tie_embeddings=hf.get("tie_word_embeddings", False),
                   num_experts=hf.get("num_local_experts", 0),
                   experts_per_token=hf.get("num_experts_per_tok", 0))


def layer_spec(index: int, L: dict) -> dict:
    """One layer of a heterogeneous stack, normalised to flat keys. `type` "attention": windowed
    softmax attention (heads, kv_heads, dim, vdim, rot_dims, rot_base, scale, window, keep_first,
    kv_from); "latent_attention": windowed softmax attention whose queries, keys and values are
    expanded from low-rank latents, with one rotated key part shared by the heads (heads, dim,
    rot_dim, vdim, kv_rank, q_rank, rot_base, scale, window); "gla": gated linear attention
    (heads, dim, vdim, tau); "biased_attention": causal softmax attention without rotation whose
    scores lose a per-head logarithmic distance bias, with a zero-logit sink and a query
    temperature that grows with the position (heads, kv_heads, dim, vdim, scale, qt_coef,
    qt_every); "diff_attention": two softmax maps per head over the same values, combined as a
    difference (heads, kv_heads, dim, vdim, maps = 2, scale, diff, chunk, rot_dims, rot_base,
    softcap), with normed and half-rotated queries and keys, visible inside chunks of `chunk`
    positions; "sloped_attention": sliding-window softmax attention without rotation whose values
    are the keys as projected, with normed queries and keys, a linear per-head distance bias and the
    query temperature (heads, kv_heads, dim, vdim = dim, scale, window, qt_coef, qt_every); "delta":
    the gated delta rule with short convolutions on its query, key and value rows (heads, kv_heads,
    dim, vdim, taps). `ffn`: None, or kind "dense" (ff) / "glu" (dense clamped GLU with biases: ff,
    limit) / "moe" (ff, limit or None for unclamped experts, experts, top)."""
    m, t = L["mixer"], L["type"]
    sp = {"index": index, "type": t, "heads": int(m["heads"]), "dim": int(m["dim"]), "vdim": int(m.get("vdim", m["dim"])),
          "kv_from": None, "kv_heads": 0, "maps": 1}
    if t == "biased_attention":
        qt = m.get("q_temp") or {"coef": 0.0, "every": 1}            # absent: no temperature
        sp.update(kv_heads=int(m.get("kv_heads", m["heads"])), scale=float(m.get("scale", sp["dim"] ** -0.5)),
                  qt_coef=float(qt.get("coef", 0.0)), qt_every=int(qt.get("every", 1)))
        if sp["kv_heads"] < 1 or sp["heads"] % sp["kv_heads"] or sp["qt_every"] < 1:
            raise ValueError(f"layer {index}: bad attention sizes")
    elif t == "diff_attention":
        rot = m.get("rot") or {"dims": 0, "base": 10000.0}          # absent: no rotation
        mask = m.get("mask") or {"size": 1 << 30}                    # absent: plain causal attention
        sp.update(kv_heads=int(m.get("kv_heads", m["heads"])), maps=2, scale=float(m.get("scale", sp["dim"] ** -0.5)),
                  diff=float(m["diff"]), chunk=int(mask["size"]), rot_dims=int(rot["dims"]),
                  rot_base=float(rot.get("base", 10000.0)), softcap=float(m.get("softcap") or 0.0))
        if sp["kv_heads"] < 1 or sp["heads"] % sp["kv_heads"] or sp["rot_dims"] % 2 or sp["rot_dims"] > sp["dim"] \
                or sp["chunk"] < 1 or sp["softcap"] < 0:
            raise ValueError(f"layer {index}: bad differential-attention sizes")
    elif t == "attention":
        rot = m.get("rot") or {"dims": 0, "base": 10000.0}          # absent: no rotation
        mask = m.get("mask") or {"size": 1 << 30}                    # absent: plain causal attention
        sp.update(kv_heads=int(m.get("kv_heads", m["heads"])), rot_dims=int(rot["dims"]),
                  rot_base=float(rot.get("base", 10000.0)), scale=float(m.get("scale", sp["dim"] ** -0.5)),
                  window=int(mask["size"]), keep_first=int(mask.get("keep_first", 0)),
                  kv_from=None if m.get("kv_from") is None else int(m["kv_from"]))
        if sp["window"] < 1 or sp["keep_first"] < 0:
            raise ValueError(f"layer {index}: window must be >= 1 and keep_first >= 0")
        if sp["heads"] % sp["kv_heads"] or sp["rot_dims"] % 2 or sp["rot_dims"] > sp["dim"]:
            raise ValueError(f"layer {index}: bad attention sizes")
    elif t == "sloped_attention":
        qt = m.get("q_temp") or {"coef": 0.0, "every": 1}            # absent: no temperature
        mask = m.get("mask") or {"size": 1 << 30}                    # absent: plain causal attention
        sp.update(kv_heads=int(m.get("kv_heads", m["heads"])), scale=float(m.get("scale", sp["dim"] ** -0.5)),
                  window=int(mask["size"]), qt_coef=float(qt.get("coef", 0.0)), qt_every=int(qt.get("every", 1)))
        if sp["kv_heads"] < 1 or sp["heads"] % sp["kv_heads"] or sp["qt_every"] < 1 or sp["window"] < 1:
            raise ValueError(f"layer {index}: bad attention sizes")
        if sp["vdim"] != sp["dim"]:
            raise ValueError(f"layer {index}: the values are the keys, so vdim must equal dim")
    elif t == "delta":
        sp.update(kv_heads=int(m.get("kv_heads", m["heads"])), taps=int(m.get("conv", 1)))
        if sp["kv_heads"] < 1 or sp["heads"] % sp["kv_heads"] or sp["taps"] < 1:
            raise ValueError(f"layer {index}: bad delta-rule sizes")
    elif t == "latent_attention":
        rot = m.get("rot") or {}
        mask = m.get("mask") or {"size": 1 << 30}
        # q_rank 0: the queries are projected from the mixer's input directly
        sp.update(rot_dim=int(m.get("rot_dim", 0)), kv_rank=int(m["kv_rank"]), q_rank=int(m.get("q_rank", 0)),
                  rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", m.get("rot_dim", 0))),
                  scale=float(m.get("scale", (sp["dim"] + int(m.get("rot_dim", 0))) ** -0.5)),
                  window=int(mask["size"]))
        if sp["rot_dims"] > sp["rot_dim"] or sp["rot_dims"] % 2:
            raise ValueError(f"layer {index}: rot.dims must be even and at most rot_dim")
        if sp["window"] < 1 or min(sp["kv_rank"], sp["dim"] + sp["rot_dim"]) < 1 or sp["q_rank"] < 0:
            raise ValueError(f"layer {index}: bad latent-attention sizes")
    elif t == "gla":
        sp.update(tau=float(m["tau"]))
    else:
        raise ValueError(f"layer {index}: unknown mixer type {t!r}")
    f = L.get("mlp")
    if f is None:
        sp["ffn"] = None
    elif f["kind"] == "dense" and t in ("biased_attention", "diff_attention"):
        lim = f.get("limit")
        sp["ffn"] = {"kind": "glu", "ff": int(f["ff"]), "limit": float("inf") if lim is None else float(lim)}
    elif f["kind"] == "dense":
        sp["ffn"] = {"kind": "dense", "ff": int(f["ff"])}
    elif f["kind"] == "moe":
        lim = f["expert"].get("limit")
        sp["ffn"] = {"kind": "moe", "ff": int(f["expert"]["ff"]), "limit": None if lim is None else float(lim),
                     "experts": int(f["router"]["experts"]), "top": int(f["router"]["top"])}
        if not 1 <= sp["ffn"]["top"] <= sp["ffn"]["experts"]:
            raise ValueError(f"layer {index}: top must be in 1..experts")
    else:
        raise ValueError(f"layer {index}: unknown feed-forward kind {f['kind']!r}")
    return sp


def layer_spec_params(h: int, sp: dict) -> int:
    H, D, Dv = sp["heads"], sp["dim"], sp["vdim"]
    if sp["type"] == "attention":
        n = h * H * D + H * Dv * h + H
        if sp["kv_from"] is None:
            n += h * sp["kv_heads"] * (D + Dv)
    elif sp["type"] in ("biased_attention", "diff_attention"):
        m = sp["maps"]
        n = h * m * D * (H + sp["kv_heads"]) + h * sp["kv_heads"] * Dv + H * Dv * h + h
        n += 2 * H if m == 1 else 6 * D + h * H * Dv
    elif sp["type"] == "sloped_attention":
        n = h * D * (H + sp["kv_heads"]) + 2 * D + H * Dv * h
    elif sp["type"] == "delta":
        c = 2 * sp["kv_heads"] * D + H * Dv
        n = h * (c + H * Dv + 2 * H) + c * sp["taps"] + 2 * H + Dv + H * Dv * h
    elif sp["type"] == "latent_attention" and not sp["q_rank"]:
        R, rd = sp["kv_rank"], sp["rot_dim"]
        n = h * (H * (D + rd) + R + rd) + R + R * H * (D + Dv) + H + H * Dv * h
    elif sp["type"] == "latent_attention":
        R, Q, rd = sp["kv_rank"], sp["q_rank"], sp["rot_dim"]
        n = h * (Q + R + rd + H) + Q + R + Q * H * (D + rd) + R * H * (D + Dv) + H * Dv * h
    else:
        n = h * H * (2 * D + 2 * Dv) + H * Dv * h + Dv
    f = sp["ffn"]
    if f:
        if f["kind"] == "glu":
            n += 3 * h * f["ff"] + 2 * f["ff"] + h
        else:
            n += 2 * h * f["ff"] if f["kind"] == "dense" else f["experts"] * ((3 if f.get("glu", True) else 2) * h * f["ff"] + h)
    return n + 2 * h


PRESETS: dict[str, dict[str, Any]] = {
    # Public architecture hyper-parameters (weights are random-init; no checkpoints here).
    "gpt2-small": dict(arch="gpt2", vocab_size=50257, hidden_size=768, intermediate_size=3072,
                       num_layers=12, num_heads=12, num_kv_heads=12, head_dim=64, max_position=1024,
                       norm="layer", act="gelu", pos_emb="learned", bias=True, tie_embeddings=True),
    "llama3-8b": dict(arch="llama", vocab_size=128256, hidden_size=4096, intermediate_size=14336,
                      num_layers=32, num_heads=32, num_kv_heads=8, head_dim=128, max_position=8192,
                      rope_theta=500000.0),
    "llama3-70b": dict(arch="llama", vocab_size=128256, hidden_size=8192, intermediate_size=28672,
                       num_layers=80, num_heads=64, num_kv_heads=8, head_dim=128, max_position=8192,
                       rope_theta=500000.0),
    "llama3.1-70b": dict(arch="llama", vocab_size=128256, hidden_size=8192, intermediate_size=28672,
                         num_layers=80, num_heads=64, num_kv_heads=8, head_dim=128,
                         max_position=131072, rope_theta=500000.0,
                         rope_scaling={"type": "llama3", "factor": 8.0, "low_freq_factor": 1.0,
                                       "high_freq_factor": 4.0,
                                       "original_max_position_embeddings": 8192}),
    "mixtral-8x7b": dict(arch="mixtral", vocab_size=32000, hidden_size=4096, intermediate_size=14336,
                         num_layers=32, num_heads=32, num_kv_heads=8, head_dim=128,
                         max_position=32768, rope_theta=1e6, num_experts=8, experts_per_token=2),
    # Small configs for tests (same code paths, GPU-kernel-compatible dims).
    "llama-tiny": dict(arch="llama", vocab_size=1024, hidden_size=256, intermediate_size=512,
                       num_layers=2, num_heads=4, num_kv_heads=2, head_dim=128, max_position=2048,
                       rope_theta=10000.0, init_std=0.05),
    "llama-small": dict(arch="llama", vocab_size=4096, hidden_size=1024, intermediate_size=2048,
                        num_layers=4, num_heads=8, num_kv_heads=2, head_dim=128, max_position=4096,
                        rope_theta=500000.0, init_std=0.05),
    "gpt2-tiny": dict(arch="gpt2", vocab_size=512, hidden_size=128, intermediate_size=512,
                      num_layers=2, num_heads=2, num_kv_heads=2, head_dim=64, max_position=256,
                      norm="layer", act="gelu", pos_emb="learned", bias=True, tie_embeddings=True,
                      init_std=0.05),
    "mixtral-tiny": dict(arch="mixtral", vocab_size=1024, hidden_size=256, intermediate_size=512,
                         num_layers=2, num_heads=4, num_kv_heads=2, head_dim=128, max_position=2048,
                         rope_theta=1e6, num_experts=4, experts_per_token=2, init_std=0.05),
}


@dataclass
class ParallelConfig:
    tp: int = 1
    pp: int = 1
    ep: int = 1
    dp: int = 1
    # layer ranges per pipeline stage ([start, end) pairs); None = balanced split
    stage_layers: Optional[list] = None

    @property
    def world_size(self) -> int:
        # EP reuses the DP x TP ranks of a stage (DP-attention + expert-parallel FFN)
        return self.tp * self.pp * self.dp

    def to_dict(self) -> dict:
        return dataclasses.asdict(self)

    @classmethod
    def from_dict(cls, d: dict) -> "ParallelConfig":
        names = {f.name for f in dataclasses.fields(cls)}
        return cls(**{k: v for k, v in d.items() if k in names})


@dataclass
class EngineConfig:
    max_batch: int = 64               # max concurrent sequences per DP replica
    max_seq_len: int = 4096           # prompt + generated tokens per sequence
    max_prefill_tokens: int = 8192    # per engine step
    block_size: int = 32              # tokens per KV page (decode kernel is specialised to 32)
    kv_cache_tokens: Optional[int] = None   # explicit KV capacity; None = size from free HBM
    hbm_utilization: float = 0.92     # fraction of device memory the engine may use
    use_graphs: bool = True           # hipGraph-captured decode steps
    graph_batch_sizes: list = field(default_factory=lambda: [1, 2, 4, 8, 16, 32, 48, 64, 96, 128, 192, 256])
    seed: int = 0
    dtype: str = "bf16"
    custom_allreduce: bool = True     # one-shot IPC all-reduce for small TP messages
    # chunked prefill mixed into decode steps (pp == 1, no EP): every step decodes all running
    # sequences and fills the rest of max_prefill_tokens with prompt chunks
    mixed_prefill: bool = True
    # automatic prefix caching (with mixed_prefill): full prompt pages are registered under a
    # hash of their token prefix and reused by later requests that start with the same tokens
    prefix_caching: bool = True
    # KV-cache element type: "auto" (= the model dtype, bf16 on GPU) or "fp8" (e4m3, unscaled,
    # |x| <= 448): half the KV bytes per token, so twice the cached tokens and half the KV
    # traffic of a decode step; attention math stays bf16 (csrc/include/bfly_kv.h)
    kv_cache_dtype: str = "auto"
    # context-parallel prefill across data-parallel replicas (pp == 1, no EP): a prompt of at
    # least this many tokens is prefilled by ALL dp replicas together (ring or Ulysses
    # attention, parallel/context_parallel.py), its K/V collected in the cache of the replica
    # that then decodes it. 0 = off. Replicas step in lockstep while it is on.
    cp_prefill_min_tokens: int = 0
    # overlapped decode for single-stage layouts (pp == 1, no EP; the serving default): the
    # asynchronous pipeline of engine/pipeline.py with one group, so the host schedules step
    # k+1 (inputs gathered on the device from step k's sampled ids) while step k still runs, and
    # token values reach the host one step late. Mixed chunked prefill and prefix caching run
    # inside it (a plan's decode rows and prompt chunks travel together). Off (synchronous
    # steps) with context-parallel prefill, whose replicas step in lockstep.
    async_decode: bool = True
    cp_attention: str = "ring"        # "ring" | "ulysses"
    # request-state snapshots (engine/state.py): every `snapshot_every` steps one rank per DP
    # replica writes <snapshot_dir>/replica-<dp>.json; LLM(..., resume=dir) replays it
    snapshot_dir: Optional[str] = None
    snapshot_every: int = 0


def load_config_file(path: str | Path) -> dict:
    p = Path(path)
    text = p.read_text()
    if p.suffix in (".yaml", ".yml"):
        import yaml

        return yaml.safe_load(text)
    return json.loads(text)
