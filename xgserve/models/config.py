"""Model registry: architecture hyper-parameters of the supported families.

BASELINE.json names Llama-3 8B / 70B, Mixtral 8x7B and GPT-2-small; the
registry also carries Llama-3.2-1B (speculative-decoding draft) and tiny
variants of every family for CPU tests. `from_hf_config` maps a HF
config.json onto the same dataclass (safetensors checkpoints).
"""
from __future__ import annotations

import json
import os
from dataclasses import asdict, dataclass, field, replace
from typing import Dict, List, Optional


@dataclass
class ModelConfig:
    name: str
    arch: str                      # "llama" | "mixtral" | "gpt2" | "dofivik" | "vizonex" | "loluzen" | "lotelix"
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position: int = 8192
    rope_theta: float = 500000.0
    rope_scaling: Optional[dict] = None
    norm_eps: float = 1e-5
    tie_embeddings: bool = False
    num_experts: int = 0
    experts_per_token: int = 0
    bos_token_id: int = 1
    eos_token_ids: List[int] = field(default_factory=lambda: [2])
    dtype: str = "bfloat16"
    # layer-list architectures ("dofivik", "vizonex"): one dict per layer {"type", "mixer", "mlp"}, the
    # residual scale of the norm-after-sum sublayers, and the taps of the input convolution
    layer_specs: Optional[List[dict]] = None
    postln_alpha: float = 1.0
    canon_taps: int = 1
    # "loluzen": factor on the embedding rows, factor on every normed sublayer output, and the run of layers
    # {"start", "stop", "times"} that is repeated with the same weights (None = every layer once)
    embed_scale: float = 1.0
    residual_mult: float = 1.0
    layer_loop: Optional[dict] = None
    # "lotelix": the equal consecutive parts of a row that its RMS norms treat separately
    norm_groups: int = 1

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    def num_params(self) -> int:
        H, F, V, L = self.hidden_size, self.intermediate_size, self.vocab_size, self.num_layers
        if self.layer_specs is not None:
            if self.arch == "vizonex":
                from .vizonex import count_params
            elif self.arch == "loluzen":
                from .loluzen import count_params
            elif self.arch == "lotelix":
                from .lotelix import count_params
            else:
                from .dofivik import count_params
            return count_params(self)
        attn = H * (self.q_size + 2 * self.kv_size) + self.q_size * H
        if self.arch == "mixtral":
            mlp = self.num_experts * 3 * H * F + H * self.num_experts
        elif self.arch == "gpt2":
            mlp = 2 * H * F
        else:
            mlp = 3 * H * F
        emb = V * H * (1 if self.tie_embeddings else 2)
        return L * (attn + mlp + 2 * H) + emb + H

    def layer_runs(self) -> List[int]:
        """Indices into layer_specs in the order the layers run (a looped run of layers appears `times` times)."""
        n = len(self.layer_specs or [])
        lp = self.layer_loop
        if not lp:
            return list(range(n))
        a, b = int(lp["start"]), int(lp["stop"])
        return list(range(a)) + list(range(a, b)) * int(lp["times"]) + list(range(b, n))

    def kv_bytes_per_token(self, tp: int = 1, dtype_bytes: int = 2) -> int:
        if self.arch == "loluzen":
            att = [(m.get("left") or m) for m in (self.layer_specs[i]["mixer"] for i in self.layer_runs())]
            return sum((m["dim"] + m["vdim"]) * m["kv_heads"] * dtype_bytes for m in att)
        if self.arch == "lotelix":
            att = [(L["mixer"].get("left") or L["mixer"]) for L in self.layer_specs if L["type"] != "mingru"]
            return sum((m["dim"] + m["vdim"]) * m["kv_heads"] * dtype_bytes for m in att)
        if self.arch == "vizonex":
            return sum((m["dim"] + m["vdim"]) * m["kv_heads"] * dtype_bytes
                       for m in (L["mixer"] for L in self.layer_specs if L["type"] == "attention"))
        if self.layer_specs is not None:
            return sum((m["kv_rank"] + m["rot_dim"]) * dtype_bytes for m in (L["mixer"] for L in self.layer_specs)
                       if "kv_rank" in m and "kv_from" not in m)
        kvh = max(1, self.num_kv_heads // tp)
        return 2 * self.num_layers * kvh * self.head_dim * dtype_bytes

    def to_dict(self) -> dict:
        return asdict(self)


_REGISTRY: Dict[str, ModelConfig] = {}


def register(cfg: ModelConfig) -> ModelConfig:
    _REGISTRY[cfg.name] = cfg
    return cfg


register(ModelConfig("llama3-8b", "llama", 4096, 32, 32, 8, 128, 14336, 128256, 8192, 500000.0,
                     bos_token_id=128000, eos_token_ids=[128001, 128009]))
register(ModelConfig("llama3-70b", "llama", 8192, 80, 64, 8, 128, 28672, 128256, 8192, 500000.0,
                     bos_token_id=128000, eos_token_ids=[128001, 128009]))
register(ModelConfig("llama3.2-1b", "llama", 2048, 16, 32, 8, 64, 8192, 128256, 8192, 500000.0,
                     rope_scaling={"rope_type": "llama3", "factor": 32.0, "low_freq_factor": 1.0,
                                   "high_freq_factor": 4.0, "original_max_position_embeddings": 8192},
                     tie_embeddings=True, bos_token_id=128000, eos_token_ids=[128001, 128009]))
register(ModelConfig("mixtral-8x7b", "mixtral", 4096, 32, 32, 8, 128, 14336, 32000, 32768, 1000000.0,
                     num_experts=8, experts_per_token=2, bos_token_id=1, eos_token_ids=[2]))
register(ModelConfig("gpt2", "gpt2", 768, 12, 12, 12, 64, 3072, 50257, 1024, 0.0, norm_eps=1e-5,
                     tie_embeddings=True, bos_token_id=50256, eos_token_ids=[50256], dtype="float32"))
# tiny variants for CPU / unit tests (same code paths, small dims)
register(ModelConfig("llama-tiny", "llama", 256, 2, 4, 2, 64, 512, 512, 1024, 10000.0,
                     bos_token_id=1, eos_token_ids=[2]))
register(ModelConfig("llama-tiny-draft", "llama", 128, 1, 2, 1, 64, 256, 512, 1024, 10000.0,
                     bos_token_id=1, eos_token_ids=[2]))
register(ModelConfig("llama-tiny-gqa8", "llama", 512, 2, 8, 8, 64, 1024, 512, 1024, 10000.0,
                     bos_token_id=1, eos_token_ids=[2]))
register(ModelConfig("mixtral-tiny", "mixtral", 256, 2, 4, 2, 64, 256, 512, 1024, 1000000.0,
                     num_experts=8, experts_per_token=2, bos_token_id=1, eos_token_ids=[2]))


def dofivik_config(name: str, width: int, vocab: int, layers: List[dict], postln_alpha: float = 2.0, taps: int = 4,
                   eps: float = 1e-6, max_position: int = 32768) -> ModelConfig:
    """A Dofivik model: a list of layers, each one mixer ("latent_attention": sliding-window attention
    over a cached low-rank latent + one shared rotary key; "general_delta": a generalized delta-rule
    recurrence) and an optional dense xIELU feed-forward, every sublayer reading h + conv(h) and
    followed by the norm of alpha * x + sublayer(x)."""
    att = [L["mixer"] for L in layers if L["type"] == "latent_attention"]
    heads = max([L["mixer"]["heads"] for L in layers] or [1])
    hd = max([m["dim"] + m["rot_dim"] for m in att] or [L["mixer"]["dim"] for L in layers] or [1])
    ff = max([L["mlp"]["ff"] for L in layers if L.get("mlp")] or [0])
    for i, L in enumerate(layers):
        if L["type"] not in ("latent_attention", "general_delta"):
            raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
        if L.get("mlp") is not None and L["mlp"].get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind {L['mlp'].get('kind')!r}")
        src = L["mixer"].get("kv_from")
        if src is not None:
            m, o = L["mixer"], (layers[src]["mixer"] if 0 <= src < i else None)
            if o is None or layers[src]["type"] != "latent_attention" or "kv_from" in o:
                raise ValueError(f"layer {i}: kv_from must name an earlier latent_attention layer with its own cache")
            if (o["kv_rank"], o["rot_dim"], o["rot"]) != (m["kv_rank"], m["rot_dim"], m["rot"]):
                raise ValueError(f"layer {i}: kv_from layer {src} has another latent size or rotation")
    return ModelConfig(name, "dofivik", width, len(layers), heads, 1, hd, ff, vocab, max_position, 0.0, None, eps,
                       False, bos_token_id=0, eos_token_ids=[], layer_specs=layers, postln_alpha=float(postln_alpha),
                       canon_taps=int(taps))


def _dofivik_tiny_layers():
    att = {"dim": 32, "heads": 4, "kv_rank": 48, "q_rank": 40, "rot_dim": 16, "vdim": 24, "scale": 48 ** -0.5,
           "mask": {"size": 24}, "rot": {"base": 10000.0, "dims": 16}}
    return [{"type": "latent_attention", "mixer": dict(att), "mlp": {"kind": "dense", "ff": 192}},
            {"type": "general_delta", "mixer": {"dim": 32, "heads": 4}, "mlp": None},
            {"type": "latent_attention", "mixer": dict(att, kv_from=0), "mlp": {"kind": "dense", "ff": 192}}]


register(dofivik_config("dofivik-tiny", 128, 512, _dofivik_tiny_layers(), max_position=1024))


def vizonex_config(name: str, width: int, vocab: int, layers: List[dict], taps: int = 4, eps: float = 1e-6,
                   max_position: int = 4096) -> ModelConfig:
    """A Vizonex model: learned position vectors and a list of parallel blocks x + a1 mixer(n + conv(n)) + a2 ff(n),
    n = rmsnorm(x). Mixers: "attention" (grouped-query, whole-vector q / k norms, chunked visibility, per-head
    temperature and softmax sink) and "mamba2" (scalar-decay state-space recurrence). Feed-forward: "dense"
    (gelu-tanh gate), "moe" (grouped sigmoid router over clamped-GLU experts + a shared expert) or none."""
    def need(d, keys, where):
        for k in keys:
            if k not in d:
                raise ValueError(f"{where}: missing {k!r}")
    if taps < 1 or taps > 8:
        raise ValueError("canon.taps must be in [1, 8]")
    for i, L in enumerate(layers):
        m, w = L.get("mixer") or {}, f"layer {i}"
        if L.get("type") == "attention":
            need(m, ("heads", "kv_heads", "dim", "vdim", "scale", "mask"), w)
            if m["heads"] % m["kv_heads"] or int(m["mask"]["size"]) < 1:
                raise ValueError(f"{w}: heads must be a multiple of kv_heads and mask.size positive")
        elif L.get("type") == "mamba2":
            need(m, ("heads", "vdim", "state", "groups", "norm_groups", "conv"), w)
            if m["heads"] % m["groups"] or (m["heads"] * m["vdim"]) % m["norm_groups"] or not 1 <= m["conv"] <= 8:
                raise ValueError(f"{w}: heads must be a multiple of groups, heads * vdim of norm_groups, conv in [1, 8]")
            if m["state"] > 256:
                raise ValueError(f"{w}: state sizes above 256 are not supported")
        else:
            raise ValueError(f"{w}: unknown mixer type {L.get('type')!r}")
        mlp = L.get("mlp")
        if mlp is None:
            continue
        if mlp.get("kind") == "dense":
            need(mlp, ("ff",), w)
        elif mlp.get("kind") == "moe":
            need(mlp, ("expert", "router"), w)
            r = mlp["router"]
            need(r, ("experts", "top", "groups", "scale"), w)
            E, c, k = r["experts"], r["groups"]["count"], r["groups"]["keep"]
            if E % c or not 1 <= k <= c or not 1 <= r["top"] <= k * (E // c) or E > 512:
                raise ValueError(f"{w}: experts must divide into groups.count groups, 1 <= keep <= count, "
                                 "top <= keep * group size, experts <= 512")
        else:
            raise ValueError(f"{w}: unknown feed-forward kind {mlp.get('kind')!r}")
    att = [L["mixer"] for L in layers if L["type"] == "attention"]
    heads = max([L["mixer"]["heads"] for L in layers] or [1])
    hd = max([max(m["dim"], m["vdim"]) for m in att] or [L["mixer"]["vdim"] for L in layers] or [1])
    ffs = [(L["mlp"]["ff"] if L["mlp"]["kind"] == "dense" else
            L["mlp"]["expert"]["ff"] * L["mlp"]["router"]["top"] + (L["mlp"].get("shared") or {}).get("ff", 0))
           for L in layers if L.get("mlp")]
    return ModelConfig(name, "vizonex", width, len(layers), heads, max([m["kv_heads"] for m in att] or [1]), hd,
                       max(ffs or [0]), vocab, max_position, 0.0, None, eps, False, bos_token_id=0, eos_token_ids=[],
                       layer_specs=layers, canon_taps=int(taps))


def _vizonex_tiny_layers():
    att = {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.2, "mask": {"size": 24}}
    ssm = {"heads": 4, "vdim": 16, "state": 16, "groups": 2, "norm_groups": 2, "conv": 3}
    moe = {"kind": "moe", "expert": {"ff": 32, "limit": 3.0}, "shared": {"ff": 48, "limit": 2.0},
           "router": {"experts": 8, "top": 2, "scale": 1.25, "groups": {"count": 4, "keep": 2}}}
    return [{"type": "attention", "mixer": dict(att), "mlp": {"kind": "dense", "ff": 192}},
            {"type": "mamba2", "mixer": dict(ssm), "mlp": moe},
            {"type": "attention", "mixer": dict(att), "mlp": None}]


register(vizonex_config("vizonex-tiny", 128, 512, _vizonex_tiny_layers(), taps=3, max_position=1024))
def loluzen_config(name: str, width: int, vocab: int, layers: List[dict], embed_scale: float = 1.0,
                   residual_mult: float = 1.0, loop: Optional[dict] = None, eps: float = 1e-5,
                   max_position: int = 131072) -> ModelConfig:
    """A Loluzen model: x <- x + m * N(mixer(N(x))), x <- x + m * N(ff(N(x))) with one-plus-weight RMS norms before
    and after every sublayer; a run of layers may repeat with shared weights (each repetition with a cache of its
    own, the scaled embedding rows added again before it). Mixers: "attention" (short convolution on q / k / v,
    per-head q / k norm, partial rotation with rescaled frequencies, per-head output gate) and "parallel" (a biased
    attention branch with a logarithmic distance penalty and post-softmax head mixing beside a gated linear
    recurrence whose forget gate also sets the write strength). Feed-forward: dense squared-relu with biases, or none."""
    def need(d, keys, where):
        for k in keys:
            if k not in d:
                raise ValueError(f"{where}: missing {k!r}")

    def gqa(m, w):
        need(m, ("heads", "kv_heads", "dim", "vdim", "scale"), w)
        if m["heads"] < 1 or m["kv_heads"] < 1 or m["heads"] % m["kv_heads"]:
            raise ValueError(f"{w}: heads must be a positive multiple of kv_heads")
    if not layers:
        raise ValueError("a model needs at least one layer")
    for i, L in enumerate(layers):
        m, w = L.get("mixer") or {}, f"layer {i}"
        if L.get("type") == "attention":
            gqa(m, w)
            if not 1 <= int(m.get("conv", 1)) <= 8:
                raise ValueError(f"{w}: conv must be in [1, 8]")
            rot = m.get("rot")
            if rot is not None:
                need(rot, ("base", "dims"), w)
                if rot["dims"] % 2 or not 0 <= rot["dims"] <= m["dim"]:
                    raise ValueError(f"{w}: rot.dims must be even and at most dim")
                if rot.get("scaling") is not None:
                    need(rot["scaling"], ("factor", "low", "high", "original"), w)
        elif L.get("type") == "parallel":
            need(m, ("left", "right"), w)
            gqa(m["left"], w + " left")
            need(m["right"], ("heads", "dim", "vdim"), w + " right")
            if m["right"]["dim"] > 256:
                raise ValueError(f"{w}: recurrent head sizes above 256 are not supported")
        else:
            raise ValueError(f"{w}: unknown mixer type {L.get('type')!r}")
        mlp = L.get("mlp")
        if mlp is not None:
            if mlp.get("kind") != "dense":
                raise ValueError(f"{w}: unknown feed-forward kind {mlp.get('kind')!r}")
            need(mlp, ("ff",), w)
    if loop is not None:
        need(loop, ("start", "stop", "times"), "loop")
        if not (0 <= loop["start"] < loop["stop"] <= len(layers)) or loop["times"] < 1:
            raise ValueError("loop: needs 0 <= start < stop <= number of layers and times >= 1")
    att = [(L["mixer"].get("left") or L["mixer"]) for L in layers]
    heads = max(m["heads"] for m in att)
    hd = max(max(m["dim"], m["vdim"]) for m in att)
    ff = max([L["mlp"]["ff"] for L in layers if L.get("mlp")] or [0])
    return ModelConfig(name, "loluzen", width, len(layers), heads, max(m["kv_heads"] for m in att), hd, ff, vocab,
                       max_position, 0.0, None, eps, False, bos_token_id=0, eos_token_ids=[], layer_specs=layers,
                       embed_scale=float(embed_scale), residual_mult=float(residual_mult), layer_loop=loop)


def _loluzen_tiny_layers():
    att = {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.2, "conv": 4,
           "rot": {"base": 10000.0, "dims": 16, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}}
    par = {"left": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.25},
           "right": {"heads": 2, "dim": 16, "vdim": 32}}
    return [{"type": "parallel", "mixer": par, "mlp": {"kind": "dense", "ff": 192}},
            {"type": "attention", "mixer": att, "mlp": None},
            {"type": "attention", "mixer": dict(att), "mlp": {"kind": "dense", "ff": 160}}]


register(loluzen_config("loluzen-tiny", 128, 512, _loluzen_tiny_layers(), embed_scale=4.0, residual_mult=0.5,
                        loop={"start": 1, "stop": 2, "times": 2}, max_position=1024))
def lotelix_config(name: str, width: int, vocab: int, layers: List[dict], embed_scale: float = 1.0, eps: float = 1e-5,
                   norm_groups: int = 1, max_position: int = 131072) -> ModelConfig:
    """A Lotelix model: pre-norm layers x <- x + mixer(N(x)), x <- x + ff(N(x)) whose RMS norm N treats `norm_groups`
    equal consecutive parts of a row separately. Mixers: "mingru" (a per-channel gated recurrence whose gate and
    candidate read the current token only), "attention" (rotation in (i, i + dims / 2) pairs with rescaled
    frequencies, sliding window, softmax sink, values blended with the first value-mixing layer's, element-wise output
    gate) and "parallel" (causal attention with unnormalised sigmoid weights, biased projections and whole-vector
    q / k norms beside a linear attention with a decay per key channel). Feed-forward: a sigmoid-routed mixture of
    squared-relu experts whose routing weight scales the expert's input, or none."""
    def need(d, keys, where):
        for k in keys:
            if k not in d:
                raise ValueError(f"{where}: missing {k!r}")

    def gqa(m, w):
        need(m, ("heads", "kv_heads", "dim", "vdim", "scale"), w)
        if m["heads"] < 1 or m["kv_heads"] < 1 or m["heads"] % m["kv_heads"]:
            raise ValueError(f"{w}: heads must be a positive multiple of kv_heads")
        rot = m.get("rot")
        if rot is not None:
            need(rot, ("base", "dims"), w)
            if rot["dims"] % 2 or not 0 <= rot["dims"] <= m["dim"]:
                raise ValueError(f"{w}: rot.dims must be even and at most dim")
            if rot.get("scaling") is not None:
                need(rot["scaling"], ("factor", "low", "high", "original"), w)
    if not layers:
        raise ValueError("a model needs at least one layer")
    if norm_groups < 1 or norm_groups > 256 or width % norm_groups:
        raise ValueError("norm.groups must be in [1, 256] and divide the width")
    mixed = None
    for i, L in enumerate(layers):
        m, w = L.get("mixer") or {}, f"layer {i}"
        if L.get("type") == "mingru":
            need(m, ("width",), w)
            if m["width"] < 1:
                raise ValueError(f"{w}: width must be positive")
        elif L.get("type") == "attention":
            gqa(m, w)
            if m.get("mask") is not None and int(m["mask"]["size"]) < 1:
                raise ValueError(f"{w}: mask.size must be positive")
            if m.get("v_mix"):
                if mixed is not None and mixed != m["kv_heads"] * m["vdim"]:
                    raise ValueError(f"{w}: value-mixing layers must have value rows of equal size")
                mixed = m["kv_heads"] * m["vdim"]
        elif L.get("type") == "parallel":
            need(m, ("left", "right"), w)
            gqa(m["left"], w + " left")
            need(m["right"], ("heads", "dim", "vdim", "tau"), w + " right")
            if m["right"]["dim"] > 256 or m["right"]["tau"] <= 0:
                raise ValueError(f"{w}: recurrent head sizes above 256 are not supported; tau must be positive")
        else:
            raise ValueError(f"{w}: unknown mixer type {L.get('type')!r}")
        mlp = L.get("mlp")
        if mlp is not None:
            if mlp.get("kind") != "moe":
                raise ValueError(f"{w}: unknown feed-forward kind {mlp.get('kind')!r}")
            need(mlp, ("expert", "router"), w)
            need(mlp["router"], ("experts", "top"), w)
            need(mlp["expert"], ("ff",), w)
            if not 1 <= mlp["router"]["top"] <= mlp["router"]["experts"] <= 512:
                raise ValueError(f"{w}: needs 1 <= top <= experts <= 512")
    att = [(L["mixer"].get("left") or L["mixer"]) for L in layers if L["type"] != "mingru"]
    heads = max([m["heads"] for m in att] or [1])
    hd = max([max(m["dim"], m["vdim"]) for m in att] or [1])
    ff = max([L["mlp"]["expert"]["ff"] * L["mlp"]["router"]["top"] for L in layers if L.get("mlp")] or [0])
    return ModelConfig(name, "lotelix", width, len(layers), heads, max([m["kv_heads"] for m in att] or [1]), hd, ff, vocab,
                       max_position, 0.0, None, eps, False, bos_token_id=0, eos_token_ids=[], layer_specs=layers,
                       embed_scale=float(embed_scale), norm_groups=int(norm_groups))


def _lotelix_tiny_layers():
    att = {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.2, "mask": {"size": 24}, "v_mix": True,
           "rot": {"base": 10000.0, "dims": 16, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}}}
    par = {"left": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "scale": 0.25, "rot": {"base": 5000.0, "dims": 8}},
           "right": {"heads": 2, "dim": 16, "vdim": 32, "tau": 8.0, "decay_rank": 8}}
    moe = {"kind": "moe", "expert": {"ff": 48}, "router": {"experts": 6, "top": 2}}
    return [{"type": "attention", "mixer": dict(att), "mlp": dict(moe)},
            {"type": "mingru", "mixer": {"width": 96}, "mlp": None},
            {"type": "parallel", "mixer": par, "mlp": dict(moe)},
            {"type": "attention", "mixer": dict(att), "mlp": dict(moe)}]


register(lotelix_config("lotelix-tiny", 128, 512, _lotelix_tiny_layers(), embed_scale=3.0, norm_groups=4,
                        max_position=1024))
register(ModelConfig("gpt2-tiny", "gpt2", 128, 2, 2, 2, 64, 512, 512, 256, 0.0, tie_embeddings=True,
                     bos_token_id=0, eos_token_ids=[0], dtype="float32"))


def get_config(name: str) -> ModelConfig:
    if name in _REGISTRY:
        return replace(_REGISTRY[name])
    if os.path.isdir(name) and os.path.exists(os.path.join(name, "config.json")):
        return from_hf_config(os.path.join(name, "config.json"), name=name)
    raise KeyError(f"unknown model {name!r}; known: {sorted(_REGISTRY)} or a HF checkpoint directory")


def list_models() -> List[str]:
    return sorted(_REGISTRY)


def from_hf_config(path: str, name: Optional[str] = None) -> ModelConfig:
    with open(path) as f:
        c = json.load(f)
    if c.get("architecture") == "Dofivik":
        return dofivik_config(name or "dofivik", c["width"], c["vocab"], c["layers"], c["postln_alpha"],
                              c["canon"]["taps"], c["norm"]["eps"], int(c.get("max_position", 32768)))
    if c.get("architecture") == "Vizonex":
        return vizonex_config(name or "vizonex", c["width"], c["vocab"], c["layers"], c["canon"]["taps"],
                              c["norm"]["eps"], int(c["max_positions"]))
    if c.get("architecture") == "Loluzen":
        return loluzen_config(name or "loluzen", c["width"], c["vocab"], c["layers"], c["embedding"]["scale"],
                              c["residual_mult"], c.get("loop"), c["norm"]["eps"], int(c.get("max_position", 131072)))
    if c.get("architecture") == "Lotelix":
        return lotelix_config(name or "lotelix", c["width"], c["vocab"], c["layers"], c["embedding"]["scale"],
                              c["norm"]["eps"], int(c["norm"].get("groups", 1)), int(c.get("max_position", 131072)))
    mt = c.get("model_type", "llama")
    eos = c.get("eos_token_id", 2)
    eos = eos if isinstance(eos, list) else [eos]
    if mt == "gpt2":
        H = c["n_embd"]
        return ModelConfig(name or "gpt2", "gpt2", H, c["n_layer"], c["n_head"], c["n_head"], H // c["n_head"],
                           c.get("n_inner") or 4 * H, c["vocab_size"], c.get("n_positions", 1024), 0.0,
                           norm_eps=c.get("layer_norm_epsilon", 1e-5), tie_embeddings=True,
                           bos_token_id=c.get("bos_token_id", 50256), eos_token_ids=eos, dtype="float32")
    H = c["hidden_size"]
    nh = c["num_attention_heads"]
    arch = "mixtral" if mt == "mixtral" else "llama"
    return ModelConfig(
        name or mt, arch, H, c["num_hidden_layers"], nh, c.get("num_key_value_heads", nh),
        c.get("head_dim", H // nh), c["intermediate_size"], c["vocab_size"],
        c.get("max_position_embeddings", 8192), float(c.get("rope_theta", 10000.0)), c.get("rope_scaling"),
        c.get("rms_norm_eps", 1e-5), bool(c.get("tie_word_embeddings", False)),
        c.get("num_local_experts", 0), c.get("num_experts_per_tok", 0), c.get("bos_token_id", 1), eos)
