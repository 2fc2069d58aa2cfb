"""Model construction + safetensors checkpoint loading with per-rank TP/EP slicing.

Checkpoints: a HF-layout directory (config.json + model.safetensors or
model-XXXXX-of-YYYYY.safetensors + model.safetensors.index.json). Each rank
reads ONLY its shard through safetensors' lazy `get_slice` (row slices for
column-parallel weights, column slices for row-parallel ones, whole experts for
EP), converts to the serving dtype on the host and copies to HBM. q/k/v and
gate/up are fused on load. `save_checkpoint` writes the same HF layout from a
TP=1 model (tests, and to materialise random-init checkpoints).
"""
from __future__ import annotations

import json
import os
from typing import Callable, Dict, Optional

import torch

from ..ops.linear import deinterleave_gate_up, interleave_gate_up
from .base import kv_head_range
from .config import ModelConfig, get_config
from .dofivik import DofivikForCausalLM
from .gpt2 import GPT2ForCausalLM
from .llama import LlamaForCausalLM
from .loluzen import LoluzenForCausalLM
from .lotelix import LotelixForCausalLM
from .vizonex import VizonexForCausalLM


def model_class(cfg: ModelConfig):
    return {"gpt2": GPT2ForCausalLM, "dofivik": DofivikForCausalLM, "vizonex": VizonexForCausalLM,
            "loluzen": LoluzenForCausalLM, "lotelix": LotelixForCausalLM}.get(cfg.arch, LlamaForCausalLM)


def _resolve_shapes(cfg: ModelConfig, checkpoint: str) -> None:
    """Sizes that only a tensor's shape gives (Dofivik: the rank of the decay projection; Loluzen: the taps of
    a short convolution when the configuration leaves them out; Lotelix: the rank of the decay projection)."""
    if cfg.arch == "lotelix":
        r = _Reader(checkpoint)
        for i, spec in enumerate(cfg.layer_specs):
            if spec["type"] == "parallel":
                spec["mixer"]["right"]["decay_rank"] = int(r.shape(f"l{i}.mix.right.a1")[0])
        return
    if cfg.arch == "loluzen":
        r = _Reader(checkpoint)
        for i, spec in enumerate(cfg.layer_specs):
            if spec["type"] == "attention" and "conv" not in spec["mixer"]:
                spec["mixer"]["conv"] = int(r.shape(f"l{i}.mix.q.conv")[1]) if r.has(f"l{i}.mix.q.conv") else 1
        return
    if cfg.arch != "dofivik":
        return
    r = _Reader(checkpoint)
    for i, spec in enumerate(cfg.layer_specs):
        if spec["type"] == "general_delta":
            spec["mixer"]["decay_rank"] = int(r.shape(f"l{i}.mix.w1")[0])


def build_model(cfg: ModelConfig, device="cpu", dtype: Optional[torch.dtype] = None,
                checkpoint: Optional[str] = None, seed: int = 0, tp: Optional[int] = None,
                rank: Optional[int] = None, weight_dtype: Optional[str] = None):
    """weight_dtype "fp8" / "int8" / "int4": also keep quantized weight copies for
    decode batches <= 64 (LlamaForCausalLM.quantize_weights); activations and
    everything else stay `dtype`."""
    if dtype is None:
        dtype = torch.float32 if (cfg.dtype == "float32" and torch.device(device).type == "cpu") else torch.bfloat16
    if checkpoint:
        _resolve_shapes(cfg, checkpoint)
    m = model_class(cfg)(cfg, device=device, dtype=dtype, tp=tp, rank=rank)
    if checkpoint:
        load_checkpoint(m, checkpoint)
    else:
        m.random_init(seed)
    if hasattr(m, "fold_norms"):
        m.fold_norms()  # RMSNorm weights into the projections (fused decode layer)
    if weight_dtype in ("fp8", "int8", "int4"):
        if not (hasattr(m, "quantize_weights") and m.quantize_weights(weight_dtype)):
            raise ValueError(f"{weight_dtype} weights are not supported for {cfg.name} on {device}")
    elif weight_dtype not in (None, "bf16", "fp16", "fp32"):
        raise ValueError(f"unknown weight_dtype {weight_dtype!r}")
    m.eval()
    return m


class _Reader:
    def __init__(self, path: str):
        from safetensors import safe_open
        self.path = path
        idx = os.path.join(path, "model.safetensors.index.json")
        files = {}
        if os.path.exists(idx):
            with open(idx) as f:
                wm = json.load(f)["weight_map"]
            for name, fn in wm.items():
                files.setdefault(fn, []).append(name)
        else:
            for fn in sorted(os.listdir(path)):
                if fn.endswith(".safetensors"):
                    files[fn] = None
        self.handles = {fn: safe_open(os.path.join(path, fn), framework="pt") for fn in files}
        self.where: Dict[str, str] = {}
        for fn, h in self.handles.items():
            for k in h.keys():
                self.where[k] = fn

    def has(self, name: str) -> bool:
        return name in self.where

    def shape(self, name: str):
        if name not in self.where:
            raise KeyError(f"missing tensor {name!r} in checkpoint {self.path}")
        return tuple(self.handles[self.where[name]].get_slice(name).get_shape())

    def get(self, name: str, dim: Optional[int] = None, start: int = 0, length: Optional[int] = None) -> torch.Tensor:
        if name not in self.where:
            raise KeyError(f"missing tensor {name!r} in checkpoint {self.path}")
        if dim is None:
            return self.handles[self.where[name]].get_tensor(name)   # (also a tensor without dimensions)
        sl = self.handles[self.where[name]].get_slice(name)
        shape = sl.get_shape()
        end = start + (length if length is not None else shape[dim] - start)
        idx = [slice(None)] * len(shape)
        idx[dim] = slice(start, end)
        return sl[tuple(idx)]


def _copy(dst: torch.nn.Parameter, src: torch.Tensor, name: str):
    if tuple(dst.shape) != tuple(src.shape):
        raise ValueError(f"shape mismatch for {name}: model {tuple(dst.shape)} vs checkpoint {tuple(src.shape)}")
    dst.data.copy_(src.to(dst.dtype))


@torch.no_grad()
def load_checkpoint(model, path: str) -> None:
    r = _Reader(path)
    cfg = model.cfg
    if cfg.arch == "gpt2":
        _load_gpt2(model, r)
    elif cfg.arch == "dofivik":
        _load_dofivik(model, r)
    elif cfg.arch == "vizonex":
        _load_vizonex(model, r)
    elif cfg.arch == "loluzen":
        _load_loluzen(model, r)
    elif cfg.arch == "lotelix":
        _load_lotelix(model, r)
    else:
        _load_llama(model, r)


def _pre(r: _Reader) -> str:
    return "model." if r.has("model.embed_tokens.weight") else ""


def _load_llama(m, r: _Reader):
    cfg, tp, rank = m.cfg, m.tp, m.rank
    D, H = cfg.head_dim, cfg.hidden_size
    p = _pre(r)
    _copy(m.embed, r.get(f"{p}embed_tokens.weight"), "embed")
    _copy(m.norm, r.get(f"{p}norm.weight"), "norm")
    if m.lm_head is not None:
        name = "lm_head.weight" if r.has("lm_head.weight") else f"{p}embed_tokens.weight"
        V = cfg.vocab_size
        per = m.V_pad // tp
        lo = rank * per
        n = max(0, min(per, V - lo))
        w = torch.zeros(per, H)
        if n > 0:
            w[:n] = r.get(name, 0, lo, n).float()
        _copy(m.lm_head, w, "lm_head")
    Hq_l = cfg.num_heads // tp
    kv0, nkv = kv_head_range(cfg, tp, rank)
    for i, L in enumerate(m.layers):
        b = f"{p}layers.{i}."
        _copy(L.input_norm, r.get(b + "input_layernorm.weight"), "input_norm")
        _copy(L.post_norm, r.get(b + "post_attention_layernorm.weight"), "post_norm")
        q = r.get(b + "self_attn.q_proj.weight", 0, rank * Hq_l * D, Hq_l * D)
        k = r.get(b + "self_attn.k_proj.weight", 0, kv0 * D, nkv * D)
        v = r.get(b + "self_attn.v_proj.weight", 0, kv0 * D, nkv * D)
        _copy(L.qkv, torch.cat([q, k, v], 0), f"layer{i}.qkv")
        _copy(L.o, r.get(b + "self_attn.o_proj.weight", 1, rank * Hq_l * D, Hq_l * D), f"layer{i}.o")
        if L.moe:
            _copy(L.router, r.get(b + "block_sparse_moe.gate.weight"), "router")
            for el in range(L.E_local):
                e = L.expert_offset + el
                eb = b + f"block_sparse_moe.experts.{e}."
                L.w13.data[el].copy_(interleave_gate_up(r.get(eb + "w1.weight"), r.get(eb + "w3.weight")).to(L.w13.dtype))
                L.w2.data[el].copy_(r.get(eb + "w2.weight").to(L.w2.dtype))
        else:
            Fl = cfg.intermediate_size // tp
            g = r.get(b + "mlp.gate_proj.weight", 0, rank * Fl, Fl)
            u = r.get(b + "mlp.up_proj.weight", 0, rank * Fl, Fl)
            _copy(L.gate_up, interleave_gate_up(g, u), f"layer{i}.gate_up")
            _copy(L.down, r.get(b + "mlp.down_proj.weight", 1, rank * Fl, Fl), f"layer{i}.down")


def _load_gpt2(m, r: _Reader):
    p = "transformer." if r.has("transformer.wte.weight") else ""
    _copy(m.wte, r.get(p + "wte.weight"), "wte")
    _copy(m.wpe, r.get(p + "wpe.weight"), "wpe")
    _copy(m.lnf_w, r.get(p + "ln_f.weight"), "ln_f")
    _copy(m.lnf_b, r.get(p + "ln_f.bias"), "ln_f.b")
    for i, L in enumerate(m.layers):
        b = f"{p}h.{i}."
        _copy(L.ln1_w, r.get(b + "ln_1.weight"), "ln1")
        _copy(L.ln1_b, r.get(b + "ln_1.bias"), "ln1b")
        _copy(L.ln2_w, r.get(b + "ln_2.weight"), "ln2")
        _copy(L.ln2_b, r.get(b + "ln_2.bias"), "ln2b")
        # HF GPT-2 uses Conv1D ([in, out]) -> transpose to the nn.Linear layout
        _copy(L.qkv_w, r.get(b + "attn.c_attn.weight").t(), "c_attn")
        _copy(L.qkv_b, r.get(b + "attn.c_attn.bias"), "c_attn.b")
        _copy(L.o_w, r.get(b + "attn.c_proj.weight").t(), "c_proj")
        _copy(L.o_b, r.get(b + "attn.c_proj.bias"), "c_proj.b")
        _copy(L.fc_w, r.get(b + "mlp.c_fc.weight").t(), "c_fc")
        _copy(L.fc_b, r.get(b + "mlp.c_fc.bias"), "c_fc.b")
        _copy(L.proj_w, r.get(b + "mlp.c_proj.weight").t(), "mlp.c_proj")
        _copy(L.proj_b, r.get(b + "mlp.c_proj.bias"), "mlp.c_proj.b")


def _dofivik_tensors(m):
    """(checkpoint name, parameter, row range of a fused parameter or None) for every tensor."""
    out = [("embed", m.embed, None), ("head", m.head, None), ("final.norm", m.final_norm, None)]
    for i, L in enumerate(m.layers):
        b, x = f"l{i}.", L.mix
        out += [(b + "norm1", L.norm1, None), (b + "canon1", L.canon1, None)]
        if L.kind == "latent_attention":
            out += [(b + "mix.dq", x.in_proj, (0, x.Rq)), (b + "mix.dq.norm", x.q_norm, None),
                    (b + "mix.g", x.in_proj, (x.off_g, x.off_g + x.H)), (b + "mix.uq", x.uq, None),
                    (b + "mix.uk", x.uk, None), (b + "mix.uv", x.uv, None), (b + "mix.o", x.o, None)]
            if x.own_kv:
                out += [(b + "mix.dkv", x.in_proj, (x.off_kv, x.off_kv + x.R + x.rd)), (b + "mix.dkv.norm", x.kv_norm, None)]
        else:
            HD = x.HD
            for j, n in enumerate(("r", "k", "v", "g", "a")):
                out.append((b + "mix." + n, x.in_proj, (j * HD, (j + 1) * HD)))
            out += [(b + "mix.w1", x.in_proj, (5 * HD, 5 * HD + x.lr)), (b + "mix.w2", x.w2, None),
                    (b + "mix.w0", x.w0, None), (b + "mix.a.b", x.a_bias, None), (b + "mix.norm", x.norm, None),
                    (b + "mix.o", x.o, None)]
        if L.mlp is not None:
            out += [(b + "norm2", L.norm2, None), (b + "canon2", L.canon2, None), (b + "mlp.up", L.mlp.up, None),
                    (b + "mlp.up.b", L.mlp.up_b, None), (b + "mlp.down", L.mlp.down, None),
                    (b + "mlp.down.b", L.mlp.down_b, None), (b + "mlp.act", L.mlp.act, None)]
    return out


def _load_dofivik(m, r: _Reader):
    """Tensors `l<i>.<norm1|norm2|canon1|canon2>`, `l<i>.mix.*`, `l<i>.mlp.*`, `embed`, `final.norm`, `head`
    ([out, in] matrices); the projections that read the same input are fused row-wise on load."""
    for name, p, rows in _dofivik_tensors(m):
        src = r.get(name)
        dst = p.data if rows is None else p.data[rows[0]:rows[1]]
        if tuple(dst.shape) != tuple(src.shape):
            raise ValueError(f"shape mismatch for {name}: model {tuple(dst.shape)} vs checkpoint {tuple(src.shape)}")
        dst.copy_(src.to(dst.dtype))
    m.finalize_weights()


def _vizonex_tensors(m):
    """(checkpoint name, parameter, index of a fused / stacked parameter or None) for every tensor."""
    out = [("embed", m.embed, None), ("pos", m.pos, None), ("head", m.head, None), ("final.norm", m.final_norm, None)]

    def glu(pre, mod):
        F_ = mod.ff
        return [(pre + "gate", mod.gate_up, slice(0, F_)), (pre + "up", mod.gate_up, slice(F_, 2 * F_)),
                (pre + "down", mod.down, None)]
    for i, L in enumerate(m.layers):
        b, x = f"l{i}.", L.mix
        out += [(b + "norm1", L.norm1, None), (b + "ls1", L.ls1, None), (b + "canon1", L.canon1, None)]
        if L.kind == "attention":
            out += [(b + "mix.q", x.qkv, slice(0, x.nq)), (b + "mix.k", x.qkv, slice(x.nq, x.nq + x.nk)),
                    (b + "mix.v", x.qkv, slice(x.nq + x.nk, x.nq + x.nk + x.nv)), (b + "mix.q.norm", x.q_norm, None),
                    (b + "mix.k.norm", x.k_norm, None), (b + "mix.temp", x.temp, None), (b + "mix.sink", x.sink, None),
                    (b + "mix.o", x.o, None)]
        else:
            out += [(b + "mix.in", x.in_proj, None), (b + "mix.conv", x.conv_w, None), (b + "mix.conv.b", x.conv_b, None),
                    (b + "mix.dt_bias", x.dt_bias, None), (b + "mix.A_log", x.A_log, None), (b + "mix.D", x.D, None),
                    (b + "mix.norm", x.norm, None), (b + "mix.o", x.o, None)]
        if L.mlp is None:
            continue
        out.append((b + "ls2", L.ls2, None))
        if not L.moe:
            out += glu(b + "mlp.", L.mlp)
            continue
        F_ = L.mlp.ff
        out += [(b + "mlp.router", L.mlp.router, None), (b + "mlp.correction", L.mlp.correction, None)]
        for e in range(L.mlp.E):
            out += [(f"{b}mlp.e{e}.gate", L.mlp.w13, (e, slice(0, F_))), (f"{b}mlp.e{e}.up", L.mlp.w13, (e, slice(F_, 2 * F_))),
                    (f"{b}mlp.e{e}.down", L.mlp.w2, e)]
        if L.mlp.shared is not None:
            out += glu(b + "mlp.shared.", L.mlp.shared)
    return out


def _load_vizonex(m, r: _Reader):
    """Tensors `embed`, `pos`, `head`, `final.norm`, `l<i>.<norm1|ls1|ls2|canon1>`, `l<i>.mix.*`, `l<i>.mlp.*`
    ([out, in] matrices). q / k / v and gate / up are fused row-wise, the experts stacked, on load."""
    for name, p, idx in _vizonex_tensors(m):
        src = r.get(name)
        dst = p.data if idx is None else p.data[idx]
        if tuple(dst.shape) != tuple(src.shape):
            raise ValueError(f"shape mismatch for {name}: model {tuple(dst.shape)} vs checkpoint {tuple(src.shape)}")
        dst.copy_(src.to(dst.dtype))


def _loluzen_tensors(m):
    """(checkpoint name, parameter, index of a fused parameter or None) for every tensor."""
    out = [("embed", m.embed, None), ("head", m.head, None), ("final.norm", m.final_norm, None)]
    for i, L in enumerate(m.layers):
        b, x = f"l{i}.", L.mix
        out += [(b + "norm1", L.norm1, None), (b + "norm1b", L.norm1b, None)]
        if L.kind == "attention":
            nq, nk, nv = x.nq, x.nk, x.nv
            out += [(b + "mix.q", x.in_proj, slice(0, nq)), (b + "mix.k", x.in_proj, slice(nq, nq + nk)),
                    (b + "mix.v", x.in_proj, slice(nq + nk, x.ch)), (b + "mix.g", x.in_proj, slice(x.ch, x.ch + x.H)),
                    (b + "mix.q.conv", x.conv_w, slice(0, nq)), (b + "mix.k.conv", x.conv_w, slice(nq, nq + nk)),
                    (b + "mix.v.conv", x.conv_w, slice(nq + nk, x.ch)), (b + "mix.q.norm", x.q_norm, None),
                    (b + "mix.k.norm", x.k_norm, None), (b + "mix.o", x.o, None)]
        else:
            a, r = x.left, x.right
            at = 0
            for name, rows, bias in (("left.q", a.nq, True), ("left.k", a.nk, True), ("left.v", a.nv, True),
                                     ("left.g", a.H, False), ("right.q", r.n, False), ("right.f", r.n, True),
                                     ("right.v", r.H * r.dv, False)):
                out.append((b + "mix." + name, x.in_proj, slice(at, at + rows)))
                if bias:
                    out.append((b + "mix." + name + ".b", x.in_bias, slice(at, at + rows)))
                at += rows
            out += [(b + "mix.left.r1", a.r1, None), (b + "mix.left.r2", a.r2, None), (b + "mix.left.talk", a.talk, None),
                    (b + "mix.left.o", a.o, None), (b + "mix.left.out", a.out_norm, None),
                    (b + "mix.right.lower", r.lower, None), (b + "mix.right.norm", r.norm, None),
                    (b + "mix.right.o", r.o, None), (b + "mix.right.out", r.out_norm, None)]
        if L.mlp is not None:
            out += [(b + "norm2", L.norm2, None), (b + "norm2b", L.norm2b, None), (b + "mlp.up", L.mlp.up, None),
                    (b + "mlp.up.b", L.mlp.up_b, None), (b + "mlp.down", L.mlp.down, None),
                    (b + "mlp.down.b", L.mlp.down_b, None)]
    return out


def _load_loluzen(m, r: _Reader):
    """Tensors `embed`, `head`, `final.norm`, `l<i>.<norm1|norm1b|norm2|norm2b>`, `l<i>.mix.*`, `l<i>.mlp.*`
    ([out, in] matrices). The projections that read the same input (and their biases) are fused row-wise on load."""
    for name, p, idx in _loluzen_tensors(m):
        src = r.get(name)
        dst = p.data if idx is None else p.data[idx]
        if tuple(dst.shape) != tuple(src.shape):
            raise ValueError(f"shape mismatch for {name}: model {tuple(dst.shape)} vs checkpoint {tuple(src.shape)}")
        dst.copy_(src.to(dst.dtype))


def _save_loluzen(model, path: str) -> None:
    from safetensors.torch import save_file
    cfg = model.cfg
    t = {}
    for name, p, idx in _loluzen_tensors(model):
        v = p.data if idx is None else p.data[idx]
        t[name] = v.detach().to(torch.bfloat16).contiguous().cpu()
    save_file(t, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump({"architecture": "Loluzen", "width": cfg.hidden_size, "vocab": cfg.vocab_size,
                   "embedding": {"scale": cfg.embed_scale}, "residual_mult": cfg.residual_mult,
                   "layers": cfg.layer_specs, "loop": cfg.layer_loop, "norm": {"eps": cfg.norm_eps},
                   "max_position": cfg.max_position}, f, indent=1)


def _lotelix_tensors(m):
    """(checkpoint name, parameter, index of a fused / stacked parameter or None) for every tensor."""
    out = [("embed", m.embed, None), ("head", m.head, None), ("final.norm", m.final_norm, None)]
    for i, L in enumerate(m.layers):
        b, x = f"l{i}.", L.mix
        out.append((b + "norm1", L.norm1, None))
        if L.kind == "mingru":
            n = x.n
            out += [(b + "mix.z", x.in_proj, slice(0, n)), (b + "mix.x", x.in_proj, slice(n, 2 * n)),
                    (b + "mix.g", x.in_proj, slice(2 * n, 3 * n)), (b + "mix.z.b", x.z_b, None),
                    (b + "mix.x.b", x.x_b, None), (b + "mix.o", x.o, None)]
        elif L.kind == "attention":
            nq, nk = x.nq, x.nk
            out += [(b + "mix.q", x.in_proj, slice(0, nq)), (b + "mix.k", x.in_proj, slice(nq, nq + nk)),
                    (b + "mix.v", x.in_proj, slice(nq + nk, x.ch)), (b + "mix.g", x.in_proj, slice(x.ch, x.ch + x.H * x.dv)),
                    (b + "mix.sink", x.sink, None), (b + "mix.o", x.o, None)]
            if x.v_mix:
                out.append((b + "mix.vmix", x.lam, "scalar"))
        else:
            a, r = x.left, x.right
            at = 0
            for name, rows, bias in (("left.q", a.nq, True), ("left.k", a.nk, True), ("left.v", a.nv, True),
                                     ("right.q", r.n, False), ("right.k", r.n, False), ("right.v", r.nv, False),
                                     ("right.g", r.nv, False), ("right.a1", r.rank, False)):
                out.append((b + "mix." + name, x.in_proj, slice(at, at + rows)))
                if bias:
                    out.append((b + "mix." + name + ".b", x.in_bias, slice(at, at + rows)))
                at += rows
            out += [(b + "mix.left.q.norm", a.q_norm, None), (b + "mix.left.k.norm", a.k_norm, None),
                    (b + "mix.left.pb", a.pb, None), (b + "mix.left.o", a.o, None), (b + "mix.left.o.b", a.o_b, None),
                    (b + "mix.left.out", a.out_norm, None), (b + "mix.right.a2", r.a2, None),
                    (b + "mix.right.a2.b", r.a2_b, None), (b + "mix.right.norm", r.norm, None),
                    (b + "mix.right.o", r.o, None), (b + "mix.right.out", r.out_norm, None)]
        if L.mlp is not None:
            out += [(b + "norm2", L.norm2, None), (b + "mlp.router", L.mlp.router, None)]
            for e in range(L.mlp.E):
                out += [(f"{b}mlp.e{e}.up", L.mlp.up, e), (f"{b}mlp.e{e}.down", L.mlp.down, e)]
    return out


def _load_lotelix(m, r: _Reader):
    """Tensors `embed`, `head`, `final.norm`, `l<i>.<norm1|norm2>`, `l<i>.mix.*`, `l<i>.mlp.*` ([out, in] matrices).
    The projections that read the same input (and their biases) are fused row-wise, the experts stacked, on load."""
    for name, p, idx in _lotelix_tensors(m):
        src = r.get(name)
        if idx == "scalar":
            src, idx = src.reshape(1), None
        dst = p.data if idx is None else p.data[idx]
        if tuple(dst.shape) != tuple(src.shape):
            raise ValueError(f"shape mismatch for {name}: model {tuple(dst.shape)} vs checkpoint {tuple(src.shape)}")
        dst.copy_(src.to(dst.dtype))


def _save_lotelix(model, path: str) -> None:
    from safetensors.torch import save_file
    cfg = model.cfg
    t = {}
    for name, p, idx in _lotelix_tensors(model):
        v = p.data.reshape(()) if idx == "scalar" else p.data if idx is None else p.data[idx]
        t[name] = v.detach().to(torch.bfloat16).contiguous().cpu()
    save_file(t, os.path.join(path, "model.safetensors"))
    layers = []
    for spec in cfg.layer_specs:
        mx = dict(spec["mixer"])
        if spec["type"] == "parallel":   # the rank of the decay projection is given by a tensor's shape
            mx["right"] = {k: v for k, v in mx["right"].items() if k != "decay_rank"}
        layers.append({"type": spec["type"], "mixer": mx, "mlp": spec.get("mlp")})
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump({"architecture": "Lotelix", "width": cfg.hidden_size, "vocab": cfg.vocab_size,
                   "embedding": {"scale": cfg.embed_scale}, "layers": layers,
                   "norm": {"eps": cfg.norm_eps, "groups": cfg.norm_groups}, "max_position": cfg.max_position}, f, indent=1)


def _save_vizonex(model, path: str) -> None:
    from safetensors.torch import save_file
    cfg = model.cfg
    t = {}
    for name, p, idx in _vizonex_tensors(model):
        v = p.data if idx is None else p.data[idx]
        t[name] = v.detach().to(torch.bfloat16).contiguous().cpu()
    save_file(t, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump({"architecture": "Vizonex", "width": cfg.hidden_size, "vocab": cfg.vocab_size,
                   "layers": cfg.layer_specs, "canon": {"taps": cfg.canon_taps}, "norm": {"eps": cfg.norm_eps},
                   "max_positions": cfg.max_position}, f, indent=1)


def _save_dofivik(model, path: str) -> None:
    from safetensors.torch import save_file
    cfg = model.cfg
    t = {}
    for name, p, rows in _dofivik_tensors(model):
        v = p.data if rows is None else p.data[rows[0]:rows[1]]
        t[name] = v.detach().to(torch.bfloat16).contiguous().cpu()
    save_file(t, os.path.join(path, "model.safetensors"))
    layers = []
    for spec in cfg.layer_specs:
        mx = {k: v for k, v in spec["mixer"].items() if k != "decay_rank"}
        layers.append({"type": spec["type"], "mixer": mx, "mlp": spec.get("mlp")})
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump({"architecture": "Dofivik", "width": cfg.hidden_size, "vocab": cfg.vocab_size, "layers": layers,
                   "postln_alpha": cfg.postln_alpha, "canon": {"taps": cfg.canon_taps},
                   "norm": {"eps": cfg.norm_eps}}, f, indent=1)


@torch.no_grad()
def save_checkpoint(model, path: str) -> None:
    """Write a TP=1 model in HF layout (safetensors + config.json)."""
    from safetensors.torch import save_file
    assert model.tp == 1, "save from a TP=1 model"
    cfg = model.cfg
    os.makedirs(path, exist_ok=True)
    if cfg.arch == "dofivik":
        return _save_dofivik(model, path)
    if cfg.arch == "vizonex":
        return _save_vizonex(model, path)
    if cfg.arch == "loluzen":
        return _save_loluzen(model, path)
    if cfg.arch == "lotelix":
        return _save_lotelix(model, path)
    t: Dict[str, torch.Tensor] = {}
    if cfg.arch == "gpt2":
        t["transformer.wte.weight"] = model.wte
        t["transformer.wpe.weight"] = model.wpe
        t["transformer.ln_f.weight"] = model.lnf_w
        t["transformer.ln_f.bias"] = model.lnf_b
        for i, L in enumerate(model.layers):
            b = f"transformer.h.{i}."
            t[b + "ln_1.weight"], t[b + "ln_1.bias"] = L.ln1_w, L.ln1_b
            t[b + "ln_2.weight"], t[b + "ln_2.bias"] = L.ln2_w, L.ln2_b
            t[b + "attn.c_attn.weight"], t[b + "attn.c_attn.bias"] = L.qkv_w.t(), L.qkv_b
            t[b + "attn.c_proj.weight"], t[b + "attn.c_proj.bias"] = L.o_w.t(), L.o_b
            t[b + "mlp.c_fc.weight"], t[b + "mlp.c_fc.bias"] = L.fc_w.t(), L.fc_b
            t[b + "mlp.c_proj.weight"], t[b + "mlp.c_proj.bias"] = L.proj_w.t(), L.proj_b
        hf = {"model_type": "gpt2", "n_embd": cfg.hidden_size, "n_layer": cfg.num_layers, "n_head": cfg.num_heads,
              "n_inner": cfg.intermediate_size, "vocab_size": cfg.vocab_size, "n_positions": cfg.max_position,
              "layer_norm_epsilon": cfg.norm_eps, "bos_token_id": cfg.bos_token_id,
              "eos_token_id": cfg.eos_token_ids[0]}
    else:
        D = cfg.head_dim
        qs, ks = cfg.num_heads * D, cfg.num_kv_heads * D
        t["model.embed_tokens.weight"] = model.embed
        t["model.norm.weight"] = model.norm
        if model.lm_head is not None:
            t["lm_head.weight"] = model.lm_head[:cfg.vocab_size]
        for i, L in enumerate(model.layers):
            b = f"model.layers.{i}."
            t[b + "input_layernorm.weight"] = L.input_norm
            t[b + "post_attention_layernorm.weight"] = L.post_norm
            t[b + "self_attn.q_proj.weight"] = L.qkv[:qs]
            t[b + "self_attn.k_proj.weight"] = L.qkv[qs:qs + ks]
            t[b + "self_attn.v_proj.weight"] = L.qkv[qs + ks:]
            t[b + "self_attn.o_proj.weight"] = L.o
            if L.moe:
                Fd = cfg.intermediate_size
                t[b + "block_sparse_moe.gate.weight"] = L.router
                for e in range(cfg.num_experts):
                    eb = b + f"block_sparse_moe.experts.{e}."
                    t[eb + "w1.weight"], t[eb + "w3.weight"] = deinterleave_gate_up(L.w13[e])
                    t[eb + "w2.weight"] = L.w2[e]
            else:
                Fd = cfg.intermediate_size
                gw, uw = deinterleave_gate_up(L.gate_up)
                t[b + "mlp.gate_proj.weight"] = gw
                t[b + "mlp.up_proj.weight"] = uw
                t[b + "mlp.down_proj.weight"] = L.down
        hf = {"model_type": "mixtral" if cfg.arch == "mixtral" else "llama", "hidden_size": cfg.hidden_size,
              "num_hidden_layers": cfg.num_layers, "num_attention_heads": cfg.num_heads,
              "num_key_value_heads": cfg.num_kv_heads, "head_dim": cfg.head_dim,
              "intermediate_size": cfg.intermediate_size, "vocab_size": cfg.vocab_size,
              "max_position_embeddings": cfg.max_position, "rope_theta": cfg.rope_theta,
              "rope_scaling": cfg.rope_scaling, "rms_norm_eps": cfg.norm_eps,
              "tie_word_embeddings": cfg.tie_embeddings, "bos_token_id": cfg.bos_token_id,
              "eos_token_id": cfg.eos_token_ids}
        if cfg.arch == "mixtral":
            hf["num_local_experts"] = cfg.num_experts
            hf["num_experts_per_tok"] = cfg.experts_per_token
    save_file({k: v.detach().contiguous().cpu() for k, v in t.items()}, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(hf, f, indent=1)
