"""Loluzen: a decoder whose sublayers are wrapped in two norms (input norm and output norm), on the paged / slotted engine.

    x_0 = embed[token] * s                                           (s = cfg.embed_scale)
    x  <- x + m * N(mixer(N(x; norm1)); norm1b)                      (m = cfg.residual_mult)
    x  <- x + m * N(ff(N(x; norm2)); norm2b)                         N(v; w) = v / rms(v) * (1 + w)

A configured run of layers may repeat with the same weights; every repetition is a *layer run* with a cache
and state of its own, and every repetition after the first starts from x + x_0. The residual stream x is
fp32 throughout; the post-norm, the residual sum and the next sublayer's input norm run in one kernel.

Mixers (reusable modules, every constant a parameter):
  * `ConvRopeAttention` ("attention"): grouped-query attention whose q / k / v pass a short causal depthwise
    convolution right after the projection, then a per-head RMS norm (q, k), then a rotation of the first
    rot.dims entries of each head (interleaved pairs, frequencies rescaled by wavelength); causal softmax; each
    head's output times the sigmoid of a gate logit projected from the mixer's input.
  * `TalkingDistanceAttention` + `LowerBoundRecurrence` ("parallel"): two branches reading the same input. Left:
    biased q / k / v, no rotation, score - r1_h ln(1 + r2_h (i - j)), causal softmax, the heads' weight maps mixed
    by a matrix AFTER the softmax, gate as above. Right: a gated linear recurrence S <- diag(f) S + (1 - f) v^T,
    o = S^T q on an fp32 [dim x vdim] state per head and slot, with q = silu(.) and f bounded below per channel;
    o RMS-normed per head. The mixer's output is the mean of the two branches, each RMS-normed over the width.
Feed-forward: `Relu2MLP`, W_down relu(W_up h + b)^2 + b.

What a sequence carries between steps (ModelRunner allocates it through alloc_cache), per layer run: K / V pages;
per state slot the last taps - 1 projected q / k / v rows of an "attention" mixer's convolution and the recurrent
state of a "parallel" mixer.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..ops import seqmix as sq
from ..parallel.state import get_state
from .base import AttnMeta
from .config import ModelConfig
from .seq_cache import LayerCache, SeqCache


def _p(t):
    return nn.Parameter(t, requires_grad=False)


class ConvRopeAttention(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, device, dtype):
        super().__init__()
        e = lambda *s: torch.empty(*s, device=device, dtype=dtype)  # noqa: E731
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.H, self.G, self.dk, self.dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        self.taps, self.scale, self.eps = int(m.get("conv", 1)), float(m["scale"]), eps
        rot = m.get("rot") or {}
        self.rot_dims, self.rot_base, self.rot_scaling = int(rot.get("dims", 0)), float(rot.get("base", 1.0)), rot.get("scaling")
        self.nq, self.nk, self.nv = self.H * self.dk, self.G * self.dk, self.G * self.dv
        self.ch = self.nq + self.nk + self.nv               # channels of the short convolution: [q | k | v]
        self.in_proj = _p(e(self.ch + self.H, width))        # fused rows [q | k | v | gate]
        self.conv_w = _p(f(self.ch, self.taps))
        self.q_norm, self.k_norm = _p(f(self.dk)), _p(f(self.dk))
        self.o = _p(e(width, self.H * self.dv))

    def rot_key(self):
        if self.rot_dims == 0:
            return None
        sc = self.rot_scaling
        return (self.rot_dims, self.rot_base, None if sc is None else tuple(sorted((k, float(v)) for k, v in sc.items())))

    def forward(self, h, sm: sq.SeqMeta, lc: LayerCache, block_size: int, rot):
        proj = F.linear(h, self.in_proj)
        q = sq.conv_head_norm_rope_cache(proj, self.conv_w, lc.mix_conv, self.H, self.G, self.dk, self.dv, self.q_norm,
                                         self.k_norm, self.eps, rot, self.rot_dims, sm, lc.k, lc.v)
        o = sq.masked_attention(q, lc.k, lc.v, self.H, self.G, self.dk, self.dv, sq.MASK_CAUSAL, 0, self.scale, None,
                                None, block_size, sm, gate=proj[:, self.ch:])
        return F.linear(o, self.o)


class TalkingDistanceAttention(nn.Module):
    """The attention branch of the "parallel" mixer; its projection rows live in the mixer's fused input matrix."""

    def __init__(self, width: int, m: dict, device, dtype):
        super().__init__()
        e = lambda *s: torch.empty(*s, device=device, dtype=dtype)  # noqa: E731
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.H, self.G, self.dk, self.dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        self.scale = float(m["scale"])
        self.nq, self.nk, self.nv = self.H * self.dk, self.G * self.dk, self.G * self.dv
        self.rows = self.nq + self.nk + self.nv + self.H     # [q | k | v | gate]
        self.r1, self.r2 = _p(f(self.H)), _p(f(self.H))
        self.talk = _p(f(self.H, self.H))
        self.o = _p(e(width, self.H * self.dv))
        self.out_norm = _p(f(width))

    def forward(self, proj, sm: sq.SeqMeta, lc: LayerCache, block_size: int):
        H, G, dv = self.H, self.G, self.dv
        n = self.nq + self.nk + self.nv
        q = sq.qk_norm_cache(proj[:, :n], self.nq, self.nk, self.nv, None, None, 0.0, sm, lc.k, lc.v)
        kw = dict(gate=None, dist=(self.r1, self.r2))
        args = (q, lc.k, lc.v, H, G, self.dk, dv, sq.MASK_CAUSAL, 0, self.scale, None, None, block_size, sm)
        if G * dv <= sq.V_ALL_MAX:
            wide = sq.masked_attention(*args, values=sq.V_ALL, **kw)
        else:   # one pass per value head
            wide = torch.stack([sq.masked_attention(*args, values=c, **kw).view(-1, H, dv) for c in range(G)], 2)
            wide = wide.reshape(-1, H * G * dv)
        o = sq.talk_mix(wide, self.talk, H, G, dv, gate=proj[:, n:n + H])
        return F.linear(o, self.o)


class LowerBoundRecurrence(nn.Module):
    """The recurrent branch of the "parallel" mixer (rows [q | f | v] of the fused input matrix)."""

    def __init__(self, width: int, m: dict, eps: float, device, dtype):
        super().__init__()
        e = lambda *s: torch.empty(*s, device=device, dtype=dtype)  # noqa: E731
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.H, self.dk, self.dv, self.eps = int(m["heads"]), int(m["dim"]), int(m["vdim"]), eps
        self.n = self.H * self.dk
        self.rows = 2 * self.n + self.H * self.dv
        self.lower = _p(f(self.n))
        self.norm = _p(f(self.dv))
        self.o = _p(e(width, self.H * self.dv))
        self.out_norm = _p(f(width))

    def forward(self, proj, sm: sq.SeqMeta, lc: LayerCache):
        n = self.n
        # the gate's bias is in the projection
        o = sq.lower_bound_recurrence(proj, 0, n, 2 * n, None, self.lower, lc.gla, self.H, self.dk, self.dv, sm)
        return F.linear(sq.gated_group_norm(o, None, self.norm, self.eps, self.H, proj.dtype), self.o)


class ParallelMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, device, dtype):
        super().__init__()
        self.left = TalkingDistanceAttention(width, m["left"], device, dtype)
        self.right = LowerBoundRecurrence(width, m["right"], eps, device, dtype)
        rows = self.left.rows + self.right.rows
        self.in_proj = _p(torch.empty(rows, width, device=device, dtype=dtype))   # [left q k v gate | right q f v]
        self.in_bias = _p(torch.zeros(rows, device=device, dtype=dtype))

    def forward(self, h, sm: sq.SeqMeta, lc: LayerCache, block_size: int):
        """The two branch outputs (their norms and mean join the residual update)."""
        proj = F.linear(h, self.in_proj, self.in_bias)
        return self.left(proj[:, :self.left.rows], sm, lc, block_size), self.right(proj[:, self.left.rows:], sm, lc)


class Relu2MLP(nn.Module):
    def __init__(self, width: int, ff: int, device, dtype):
        super().__init__()
        self.ff = int(ff)
        self.up = _p(torch.empty(self.ff, width, device=device, dtype=dtype))
        self.up_b = _p(torch.zeros(self.ff, device=device, dtype=torch.float32))
        self.down = _p(torch.empty(width, self.ff, device=device, dtype=dtype))
        self.down_b = _p(torch.zeros(width, device=device, dtype=torch.float32))

    def forward(self, h):
        """W_down relu(W_up h + b)^2; the output bias down_b is added by the residual update."""
        return F.linear(sq.relu2(F.linear(h, self.up), self.up_b), self.down)


class LoluzenLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, spec: dict, device, dtype):
        super().__init__()
        W = cfg.hidden_size
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.kind, self.eps, self.mult = spec["type"], cfg.norm_eps, cfg.residual_mult
        if self.kind == "attention":
            self.mix = ConvRopeAttention(W, spec["mixer"], cfg.norm_eps, device, dtype)
        else:
            self.mix = ParallelMixer(W, spec["mixer"], cfg.norm_eps, device, dtype)
        self.norm1, self.norm1b = _p(f(W)), _p(f(W))
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            self.norm2, self.norm2b = _p(f(W)), _p(f(W))
            self.mlp = Relu2MLP(W, mlp["ff"], device, dtype)

    def forward(self, x, n, sm: sq.SeqMeta, lc: LayerCache, block_size: int, rot, extra, next_norm):
        """x: fp32 residual (updated in place); n: N(x; norm1) as an activation tensor. `extra` (fp32 rows or None)
        is added to x after the layer; returns N(x; next_norm) of the result."""
        dt, last = n.dtype, self.mlp is None
        after = (extra, next_norm) if last else (None, self.norm2)
        if self.kind == "attention":
            y = self.mix(n, sm, lc, block_size, rot)
            n = sq.post_norm_residual(x, y, None, self.norm1b, self.mult, after[0], after[1], self.eps, dt)
        else:
            ya, yb = self.mix(n, sm, lc, block_size)
            n = sq.post_norm_residual(x, ya, None, self.norm1b, self.mult, after[0], after[1], self.eps, dt, y2=yb,
                                      pre_w=(self.mix.left.out_norm, self.mix.right.out_norm))
        if not last:
            n = sq.post_norm_residual(x, self.mlp(n), self.mlp.down_b, self.norm2b, self.mult, extra, next_norm,
                                      self.eps, dt)
        return n


class LoluzenForCausalLM(nn.Module):
    has_sequence_state = True   # recurrent / convolution state per slot: no prefix reuse, no draft verification

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, tp: Optional[int] = None,
                 rank: Optional[int] = None):
        super().__init__()
        tp = get_state().tp_size if tp is None else tp
        if tp != 1:
            raise ValueError("Loluzen runs with tp=1 (use DP replicas to scale)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Loluzen runs in bfloat16 or float32")
        self.cfg, self.tp, self.rank = cfg, 1, 0
        self.device, self.dtype = torch.device(device), dtype
        W = cfg.hidden_size
        self.embed = _p(torch.empty(cfg.vocab_size, W, device=device, dtype=dtype))
        self.layers = nn.ModuleList([LoluzenLayer(cfg, spec, device, dtype) for spec in cfg.layer_specs])
        self.final_norm = _p(torch.zeros(W, device=device, dtype=torch.float32))
        self.head = _p(torch.empty(cfg.vocab_size, W, device=device, dtype=dtype))
        self.num_kv_heads_local = 1
        # the order the layers run in, and the runs before which the embedding rows are added again
        self.runs: List[int] = cfg.layer_runs()
        lp = cfg.layer_loop
        self.pass_starts = set() if not lp else \
            {int(lp["start"]) + r * (int(lp["stop"]) - int(lp["start"])) for r in range(1, int(lp["times"]))}
        self._rot: Dict[tuple, torch.Tensor] = {}
        self._rot_len = 0
        self.set_max_positions(min(cfg.max_position, 4096))
        self.keep_residuals = None   # tests: a list that collects x after every layer run

    # ------------------------------------------------------------------ positions
    def set_max_positions(self, n: int) -> None:
        """(Re)build the rotation tables for positions [0, n) -- the runner passes its max_model_len."""
        if n <= self._rot_len:
            return
        self._rot = {}
        for L in self.layers:
            key = L.mix.rot_key() if L.kind == "attention" else None
            if key is not None and key not in self._rot:
                self._rot[key] = sq.build_rot_table(L.mix.rot_dims, L.mix.rot_base, n, self.device, L.mix.rot_scaling)
        self._rot_len = n

    # ------------------------------------------------------------------ cache / state
    def alloc_cache(self, num_blocks: int, block_size: int, max_num_seqs: int) -> SeqCache:
        dev = self.device
        f32 = dict(dtype=torch.float32, device=dev)
        sc = SeqCache(block_size=block_size)
        rows = num_blocks * block_size
        for i in self.runs:            # one cache per layer run: a repeated layer shares weights, not cache
            L = self.layers[i]
            a = L.mix if L.kind == "attention" else L.mix.left
            lc = LayerCache(k=torch.zeros(rows, a.nk, dtype=self.dtype, device=dev),
                            v=torch.zeros(rows, a.nv, dtype=self.dtype, device=dev))
            if L.kind == "attention":
                lc.mix_conv = torch.zeros(max_num_seqs, a.taps - 1, a.ch, **f32)
            else:
                r = L.mix.right
                lc.gla = torch.zeros(max_num_seqs, r.H, r.dk, r.dv, **f32)
            sc.layers.append(lc)
        return sc

    def _attn(self, i):
        L = self.layers[i]
        return L.mix if L.kind == "attention" else L.mix.left

    def cache_bytes_per_block(self, block_size: int) -> int:
        esz = torch.tensor([], dtype=self.dtype).element_size()
        return block_size * sum((self._attn(i).nk + self._attn(i).nv) * esz for i in self.runs)

    def state_bytes_per_slot(self) -> int:
        n = 0
        for i in self.runs:
            L = self.layers[i]
            if L.kind == "attention":
                n += (L.mix.taps - 1) * L.mix.ch
            else:
                n += L.mix.right.H * L.mix.right.dk * L.mix.right.dv
        return 4 * n

    # ------------------------------------------------------------------ weights
    @torch.no_grad()
    def random_init(self, seed: int = 0):
        g = torch.Generator().manual_seed(seed)

        def mat(p, gain=1.0):
            p.copy_((torch.randn(p.shape, generator=g) * gain / math.sqrt(p.shape[-1])).to(p.dtype))

        def vec(p, std, mean=0.0):
            p.copy_((torch.randn(p.shape, generator=g) * std + mean).to(p.dtype))
        self.embed.copy_((torch.randn(self.embed.shape, generator=g) * 0.3).to(self.dtype))
        mat(self.head)
        vec(self.final_norm, 0.1)
        for L in self.layers:
            for w in (L.norm1, L.norm1b):
                vec(w, 0.1)
            m = L.mix
            if L.kind == "attention":
                mat(m.in_proj)
                mat(m.o)
                vec(m.conv_w, 0.4, 1.0 / m.taps)
                vec(m.q_norm, 0.1, 1.0)
                vec(m.k_norm, 0.1, 1.0)
            else:
                mat(m.in_proj)
                vec(m.in_bias, 0.1)
                a, r = m.left, m.right
                with torch.no_grad():   # the gate rows of the left branch and q / v of the right one have no bias
                    n = a.nq + a.nk + a.nv
                    m.in_bias[n:n + a.H] = 0
                    m.in_bias[a.rows:a.rows + r.n] = 0
                    m.in_bias[a.rows + 2 * r.n:] = 0
                mat(a.o)
                mat(r.o)
                a.r1.copy_(torch.rand(a.H, generator=g) * 1.5)
                a.r2.copy_(torch.rand(a.H, generator=g) * 2.0 + 0.05)
                a.talk.copy_(torch.eye(a.H) + torch.randn(a.H, a.H, generator=g) * 0.3)
                r.lower.copy_(torch.rand(r.n, generator=g) * 0.9)
                vec(r.norm, 0.1, 1.0)
                vec(a.out_norm, 0.1, 1.0)
                vec(r.out_norm, 0.1, 1.0)
            if L.mlp is not None:
                for w in (L.norm2, L.norm2b):
                    vec(w, 0.1)
                mat(L.mlp.up)
                mat(L.mlp.down)
                vec(L.mlp.up_b, 0.1)
                vec(L.mlp.down_b, 0.1)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, cache: SeqCache):
        sm = meta.seq
        if sm is None:
            raise ValueError("Loluzen needs the step's per-sequence metadata (AttnMeta.seq)")
        cfg, eps = self.cfg, self.cfg.norm_eps
        x = sq.embed_rows(input_ids, self.embed, scale=cfg.embed_scale)
        e = x.clone() if self.pass_starts else None
        n = sq.post_norm_residual(x, None, None, None, 0.0, None, self.layers[self.runs[0]].norm1, eps, self.dtype)
        last = len(self.runs) - 1
        keep = self.keep_residuals
        for r, (i, lc) in enumerate(zip(self.runs, cache.layers)):
            L = self.layers[i]
            nxt = self.layers[self.runs[r + 1]].norm1 if r < last else self.final_norm
            extra = e if (r + 1) in self.pass_starts else None
            rot = self._rot.get(L.mix.rot_key()) if L.kind == "attention" else None
            if keep is None:
                n = L(x, n, sm, lc, cache.block_size, rot, extra, nxt)
            else:   # x after the layer, before what precedes the next one
                L(x, n, sm, lc, cache.block_size, rot, None, None)
                keep.append(x.clone())
                n = sq.post_norm_residual(x, None, None, None, 0.0, extra, nxt, eps, self.dtype)
        self.last_hidden = x
        return n

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(h, self.head)

    def set_moe_comm(self, mode: str):
        pass


def count_params(cfg: ModelConfig) -> int:
    W, V = cfg.hidden_size, cfg.vocab_size
    n = 2 * V * W + W

    def gqa(m):
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        return (H * dk + G * dk + G * dv + H) * W + W * H * dv
    for spec in cfg.layer_specs:
        m = spec["mixer"]
        n += 2 * W
        if spec["type"] == "attention":
            n += gqa(m) + (m["heads"] * m["dim"] + m["kv_heads"] * (m["dim"] + m["vdim"])) * m.get("conv", 1) + 2 * m["dim"]
        else:
            a, r = m["left"], m["right"]
            n += gqa(a) + a["heads"] * a["dim"] + a["kv_heads"] * (a["dim"] + a["vdim"]) + 2 * a["heads"] + a["heads"] ** 2
            n += (2 * r["heads"] * r["dim"] + r["heads"] * r["vdim"]) * W + 2 * r["heads"] * r["dim"] + r["vdim"]
            n += W * r["heads"] * r["vdim"] + 2 * W
        if spec.get("mlp") is not None:
            n += 2 * W + 2 * W * spec["mlp"]["ff"] + spec["mlp"]["ff"] + W
    return n
