"""Lotelix: a pre-norm decoder of a configured list of layers with a group RMS norm, on the paged / slotted engine.

    x_0 = embed[token] * s                                   (s = cfg.embed_scale)
    x  <- x + mixer(N(x; norm1));   x <- x + ff(N(x; norm2))
    N(v; w): v in cfg.norm_groups equal consecutive parts, each divided by its own root mean square; times w

The residual stream x is fp32 throughout; a residual sum and the norm that follows it run in one kernel.

Mixers (reusable modules, every constant a parameter):
  * `MinGRUMixer` ("mingru"): per channel S <- (1 - z) S + z c with gate z and candidate c functions of the current
    token only; output W_o (S * silu(W_g h)); an fp32 state row per slot.
  * `WindowSinkAttention` ("attention"): grouped-query attention, the first rot.dims entries of each head rotated in
    (i, i + dims / 2) pairs with wavelength-rescaled frequencies; sliding window; a sink term in the softmax denominator;
    the values of every value-mixing layer after the first are blended with the first one's values of the same token
    before they are cached; the concatenated heads times sigmoid(W_g h), entry by entry.
  * `ParallelMixer` ("parallel"): `SigmoidAttention` (biased projections, whole-vector q / k norms, (2i, 2i + 1)
    rotation, causal, weights sigmoid(score + b_h) without normalisation) beside `DecayedLinearAttention` (per head
    S <- diag(a) S + k v^T, o = S^T q with a decay per key channel from a low-rank projection; o RMS-normed per head,
    times silu(W_g h)); the mixer's output is the mean of the two branches, each RMS-normed over the width.
Feed-forward: `InputScaledMoE`: sigmoid router, the `top` largest scores, each chosen expert W_down relu(W_up .)^2 reads
the token times its score; or none.

What a sequence carries between steps (ModelRunner allocates it through alloc_cache): K / V pages of the attention
layers and of the left branches; per state slot the minGRU rows and the linear-attention states.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

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


def _rot_key(rot):
    if not rot or int(rot.get("dims", 0)) == 0:
        return None
    sc = rot.get("scaling")
    return (int(rot["dims"]), float(rot["base"]), None if sc is None else tuple(sorted((k, float(v)) for k, v in sc.items())))


class MinGRUMixer(nn.Module):
    def __init__(self, width: int, m: dict, device, dtype):
        super().__init__()
        self.n = int(m["width"])
        self.in_proj = _p(torch.empty(3 * self.n, width, device=device, dtype=dtype))    # fused rows [z | x | g]
        self.z_b = _p(torch.zeros(self.n, device=device, dtype=torch.float32))
        self.x_b = _p(torch.zeros(self.n, device=device, dtype=torch.float32))
        self.o = _p(torch.empty(width, self.n, device=device, dtype=dtype))

    def forward(self, h, sm: sq.SeqMeta, lc: LayerCache):
        n = self.n
        proj = F.linear(h, self.in_proj)
        return F.linear(sq.mingru_scan(proj, 0, n, 2 * n, n, self.z_b, self.x_b, lc.gru, sm, h.dtype), self.o)


class WindowSinkAttention(nn.Module):
    def __init__(self, width: int, m: dict, device, dtype):
        super().__init__()
        e = lambda *s: torch.empty(*s, device=device, dtype=dtype)  # noqa: E731
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.H, self.G, self.dk, self.dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        self.scale = float(m["scale"])
        mask = m.get("mask")
        self.mask, self.size = (sq.MASK_WINDOW, int(mask["size"])) if mask else (sq.MASK_CAUSAL, 0)
        self.rot = m.get("rot") or None
        self.rot_dims = int(self.rot["dims"]) if self.rot else 0
        self.v_mix = bool(m.get("v_mix", False))
        self.nq, self.nk, self.nv = self.H * self.dk, self.G * self.dk, self.G * self.dv
        self.ch = self.nq + self.nk + self.nv
        self.in_proj = _p(e(self.ch + self.H * self.dv, width))     # fused rows [q | k | v | gate]
        self.sink = _p(f(self.H))
        self.lam = _p(f(1))                                          # value-mixing weight (unused by the first mixing layer)
        self.o = _p(e(width, self.H * self.dv))

    def forward(self, h, sm: sq.SeqMeta, lc: LayerCache, block_size: int, rot, v_first):
        """(output, this layer's own projected values as a view of the fused projection)."""
        proj = F.linear(h, self.in_proj)
        own = proj[:, self.nq + self.nk:self.ch]
        q = sq.head_norm_rope_cache(proj, self.H, self.G, self.dk, self.dv, None, None, 0.0, rot, self.rot_dims, sm, lc.k,
                                    lc.v, h.dtype, half=True, v_first=v_first, v_mix=self.lam if v_first is not None else None)
        o = sq.masked_attention(q, lc.k, lc.v, self.H, self.G, self.dk, self.dv, self.mask, self.size, self.scale, None,
                                self.sink, block_size, sm, gate=proj[:, self.ch:], gate_elem=True)
        return F.linear(o, self.o), own


class SigmoidAttention(nn.Module):
    """The attention branch of the "parallel" mixer; its projection rows live in the mixer's fused input matrix."""

    def __init__(self, width: int, m: dict, eps: float, device, dtype):
        super().__init__()
        e = lambda *s: torch.empty(*s, device=device, dtype=dtype)  # noqa: E731
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.H, self.G, self.dk, self.dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        self.scale, self.eps = float(m["scale"]), eps
        self.rot = m.get("rot") or None
        self.rot_dims = int(self.rot["dims"]) if self.rot else 0
        self.nq, self.nk, self.nv = self.H * self.dk, self.G * self.dk, self.G * self.dv
        self.rows = self.nq + self.nk + self.nv                    # [q | k | v]
        self.q_norm, self.k_norm = _p(f(self.nq)), _p(f(self.nk))
        self.pb = _p(f(self.H))
        self.o = _p(e(width, self.H * self.dv))
        self.o_b = _p(e(width))
        self.out_norm = _p(f(width))

    def forward(self, proj, sm: sq.SeqMeta, lc: LayerCache, block_size: int, rot):
        q = sq.head_norm_rope_cache(proj, self.H, self.G, self.dk, self.dv, self.q_norm, self.k_norm, self.eps, rot,
                                    self.rot_dims, sm, lc.k, lc.v, proj.dtype, whole=True)
        o = sq.masked_attention(q, lc.k, lc.v, self.H, self.G, self.dk, self.dv, sq.MASK_CAUSAL, 0, self.scale, None, None,
                                block_size, sm, weights=sq.W_SIGMOID, score_bias=self.pb)
        return F.linear(o, self.o, self.o_b)


class DecayedLinearAttention(nn.Module):
    """The recurrent branch of the "parallel" mixer (rows [q | k | v | gate | a1] of the fused input matrix)."""

    def __init__(self, width: int, m: dict, eps: float, device, dtype):
        super().__init__()
        e = lambda *s: torch.empty(*s, device=device, dtype=dtype)  # noqa: E731
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.H, self.dk, self.dv, self.eps = int(m["heads"]), int(m["dim"]), int(m["vdim"]), eps
        self.tau, self.rank = float(m["tau"]), int(m["decay_rank"])
        self.n, self.nv = self.H * self.dk, self.H * self.dv
        self.rows = 2 * self.n + 2 * self.nv + self.rank
        self.a2 = _p(e(self.n, self.rank))
        self.a2_b = _p(f(self.n))
        self.norm = _p(f(self.dv))
        self.o = _p(e(width, self.nv))
        self.out_norm = _p(f(width))

    def forward(self, proj, sm: sq.SeqMeta, lc: LayerCache):
        n, nv = self.n, self.nv
        z = F.linear(proj[:, 2 * n + 2 * nv:], self.a2)
        q, f, k = sq.decay_gates(proj, 0, n, n, self.dk ** -0.5, z, self.a2_b, self.tau)
        o = sq.gated_linear_scan(q, f, k, proj[:, 2 * n:2 * n + nv], lc.gla, self.H, self.dk, self.dv, sm)
        y = sq.gated_group_norm(o, proj[:, 2 * n + nv:2 * n + 2 * nv], self.norm, self.eps, self.H, proj.dtype,
                                gate_after=True)
        return F.linear(y, self.o)


class ParallelMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, device, dtype):
        super().__init__()
        self.left = SigmoidAttention(width, m["left"], eps, device, dtype)
        self.right = DecayedLinearAttention(width, m["right"], eps, device, dtype)
        rows = self.left.rows + self.right.rows
        self.in_proj = _p(torch.empty(rows, width, device=device, dtype=dtype))   # [left q k v | right q k v gate a1]
        self.in_bias = _p(torch.zeros(rows, device=device, dtype=dtype))          # zero where the design has none

    def forward(self, h, sm: sq.SeqMeta, lc: LayerCache, block_size: int, rot):
        """The two branch outputs (their norms and mean join the residual update)."""
        proj = F.linear(h, self.in_proj, self.in_bias)
        return (self.left(proj[:, :self.left.rows], sm, lc, block_size, rot),
                self.right(proj[:, self.left.rows:], sm, lc))


class InputScaledMoE(nn.Module):
    def __init__(self, width: int, mlp: dict, device, dtype):
        super().__init__()
        self.E, self.top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
        self.ff = int(mlp["expert"]["ff"])
        self.router = _p(torch.zeros(self.E, width, device=device, dtype=torch.float32))
        self.up = _p(torch.empty(self.E, self.ff, width, device=device, dtype=dtype))
        self.down = _p(torch.empty(self.E, width, self.ff, device=device, dtype=dtype))

    def forward(self, n32, nact):
        """The experts' output rows; the residual update sums them per token."""
        ids, wts = sq.grouped_router(None, None, 1, 1, self.top, 1.0, rows=n32, router_w=self.router)
        return sq.routed_experts(nact, self.up, self.down, ids, wts, sq.ACT_RELU2, scale_input=True, combine=False)


class LotelixLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, spec: dict, device, dtype):
        super().__init__()
        W = cfg.hidden_size
        f = lambda *s: torch.zeros(*s, device=device, dtype=torch.float32)  # noqa: E731
        self.kind, self.eps, self.groups = spec["type"], cfg.norm_eps, cfg.norm_groups
        if self.kind == "mingru":
            self.mix = MinGRUMixer(W, spec["mixer"], device, dtype)
        elif self.kind == "attention":
            self.mix = WindowSinkAttention(W, spec["mixer"], device, dtype)
        else:
            self.mix = ParallelMixer(W, spec["mixer"], cfg.norm_eps, device, dtype)
        self.norm1 = _p(f(W))
        self.mlp = None
        if spec.get("mlp") is not None:
            self.norm2 = _p(f(W))
            self.mlp = InputScaledMoE(W, spec["mlp"], device, dtype)

    def attn(self):
        return self.mix if self.kind == "attention" else self.mix.left if self.kind == "parallel" else None


class LotelixForCausalLM(nn.Module):
    has_sequence_state = True   # recurrent state per slot: no prefix reuse, no draft verification

    def __init__(self, cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, tp: Optional[int] = None,
                 rank: Optional[int] = None):
        super().__init__()
        tp = get_state().tp_size if tp is None else tp
        if tp != 1:
            raise ValueError("Lotelix runs with tp=1 (use DP replicas to scale)")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("Lotelix runs in bfloat16 or float32")
        self.cfg, self.tp, self.rank = cfg, 1, 0
        self.device, self.dtype = torch.device(device), dtype
        W = cfg.hidden_size
        self.embed = _p(torch.empty(cfg.vocab_size, W, device=device, dtype=dtype))
        self.layers = nn.ModuleList([LotelixLayer(cfg, spec, device, dtype) for spec in cfg.layer_specs])
        self.final_norm = _p(torch.zeros(W, device=device, dtype=torch.float32))
        self.head = _p(torch.empty(cfg.vocab_size, W, device=device, dtype=dtype))
        self.num_kv_heads_local = 1
        self._rot: Dict[tuple, torch.Tensor] = {}
        self._rot_len = 0
        self.set_max_positions(min(cfg.max_position, 4096))
        self.keep_residuals = None   # tests: a list that collects x after every layer

    # ------------------------------------------------------------------ positions
    def set_max_positions(self, n: int) -> None:
        """(Re)build the rotation tables for positions [0, n) -- the runner passes its max_model_len."""
        if n <= self._rot_len:
            return
        self._rot = {}
        for L in self.layers:
            a = L.attn()
            key = _rot_key(a.rot) if a is not None else None
            if key is not None and key not in self._rot:
                self._rot[key] = sq.build_rot_table(a.rot_dims, float(a.rot["base"]), n, self.device, a.rot.get("scaling"))
        self._rot_len = n

    # ------------------------------------------------------------------ cache / state
    def alloc_cache(self, num_blocks: int, block_size: int, max_num_seqs: int) -> SeqCache:
        dev = self.device
        f32 = dict(dtype=torch.float32, device=dev)
        sc = SeqCache(block_size=block_size)
        rows = num_blocks * block_size
        for L in self.layers:
            lc, a = LayerCache(), L.attn()
            if a is not None:
                lc.k = torch.zeros(rows, a.nk, dtype=self.dtype, device=dev)
                lc.v = torch.zeros(rows, a.nv, dtype=self.dtype, device=dev)
            if L.kind == "mingru":
                lc.gru = torch.zeros(max_num_seqs, L.mix.n, **f32)
            elif L.kind == "parallel":
                r = L.mix.right
                lc.gla = torch.zeros(max_num_seqs, r.H, r.dk, r.dv, **f32)
            sc.layers.append(lc)
        return sc

    def cache_bytes_per_block(self, block_size: int) -> int:
        esz = torch.tensor([], dtype=self.dtype).element_size()
        return max(1, block_size * sum((a.nk + a.nv) * esz for a in (L.attn() for L in self.layers) if a is not None))

    def state_bytes_per_slot(self) -> int:
        n = 0
        for L in self.layers:
            if L.kind == "mingru":
                n += L.mix.n
            elif L.kind == "parallel":
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
        vec(self.final_norm, 0.1, 1.0)
        for L in self.layers:
            vec(L.norm1, 0.1, 1.0)
            m = L.mix
            if L.kind == "mingru":
                mat(m.in_proj)
                mat(m.o)
                vec(m.z_b, 0.5)
                vec(m.x_b, 0.3)
            elif L.kind == "attention":
                mat(m.in_proj)
                mat(m.o)
                vec(m.sink, 0.7)
                m.lam.fill_(0.2 + 0.5 * float(torch.rand(1, generator=g)))
            else:
                a, r = m.left, m.right
                mat(m.in_proj)
                m.in_bias.zero_()
                vec(m.in_bias[:a.rows], 0.2)
                vec(a.q_norm, 0.1, 1.0)
                vec(a.k_norm, 0.1, 1.0)
                vec(a.pb, 0.5, -2.0)
                mat(a.o)
                vec(a.o_b, 0.1)
                mat(r.a2, 2.0)
                vec(r.a2_b, 0.5, 2.0)
                vec(r.norm, 0.1, 1.0)
                mat(r.o)
                vec(a.out_norm, 0.1, 1.0)
                vec(r.out_norm, 0.1, 1.0)
            if L.mlp is not None:
                vec(L.norm2, 0.1, 1.0)
                mat(L.mlp.router, 2.0)
                mat(L.mlp.up)
                mat(L.mlp.down)

    # ------------------------------------------------------------------ forward
    def forward(self, input_ids: torch.Tensor, meta: AttnMeta, cache: SeqCache):
        sm = meta.seq
        if sm is None:
            raise ValueError("Lotelix needs the step's per-sequence metadata (AttnMeta.seq)")
        cfg, eps, groups, dt = self.cfg, self.cfg.norm_eps, self.cfg.norm_groups, self.dtype
        x = sq.embed_rows(input_ids, self.embed, scale=cfg.embed_scale)
        first = self.layers[0]
        n32, n = sq.residual_norm(x, None, None, None, None, None, first.norm1, eps, dt, False, groups)
        v_first, last, keep = None, len(self.layers) - 1, self.keep_residuals
        for i, (L, lc) in enumerate(zip(self.layers, cache.layers)):
            nxt = self.layers[i + 1].norm1 if i < last else self.final_norm
            after = L.norm2 if L.mlp is not None else nxt       # the norm that follows the mixer's residual sum
            f32 = L.mlp is not None                             # the router reads the fp32 norm
            a = L.attn()
            rot = self._rot.get(_rot_key(a.rot)) if a is not None else None
            if L.kind == "mingru":
                n32, n = sq.residual_norm(x, L.mix(n, sm, lc), None, None, None, None, after, eps, dt, f32, groups)
            elif L.kind == "attention":
                y, own = L.mix(n, sm, lc, cache.block_size, rot, v_first if L.mix.v_mix else None)
                if L.mix.v_mix and v_first is None:
                    v_first = own
                n32, n = sq.residual_norm(x, y, None, None, None, None, after, eps, dt, f32, groups)
            else:
                ya, yb = L.mix(n, sm, lc, cache.block_size, rot)
                n32, n = sq.residual_norm(x, ya, None, yb, None, None, after, eps, dt, f32, groups,
                                          branch_w=(L.mix.left.out_norm, L.mix.right.out_norm))
            if L.mlp is not None:
                n32, n = sq.residual_norm(x, None, None, None, L.mlp(n32, n), None, nxt, eps, dt, False, groups)
            if keep is not None:
                keep.append(x.clone())
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
        return (m["heads"] * m["dim"] + m["kv_heads"] * (m["dim"] + m["vdim"])) * W + W * m["heads"] * m["vdim"]
    for spec in cfg.layer_specs:
        m = spec["mixer"]
        n += W
        if spec["type"] == "mingru":
            n += 4 * m["width"] * W + 2 * m["width"]
        elif spec["type"] == "attention":
            n += gqa(m) + m["heads"] * m["vdim"] * W + m["heads"] + 1
        else:
            a, r = m["left"], m["right"]
            n += gqa(a) + 2 * (a["heads"] * a["dim"] + a["kv_heads"] * a["dim"]) + a["kv_heads"] * a["vdim"] + a["heads"] + W
            nk, nv, rk = r["heads"] * r["dim"], r["heads"] * r["vdim"], r.get("decay_rank", 16)
            n += (2 * nk + 2 * nv + rk) * W + nk * rk + nk + r["vdim"] + W * nv + 2 * W
        mlp = spec.get("mlp")
        if mlp is not None:
            E = mlp["router"]["experts"]
            n += W + E * W + 2 * E * W * mlp["expert"]["ff"]
    return n
