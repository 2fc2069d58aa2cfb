"""Operators of the stateful / latent-cache decoder layers (csrc/mixers).

A ragged step is described by a `SeqMeta`: per sequence its first row (`qsl`), the
tokens it holds after the step (`seq_lens`), its state row (`slots`, < 0: padding) and
its page table; per token its position, cache row (`slot_mapping`) and sequence
(`token_seq`). A sequence with an empty context starts from zero state whatever its
slot holds. GPU tensors run on the HIP kernels; CPU tensors on the PyTorch forms below
(the same paged / carried semantics, used by the CPU engine).

The residual stream, norms, softmax, rotations and recurrences are fp32; `act` tensors
(GEMM inputs / outputs, caches) are bfloat16 or float32.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional

import torch

from .. import tune
from ._native import is_f32, mixers, native_device, stream_ptr


@dataclass
class SeqMeta:
    num_seqs: int
    max_q: int
    qsl: torch.Tensor            # int32 [num_seqs + 1]
    seq_lens: torch.Tensor       # int32 [num_seqs]
    slots: torch.Tensor          # int32 [num_seqs]
    block_tables: torch.Tensor   # int32 [num_seqs, width]
    token_seq: torch.Tensor      # int32 [T]
    positions: torch.Tensor      # int32 [T]
    slot_mapping: torch.Tensor   # int32 [T]


def _p(t: Optional[torch.Tensor]) -> int:
    return 0 if t is None else t.data_ptr()


def _i32(t: torch.Tensor) -> torch.Tensor:
    assert t.dtype == torch.int32 and t.is_contiguous()
    return t


# ---------------------------------------------------------------------------- embedding
def embed_rows(ids: torch.Tensor, table: torch.Tensor, pos_table: Optional[torch.Tensor] = None,
               positions: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """fp32 rows table[ids] * scale (zero rows for ids outside the table); with `pos_table` the learned vector
    pos_table[positions] is added (unscaled)."""
    V, W = table.shape
    if not native_device(table):
        ok = (ids >= 0) & (ids < V)
        out = table[ids.long().clamp(0, V - 1)].float() * scale
        out[~ok] = 0
        if pos_table is not None:
            pk = (positions >= 0) & (positions < pos_table.shape[0])
            add = pos_table[positions.long().clamp(0, pos_table.shape[0] - 1)].float()
            add[~pk] = 0
            out = out + add
        return out
    out = torch.empty(ids.shape[0], W, dtype=torch.float32, device=table.device)
    if pos_table is not None:
        assert pos_table.dtype == table.dtype and pos_table.shape[1] == W and pos_table.is_contiguous()
    mixers().embed_rows(_i32(ids).data_ptr(), table.data_ptr(), is_f32(table), out.data_ptr(), ids.shape[0], W, V,
                        _p(pos_table), _i32(positions).data_ptr() if pos_table is not None else 0,
                        pos_table.shape[0] if pos_table is not None else 0, float(scale), stream_ptr())
    return out


# ---------------------------------------------------------------------------- input convolution
def causal_conv_residual(x: torch.Tensor, w: torch.Tensor, state: torch.Tensor, sm: SeqMeta,
                         out_dtype: torch.dtype) -> torch.Tensor:
    """h + conv(h) per channel over time: out_t = x_t + sum_j w[:, j] x_(t - taps + 1 + j), zeros
    before a sequence's start. x fp32 [T, W]; w fp32 [W, taps]; state fp32 [slots, taps - 1, W]
    holds each sequence's last taps - 1 inputs and is updated."""
    T, W = x.shape
    taps = w.shape[1]
    out = torch.empty(T, W, dtype=out_dtype, device=x.device)
    if native_device(x):
        assert x.dtype == torch.float32 and x.is_contiguous() and w.dtype == torch.float32 and w.is_contiguous()
        assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (taps - 1, W)
        mixers().canon_conv(x.data_ptr(), w.data_ptr(), state.data_ptr(), _i32(sm.qsl).data_ptr(),
                            _i32(sm.seq_lens).data_ptr(), _i32(sm.slots).data_ptr(), out.data_ptr(), is_f32(out),
                            sm.num_seqs, sm.max_q, W, taps, stream_ptr())
        return out
    nh = taps - 1
    qsl, sl, slots = sm.qsl.tolist(), sm.seq_lens.tolist(), sm.slots.tolist()
    for s in range(sm.num_seqs):
        a, b = qsl[s], qsl[s + 1]
        if slots[s] < 0 or b <= a:
            continue
        ctx = sl[s] - (b - a)
        hist = state[slots[s]] if ctx > 0 else torch.zeros(nh, W)
        ext = torch.cat([hist, x[a:b]], 0)
        y = x[a:b].clone()
        for j in range(taps):
            y += w[:, j] * ext[j:j + b - a]
        out[a:b] = y.to(out_dtype)
        if nh:
            state[slots[s]] = ext[-nh:]
    return out


def causal_conv(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor, sm: SeqMeta,
                out_dtype: torch.dtype, residual: bool = False, silu: bool = False) -> torch.Tensor:
    """Causal depthwise convolution over time of a row-strided activation block x [T, C] (float32 or
    bfloat16): out_t = [x_t] + bias + sum_j w[:, j] x_(t - taps + 1 + j), optionally through silu; zeros
    before a sequence's start. state fp32 [slots, taps - 1, C] holds each sequence's last taps - 1 raw
    inputs and is updated."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.empty(T, C, dtype=out_dtype, device=x.device)
    if native_device(x):
        assert x.stride(1) == 1 and w.dtype == torch.float32 and w.is_contiguous() and w.shape[0] == C
        assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (taps - 1, C)
        mixers().causal_conv(x.data_ptr(), is_f32(x), x.stride(0), w.data_ptr(), _p(bias), state.data_ptr(),
                             _i32(sm.qsl).data_ptr(), _i32(sm.seq_lens).data_ptr(), _i32(sm.slots).data_ptr(),
                             out.data_ptr(), is_f32(out), sm.num_seqs, sm.max_q, C, taps, residual, silu, stream_ptr())
        return out
    nh = taps - 1
    qsl, sl, slots = sm.qsl.tolist(), sm.seq_lens.tolist(), sm.slots.tolist()
    xf = x.float()
    for s in range(sm.num_seqs):
        a, b = qsl[s], qsl[s + 1]
        if slots[s] < 0 or b <= a:
            continue
        ctx = sl[s] - (b - a)
        hist = state[slots[s]] if ctx > 0 else torch.zeros(nh, C)
        ext = torch.cat([hist, xf[a:b]], 0)
        y = xf[a:b].clone() if residual else torch.zeros(b - a, C)
        if bias is not None:
            y = y + bias
        for j in range(taps):
            y = y + w[:, j] * ext[j:j + b - a]
        if silu:
            y = y * torch.sigmoid(y)
        out[a:b] = y.to(out_dtype)
        if nh:
            state[slots[s]] = ext[-nh:]
    return out


# ---------------------------------------------------------------------------- norm after the sum
def scaled_add_rmsnorm(x: torch.Tensor, y: Optional[torch.Tensor], w: torch.Tensor, eps: float, alpha: float = 1.0,
                       bias: Optional[torch.Tensor] = None, w_offset: float = 0.0, inplace: bool = True,
                       out_dtype: Optional[torch.dtype] = None):
    """v = alpha * x + y + bias; r = v / sqrt(mean(v^2) + eps) * (w_offset + w), in fp32.
    x fp32 [T, W] (overwritten with r when `inplace`); y an activation tensor or None.
    Returns r as fp32 (inplace) or as `out_dtype`."""
    T, W = x.shape
    if not native_device(x):
        v = alpha * x
        if y is not None:
            v = v + y.float()
        if bias is not None:
            v = v + bias
        r = v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * (w_offset + w)
        if inplace:
            x.copy_(r)
            return x
        return r.to(out_dtype or torch.float32)
    assert x.dtype == torch.float32 and x.is_contiguous() and w.dtype == torch.float32
    out = None if inplace else torch.empty(T, W, dtype=out_dtype or torch.float32, device=x.device)
    if y is not None:
        assert y.stride(-1) == 1 and y.shape == x.shape
    mixers().scaled_add_rmsnorm(x.data_ptr(), _p(y), is_f32(y) if y is not None else True,
                                y.stride(0) if y is not None else 0, _p(bias), float(alpha), w.data_ptr(),
                                float(w_offset), float(eps), x.data_ptr() if inplace else 0, _p(out),
                                is_f32(out) if out is not None else True, T, W, stream_ptr())
    return x if inplace else out


# ---------------------------------------------------------------------------- rotation table
def rot_frequencies(dims: int, base: float, scaling: Optional[dict] = None) -> torch.Tensor:
    """fp64 [dims / 2]: f_i = base^(-2 i / dims); with `scaling` {factor, low, high, original} each frequency is
    rescaled by its wavelength l = 2 pi / f: kept where l < original / high, divided by factor where
    l > original / low, and in between blended, (1 - s) f / factor + s f with s = (original / l - low) / (high - low)."""
    inv = base ** (-torch.arange(0, dims, 2, dtype=torch.float64) / dims)
    if scaling is None:
        return inv
    factor, low, high, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    wave = 2.0 * math.pi / inv
    s = ((orig / wave - low) / (high - low)) if high != low else torch.ones_like(inv)
    mid = (1.0 - s) * inv / factor + s * inv
    return torch.where(wave < orig / high, inv, torch.where(wave > orig / low, inv / factor, mid))


def build_rot_table(dims: int, base: float, max_pos: int, device="cpu", scaling: Optional[dict] = None) -> torch.Tensor:
    """fp32 [max_pos, dims / 2, 2] = (cos, sin) of position * f_i (rot_frequencies): the angles of the
    interleaved-pair rotation (dimension 2i with 2i + 1), evaluated in fp64."""
    inv = rot_frequencies(dims, base, scaling)
    ang = torch.outer(torch.arange(max_pos, dtype=torch.float64), inv)
    return torch.stack([ang.cos(), ang.sin()], -1).float().contiguous().to(device)


def _rotate_pairs(v: torch.Tensor, rot: torch.Tensor, pos: torch.Tensor, dims: int, half: bool = False) -> torch.Tensor:
    """v [T, ..., n] fp32: rotate the first `dims` entries pairwise by the table rows of `pos`; pair i is entries
    (2 i, 2 i + 1), or (i, i + dims / 2) with `half`."""
    cs = rot[pos.long()]  # [T, dims/2, 2]
    while cs.dim() < v.dim() + 1:
        cs = cs.unsqueeze(1)
    c, s = cs[..., 0], cs[..., 1]
    ia, ib = (slice(0, dims // 2), slice(dims // 2, dims)) if half else (slice(0, dims, 2), slice(1, dims, 2))
    a, b = v[..., ia], v[..., ib]
    out = v.clone()
    out[..., ia] = a * c - b * s
    out[..., ib] = b * c + a * s
    return out


# ---------------------------------------------------------------------------- latent attention
# XGS_TUNE latent_mfma=0: the general (any size, fp32-capable) kernel for bf16 too (A/B and tests)
LATENT_MFMA = tune.get_bool("latent_mfma", True)
LATENT_MAX_SPLITS = 16    # key shares per single-token row, at most
LATENT_SPLIT_WGS = 1024   # ... while the launch stays under about this many workgroups


def latent_prep(proj: torch.Tensor, off_q: int, Rq: int, off_kv: int, R: int, rd: int, wq: torch.Tensor,
                wkv: Optional[torch.Tensor], eps: float, rot: torch.Tensor, rot_dims: int, sm: SeqMeta,
                cache: Optional[torch.Tensor]) -> torch.Tensor:
    """From a fused projection row: the query latent (RMS-normed, weight wq) is returned; with
    off_kv >= 0 the key/value latent (RMS-normed, weight wkv) and the shared rotary key (rotated by
    its position) are written to cache row slot_mapping[t] as [latent (R) | key (rd)]."""
    T = proj.shape[0]
    cq = torch.empty(T, Rq, dtype=proj.dtype, device=proj.device)
    if native_device(proj):
        assert proj.stride(1) == 1 and rot.dtype == torch.float32
        if off_kv >= 0:
            assert cache.is_contiguous() and cache.dtype == proj.dtype and cache.shape[-1] == R + rd
        mixers().latent_prep(proj.data_ptr(), is_f32(proj), proj.stride(0), off_q, Rq, off_kv, R, rd, wq.data_ptr(),
                             _p(wkv), float(eps), _i32(sm.positions).data_ptr(), _i32(sm.slot_mapping).data_ptr(),
                             rot.data_ptr(), rot_dims, cq.data_ptr(), _p(cache) if off_kv >= 0 else 0, T, stream_ptr())
        return cq
    pf = proj.float()
    v = pf[:, off_q:off_q + Rq]
    cq.copy_((v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * wq).to(proj.dtype))
    if off_kv >= 0:
        c = pf[:, off_kv:off_kv + R]
        c = c / torch.sqrt(c.pow(2).mean(-1, keepdim=True) + eps) * wkv
        kr = _rotate_pairs(pf[:, off_kv + R:off_kv + R + rd], rot, sm.positions, rot_dims)
        rows = torch.cat([c, kr], -1).to(cache.dtype)
        ok = sm.slot_mapping >= 0
        cache.view(-1, R + rd)[sm.slot_mapping[ok].long()] = rows[ok]
    return cq


def latent_attention(qabs: torch.Tensor, q: torch.Tensor, dn: int, gate: torch.Tensor, cache: torch.Tensor,
                     rot: torch.Tensor, rot_dims: int, window: int, scale: float, block_size: int,
                     sm: SeqMeta) -> torch.Tensor:
    """Sliding-window softmax attention in latent space. Every head scores the same cached rows
    [latent (R) | rotated key (rd)]: head h of token t uses qabs[h, t] (its unrotated query mapped into
    latent space) and the rotary part q[t, h, dn:], rotated here; the output is the softmax-weighted
    mean of the latents, times sigmoid(gate[t, h]). Position i sees j with 0 <= i - j < window.
    qabs [H, T, R]; q [T, H, dn + rd]; gate [T, >= H] (row-strided); returns [H, T, R]."""
    H, T, R = qabs.shape
    dq = q.shape[-1]
    rd = dq - dn
    out = torch.empty(H, T, R, dtype=qabs.dtype, device=qabs.device)
    if native_device(qabs):
        assert qabs.is_contiguous() and q.is_contiguous() and cache.is_contiguous() and gate.stride(1) == 1
        assert cache.dtype == qabs.dtype == q.dtype == gate.dtype and cache.shape[-1] == R + rd
        bt = _i32(sm.block_tables)
        if LATENT_MFMA and qabs.dtype == torch.bfloat16 and R % 16 == 0 and 16 <= R <= 512 and rd % 8 == 0 and rd <= 128:
            # matrix-core form: 16 query slots per wave, 64 cached rows per LDS tile; a step of single tokens
            # divides each window's key tiles over several workgroups (merged by a second launch)
            nsplit, part_o, part_ml = 1, None, None
            if sm.max_q == 1 and T == sm.num_seqs:
                groups = T * ((H + 4 * min(16, H) - 1) // (4 * min(16, H)))
                nsplit = max(1, min(LATENT_MAX_SPLITS, (window + 63) // 64, LATENT_SPLIT_WGS // max(1, groups)))
                if nsplit > 1:
                    part_o = torch.empty(nsplit * H * T * R, dtype=torch.float32, device=q.device)
                    part_ml = torch.empty(nsplit * H * T * 2, dtype=torch.float32, device=q.device)
            mixers().latent_attention_mfma(qabs.data_ptr(), q.data_ptr(), dq, dn, gate.data_ptr(), gate.stride(0),
                                           cache.data_ptr(), bt.data_ptr(), bt.shape[1], block_size,
                                           _i32(sm.qsl).data_ptr(), _i32(sm.seq_lens).data_ptr(),
                                           _i32(sm.slots).data_ptr(), rot.data_ptr(), rot_dims, out.data_ptr(), T,
                                           sm.num_seqs, sm.max_q, H, R, rd, int(window), float(scale), nsplit,
                                           _p(part_o), _p(part_ml), stream_ptr())
            return out
        mixers().latent_attention(qabs.data_ptr(), q.data_ptr(), is_f32(q), H * dq, dq, dn, gate.data_ptr(),
                                  gate.stride(0), cache.data_ptr(), bt.data_ptr(), bt.shape[1], block_size,
                                  _i32(sm.positions).data_ptr(), _i32(sm.token_seq).data_ptr(), rot.data_ptr(), rot_dims,
                                  out.data_ptr(), T, H, R, rd, int(window), float(scale), stream_ptr())
        return out
    rows = cache.view(-1, R + rd)
    qr = _rotate_pairs(q.float()[..., dn:], rot, sm.positions, rot_dims)  # [T, H, rd]
    qa = qabs.float()
    tseq, pos = sm.token_seq.tolist(), sm.positions.tolist()
    for t in range(T):
        s = tseq[t]
        if s < 0:
            out[:, t] = 0
            continue
        j0 = max(0, pos[t] - window + 1)
        keys = torch.arange(j0, pos[t] + 1)
        idx = sm.block_tables[s][(keys // block_size).long()].long() * block_size + keys % block_size
        kv = rows[idx].float()  # [n, R + rd]
        sc = (qa[:, t] @ kv[:, :R].T + qr[t] @ kv[:, R:].T) * scale
        p = torch.softmax(sc, -1)
        out[:, t] = ((p @ kv[:, :R]) * torch.sigmoid(gate[t, :H].float())[:, None]).to(out.dtype)
    return out


def heads_to_rows(x: torch.Tensor) -> torch.Tensor:
    """[H, T, n] -> [T, H * n]."""
    H, T, n = x.shape
    if not native_device(x):
        return x.transpose(0, 1).reshape(T, H * n)
    out = torch.empty(T, H * n, dtype=x.dtype, device=x.device)
    mixers().heads_to_rows(x.contiguous().data_ptr(), is_f32(x), out.data_ptr(), T, H, n, stream_ptr())
    return out


# ---------------------------------------------------------------------------- generalized delta rule
DECAY_SCALE = math.exp(-0.5)
# XGS_TUNE delta_two_pass=0: the one-pass scan kernel (any head size; A/B and tests)
DELTA_TWO_PASS = tune.get_bool("delta_two_pass", True)
UNIT_KEY_EPS = 1e-6


def delta_rule_scan(proj: torch.Tensor, off_r: int, off_k: int, off_v: int, off_a: int, wl: torch.Tensor,
                    a_bias: torch.Tensor, w0: torch.Tensor, state: torch.Tensor, H: int, D: int,
                    sm: SeqMeta) -> torch.Tensor:
    """Per head, with r, k, v, a-logits at column offsets of the fused projection row and the decay
    logits wl [T, H * D]:  w = exp(-e^(-1/2) sigmoid(wl + w0)), a = sigmoid(a_logit + a_bias),
    u = k / sqrt(|k|^2 + 1e-6);  S <- diag(w) S - (a u)(u^T S) + k v^T (both read the old S);
    o = S^T r. state fp32 [slots, H, D, D] is carried and updated. Returns o fp32 [T, H * D]."""
    T = proj.shape[0]
    o = torch.empty(T, H * D, dtype=torch.float32, device=proj.device)
    if native_device(proj):
        assert proj.stride(1) == 1 and wl.stride(1) == 1 and wl.dtype == proj.dtype
        assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, D, D)
        # state-independent terms (decay, removal rate, unit key) in a parallel pass of their own
        prep = torch.empty(T * H * 5 * D, dtype=torch.float32, device=proj.device) if DELTA_TWO_PASS else None
        mixers().delta_scan(proj.data_ptr(), is_f32(proj), proj.stride(0), off_r, off_k, off_v, off_a, wl.data_ptr(),
                            wl.stride(0), a_bias.data_ptr(), w0.data_ptr(), state.data_ptr(), _i32(sm.qsl).data_ptr(),
                            _i32(sm.seq_lens).data_ptr(), _i32(sm.slots).data_ptr(), o.data_ptr(), sm.num_seqs, H, D,
                            _p(prep), T, stream_ptr())
        return o
    pf = proj.float()
    HD = H * D
    r, k, v = (pf[:, off:off + HD].view(T, H, D) for off in (off_r, off_k, off_v))
    a = torch.sigmoid(pf[:, off_a:off_a + HD] + a_bias).view(T, H, D)
    w = torch.exp(-DECAY_SCALE * torch.sigmoid(wl.float() + w0)).view(T, H, D)
    u = k / torch.sqrt(k.pow(2).sum(-1, keepdim=True) + UNIT_KEY_EPS)
    qsl, sl, slots = sm.qsl.tolist(), sm.seq_lens.tolist(), sm.slots.tolist()
    for s in range(sm.num_seqs):
        lo, hi = qsl[s], qsl[s + 1]
        if slots[s] < 0 or hi <= lo:
            continue
        S = state[slots[s]].clone() if sl[s] - (hi - lo) > 0 else torch.zeros(H, D, D)
        for t in range(lo, hi):
            uS = torch.einsum("hi,hij->hj", u[t], S)
            S = w[t][:, :, None] * S - (a[t] * u[t])[:, :, None] * uS[:, None, :] + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hij,hi->hj", S, r[t]).reshape(HD)
        state[slots[s]] = S
    return o


def delta_rule_out(o: torch.Tensor, norm_w: torch.Tensor, gate: torch.Tensor, eps: float, H: int, D: int,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """Each head's o / rms(o), times norm_w, times sigmoid(gate). o fp32 [T, H * D]; gate [T, H * D] (row-strided)."""
    T = o.shape[0]
    if not native_device(o):
        v = o.view(T, H, D)
        v = (v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, H * D)
        return (v * norm_w * torch.sigmoid(gate.float())).to(out_dtype)
    out = torch.empty(T, H * D, dtype=out_dtype, device=o.device)
    assert gate.stride(1) == 1 and gate.dtype == out_dtype
    mixers().delta_out(o.data_ptr(), norm_w.data_ptr(), gate.data_ptr(), is_f32(gate), gate.stride(0), float(eps),
                       out.data_ptr(), T, H, D, stream_ptr())
    return out


# ---------------------------------------------------------------------------- activations
def xielu(z: torch.Tensor, bias: Optional[torch.Tensor], sp: float, cn: float) -> torch.Tensor:
    """xIELU of z + bias with sp = softplus(p), cn = 1/2 + softplus(q):
    z > 0: sp z^2 + z / 2;  z <= 0: cn (exp(z) - 1 - z) + z / 2."""
    if not native_device(z):
        v = z.float() + (bias if bias is not None else 0)
        neg = cn * (torch.expm1(v.clamp(max=0)) - v) + 0.5 * v
        return torch.where(v > 0, sp * v * v + 0.5 * v, neg).to(z.dtype)
    assert z.is_contiguous()
    out = torch.empty_like(z)
    mixers().xielu(z.data_ptr(), is_f32(z), _p(bias), float(sp), float(cn), out.data_ptr(), z.numel(), z.shape[-1],
                   stream_ptr())
    return out


def tanh_cols(x: torch.Tensor, off: int, n: int) -> torch.Tensor:
    """tanh of columns [off, off + n) of a row-strided activation tensor, as a contiguous [T, n]."""
    T = x.shape[0]
    if not native_device(x):
        return torch.tanh(x[:, off:off + n].float()).to(x.dtype)
    out = torch.empty(T, n, dtype=x.dtype, device=x.device)
    mixers().tanh_cols(x.data_ptr() + off * x.element_size(), is_f32(x), x.stride(0), out.data_ptr(), T, n, stream_ptr())
    return out


# ---------------------------------------------------------------------------- parallel-block residual + next norm
def residual_norm(x: torch.Tensor, y1: Optional[torch.Tensor], a1: Optional[torch.Tensor], y2: Optional[torch.Tensor],
                  y3: Optional[torch.Tensor], a2: Optional[torch.Tensor], norm_w: Optional[torch.Tensor], eps: float,
                  out_dtype: Optional[torch.dtype] = None, want_f32: bool = False, groups: int = 1,
                  branch_w: Optional[tuple] = None):
    """x <- x + a1 * y1 + a2 * (y2 + y3) in place (x fp32 [T, W]; y1 / y2 activation tensors, y3 fp32; a1 / a2
    per-channel scales, None = 1; any y may be None), then, with `norm_w`, the RMS norm of the new x:
    n = x / sqrt(mean(x^2) + eps) * norm_w, returned as (n fp32 or None, n as out_dtype or None).
    y3 may be the `RoutedRows` of routed_experts(combine=False): the weighted sum over a token's choices is then formed here.
    `groups` > 1: the norm splits a row into that many equal consecutive parts, each divided by its own root mean
    square. `branch_w` = (w1, w2): y1 and y2 are the outputs of two branches that are averaged after each is
    RMS-normed over the row with its plain weight, x <- x + (N0(y1) w1 + N0(y2) w2) / 2 + y3 (no a1 / a2)."""
    T, W = x.shape
    assert groups >= 1 and W % groups == 0
    routed = None
    if isinstance(y3, RoutedRows):   # the rows of a routed mixture, summed per token here
        if y3.dest is None:
            y3 = y3.y
        else:
            routed, y3 = y3, y3.y
    if not native_device(x):
        def n0(v):
            return v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)
        if routed is not None:
            rows = y3[routed.dest.long()]                         # [T, top, W]
            y3 = (rows * routed.wts[:, :, None]).sum(1) if routed.wts is not None else rows.sum(1)
        v = x
        if branch_w is not None:
            v = v + 0.5 * (n0(y1.float()) * branch_w[0] + n0(y2.float()) * branch_w[1])
            if y3 is not None:
                v = v + y3
        else:
            if y1 is not None:
                v = v + (a1 if a1 is not None else 1.0) * y1.float()
            if y2 is not None or y3 is not None:
                f = (y2.float() if y2 is not None else 0.0) + (y3 if y3 is not None else 0.0)
                v = v + (a2 if a2 is not None else 1.0) * f
        x.copy_(v)
        if norm_w is None:
            return None, None
        n = n0(x.view(T, groups, W // groups)).reshape(T, W) * norm_w
        return (n if want_f32 else None), (n.to(out_dtype) if out_dtype is not None else None)
    assert branch_w is None or (y1 is not None and y2 is not None and a1 is None and a2 is None)
    assert x.dtype == torch.float32 and x.is_contiguous()
    ys = [y for y in (y1, y2) if y is not None]
    assert all(y.stride(1) == 1 and y.shape == x.shape for y in ys) and len({y.dtype for y in ys}) <= 1
    assert y3 is None or (y3.dtype == torch.float32 and y3.is_contiguous() and (routed is not None or y3.shape == x.shape))
    if routed is not None:
        assert y3.shape[1] == W and routed.dest.dtype == torch.int32 and routed.dest.is_contiguous()
        assert routed.dest.shape[0] == T and (routed.wts is None or routed.wts.shape == routed.dest.shape)
    n32 = torch.empty_like(x) if (norm_w is not None and want_f32) else None
    nact = torch.empty(T, W, dtype=out_dtype, device=x.device) if (norm_w is not None and out_dtype is not None) else None
    mixers().residual_norm(x.data_ptr(), _p(y1), y1.stride(0) if y1 is not None else 0, _p(a1), _p(y2),
                           y2.stride(0) if y2 is not None else 0, _p(y3), _p(a2), is_f32(ys[0]) if ys else True,
                           _p(norm_w), float(eps), _p(n32), _p(nact), is_f32(nact) if nact is not None else True, T, W,
                           int(groups), _p(branch_w[0]) if branch_w else 0, _p(branch_w[1]) if branch_w else 0,
                           _p(routed.dest) if routed else 0, _p(routed.wts) if routed else 0,
                           routed.dest.shape[1] if routed else 0, stream_ptr())
    return n32, nact


# ---------------------------------------------------------------------------- grouped-query attention, masked
MASK_CAUSAL, MASK_WINDOW, MASK_CHUNK = 0, 1, 2
# XGS_TUNE attn_mfma=0: the general (any size, fp32-capable) kernel for bf16 too (A/B and tests)
ATTN_MFMA = tune.get_bool("attn_mfma", True)
# XGS_TUNE attn_waves=4|8|16: waves per workgroup of the matrix-core kernel on prompt portions (0: by portion length)
ATTN_WAVES = tune.get_int("attn_waves", 0)
ATTN_MAX_SPLITS = 8      # key shares per single-token row, at most
ATTN_SPLIT_WGS = 2048    # ... while the launch stays under about this many workgroups


def first_visible(mask: int, size: int, pos: int) -> int:
    """The first key position a query at `pos` sees: 0 (causal), pos - size + 1 (sliding window), or the
    start of its chunk of `size` positions counted from the sequence's start (chunked)."""
    if mask == MASK_WINDOW:
        return max(0, pos - size + 1)
    if mask == MASK_CHUNK:
        return (pos // size) * size
    return 0


def qk_norm_cache(proj: torch.Tensor, nq: int, nk: int, nv: int, wq: Optional[torch.Tensor], wk: Optional[torch.Tensor],
                  eps: float, sm: SeqMeta, kcache: torch.Tensor, vcache: torch.Tensor) -> torch.Tensor:
    """From a fused projection row [q (nq) | k (nk) | v (nv)]: q and k are RMS-normed over their WHOLE
    vectors (all heads at once; weights wq / wk, None = no norm); q is returned [T, nq], k and v go to
    cache rows slot_mapping[t] (kcache [rows, nk], vcache [rows, nv])."""
    T = proj.shape[0]
    q = torch.empty(T, nq, dtype=proj.dtype, device=proj.device)
    if native_device(proj):
        assert proj.stride(1) == 1 and kcache.is_contiguous() and vcache.is_contiguous()
        assert kcache.dtype == vcache.dtype == proj.dtype and kcache.shape[-1] == nk and vcache.shape[-1] == nv
        mixers().qk_norm_cache(proj.data_ptr(), is_f32(proj), proj.stride(0), nq, nk, nv, _p(wq), _p(wk), float(eps),
                               _i32(sm.slot_mapping).data_ptr(), q.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), T,
                               stream_ptr())
        return q
    pf = proj.float()

    def nrm(v, w):
        return v if w is None else v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w
    q.copy_(nrm(pf[:, :nq], wq).to(proj.dtype))
    ok = sm.slot_mapping >= 0
    rows = sm.slot_mapping[ok].long()
    kcache.view(-1, nk)[rows] = nrm(pf[:, nq:nq + nk], wk)[ok].to(kcache.dtype)
    vcache.view(-1, nv)[rows] = proj[:, nq + nk:nq + nk + nv][ok].to(vcache.dtype)
    return q


V_OWN, V_ALL = -1, -2   # masked_attention(values=...): the query head's own key/value head, or every head's values
V_ALL_MAX = 256         # ... V_ALL serves up to this many value columns (G * dv) per query head
W_SOFTMAX, W_SIGMOID = 0, 1   # masked_attention(weights=...): how scores become weights


def masked_attention(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, H: int, G: int, dk: int, dv: int,
                     mask: int, size: int, scale: float, temp: Optional[torch.Tensor], sink: Optional[torch.Tensor],
                     block_size: int, sm: SeqMeta, gate: Optional[torch.Tensor] = None,
                     dist: Optional[tuple] = None, values: int = V_OWN, gate_elem: bool = False,
                     weights: int = W_SOFTMAX, score_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Softmax attention of H query heads over G cached key/value heads (query head h reads head h // (H / G)).
    A query at position i sees keys first_visible(mask, size, i) .. i of its own sequence. score = (q . k) * scale
    * temp[h]; with `dist` = (r1, r2) (fp32 [H] each) the score of key j loses r1[h] * ln(1 + r2[h] * (i - j)),
    otherwise positions do not enter the scores; with `sink` the denominator also holds exp(sink[h]), a term with no
    key and no value; with `gate` ([T, >= H], row-strided) head h's output is multiplied by sigmoid(gate[t, h]), or,
    with `gate_elem` (gate [T, >= H dv]), entry d of head h by sigmoid(gate[t, h dv + d]).
    `weights` = W_SIGMOID: no softmax; the weight of a visible key is sigmoid(score + score_bias[h]) (fp32 [H], None =
    0), not normalised over the keys (no sink).
    `values`: V_OWN: head h weighs the values of its own key/value head, returns [T, H * dv]; V_ALL: the values of
    all G heads concatenated, returns [T, H * G * dv] (what mixing of the heads' weight maps needs);
    c >= 0: the values of head c for every query head.
    q [T, H * dk]; caches [rows, G * dk] / [rows, G * dv]."""
    T = q.shape[0]
    dvo = G * dv if values == V_ALL else dv           # value columns per query head
    out = torch.empty(T, H * dvo, dtype=q.dtype, device=q.device)
    if native_device(q):
        assert q.is_contiguous() and kcache.is_contiguous() and vcache.is_contiguous()
        assert kcache.dtype == vcache.dtype == q.dtype and -2 <= values < G
        assert gate is None or (gate.stride(1) == 1 and gate.dtype == q.dtype and
                                gate.shape[1] >= (H * dv if gate_elem else H))
        assert not gate_elem or values == V_OWN
        assert weights == W_SOFTMAX or (sink is None and weights == W_SIGMOID)
        assert score_bias is None or (score_bias.dtype == torch.float32 and score_bias.numel() == H)
        r1, r2 = dist if dist is not None else (None, None)
        bt = _i32(sm.block_tables)
        single = sm.max_q == 1 and T == sm.num_seqs
        if ATTN_MFMA and q.dtype == torch.bfloat16 and dk % 32 == 0 and dv % 16 == 0 and dk <= 128 and dvo <= 256 \
                and (not single or H // G <= 64):
            # matrix cores: prompt portions (also beside single tokens) as 16 tokens x one head per wave, steps of
            # single tokens as the query heads of one key/value head per wave
            nsplit, part_o, part_ml = 1, None, None
            if single:  # divide the visible key tiles over several workgroups (merged by a second launch)
                tiles = (size + 63) // 64 if mask != MASK_CAUSAL else ATTN_MAX_SPLITS
                nsplit = max(1, min(ATTN_MAX_SPLITS, tiles, ATTN_SPLIT_WGS // max(1, T * G)))
                if nsplit > 1:
                    part_o = torch.empty(nsplit * T * H * dvo, dtype=torch.float32, device=q.device)
                    part_ml = torch.empty(nsplit * T * H * 2, dtype=torch.float32, device=q.device)
            mixers().masked_attention_mfma(q.data_ptr(), kcache.data_ptr(), vcache.data_ptr(), bt.data_ptr(), bt.shape[1],
                                           block_size, _i32(sm.qsl).data_ptr(), _i32(sm.seq_lens).data_ptr(),
                                           _i32(sm.slots).data_ptr(), _p(temp), _p(sink), out.data_ptr(), T, sm.num_seqs,
                                           sm.max_q, H, G, dk, dv, int(mask), int(size), float(scale), nsplit,
                                           _p(part_o), _p(part_ml), _p(gate), gate.stride(0) if gate is not None else 0,
                                           _p(r1), _p(r2), int(values), ATTN_WAVES, bool(gate_elem), int(weights),
                                           _p(score_bias), stream_ptr())
            return out
        mixers().masked_attention(q.data_ptr(), is_f32(q), kcache.data_ptr(), vcache.data_ptr(), bt.data_ptr(),
                                  bt.shape[1], block_size, _i32(sm.positions).data_ptr(), _i32(sm.token_seq).data_ptr(),
                                  _p(temp), _p(sink), out.data_ptr(), T, H, G, dk, dv, int(mask), int(size), float(scale),
                                  _p(gate), gate.stride(0) if gate is not None else 0, _p(r1), _p(r2), int(values),
                                  bool(gate_elem), int(weights), _p(score_bias), stream_ptr())
        return out
    kr, vr = kcache.view(-1, G, dk), vcache.view(-1, G, dv)
    qf = q.float().view(T, H, dk)
    rep = H // G
    tseq, pos = sm.token_seq.tolist(), sm.positions.tolist()
    tmp = temp if temp is not None else torch.ones(H)
    for t in range(T):
        s = tseq[t]
        if s < 0:
            out[t] = 0
            continue
        keys = torch.arange(first_visible(mask, size, pos[t]), pos[t] + 1)
        idx = sm.block_tables[s][(keys // block_size).long()].long() * block_size + keys % block_size
        kk = kr[idx].float().repeat_interleave(rep, 1)   # [n, H, dk]
        sc = torch.einsum("hd,nhd->hn", qf[t], kk) * (scale * tmp)[:, None]
        if dist is not None:
            sc = sc - dist[0][:, None] * torch.log1p(dist[1][:, None] * (pos[t] - keys).float()[None, :])
        if weights == W_SIGMOID:
            p = torch.sigmoid(sc + (score_bias[:, None] if score_bias is not None else 0.0))
        else:
            if sink is not None:
                sc = torch.cat([sc, sink[:, None]], 1)
            p = torch.softmax(sc, -1)[:, :keys.numel()]
        if values == V_ALL:
            o = torch.einsum("hn,nd->hd", p, vr[idx].float().reshape(keys.numel(), G * dv))
        elif values >= 0:
            o = torch.einsum("hn,nd->hd", p, vr[idx][:, values].float())
        else:
            o = torch.einsum("hn,nhd->hd", p, vr[idx].float().repeat_interleave(rep, 1))
        if gate is not None and gate_elem:
            o = o * torch.sigmoid(gate[t, :H * dv].float()).view(H, dv)
        elif gate is not None:
            o = o * torch.sigmoid(gate[t, :H].float())[:, None]
        out[t] = o.reshape(H * dvo).to(out.dtype)
    return out


# ---------------------------------------------------------------------------- state-space recurrence
def ssm_scan(xbc: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, A_log: torch.Tensor, D: torch.Tensor,
             state: torch.Tensor, H: int, G: int, N: int, P: int, sm: SeqMeta) -> torch.Tensor:
    """Per head h (group h // (H / G)), with x / B / C the column blocks [H P | G N | G N] of `xbc` and
    dt = softplus(dt_raw + dt_bias) (not limited to a range):  S <- exp(-exp(A_log_h) dt) S + dt B x^T  (S is N x P),
    y = S^T C + D_h x. state fp32 [slots, H, N, P] is carried and updated. Returns y fp32 [T, H * P]."""
    T = xbc.shape[0]
    y = torch.empty(T, H * P, dtype=torch.float32, device=xbc.device)
    if native_device(xbc):
        assert xbc.stride(1) == 1 and dt_raw.stride(1) == 1 and dt_raw.dtype == xbc.dtype
        assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, N, P)
        mixers().ssm_scan(xbc.data_ptr(), is_f32(xbc), xbc.stride(0), dt_raw.data_ptr(), dt_raw.stride(0),
                          dt_bias.data_ptr(), A_log.data_ptr(), D.data_ptr(), state.data_ptr(), _i32(sm.qsl).data_ptr(),
                          _i32(sm.seq_lens).data_ptr(), _i32(sm.slots).data_ptr(), y.data_ptr(), sm.num_seqs, H, G, N, P,
                          stream_ptr())
        return y
    xf = xbc.float()
    x = xf[:, :H * P].view(T, H, P)
    B = xf[:, H * P:H * P + G * N].view(T, G, N).repeat_interleave(H // G, 1)
    C = xf[:, H * P + G * N:H * P + 2 * G * N].view(T, G, N).repeat_interleave(H // G, 1)
    dt = torch.nn.functional.softplus(dt_raw.float()[:, :H] + dt_bias, threshold=20.0)
    dec = torch.exp(-torch.exp(A_log) * dt)
    qsl, sl, slots = sm.qsl.tolist(), sm.seq_lens.tolist(), sm.slots.tolist()
    for s in range(sm.num_seqs):
        lo, hi = qsl[s], qsl[s + 1]
        if slots[s] < 0 or hi <= lo:
            continue
        S = state[slots[s]].clone() if sl[s] - (hi - lo) > 0 else torch.zeros(H, N, P)
        for t in range(lo, hi):
            S = dec[t][:, None, None] * S + (dt[t][:, None] * B[t])[:, :, None] * x[t][:, None, :]
            y[t] = (torch.einsum("hnp,hn->hp", S, C[t]) + D[:, None] * x[t]).reshape(H * P)
        state[slots[s]] = S
    return y


def gated_group_norm(y: torch.Tensor, z: Optional[torch.Tensor], w: torch.Tensor, eps: float, groups: int,
                     out_dtype: torch.dtype, gate_after: bool = False) -> torch.Tensor:
    """v = y * silu(z) (v = y when z is None); each of `groups` equal parts of a row divided by its own root mean
    square; times w, which holds one weight per column or one period of a repeating pattern (e.g. a weight of one
    head's size shared by all heads). With `gate_after` the norm is taken of y itself and silu(z) multiplies the
    normed, weighted result. y fp32 [T, n]; z [T, n] (row-strided activation)."""
    T, n = y.shape
    assert n % groups == 0 and n % w.numel() == 0
    if not native_device(y):
        v = y
        gate = None
        if z is not None:
            zf = z.float()
            gate = zf * torch.sigmoid(zf)
            if not gate_after:
                v = y * gate
        v = v.view(T, groups, n // groups)
        v = (v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)).reshape(T, n) * w.repeat(n // w.numel())
        if gate_after and gate is not None:
            v = v * gate
        return v.to(out_dtype)
    out = torch.empty(T, n, dtype=out_dtype, device=y.device)
    assert y.is_contiguous() and y.dtype == torch.float32 and w.dtype == torch.float32
    assert z is None or (z.stride(1) == 1 and z.dtype == out_dtype)
    mixers().gated_group_norm(y.data_ptr(), _p(z), is_f32(out), z.stride(0) if z is not None else 0, w.data_ptr(),
                              w.numel(), float(eps), out.data_ptr(), T, n, groups, bool(gate_after), stream_ptr())
    return out


# ---------------------------------------------------------------------------- gated feed-forward, routed experts
GLU_GELU_TANH, GLU_CLAMPED = 0, 1
ACT_RELU2 = 2   # routed_experts(kind=...): an expert without a gate, W_down relu(W_up h)^2
# XGS_TUNE moe_mfma=0: the general grouped GEMM for bf16 too (A/B and tests)
MOE_MFMA = tune.get_bool("moe_mfma", True)
MOE_TILE_SMALL, MOE_TILES_BIG = 16, (128, 64, 32)   # rows per expert tile of the sorted layout
MOE_TILE32_MIN = 12   # average rows per expert from which 32-row tiles replace 16-row ones (XGS_TUNE moe_tile32_min)
MOE_TILE32_MIN = tune.get_int("moe_tile32_min", MOE_TILE32_MIN)


def _glu_ref(g, u, kind, limit, alpha):
    if kind == GLU_GELU_TANH:
        return 0.5 * g * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (g + 0.044715 * g ** 3))) * u
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    return g * torch.sigmoid(alpha * g) * (u + 1.0)


def glu_act(x: torch.Tensor, kind: int, limit: float = 0.0, alpha: float = 1.702) -> torch.Tensor:
    """Rows [gate (F) | up (F)] -> [F]: GLU_GELU_TANH: gelu_tanh(gate) * up; GLU_CLAMPED: with g = min(gate, limit),
    u = clamp(up, -limit, limit): g * sigmoid(alpha g) * (u + 1)."""
    T, F2 = x.shape
    F_ = F2 // 2
    if not native_device(x):
        xf = x.float()
        return _glu_ref(xf[:, :F_], xf[:, F_:], kind, limit, alpha).to(x.dtype)
    assert x.stride(1) == 1
    out = torch.empty(T, F_, dtype=x.dtype, device=x.device)
    mixers().glu_act(x.data_ptr(), is_f32(x), x.stride(0), out.data_ptr(), T, F_, int(kind), float(limit), float(alpha),
                     stream_ptr())
    return out


ROUTER_FUSED_MAX_ROWS = 256     # steps of up to this many rows form the router logits inside the router kernel ...
ROUTER_FUSED_MAX_WORK = 16384   # ... when experts x width stays within this (measured on 64 rows: 13 against 16 us at
                                # 8 x 2048, 20 against 16 us at 8 x 4096)


def grouped_router(logits: Optional[torch.Tensor], correction: Optional[torch.Tensor], count: int, keep: int, top: int,
                   scale: float, rows: Optional[torch.Tensor] = None, router_w: Optional[torch.Tensor] = None):
    """fp32 router logits [T, E] -> (expert ids int32 [T, top], weights fp32 [T, top]). With `rows` (fp32 [T, W]) and
    `router_w` (fp32 [E, W]) in place of `logits` the logits are rows . router_w[e] in fp32: inside the router kernel
    for steps of few rows on the GPU (a launch less; the library product wins on long steps), else a matrix product. Scores are
    sigmoid(logits). Selection uses score + correction: the experts form `count` contiguous groups of equal
    size, a group is rated by the sum of its two highest selection scores, and only members of the `keep`
    highest-rated groups are eligible (everything else is excluded outright, selection score -inf). The
    returned weights are score * scale: the correction does not enter them and they are not normalised."""
    fused = False
    if logits is None:
        assert rows.dtype == router_w.dtype == torch.float32 and rows.shape[1] == router_w.shape[1]
        fused = native_device(rows) and rows.shape[0] <= ROUTER_FUSED_MAX_ROWS and rows.is_contiguous() \
            and router_w.is_contiguous() and router_w.numel() <= ROUTER_FUSED_MAX_WORK
        if not fused:
            logits = torch.nn.functional.linear(rows, router_w)
    T, E = (rows.shape[0], router_w.shape[0]) if fused else logits.shape
    if not fused and not native_device(logits):
        s = torch.sigmoid(logits.float())
        c = s + (correction if correction is not None else 0.0)
        per = E // count
        gsc = c.view(T, count, per).topk(min(2, per), -1).values.sum(-1)
        kept = torch.zeros(T, count, dtype=torch.bool)
        kept.scatter_(1, gsc.topk(keep, -1).indices, True)
        c = c.masked_fill(~kept.repeat_interleave(per, 1), float("-inf"))
        ids = c.topk(top, -1).indices
        return ids.to(torch.int32), s.gather(1, ids) * scale
    assert fused or (logits.dtype == torch.float32 and logits.is_contiguous())
    dev = rows.device if fused else logits.device
    ids = torch.empty(T, top, dtype=torch.int32, device=dev)
    wts = torch.empty(T, top, dtype=torch.float32, device=dev)
    mixers().grouped_router(0 if fused else logits.data_ptr(), _p(correction), T, E, int(count), int(keep), int(top),
                            float(scale), ids.data_ptr(), wts.data_ptr(), rows.data_ptr() if fused else 0,
                            router_w.data_ptr() if fused else 0, rows.shape[1] if fused else 0, stream_ptr())
    return ids, wts


def _act_ref(z, kind):
    assert kind == ACT_RELU2
    return torch.relu(z).pow(2)


@dataclass
class RoutedRows:
    """The experts' output rows before they are summed per token (routed_experts(combine=False)): row dest[t, j] of
    `y` (fp32, the sorted layout) is token t's j-th choice, to be weighted by wts[t, j] (None: 1). residual_norm takes
    it in place of its fp32 term and forms the sum itself. `dest` None: `y` is the finished sum [T, W]."""
    y: torch.Tensor
    dest: Optional[torch.Tensor] = None
    wts: Optional[torch.Tensor] = None


def routed_experts(h: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, kind: int,
                   limit: float = 0.0, alpha: float = 1.702, scale_input: bool = False, combine: bool = True):
    """sum_j wts[t, j] * W2[e] glu(W13[e] h_t), e = ids[t, j]. w13 [E, 2 F, K] holds each expert's gate rows then
    its up rows, w2 [E, W, F]. With an ungated `kind` (ACT_RELU2) w13 is [E, F, K] and the expert is W2 act(W13 h).
    `scale_input`: the weight multiplies the expert's INPUT instead of its output, sum_j expert_e(wts[t, j] h_t); the
    first product being linear, the weight is applied to its fp32 accumulator, act(wts * (W13 h)).
    Returns fp32 [T, W] (a sum in a fixed order per row), or with combine=False the rows as `RoutedRows`."""
    T, K = h.shape
    E = w13.shape[0]
    gated = kind in (GLU_GELU_TANH, GLU_CLAMPED)
    F_ = w13.shape[1] // 2 if gated else w13.shape[1]
    W, top = w2.shape[1], ids.shape[1]
    if not native_device(h):
        out = torch.zeros(T, W)
        hf = h.float()
        for e in range(E):
            tt, jj = torch.nonzero(ids == e, as_tuple=True)
            if tt.numel() == 0:
                continue
            wt = wts[tt, jj][:, None]
            gu = hf[tt] @ w13[e].float().t()
            if scale_input:
                gu = gu * wt
            gu = gu.to(h.dtype).float()
            a = _glu_ref(gu[:, :F_], gu[:, F_:], kind, limit, alpha) if gated else _act_ref(gu, kind)
            y = a.to(h.dtype).float() @ w2[e].float().t()
            out.index_add_(0, tt, y if scale_input else y * wt)
        return out if combine else RoutedRows(out)
    M = mixers()
    assert h.is_contiguous() and w13.is_contiguous() and w2.is_contiguous() and w13.dtype == w2.dtype == h.dtype
    assert wts.dtype == torch.float32 and wts.is_contiguous()
    pairs = T * top
    # rows of an expert are padded to whole tiles: 128 / 64-row tiles once the average expert has that many; 32-row
    # tiles once many experts would need a second 16-row tile (their weights would be streamed twice); else 16
    tm = next((t for t in MOE_TILES_BIG if pairs >= (t if t > 32 else MOE_TILE32_MIN) * E), MOE_TILE_SMALL)
    cap = (pairs + E * (tm - 1) + tm - 1) // tm * tm
    dev = h.device
    meta = torch.empty(cap + cap // tm + pairs, dtype=torch.int32, device=dev)
    rows, tile_e, dest = meta[:cap], meta[cap:cap + cap // tm], meta[cap + cap // tm:]
    M.moe_align(_i32(ids).data_ptr(), pairs, E, cap, tm, rows.data_ptr(), tile_e.data_ptr(), dest.data_ptr(), stream_ptr())
    act = torch.empty(cap, F_, dtype=h.dtype, device=dev)
    M.grouped_gemm(h.data_ptr(), is_f32(h), h.stride(0), w13.data_ptr(), rows.data_ptr(), tile_e.data_ptr(), cap, tm, top,
                   F_, K, 1 if gated else 2, act.data_ptr(), int(kind), float(limit), float(alpha),
                   wts.data_ptr() if scale_input else 0, MOE_MFMA, stream_ptr())
    y = torch.empty(cap, W, dtype=torch.float32, device=dev)
    M.grouped_gemm(act.data_ptr(), is_f32(act), F_, w2.data_ptr(), rows.data_ptr(), tile_e.data_ptr(), cap, tm, top, W, F_,
                   0, y.data_ptr(), 0, 0.0, 0.0, 0, MOE_MFMA, stream_ptr())
    if not combine:
        return RoutedRows(y, dest.view(T, top), None if scale_input else wts)
    out = torch.empty(T, W, dtype=torch.float32, device=dev)
    M.moe_combine(y.data_ptr(), dest.data_ptr(), 0 if scale_input else wts.data_ptr(), T, top, W, out.data_ptr(),
                  stream_ptr())
    return out


# ---------------------------------------------------------------------------- output norm, residual sum, next input norm
def post_norm_residual(x: torch.Tensor, y: Optional[torch.Tensor], y_bias: Optional[torch.Tensor],
                       post_w: Optional[torch.Tensor], mult: float, extra: Optional[torch.Tensor],
                       next_w: Optional[torch.Tensor], eps: float, out_dtype: Optional[torch.dtype] = None,
                       w_offset: float = 1.0, y2: Optional[torch.Tensor] = None,
                       pre_w: Optional[tuple] = None) -> Optional[torch.Tensor]:
    """A sublayer's output is normed before it joins the residual, and the next sublayer's input norm follows:
        u  = y + y_bias                                    (pre_w is None)
        u  = (N0(y) * pre_w[0] + N0(y2) * pre_w[1]) / 2    (two branches, each normed with a plain weight first)
        x <- x + mult * N0(u) * (w_offset + post_w) + extra
        n  = N0(x) * (w_offset + next_w)
    with N0(v) = v / sqrt(mean(v^2) + eps). x fp32 [T, W] is updated in place; y / y2 activation tensors or fp32,
    row-strided; y_bias, the weights fp32 [W]; extra fp32 [T, W]. y None: only `extra` is added. Returns n as
    `out_dtype` (None when next_w is None)."""
    T, W = x.shape

    def n0(v):
        return v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    if not native_device(x):
        if y is not None:
            u = y.float()
            if pre_w is not None:
                u = 0.5 * (n0(u) * pre_w[0] + n0(y2.float()) * pre_w[1])
            elif y_bias is not None:
                u = u + y_bias
            x.add_(mult * n0(u) * (w_offset + post_w))
        if extra is not None:
            x.add_(extra)
        return None if next_w is None else (n0(x) * (w_offset + next_w)).to(out_dtype)
    assert x.dtype == torch.float32 and x.is_contiguous()
    for t in (y, y2):
        assert t is None or (t.stride(1) == 1 and t.shape == x.shape)
    assert (pre_w is None) == (y2 is None) and (y2 is None or y2.dtype == y.dtype)
    assert extra is None or (extra.dtype == torch.float32 and extra.is_contiguous() and extra.shape == x.shape)
    out = torch.empty(T, W, dtype=out_dtype, device=x.device) if next_w is not None else None
    mixers().post_norm_residual(x.data_ptr(), _p(y), is_f32(y) if y is not None else True,
                                y.stride(0) if y is not None else 0, _p(y_bias), _p(y2),
                                y2.stride(0) if y2 is not None else 0, _p(pre_w[0]) if pre_w else 0,
                                _p(pre_w[1]) if pre_w else 0, _p(post_w), float(mult), _p(extra), _p(next_w),
                                float(w_offset), float(eps), _p(out), is_f32(out) if out is not None else True, T, W,
                                stream_ptr())
    return out


# ---------------------------------------------------------------------------- per-head q / k norm, rotation, cache append
def head_norm_rope_cache(src: torch.Tensor, H: int, G: int, dk: int, dv: int, wq: Optional[torch.Tensor],
                         wk: Optional[torch.Tensor], eps: float, rot: Optional[torch.Tensor], rot_dims: int, sm: SeqMeta,
                         kcache: torch.Tensor, vcache: torch.Tensor, out_dtype: torch.dtype, whole: bool = False,
                         half: bool = False, v_first: Optional[torch.Tensor] = None,
                         v_mix: Optional[torch.Tensor] = None) -> torch.Tensor:
    """From rows [q (H dk) | k (G dk) | v (G dv)] (fp32 or an activation tensor, row-strided): every q head and
    every k head is RMS-normed over its own dk entries with one weight of size dk shared by the heads (wq / wk, None
    = no norm) -- or, with `whole`, q and k are each normed over ALL their entries at once with weights of size H dk /
    G dk -- then the first rot_dims entries of each head are rotated pairwise (entry 2i with 2i + 1, or, with `half`,
    entry i with i + rot_dims / 2) by the table row of the token's position (rot fp32 [positions, rot_dims / 2, 2],
    None = no rotation). With `v_first` ([T, G dv], row-strided, the values another layer projected for the same
    tokens) and `v_mix` (fp32, one element, lambda) the values become (1 - lambda) v + lambda v_first. q is returned
    [T, H dk]; k and the (mixed) v go to cache rows slot_mapping[t]."""
    T = src.shape[0]
    nq, nk, nv = H * dk, G * dk, G * dv
    q = torch.empty(T, nq, dtype=out_dtype, device=src.device)
    assert (v_first is None) == (v_mix is None)
    if native_device(src):
        assert src.stride(1) == 1 and kcache.is_contiguous() and vcache.is_contiguous()
        assert kcache.dtype == vcache.dtype == out_dtype and kcache.shape[-1] == nk and vcache.shape[-1] == nv
        assert rot is None or (rot.dtype == torch.float32 and rot.is_contiguous() and rot.shape[1] * 2 == rot_dims)
        assert rot_dims % 2 == 0 and rot_dims <= dk
        assert not whole or ((wq is None or wq.numel() == nq) and (wk is None or wk.numel() == nk))
        if v_first is not None:
            assert v_first.stride(1) == 1 and v_first.shape == (T, nv) and v_first.dtype == src.dtype
            assert v_mix.dtype == torch.float32 and v_mix.numel() == 1
        mixers().head_norm_rope_cache(src.data_ptr(), is_f32(src), src.stride(0), H, G, dk, dv, _p(wq), _p(wk),
                                      float(eps), _p(rot), rot.shape[0] if rot is not None else 0,
                                      rot_dims if rot is not None else 0, _i32(sm.positions).data_ptr(),
                                      _i32(sm.slot_mapping).data_ptr(), q.data_ptr(), kcache.data_ptr(),
                                      vcache.data_ptr(), is_f32(q), T, bool(whole), bool(half), _p(v_first),
                                      v_first.stride(0) if v_first is not None else 0, _p(v_mix), stream_ptr())
        return q
    pf = src.float()

    def prep(v, n, w):
        if w is not None and whole:
            v = v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w
        v = v.reshape(T, n, dk)
        if w is not None and not whole:
            v = v / torch.sqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w
        if rot is not None and rot_dims:
            v = _rotate_pairs(v, rot, sm.positions, rot_dims, half)
        return v.reshape(T, n * dk)
    q.copy_(prep(pf[:, :nq], H, wq).to(out_dtype))
    ok = sm.slot_mapping >= 0
    rows = sm.slot_mapping[ok].long()
    kcache.view(-1, nk)[rows] = prep(pf[:, nq:nq + nk], G, wk)[ok].to(kcache.dtype)
    vals = pf[:, nq + nk:nq + nk + nv]
    if v_first is not None:
        vals = (1.0 - v_mix) * vals + v_mix * v_first.float()
    vcache.view(-1, nv)[rows] = vals[ok].to(vcache.dtype)
    return q


CONV_PREP_FUSED = tune.get_bool("conv_prep_fused", True)   # XGS_TUNE conv_prep_fused=0: convolution and norm apart
# steps of more rows run the convolution as a kernel of its own: over a long portion it slides a register window along
# the tokens (one load per input), where the one-pass kernel loads every tap of every output
CONV_PREP_FUSED_MAX_ROWS = 1024


def conv_head_norm_rope_cache(proj: torch.Tensor, conv_w: torch.Tensor, state: torch.Tensor, H: int, G: int, dk: int,
                              dv: int, wq: Optional[torch.Tensor], wk: Optional[torch.Tensor], eps: float,
                              rot: Optional[torch.Tensor], rot_dims: int, sm: SeqMeta, kcache: torch.Tensor,
                              vcache: torch.Tensor) -> torch.Tensor:
    """causal_conv (no bias, no activation) of the columns [q | k | v] of a fused projection row, then
    head_norm_rope_cache of the result; in one pass on the GPU for steps of single tokens and short portions (the
    convolution's output never reaches memory).
    conv_w fp32 [channels, taps]; state fp32 [slots, taps - 1, channels] is updated."""
    C = (H + G) * dk + G * dv
    taps = conv_w.shape[1]
    if not (native_device(proj) and CONV_PREP_FUSED and dk <= 256 and proj.shape[0] <= CONV_PREP_FUSED_MAX_ROWS):
        qkv = causal_conv(proj[:, :C], conv_w, None, state, sm, torch.float32)
        return head_norm_rope_cache(qkv, H, G, dk, dv, wq, wk, eps, rot, rot_dims, sm, kcache, vcache, proj.dtype)
    T = proj.shape[0]
    q = torch.empty(T, H * dk, dtype=proj.dtype, device=proj.device)
    assert proj.stride(1) == 1 and conv_w.dtype == torch.float32 and conv_w.is_contiguous() and conv_w.shape[0] == C
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (taps - 1, C)
    assert kcache.is_contiguous() and vcache.is_contiguous() and kcache.dtype == vcache.dtype == proj.dtype
    assert kcache.shape[-1] == G * dk and vcache.shape[-1] == G * dv and rot_dims % 2 == 0 and rot_dims <= dk
    assert rot is None or (rot.dtype == torch.float32 and rot.is_contiguous() and rot.shape[1] * 2 == rot_dims)
    mixers().conv_head_norm_rope_cache(proj.data_ptr(), is_f32(proj), proj.stride(0), conv_w.data_ptr(), taps,
                                       state.data_ptr(), _i32(sm.qsl).data_ptr(), _i32(sm.seq_lens).data_ptr(),
                                       _i32(sm.slots).data_ptr(), _i32(sm.token_seq).data_ptr(), sm.num_seqs, sm.max_q,
                                       H, G, dk, dv, _p(wq), _p(wk), float(eps), _p(rot),
                                       rot.shape[0] if rot is not None else 0, rot_dims if rot is not None else 0,
                                       _i32(sm.slot_mapping).data_ptr(), q.data_ptr(), kcache.data_ptr(),
                                       vcache.data_ptr(), is_f32(q), T, stream_ptr())
    return q


# ---------------------------------------------------------------------------- mixing the heads' weight maps
def talk_mix(o_all: torch.Tensor, talk: torch.Tensor, H: int, G: int, dv: int,
             gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Softmax weights mixed over heads AFTER the softmax, p'_h = sum_g talk[h, g] p_g, applied to the values of head
    h's own key/value head c(h) = h // (H / G), equal  sum_g talk[h, g] * (p_g V_c(h)). o_all [T, H * G * dv] holds
    p_g V_c for every (g, c) (masked_attention with values=V_ALL); returns [T, H * dv], head h's row times
    sigmoid(gate[t, h]) when `gate` ([T, >= H], row-strided) is given. The sum over g is fp32."""
    T = o_all.shape[0]
    if not native_device(o_all):
        o = o_all.float().view(T, H, G, dv)
        sel = o[:, :, torch.arange(H) // (H // G), :]            # [T, g, h, dv]: head g's weights on h's values
        out = torch.einsum("hg,tghd->thd", talk.float(), sel)
        if gate is not None:
            out = out * torch.sigmoid(gate[:, :H].float())[:, :, None]
        return out.reshape(T, H * dv).to(o_all.dtype)
    assert o_all.is_contiguous() and talk.dtype == torch.float32 and talk.is_contiguous() and talk.shape == (H, H)
    assert gate is None or (gate.stride(1) == 1 and gate.dtype == o_all.dtype)
    out = torch.empty(T, H * dv, dtype=o_all.dtype, device=o_all.device)
    mixers().talk_mix(o_all.data_ptr(), is_f32(o_all), talk.data_ptr(), _p(gate), gate.stride(0) if gate is not None else 0,
                      out.data_ptr(), T, H, G, dv, stream_ptr())
    return out


# ---------------------------------------------------------------------------- gated linear recurrence
# XGS_TUNE scan_cols=32|64: state columns per workgroup of the gated linear scan (0: by the size of the step)
SCAN_COLS = tune.get_int("scan_cols", 0)
# XGS_TUNE scan_two_pass=0: every portion in one workgroup per (sequence, head, column block) (A/B and tests)
SCAN_TWO_PASS = tune.get_bool("scan_two_pass", True)
SCAN_TWO_PASS_MIN = 512   # portions longer than this may be scanned as chunks of 256 tokens over the whole grid ...
SCAN_FILL_WGS = 192       # ... when their one-launch form would start at most this many workgroups (256 compute units)


def _scan_scratch(T: int, sm: SeqMeta, H: int, dk: int, dv: int, device) -> Optional[torch.Tensor]:
    """Chunk summaries of a long portion (gated_linear_scan in two launches); None for short steps and for steps whose
    long sequences fill the chip by themselves (the chunked form runs the recurrence twice: measured 1.7x - 3.7x faster
    on 128 - 32 workgroups, 10 % slower on 256)."""
    if not SCAN_TWO_PASS or sm.max_q <= SCAN_TWO_PASS_MIN:
        return None
    cols = 32 if (SCAN_COLS == 32 or (SCAN_COLS != 64 and dv <= 32)) else 64
    if max(1, T // sm.max_q) * H * ((dv + cols - 1) // cols) > SCAN_FILL_WGS:
        return None
    return torch.empty(mixers().gated_linear_scan_scratch_floats(T, sm.num_seqs, H, dk, dv), dtype=torch.float32,
                       device=device)


def lower_bound_gates(proj: torch.Tensor, off_q: int, off_f: int, n: int, f_bias: Optional[torch.Tensor],
                      lower: torch.Tensor):
    """From a fused projection row: q = silu(proj[off_q : off_q + n]) and the forget gate
    f = l + (1 - l) * sigmoid(proj[off_f : off_f + n] + f_bias), bounded below by l = `lower` (fp32 [n]).
    Returns (q, f), fp32 [T, n] each."""
    T = proj.shape[0]
    if not native_device(proj):
        pf = proj.float()
        z = pf[:, off_q:off_q + n]
        g = pf[:, off_f:off_f + n] + (f_bias if f_bias is not None else 0.0)
        return z * torch.sigmoid(z), lower + (1.0 - lower) * torch.sigmoid(g)
    assert proj.stride(1) == 1 and lower.dtype == torch.float32
    qf = torch.empty(2, T, n, dtype=torch.float32, device=proj.device)
    mixers().lower_bound_gates(proj.data_ptr(), is_f32(proj), proj.stride(0), off_q, off_f, n, _p(f_bias),
                               lower.data_ptr(), qf[0].data_ptr(), qf[1].data_ptr(), T, stream_ptr())
    return qf[0], qf[1]


def gated_linear_scan(q: torch.Tensor, f: torch.Tensor, k: Optional[torch.Tensor], v: torch.Tensor, state: torch.Tensor,
                      H: int, dk: int, dv: int, sm: SeqMeta) -> torch.Tensor:
    """Per head a [dk x dv] fp32 state with one decay per row:  S <- diag(f) S + k v^T,  o = S^T q;  k = 1 - f when
    `k` is None (write strength = complement of the forget gate). q, f, k fp32 [T, H dk]; v [T, H dv] (row-strided
    activation). state fp32 [slots, H, dk, dv] is carried and updated. Returns o fp32 [T, H dv]."""
    T = q.shape[0]
    o = torch.empty(T, H * dv, dtype=torch.float32, device=q.device)
    if native_device(q):
        assert q.dtype == f.dtype == torch.float32 and q.is_contiguous() and f.is_contiguous() and v.stride(1) == 1
        assert k is None or (k.dtype == torch.float32 and k.is_contiguous())
        assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, dk, dv)
        scratch = _scan_scratch(T, sm, H, dk, dv, q.device)
        mixers().gated_linear_scan(q.data_ptr(), f.data_ptr(), _p(k), 0, 0, 0, 0, 0, 0, v.data_ptr(), is_f32(v),
                                   v.stride(0), state.data_ptr(), _i32(sm.qsl).data_ptr(), _i32(sm.seq_lens).data_ptr(),
                                   _i32(sm.slots).data_ptr(), o.data_ptr(), sm.num_seqs, H, dk, dv, SCAN_COLS,
                                   _p(scratch), sm.max_q, T, stream_ptr())
        return o
    qh, fh = q.view(T, H, dk), f.view(T, H, dk)
    kh = (1.0 - fh) if k is None else k.view(T, H, dk)
    vh = v.float().reshape(T, H, dv)
    qsl, sl, slots = sm.qsl.tolist(), sm.seq_lens.tolist(), sm.slots.tolist()
    for s in range(sm.num_seqs):
        lo, hi = qsl[s], qsl[s + 1]
        if slots[s] < 0 or hi <= lo:
            continue
        S = state[slots[s]].clone() if sl[s] - (hi - lo) > 0 else torch.zeros(H, dk, dv)
        for t in range(lo, hi):
            S = fh[t][:, :, None] * S + kh[t][:, :, None] * vh[t][:, None, :]
            o[t] = torch.einsum("hkd,hk->hd", S, qh[t]).reshape(H * dv)
        state[slots[s]] = S
    return o


def lower_bound_recurrence(proj: torch.Tensor, off_q: int, off_f: int, off_v: int, f_bias: Optional[torch.Tensor],
                           lower: torch.Tensor, state: torch.Tensor, H: int, dk: int, dv: int, sm: SeqMeta) -> torch.Tensor:
    """lower_bound_gates + gated_linear_scan with k = 1 - f on the columns [q | f | v] of one fused projection row:
    on the GPU the gates are formed while the scan stages its inputs. Returns o fp32 [T, H dv]."""
    n = H * dk
    v = proj[:, off_v:off_v + H * dv]
    if not native_device(proj):
        q, f = lower_bound_gates(proj, off_q, off_f, n, f_bias, lower)
        return gated_linear_scan(q, f, None, v, state, H, dk, dv, sm)
    assert proj.stride(1) == 1 and lower.dtype == torch.float32 and lower.numel() == n
    assert state.dtype == torch.float32 and state.is_contiguous() and state.shape[1:] == (H, dk, dv)
    o = torch.empty(proj.shape[0], H * dv, dtype=torch.float32, device=proj.device)
    scratch = _scan_scratch(proj.shape[0], sm, H, dk, dv, proj.device)
    mixers().gated_linear_scan(0, 0, 0, proj.data_ptr(), proj.stride(0), off_q, off_f, _p(f_bias), lower.data_ptr(),
                               v.data_ptr(), is_f32(proj), proj.stride(0), state.data_ptr(), _i32(sm.qsl).data_ptr(),
                               _i32(sm.seq_lens).data_ptr(), _i32(sm.slots).data_ptr(), o.data_ptr(), sm.num_seqs, H, dk,
                               dv, SCAN_COLS, _p(scratch), sm.max_q, proj.shape[0], stream_ptr())
    return o


# ---------------------------------------------------------------------------- squared relu
def relu2(z: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """max(z + bias, 0)^2 (bias fp32 per column)."""
    if not native_device(z):
        v = z.float() + (bias if bias is not None else 0)
        return torch.relu(v).pow(2).to(z.dtype)
    assert z.is_contiguous()
    out = torch.empty_like(z)
    mixers().relu2(z.data_ptr(), is_f32(z), _p(bias), out.data_ptr(), z.numel(), z.shape[-1], stream_ptr())
    return out


# ---------------------------------------------------------------------------- minimal gated recurrence
# XGS_TUNE mingru_two_pass=0: every portion in one workgroup per (sequence, 64 channels) (A/B and tests)
MINGRU_TWO_PASS = tune.get_bool("mingru_two_pass", True)
MINGRU_TWO_PASS_MIN = 512   # portions longer than this are scanned as chunks of 256 tokens over the whole grid


def mingru_scan(proj: torch.Tensor, off_z: int, off_x: int, off_g: int, n: int, bias_z: Optional[torch.Tensor],
                bias_x: Optional[torch.Tensor], state: torch.Tensor, sm: SeqMeta, out_dtype: torch.dtype) -> torch.Tensor:
    """Per channel, with z = sigmoid(proj[off_z + c] + bias_z[c]) and u = proj[off_x + c] + bias_x[c]:
        S <- (1 - z) S + z * cand(u),   cand(u) = u + 1/2 (u >= 0), sigmoid(u) (u < 0)
    (both gate and candidate read only the current token), and the output S * silu(proj[off_g + c]). proj [T, >= ...]
    is a row-strided activation tensor; state fp32 [slots, n] is carried and updated. Returns [T, n] as out_dtype."""
    T = proj.shape[0]
    out = torch.empty(T, n, dtype=out_dtype, device=proj.device)
    if native_device(proj):
        assert proj.stride(1) == 1 and state.dtype == torch.float32 and state.is_contiguous() and state.shape[1] == n
        assert max(off_z, off_x, off_g) + n <= proj.shape[1]
        scratch = None
        if MINGRU_TWO_PASS and sm.max_q > MINGRU_TWO_PASS_MIN:   # a long portion: its pieces spread over the whole grid
            scratch = torch.empty(mixers().mingru_scratch_floats(T, sm.num_seqs, n), dtype=torch.float32, device=proj.device)
        mixers().mingru_scan(proj.data_ptr(), is_f32(proj), proj.stride(0), off_z, off_x, off_g, n, _p(bias_z), _p(bias_x),
                             state.data_ptr(), _i32(sm.qsl).data_ptr(), _i32(sm.seq_lens).data_ptr(),
                             _i32(sm.slots).data_ptr(), out.data_ptr(), is_f32(out), sm.num_seqs, sm.max_q, _p(scratch), T,
                             stream_ptr())
        return out
    pf = proj.float()
    z = torch.sigmoid(pf[:, off_z:off_z + n] + (bias_z if bias_z is not None else 0.0))
    u = pf[:, off_x:off_x + n] + (bias_x if bias_x is not None else 0.0)
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = pf[:, off_g:off_g + n]
    g = g * torch.sigmoid(g)
    qsl, sl, slots = sm.qsl.tolist(), sm.seq_lens.tolist(), sm.slots.tolist()
    for s in range(sm.num_seqs):
        lo, hi = qsl[s], qsl[s + 1]
        if slots[s] < 0 or hi <= lo:
            out[lo:hi] = 0
            continue
        S = state[slots[s]].clone() if sl[s] - (hi - lo) > 0 else torch.zeros(n)
        for t in range(lo, hi):
            S = (1.0 - z[t]) * S + z[t] * cand[t]
            out[t] = (S * g[t]).to(out_dtype)
        state[slots[s]] = S
    return out


# ---------------------------------------------------------------------------- per-channel decay of a linear recurrence
def decay_gates(proj: torch.Tensor, off_q: int, off_k: int, n: int, q_scale: float, z: torch.Tensor,
                z_bias: Optional[torch.Tensor], tau: float):
    """Inputs of gated_linear_scan with a decay per key channel: q = proj[off_q : off_q + n] * q_scale,
    k = proj[off_k : off_k + n] and f = sigmoid(z + z_bias)^(1 / tau), evaluated as exp(-softplus(-(z + z_bias)) / tau).
    proj / z row-strided activation tensors. Returns (q, f, k), fp32 [T, n] each."""
    T = proj.shape[0]
    if not native_device(proj):
        pf = proj.float()
        zz = z.float() + (z_bias if z_bias is not None else 0.0)
        f = torch.exp(-torch.nn.functional.softplus(-zz) / tau)
        return pf[:, off_q:off_q + n] * q_scale, f, pf[:, off_k:off_k + n].clone()
    assert proj.stride(1) == 1 and z.stride(1) == 1 and z.dtype == proj.dtype and z.shape == (T, n)
    out = torch.empty(3, T, n, dtype=torch.float32, device=proj.device)
    mixers().decay_gates(proj.data_ptr(), is_f32(proj), proj.stride(0), off_q, off_k, n, float(q_scale), z.data_ptr(),
                         z.stride(0), _p(z_bias), float(1.0 / tau), out[0].data_ptr(), out[1].data_ptr(),
                         out[2].data_ptr(), T, stream_ptr())
    return out[0], out[1], out[2]
