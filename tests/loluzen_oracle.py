"""Slow, dense, fp64 oracle of the Loluzen design: one function per mechanism, whole sequences,
no cache, no batching. It shares nothing with xgserve's model or ops; the tests compare the
framework against it. Weights are a dict of checkpoint tensor names -> fp64 tensors.

Notation: x_t is the residual row of token t (t = 0 is the sequence's first token). A layer is
    x <- x + m * N(mixer(N(x; norm1)); norm1b),   x <- x + m * N(ff(N(x; norm2)); norm2b)
with N(v; w) = v / sqrt(mean(v^2) + eps) * (1 + w). A run of layers may be repeated with the same
weights; every repetition after the first starts from x + e, e being the scaled embedding rows.
"""
import math

import torch

F64 = torch.float64


# ------------------------------------------------------------------------------ small pieces
def unit_rms(v, eps):
    """v / sqrt(mean(v^2) + eps) over the last axis."""
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def silu(z):
    return z / (1.0 + torch.exp(-z))


def shifted_conv(u, w):
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j); rows before t = 0 are zero. u [T, C], w [C, taps]."""
    T, C = u.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            src = t - taps + 1 + j
            if src >= 0:
                out[t] += w[:, j] * u[src]
    return out


def rot_frequencies(rot):
    """Per pair i: base^(-2i / dims), then the wavelength-dependent rescaling (long waves slowed by
    `factor`, short ones kept, a linear blend in between)."""
    dims = int(rot["dims"])
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    sc = rot.get("scaling")
    if sc is None:
        return f
    factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
    out = f.clone()
    for i in range(f.numel()):
        wave = 2.0 * math.pi / float(f[i])
        if wave < orig / high:
            continue
        if wave > orig / low:
            out[i] = f[i] / factor
        else:
            s = (orig / wave - low) / (high - low)
            out[i] = (1.0 - s) * f[i] / factor + s * f[i]
    return out


def rotate_pairs(v, freqs, dims):
    """v [T, heads, n]: entries (2i, 2i + 1), i < dims / 2, of token t turn by the angle t * freqs[i]."""
    T = v.shape[0]
    ang = torch.arange(T, dtype=F64)[:, None] * freqs[None, :]          # [T, dims / 2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out = v.clone()
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def causal_weights(q, k, scale, r1=None, r2=None):
    """Softmax weights [H, T, T] of H query heads over G key heads (head h reads key head h // (H / G)); query i
    sees keys j <= i; with r1 / r2 the score loses r1_h * ln(1 + r2_h * (i - j))."""
    T, H, _ = q.shape
    G = k.shape[1]
    P = torch.zeros(H, T, T, dtype=F64)
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).clamp(min=0).to(F64)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if r1 is not None:
            s = s - r1[h] * torch.log1p(r2[h] * dist)
        s = s.masked_fill(torch.arange(T)[None, :] > torch.arange(T)[:, None], float("-inf"))
        P[h] = torch.softmax(s, -1)
    return P


# ------------------------------------------------------------------------------ mixer "attention"
def conv_rope_attention(Wt, pre, m, h, eps):
    """Projections -> short causal convolution per channel -> per-head RMS norm of q and k (one weight of size
    dim for all heads) -> rotation of the first rot.dims entries of each head -> causal softmax -> each head's
    output times sigmoid of its gate logit -> output projection."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = shifted_conv(h @ Wt[pre + "q"].T, Wt[pre + "q.conv"]).reshape(T, H, dk)
    k = shifted_conv(h @ Wt[pre + "k"].T, Wt[pre + "k.conv"]).reshape(T, G, dk)
    v = shifted_conv(h @ Wt[pre + "v"].T, Wt[pre + "v.conv"]).reshape(T, G, dv)
    q = unit_rms(q, eps) * Wt[pre + "q.norm"]
    k = unit_rms(k, eps) * Wt[pre + "k.norm"]
    if m.get("rot") and int(m["rot"]["dims"]) > 0:
        fr = rot_frequencies(m["rot"])
        q, k = rotate_pairs(q, fr, int(m["rot"]["dims"])), rotate_pairs(k, fr, int(m["rot"]["dims"]))
    P = causal_weights(q, k, float(m["scale"]))
    gate = torch.sigmoid(h @ Wt[pre + "g"].T)                            # [T, H]
    o = torch.stack([P[hd] @ v[:, hd // (H // G)] for hd in range(H)], 1) * gate[:, :, None]
    return o.reshape(T, H * dv) @ Wt[pre + "o"].T


# ------------------------------------------------------------------------------ mixer "parallel": left branch
def talking_attention(Wt, pre, m, h):
    """Biased projections, no rotation, a logarithmic distance penalty on the scores, causal softmax, then the
    heads' weight maps are mixed by T[h, g] before head h applies them to the values of its own key/value head."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ Wt[pre + "q"].T + Wt[pre + "q.b"]).reshape(T, H, dk)
    k = (h @ Wt[pre + "k"].T + Wt[pre + "k.b"]).reshape(T, G, dk)
    v = (h @ Wt[pre + "v"].T + Wt[pre + "v.b"]).reshape(T, G, dv)
    P = causal_weights(q, k, float(m["scale"]), Wt[pre + "r1"], Wt[pre + "r2"])
    P = torch.einsum("hg,gij->hij", Wt[pre + "talk"], P)
    gate = torch.sigmoid(h @ Wt[pre + "g"].T)
    o = torch.stack([P[hd] @ v[:, hd // (H // G)] for hd in range(H)], 1) * gate[:, :, None]
    return o.reshape(T, H * dv) @ Wt[pre + "o"].T


# ------------------------------------------------------------------------------ mixer "parallel": right branch
def gated_linear_recurrence(Wt, pre, m, h, eps, states=None):
    """Per head a [dim x vdim] state: S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t, with
    q = silu(W_q h) and f = l + (1 - l) * sigmoid(W_f h + b) bounded below by l; o is RMS-normed per head."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ Wt[pre + "q"].T).reshape(T, H, dk)
    low = Wt[pre + "lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ Wt[pre + "f"].T + Wt[pre + "f.b"])).reshape(T, H, dk)
    v = (h @ Wt[pre + "v"].T).reshape(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = f[t, hd][:, None] * S + torch.outer(1.0 - f[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
        if states is not None:
            states.append(S)
    o = unit_rms(o, eps) * Wt[pre + "norm"]
    return o.reshape(T, H * dv) @ Wt[pre + "o"].T


def parallel_mixer(Wt, pre, m, h, eps):
    """Mean of the two branches, each RMS-normed over the model width with its own plain weight."""
    a = unit_rms(talking_attention(Wt, pre + "left.", m["left"], h), eps) * Wt[pre + "left.out"]
    b = unit_rms(gated_linear_recurrence(Wt, pre + "right.", m["right"], h, eps), eps) * Wt[pre + "right.out"]
    return 0.5 * (a + b)


# ------------------------------------------------------------------------------ feed-forward
def relu2_ff(Wt, pre, h):
    z = torch.relu(h @ Wt[pre + "up"].T + Wt[pre + "up.b"])
    return (z * z) @ Wt[pre + "down"].T + Wt[pre + "down.b"]


# ------------------------------------------------------------------------------ the model
def layer_order(cfg):
    """Indices of the layers in the order they run."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def pass_starts(cfg):
    """Positions in layer_order() at which a repetition after the first begins."""
    lp = cfg.get("loop")
    if not lp:
        return set()
    a, b = int(lp["start"]), int(lp["stop"])
    return {a + r * (b - a) for r in range(1, int(lp["times"]))}


def forward(cfg, Wt, tokens, residuals=None):
    """Logits [T, vocab] of one sequence; `residuals` collects x after every layer run."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])

    def N(v, name):
        return unit_rms(v, eps) * (1.0 + Wt[name])
    e = Wt["embed"][torch.as_tensor(tokens)] * float(cfg["embedding"]["scale"])
    x = e.clone()
    again = pass_starts(cfg)
    for run, i in enumerate(layer_order(cfg)):
        L, b = cfg["layers"][i], f"l{i}."
        if run in again:
            x = x + e
        h = N(x, b + "norm1")
        if L["type"] == "attention":
            y = conv_rope_attention(Wt, b + "mix.", L["mixer"], h, eps)
        else:
            y = parallel_mixer(Wt, b + "mix.", L["mixer"], h, eps)
        x = x + mult * N(y, b + "norm1b")
        if L.get("mlp") is not None:
            x = x + mult * N(relu2_ff(Wt, b + "mlp.", N(x, b + "norm2")), b + "norm2b")
        if residuals is not None:
            residuals.append(x.clone())
    return N(x, "final.norm") @ Wt["head"].T


# ------------------------------------------------------------------------------ test models
def random_weights(config, seed=0):
    """Random weights of a configuration, rounded to bfloat16 (what a checkpoint stores)."""
    g = torch.Generator().manual_seed(seed)
    W, V = config["width"], config["vocab"]
    out = {}

    def mat(name, o, i, gain=1.0):
        out[name] = torch.randn(o, i, generator=g) * gain / math.sqrt(i)

    def vec(name, n, std, mean=0.0):
        out[name] = torch.randn(n, generator=g) * std + mean
    out["embed"] = torch.randn(V, W, generator=g) * 0.5
    mat("head", V, W)
    vec("final.norm", W, 0.2)
    for n, layer in enumerate(config["layers"]):
        pre, m = f"l{n}.", layer["mixer"]
        vec(pre + "norm1", W, 0.2)
        vec(pre + "norm1b", W, 0.2)
        if layer["type"] == "attention":
            H, G, dk, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            for nm, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
                mat(pre + "mix." + nm, rows, W, 2.0)
                out[pre + "mix." + nm + ".conv"] = torch.randn(rows, taps, generator=g) * 0.5 + 1.0 / taps
            vec(pre + "mix.q.norm", dk, 0.3, 1.5)
            vec(pre + "mix.k.norm", dk, 0.3, 1.5)
            mat(pre + "mix.g", H, W, 2.0)
            mat(pre + "mix.o", W, H * dv)
        else:
            a, r = m["left"], m["right"]
            H, G, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            for nm, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
                mat(pre + "mix.left." + nm, rows, W, 2.0)
                vec(pre + "mix.left." + nm + ".b", rows, 0.3)
            out[pre + "mix.left.r1"] = torch.rand(H, generator=g) * 2.0
            out[pre + "mix.left.r2"] = torch.rand(H, generator=g) * 3.0 + 0.05
            out[pre + "mix.left.talk"] = torch.eye(H) * 0.7 + torch.randn(H, H, generator=g) * 0.4
            mat(pre + "mix.left.g", H, W, 2.0)
            mat(pre + "mix.left.o", W, H * dv)
            n_, Hr = r["heads"] * r["dim"], r["heads"]
            mat(pre + "mix.right.q", n_, W, 2.0)
            mat(pre + "mix.right.f", n_, W, 2.0)
            vec(pre + "mix.right.f.b", n_, 0.5, 1.0)
            out[pre + "mix.right.lower"] = torch.rand(n_, generator=g) * 0.95
            mat(pre + "mix.right.v", Hr * r["vdim"], W, 2.0)
            vec(pre + "mix.right.norm", r["vdim"], 0.3, 1.0)
            mat(pre + "mix.right.o", W, Hr * r["vdim"])
            vec(pre + "mix.left.out", W, 0.3, 1.0)
            vec(pre + "mix.right.out", W, 0.3, 1.0)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        vec(pre + "norm2", W, 0.2)
        vec(pre + "norm2b", W, 0.2)
        mat(pre + "mlp.up", mlp["ff"], W, 1.5)
        vec(pre + "mlp.up.b", mlp["ff"], 0.3)
        mat(pre + "mlp.down", W, mlp["ff"])
        vec(pre + "mlp.down.b", W, 0.3)
    return {k: v.to(torch.bfloat16).to(F64) for k, v in out.items()}


def write_checkpoint(path, config, Wt):
    import json
    import os

    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in Wt.items()}, os.path.join(path, "model.safetensors"))
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
