"""Dense fp64 forms of every Lotelix mechanism, one function per mechanism, for whole sequences at once.

Written from the design's equations; shares no code with xgserve. `weights` maps checkpoint tensor names to tensors,
`cfg` is the checkpoint's configuration dictionary. Everything is O(T^2) / token-by-token and meant for short inputs.
"""
import math

import torch

F64 = torch.float64


def d(t):
    return t.to(F64)


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    """The vector in `groups` equal consecutive parts, each divided by its own root mean square; times w."""
    T, W = x.shape
    return unit_rms(x.reshape(T, groups, W // groups), eps).reshape(T, W) * w


def frequencies(rot):
    n = int(rot["dims"])
    f = torch.tensor([float(rot["base"]) ** (-2.0 * i / n) for i in range(n // 2)], dtype=F64)
    sc = rot.get("scaling")
    if sc is None:
        return f
    factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
    out = []
    for fi in f.tolist():
        wave = 2 * math.pi / fi
        if wave < orig / high:
            out.append(fi)
        elif wave > orig / low:
            out.append(fi / factor)
        else:
            s = (orig / wave - low) / (high - low)
            out.append((1 - s) * fi / factor + s * fi)
    return torch.tensor(out, dtype=F64)


def rotate(x, pos, rot, layout):
    """x [T, heads, dim]; the first rot.dims entries of each head turn by pos * f_i. layout "half": entry i pairs with
    i + dims / 2; "pairs": entry 2 i with 2 i + 1."""
    n = int(rot["dims"])
    if n == 0:
        return x
    ang = pos.to(F64)[:, None] * frequencies(rot)[None, :]      # [T, n / 2]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    out = x.clone()
    if layout == "half":
        u, v = x[..., :n // 2], x[..., n // 2:n]
        out[..., :n // 2] = u * c - v * s
        out[..., n // 2:n] = v * c + u * s
    else:
        u, v = x[..., 0:n:2], x[..., 1:n:2]
        out[..., 0:n:2] = u * c - v * s
        out[..., 1:n:2] = v * c + u * s
    return out


def mingru(h, w, pre):
    """h [T, W] -> [T, W]: the minimal gated recurrence on a zero initial state."""
    z = torch.sigmoid(h @ d(w[pre + "z"]).T + d(w[pre + "z.b"]))
    u = h @ d(w[pre + "x"]).T + d(w[pre + "x.b"])
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    g = h @ d(w[pre + "g"]).T
    S = torch.zeros(z.shape[1], dtype=F64)
    rows = []
    for t in range(h.shape[0]):
        S = (1 - z[t]) * S + z[t] * cand[t]
        rows.append(S * g[t] * torch.sigmoid(g[t]))
    return torch.stack(rows) @ d(w[pre + "o"]).T


def window_attention(h, w, pre, m, v_first):
    """Sliding-window softmax attention with a sink, rotate-half positions, value mixing and an output gate.
    Returns (output [T, W], this layer's own projected values [T, G vdim])."""
    T = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = (h @ d(w[pre + "q"]).T).reshape(T, H, dk)
    k = (h @ d(w[pre + "k"]).T).reshape(T, G, dk)
    v_own = h @ d(w[pre + "v"]).T
    v = v_own
    if v_first is not None:
        lam = float(w[pre + "vmix"])
        v = (1 - lam) * v_own + lam * v_first
    v = v.reshape(T, G, dv)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"], "half"), rotate(k, pos, m["rot"], "half")
    size = int(m["mask"]["size"]) if m.get("mask") else T + 1
    sink = d(w[pre + "sink"])
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        lo = max(0, i - size + 1)
        for hh in range(H):
            c = hh // (H // G)
            sc = (k[lo:i + 1, c] @ q[i, hh]) * float(m["scale"])
            mx = max(float(sc.max()), float(sink[hh]))
            e = torch.exp(sc - mx)
            den = e.sum() + math.exp(float(sink[hh]) - mx)
            out[i, hh] = (e / den) @ v[lo:i + 1, c]
    gate = torch.sigmoid(h @ d(w[pre + "g"]).T)
    return (out.reshape(T, H * dv) * gate) @ d(w[pre + "o"]).T, v_own


def sigmoid_attention(h, w, pre, m, eps):
    """Causal attention whose weights are sigmoid(score + bias_h), not normalised; biased projections, whole-vector
    q / k norms before the interleaved rotation."""
    T = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    pos = torch.arange(T)
    q = unit_rms(h @ d(w[pre + "q"]).T + d(w[pre + "q.b"]), eps) * d(w[pre + "q.norm"])
    k = unit_rms(h @ d(w[pre + "k"]).T + d(w[pre + "k.b"]), eps) * d(w[pre + "k.norm"])
    v = (h @ d(w[pre + "v"]).T + d(w[pre + "v.b"])).reshape(T, G, dv)
    q, k = q.reshape(T, H, dk), k.reshape(T, G, dk)
    if m.get("rot"):
        q, k = rotate(q, pos, m["rot"], "pairs"), rotate(k, pos, m["rot"], "pairs")
    pb = d(w[pre + "pb"])
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        for hh in range(H):
            c = hh // (H // G)
            p = torch.sigmoid((k[:i + 1, c] @ q[i, hh]) * float(m["scale"]) + pb[hh])
            out[i, hh] = p @ v[:i + 1, c]
    return out.reshape(T, H * dv) @ d(w[pre + "o"]).T + d(w[pre + "o.b"])


def decayed_linear_attention(h, w, pre, m, eps):
    """Per head S <- diag(alpha) S + k v^T, o = S^T q with one decay per key channel, alpha = sigmoid(z)^(1 / tau)."""
    T = h.shape[0]
    H, dk, dv, tau = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"])
    q = (h @ d(w[pre + "q"]).T).reshape(T, H, dk) * dk ** -0.5
    k = (h @ d(w[pre + "k"]).T).reshape(T, H, dk)
    v = (h @ d(w[pre + "v"]).T).reshape(T, H, dv)
    z = (h @ d(w[pre + "a1"]).T) @ d(w[pre + "a2"]).T + d(w[pre + "a2.b"])
    alpha = torch.sigmoid(z).pow(1.0 / tau).reshape(T, H, dk)
    S = torch.zeros(H, dk, dv, dtype=F64)
    rows = []
    for t in range(T):
        S = alpha[t][:, :, None] * S + k[t][:, :, None] * v[t][:, None, :]
        rows.append(torch.einsum("hkv,hk->hv", S, q[t]))
    o = unit_rms(torch.stack(rows), eps) * d(w[pre + "norm"])
    g = h @ d(w[pre + "g"]).T
    return (o.reshape(T, H * dv) * g * torch.sigmoid(g)) @ d(w[pre + "o"]).T


def parallel_mixer(h, w, pre, m, eps):
    a = unit_rms(sigmoid_attention(h, w, pre + "left.", m["left"], eps), eps) * d(w[pre + "left.out"])
    b = unit_rms(decayed_linear_attention(h, w, pre + "right.", m["right"], eps), eps) * d(w[pre + "right.out"])
    return 0.5 * (a + b)


def moe(h, w, pre, mlp):
    """Sigmoid router, the `top` largest scores, the score multiplies the chosen expert's INPUT; squared relu."""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    s = torch.sigmoid(h @ d(w[pre + "router"]).T)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            a = torch.relu(d(w[f"{pre}e{e}.up"]) @ (s[t, e] * h[t])) ** 2
            out[t] += d(w[f"{pre}e{e}.down"]) @ a
    return out


def forward(cfg, w, tokens, keep=None):
    """Logits [T, vocab] of one whole sequence; `keep` collects the residual stream after every layer."""
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"]["groups"])
    x = d(w["embed"])[torch.as_tensor(tokens).long()] * float(cfg["embedding"]["scale"])
    v_first = None
    for i, L in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = group_norm(x, d(w[pre + "norm1"]), groups, eps)
        if L["type"] == "mingru":
            y = mingru(h, w, pre + "mix.")
        elif L["type"] == "attention":
            mixes = bool(L["mixer"].get("v_mix"))
            y, v_own = window_attention(h, w, pre + "mix.", L["mixer"], v_first if mixes else None)
            if mixes and v_first is None:
                v_first = v_own
        else:
            y = parallel_mixer(h, w, pre + "mix.", L["mixer"], eps)
        x = x + y
        if L.get("mlp") is not None:
            x = x + moe(group_norm(x, d(w[pre + "norm2"]), groups, eps), w, pre + "mlp.", L["mlp"])
        if keep is not None:
            keep.append(x.clone())
    return group_norm(x, d(w["final.norm"]), groups, eps) @ d(w["head"]).T


def random_weights(cfg, seed=0):
    """Random weights of a configuration, rounded to bfloat16 (what a checkpoint stores). `decay_rank` of a right
    branch (the rank of its decay projection) is read from the mixer's dictionary and not written to config.json."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]
    out = {}

    def mat(name, o, i, gain=1.0):
        out[name] = torch.randn(o, i, generator=g) * gain / math.sqrt(i)

    def vec(name, n, std, mean=0.0):
        out[name] = torch.randn(n, generator=g) * std + mean
    out["embed"] = torch.randn(V, W, generator=g) * 0.5
    mat("head", V, W)
    vec("final.norm", W, 0.2, 1.0)
    for n, L in enumerate(cfg["layers"]):
        pre, m = f"l{n}.", L["mixer"]
        vec(pre + "norm1", W, 0.2, 1.0)
        if L["type"] == "mingru":
            C = m["width"]
            for nm in ("z", "x", "g"):
                mat(pre + "mix." + nm, C, W, 2.0)
            vec(pre + "mix.z.b", C, 0.7)
            vec(pre + "mix.x.b", C, 0.5)
            mat(pre + "mix.o", W, C)
        elif L["type"] == "attention":
            H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for nm, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv), ("g", H * dv)):
                mat(pre + "mix." + nm, rows, W, 2.0)
            vec(pre + "mix.sink", H, 1.0, 0.5)
            if m.get("v_mix"):
                out[pre + "mix.vmix"] = torch.rand((), generator=g) * 0.6 + 0.2
            mat(pre + "mix.o", W, H * dv)
        else:
            a, r = m["left"], m["right"]
            H, G, dk, dv = a["heads"], a["kv_heads"], a["dim"], a["vdim"]
            for nm, rows in (("q", H * dk), ("k", G * dk), ("v", G * dv)):
                mat(pre + "mix.left." + nm, rows, W, 2.0)
                vec(pre + "mix.left." + nm + ".b", rows, 0.3)
            vec(pre + "mix.left.q.norm", H * dk, 0.3, 1.5)
            vec(pre + "mix.left.k.norm", G * dk, 0.3, 1.5)
            vec(pre + "mix.left.pb", H, 0.7, -1.5)
            mat(pre + "mix.left.o", W, H * dv)
            vec(pre + "mix.left.o.b", W, 0.2)
            nk, nv, rk = r["heads"] * r["dim"], r["heads"] * r["vdim"], r.get("decay_rank", 4)
            mat(pre + "mix.right.q", nk, W, 2.0)
            mat(pre + "mix.right.k", nk, W, 2.0)
            mat(pre + "mix.right.v", nv, W, 2.0)
            mat(pre + "mix.right.g", nv, W, 2.0)
            mat(pre + "mix.right.a1", rk, W, 2.0)
            mat(pre + "mix.right.a2", nk, rk, 2.0)
            vec(pre + "mix.right.a2.b", nk, 1.0, 1.5)
            vec(pre + "mix.right.norm", r["vdim"], 0.3, 1.0)
            mat(pre + "mix.right.o", W, nv)
            vec(pre + "mix.left.out", W, 0.3, 1.0)
            vec(pre + "mix.right.out", W, 0.3, 1.0)
        mlp = L.get("mlp")
        if mlp is None:
            continue
        vec(pre + "norm2", W, 0.2, 1.0)
        E, ff = mlp["router"]["experts"], mlp["expert"]["ff"]
        mat(pre + "mlp.router", E, W, 4.0)
        for e in range(E):
            mat(f"{pre}mlp.e{e}.up", ff, W, 1.5)
            mat(f"{pre}mlp.e{e}.down", W, ff)
    return {k: v.to(torch.bfloat16).to(F64) for k, v in out.items()}


def write_checkpoint(path, cfg, Wt):
    """config.json + model.safetensors (bfloat16) of a test model."""
    import copy
    import json
    import os

    from safetensors.torch import save_file
    c = copy.deepcopy(cfg)
    for L in c["layers"]:
        if L["type"] == "parallel":
            L["mixer"]["right"].pop("decay_rank", None)
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(c, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in Wt.items()}, os.path.join(path, "model.safetensors"))
