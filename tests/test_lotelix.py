"""Lotelix on the engine against the dense fp64 oracle (tests/lotelix_oracle.py).

Every test runs on the CPU (PyTorch forms of the ops, same scheduler / cache / state code) and,
marked `gpu`, on the HIP kernels in float32 and bfloat16. Configurations and weights are made
here; the oracle shares no code with xgserve.
"""
import copy
import json
import math
import os
import subprocess
import sys

import pytest
import torch

import lotelix_oracle as orc
from xgserve.engine import EngineConfig, LLMEngine, SamplingParams
from xgserve.models import build_model, get_config
from xgserve.models.config import lotelix_config
from xgserve.ops import seqmix as sq

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F64 = torch.float64

CASES = [pytest.param("cpu", "float32", id="cpu-f32"),
         pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)]
OP_CASES = [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]
TOL = {"float32": 2e-4, "bfloat16": 6e-2}


def config_a():
    """Parallel layer first; three query heads per key head; key sizes unlike value sizes; a window of five tokens and
    a layer that sees everything; the first value-mixing layer is not the first attention layer; rotation of a part of
    a head with all three wavelength ranges, of a whole head, and none; a layer without feed-forward; two of five
    experts; norms in four parts."""
    par = {"left": {"heads": 6, "kv_heads": 2, "dim": 12, "vdim": 20, "scale": 0.35, "rot": {"base": 300.0, "dims": 8}},
           "right": {"heads": 3, "dim": 20, "vdim": 12, "tau": 5.0, "decay_rank": 6}}
    a0 = {"heads": 6, "kv_heads": 2, "dim": 20, "vdim": 12, "scale": 0.31}
    a1 = {"heads": 3, "kv_heads": 3, "dim": 24, "vdim": 8, "scale": 0.2, "mask": {"size": 5}, "v_mix": True,
          "rot": {"base": 5000.0, "dims": 16, "scaling": {"factor": 6.0, "low": 1.0, "high": 8.0, "original": 160}}}
    a2 = {"heads": 4, "kv_heads": 1, "dim": 10, "vdim": 24, "scale": 0.4, "mask": {"size": 19}, "v_mix": True,
          "rot": {"base": 100.0, "dims": 10}}
    moe = {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 5, "top": 2}}
    return {"architecture": "Lotelix", "width": 88, "vocab": 150, "norm": {"eps": 1e-5, "groups": 4},
            "embedding": {"scale": 9.0},
            "layers": [{"type": "parallel", "mixer": par, "mlp": dict(moe)},
                       {"type": "attention", "mixer": a0, "mlp": None},
                       {"type": "mingru", "mixer": {"width": 70}, "mlp": dict(moe)},
                       {"type": "attention", "mixer": a1, "mlp": dict(moe)},
                       {"type": "attention", "mixer": a2, "mlp": {"kind": "moe", "expert": {"ff": 40},
                                                                   "router": {"experts": 3, "top": 3}}}]}


def config_b():
    """Values that make mechanisms trivial: one head, one norm part, one expert, a window of one token, tau and the
    embedding factor equal to one, a rotation of two entries, a single value-mixing layer (nothing to mix with)."""
    a1 = {"heads": 1, "kv_heads": 1, "dim": 32, "vdim": 32, "scale": 0.2, "mask": {"size": 1}, "v_mix": True,
          "rot": {"base": 10.0, "dims": 2, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 8}}}
    par = {"left": {"heads": 1, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.25},
           "right": {"heads": 1, "dim": 16, "vdim": 16, "tau": 1.0, "decay_rank": 1}}
    one = {"kind": "moe", "expert": {"ff": 32}, "router": {"experts": 1, "top": 1}}
    return {"architecture": "Lotelix", "width": 48, "vocab": 97, "norm": {"eps": 1e-6, "groups": 1},
            "embedding": {"scale": 1.0},
            "layers": [{"type": "mingru", "mixer": {"width": 48}, "mlp": None},
                       {"type": "attention", "mixer": a1, "mlp": dict(one)},
                       {"type": "parallel", "mixer": par, "mlp": {"kind": "moe", "expert": {"ff": 16},
                                                                   "router": {"experts": 4, "top": 1}}}]}


def config_c():
    """Sizes the matrix-core kernels take (key sizes multiples of 32, value sizes of 16; expert sizes multiples of
    32 / 16); a window longer than a key tile; value mixing over three layers."""
    att = {"heads": 8, "kv_heads": 2, "dim": 64, "vdim": 32, "scale": 0.125, "mask": {"size": 70}, "v_mix": True,
           "rot": {"base": 10000.0, "dims": 32, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}}
    att2 = dict(att, heads=4, kv_heads=4, dim=32, vdim=16, mask={"size": 9}, rot={"base": 1000.0, "dims": 32})
    par = {"left": {"heads": 8, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.18, "rot": {"base": 1e6, "dims": 32}},
           "right": {"heads": 2, "dim": 64, "vdim": 80, "tau": 16.0, "decay_rank": 8}}
    moe = {"kind": "moe", "expert": {"ff": 64}, "router": {"experts": 6, "top": 2}}
    return {"architecture": "Lotelix", "width": 128, "vocab": 200, "norm": {"eps": 1e-5, "groups": 2},
            "embedding": {"scale": 11.3},
            "layers": [{"type": "attention", "mixer": att, "mlp": dict(moe)},
                       {"type": "mingru", "mixer": {"width": 160}, "mlp": dict(moe)},
                       {"type": "attention", "mixer": att2, "mlp": None},
                       {"type": "parallel", "mixer": par, "mlp": dict(moe)},
                       {"type": "attention", "mixer": dict(att, mask={"size": 33}), "mlp": dict(moe)}]}


_MADE = {}


def made(name, tmp_path_factory):
    """(config, oracle weights, checkpoint dir) of a test model, written once per session."""
    if name not in _MADE:
        cfg = {"a": config_a, "b": config_b, "c": config_c}[name]()
        Wt = orc.random_weights(cfg, seed={"a": 5, "b": 13, "c": 21}[name])
        path = str(tmp_path_factory.mktemp("lotelix_" + name))
        orc.write_checkpoint(path, cfg, Wt)
        _MADE[name] = (cfg, Wt, path)
    return _MADE[name]


def engine(path, device, dtype, **kw):
    args = dict(model=path, checkpoint=path, device=device, dtype=dtype, block_size=4, num_blocks=64, max_num_seqs=3,
                max_num_batched_tokens=256, max_model_len=200, use_graphs=False)
    args.update(kw)
    return LLMEngine(EngineConfig(**args))


def tokens_of(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def row_errs(got, ref):
    got, ref = got.detach().to("cpu", F64), ref.to(F64)
    d = got - ref
    d = d - d.mean(-1, keepdim=True)
    r = ref - ref.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / r.pow(2).mean(-1).sqrt()


def rel_err(got, ref):
    return float(row_errs(got, ref).max())


def close(got, ref, dtype):
    """float32: every position within 2e-4. bfloat16: rounding can tip a router's close call at a token; where one
    expert of few is chosen that token's feed-forward output is then another one altogether, and the tokens after it
    feel it through the state. So a few positions may exceed the rounding level, while most stay within it; a wrong
    mechanism is caught by the float32 runs and moves most positions."""
    e = row_errs(got, ref)
    if dtype == "float32":
        return float(e.max()) < TOL[dtype]
    return bool(torch.isfinite(e).all()) and float((e > TOL[dtype]).double().mean()) <= 0.15 and \
        float(e.median()) < TOL[dtype] / 2


def run_portions(eng, rid, toks, portions):
    """Feed `toks` in the given portion sizes (the rest one by one); logits of every position."""
    out, at = [], 0
    sizes = list(portions)
    while at < len(toks):
        n = sizes.pop(0) if sizes else 1
        n = min(n, len(toks) - at)
        end = [rid] if at + n == len(toks) else []
        out.append(eng.score_step([(rid, toks[at:at + n], list(range(n)))], end))
        at += n
    return torch.cat(out, 0)


# ---------------------------------------------------------------------------------- whole model
@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_whole_prompt_matches_oracle(name, device, dtype, tmp_path_factory):
    cfg, Wt, path = made(name, tmp_path_factory)
    toks = tokens_of(cfg, 90 if name == "c" else 45, 1)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype)
    got = eng.score_step([("w", toks, list(range(len(toks))))], ["w"])
    assert close(got, ref, dtype)
    assert eng.sched.num_used_blocks() == 0


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", ["a", "c"])
def test_residual_after_every_layer(name, device, dtype, tmp_path_factory):
    cfg, Wt, path = made(name, tmp_path_factory)
    toks = tokens_of(cfg, 17, 2)
    res = []
    orc.forward(cfg, Wt, toks, res)
    m = build_model(get_config(path), device=device, dtype=getattr(torch, dtype), checkpoint=path)
    eng = LLMEngine(EngineConfig(model=path, device=device, dtype=dtype, block_size=4, num_blocks=16, max_num_seqs=2,
                                 max_model_len=64, use_graphs=False), model=m)
    m.keep_residuals = seen = []
    eng.score_step([("x", toks, [0, 16])], ["x"])
    m.keep_residuals = None
    tol = 1e-4 if dtype == "float32" else 8e-2
    assert len(seen) == len(res) == len(cfg["layers"])
    for got, ref in zip(seen, res):
        assert float((got.detach().to("cpu", F64) - ref).abs().max()) < tol * float(ref.abs().max())


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_decode_token_by_token_equals_prefill(name, device, dtype, tmp_path_factory):
    cfg, Wt, path = made(name, tmp_path_factory)
    toks = tokens_of(cfg, 40, 3)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype)
    got = run_portions(eng, "d", toks, [])
    assert close(got, ref, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("portions", [[2, 2, 3, 2, 9, 1, 1, 5, 2], [7, 1, 13, 2], [33, 2], [1, 2, 4, 8, 16]])
def test_portions_of_any_size(portions, device, dtype, tmp_path_factory):
    cfg, Wt, path = made("a", tmp_path_factory)
    toks = tokens_of(cfg, 42, 4)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype)
    got = run_portions(eng, "p", toks, portions)
    assert close(got, ref, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", ["b", "c"])
def test_long_decoding(name, device, dtype, tmp_path_factory):
    cfg, Wt, path = made(name, tmp_path_factory)   # positions up to 170: many pages, windows pass over decoded tokens
    toks = tokens_of(cfg, 170, 5)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype, num_blocks=48)
    got = run_portions(eng, "l", toks, [9])
    assert close(got, ref, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
def test_long_portion_is_scanned_in_pieces(device, dtype, tmp_path_factory):
    """A portion of several hundred tokens after a short one: the recurrences scan it in pieces that start from
    the carried state."""
    cfg, Wt, path = made("c", tmp_path_factory)
    toks = tokens_of(cfg, 333, 6)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype, block_size=16, num_blocks=24, max_num_batched_tokens=512, max_model_len=400)
    got = run_portions(eng, "s", toks, [3, 290, 2, 37])
    assert close(got, ref, dtype)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", ["a", "c"])
def test_mixed_batches_reused_pages_and_slots(name, device, dtype, tmp_path_factory):
    """Unequal requests share steps (portions beside single tokens), sit steps out, end, and later ones take
    over their slots and pages: two slots and a pool that holds only the live requests."""
    cfg, Wt, path = made(name, tmp_path_factory)
    lens = {"r0": 23, "r1": 9, "r2": 31, "r3": 1, "r4": 14}
    toks = {k: tokens_of(cfg, n, 10 + i) for i, (k, n) in enumerate(lens.items())}
    ref = {k: orc.forward(cfg, Wt, v) for k, v in toks.items()}
    eng = engine(path, device, dtype, num_blocks=14, max_num_seqs=2)
    steps = [[("r0", 5), ("r1", 2)], [("r0", 1), ("r1", 3)], [("r1", 4)], [("r0", 9)], [("r2", 6), ("r0", 1)],
             [("r0", 7), ("r2", 1)], [("r2", 2)], [("r3", 1), ("r2", 13)], [("r4", 3), ("r2", 1)], [("r2", 8), ("r4", 1)],
             [("r4", 10)]]
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for st in steps:
        entries, end = [], []
        for k, n in st:
            entries.append((k, toks[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == lens[k]:
                end.append(k)
        lg = eng.score_step(entries, end)
        o = 0
        for k, n in st:
            got[k].append(lg[o:o + n])
            o += n
    assert at == lens
    for k in lens:
        assert close(torch.cat(got[k], 0), ref[k], dtype), k
    assert eng.sched.num_used_blocks() == 0 and eng.sched.num_running() == 0


@pytest.mark.parametrize("device,dtype", CASES)
def test_batch_rows_equal_alone(device, dtype, tmp_path_factory):
    cfg, Wt, path = made("a", tmp_path_factory)
    a, b, c = tokens_of(cfg, 30, 20), tokens_of(cfg, 5, 21), tokens_of(cfg, 12, 22)
    eng = engine(path, device, dtype)
    alone = [eng.score_step([(n, t, list(range(len(t))))], [n]) for n, t in (("a", a), ("b", b), ("c", c))]
    both = eng.score_step([("a", a, list(range(30))), ("b", b, list(range(5))), ("c", c, list(range(12)))], ["a", "b", "c"])
    tol = 1e-5 if dtype == "float32" else 2e-2
    assert rel_err(both[:30], alone[0].cpu()) < tol and rel_err(both[30:35], alone[1].cpu()) < tol
    assert rel_err(both[35:], alone[2].cpu()) < tol


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", ["a", "c"])
def test_greedy_generation_through_the_scheduler(name, device, dtype, tmp_path_factory):
    """add_request / step with the engine's own scheduler (chunked prompts, several requests at once; HIP graphs
    on the GPU): every generated token is the oracle's argmax on the same history, up to rounding."""
    cfg, Wt, path = made(name, tmp_path_factory)
    prompts = [tokens_of(cfg, n, 30 + i) for i, n in enumerate((19, 3, 11, 1))]
    eng = engine(path, device, dtype, max_num_batched_tokens=8, max_num_seqs=3, use_graphs=True,
                 graph_batch_sizes=[1, 2, 4])
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in outs] == [12] * 4
    bad = 0
    for p, o in zip(prompts, outs):
        ref = orc.forward(cfg, Wt, p + o[:-1])
        for i, tok in enumerate(o):
            row = ref[len(p) - 1 + i]
            gap = float(row.max() - row[tok])
            bad += gap > (1e-3 if dtype == "float32" else 0.15) * float(row.std())
    assert bad <= (0 if dtype == "float32" else 2)     # bfloat16: a router's close call may tip at a token
    assert eng.sched.num_used_blocks() == 0


def test_registered_tiny_model_generates():
    eng = LLMEngine(EngineConfig(model="lotelix-tiny", device="cpu", dtype="float32", block_size=4, num_blocks=32,
                                 max_num_seqs=2, max_model_len=64, use_graphs=False))
    outs = eng.generate([[1, 2, 3, 4, 5], [7]], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))
    assert [len(o) for o in outs] == [6, 6]


def test_trace_runner_cli(tmp_path, tmp_path_factory):
    cfg, Wt, path = made("b", tmp_path_factory)
    a, b = tokens_of(cfg, 21, 40), tokens_of(cfg, 6, 41)
    lines = [{"step": 0, "entries": [{"id": "a", "tokens": a[:10], "want": [0, 9]}, {"id": "b", "tokens": b[:2], "want": []}],
              "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": [3]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[10:], "want": [10]}], "end": ["a"]}]
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                        "--out", str(tmp_path / "o"), "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(x) for x in lines) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    import numpy as np
    V = cfg["vocab"]
    ra, rb = orc.forward(cfg, Wt, a), orc.forward(cfg, Wt, b)
    g0 = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4").reshape(-1, V))
    g1 = torch.from_numpy(np.fromfile(tmp_path / "o" / "1.f32", dtype="<f4").reshape(-1, V))
    g2 = torch.from_numpy(np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4").reshape(-1, V))
    assert rel_err(g0, ra[[0, 9]]) < 2e-4 and rel_err(g1, rb[[5]]) < 2e-4 and rel_err(g2, ra[[20]]) < 2e-4


def test_save_and_reload_checkpoint(tmp_path):
    from xgserve.models import save_checkpoint
    m = build_model(get_config("lotelix-tiny"), device="cpu", dtype=torch.float32, seed=3)
    save_checkpoint(m, str(tmp_path / "ck"))
    cfg2 = get_config(str(tmp_path / "ck"))
    assert cfg2.norm_groups == m.cfg.norm_groups and cfg2.embed_scale == m.cfg.embed_scale
    assert "decay_rank" not in cfg2.layer_specs[2]["mixer"]["right"]       # read from a tensor's shape on load
    m2 = build_model(cfg2, device="cpu", dtype=torch.float32, checkpoint=str(tmp_path / "ck"))
    for (n1, p1), (n2, p2) in zip(m.named_parameters(), m2.named_parameters()):
        assert n1 == n2 and torch.equal(p1.to(torch.bfloat16).float(), p2), n1
    assert m.cfg.num_params() == sum(p.numel() for n, p in m.named_parameters()) - \
        sum(L.mix.lam.numel() for L in m.layers if L.kind == "attention" and not L.mix.v_mix) - \
        sum(int((L.mix.in_bias == 0).sum()) for L in m.layers if L.kind == "parallel")


def test_config_rejects_what_the_design_does_not_have():
    cfg = config_a()
    for edit in (lambda L: L[0].__setitem__("type", "something_else"),
                 lambda L: L[1]["mixer"].__setitem__("kv_heads", 4),           # 6 heads do not divide over 4
                 lambda L: L[0]["mixer"]["left"].__setitem__("kv_heads", 4),
                 lambda L: L[3]["mixer"]["rot"].__setitem__("dims", 26),       # more than the head holds
                 lambda L: L[3]["mixer"]["mask"].__setitem__("size", 0),
                 lambda L: L[4]["mixer"].__setitem__("vdim", 8),               # value rows of mixing layers differ
                 lambda L: L[0]["mixer"]["right"].__setitem__("tau", 0.0),
                 lambda L: L[0]["mlp"]["router"].__setitem__("top", 6),
                 lambda L: L[0]["mlp"].__setitem__("kind", "dense")):
        bad = copy.deepcopy(cfg["layers"])
        edit(bad)
        with pytest.raises(ValueError):
            lotelix_config("x", 88, 150, bad, norm_groups=4)
    with pytest.raises(ValueError):
        lotelix_config("x", 88, 150, cfg["layers"], norm_groups=3)             # 88 columns do not split into 3 parts
    with pytest.raises(ValueError):
        LLMEngine(EngineConfig(model="lotelix-tiny", device="cpu", num_blocks=8, max_num_seqs=2, max_model_len=32,
                               use_graphs=False, draft_model="llama-tiny-draft", num_speculative_tokens=2))


# ---------------------------------------------------------------------------------- mechanisms alone
def seq_meta(device, rows, block_size, tables):
    """rows: [(slot, context length, tokens in this step)] -> SeqMeta; tables: page list per row."""
    qsl, sl, slots, tseq, pos, smap = [0], [], [], [], [], []
    width = max(len(t) for t in tables)
    for i, (slot, ctx, q) in enumerate(rows):
        qsl.append(qsl[-1] + q)
        sl.append(ctx + q)
        slots.append(slot)
        for p in range(ctx, ctx + q):
            tseq.append(i)
            pos.append(p)
            smap.append(tables[i][p // block_size] * block_size + p % block_size)
    bt = [t + [0] * (width - len(t)) for t in tables]
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)  # noqa: E731
    return sq.SeqMeta(len(rows), max(r[2] for r in rows), i32(qsl), i32(sl), i32(slots), i32(bt), i32(tseq), i32(pos),
                      i32(smap))


def in_portions(device, xs, cuts, slots, fn, tables=None, block_size=4):
    """Run fn(rows of this step [n, C] on `device`, SeqMeta) over several sequences cut into portions that
    share steps; returns each sequence's outputs in order."""
    got, at = [[] for _ in xs], [0] * len(xs)
    cuts = [list(c) for c in cuts]
    while any(cuts):
        rows, parts, who = [], [], []
        for i in range(len(xs)):
            if cuts[i]:
                q = cuts[i].pop(0)
                rows.append((slots[i], at[i], q))
                parts.append(xs[i][at[i]:at[i] + q])
                who.append((i, q))
                at[i] += q
        sm = seq_meta(device, rows, block_size, [tables[i] if tables else [0] * 512 for i, _ in who])
        y = fn(torch.cat(parts).to(device), sm)
        o = 0
        for i, q in who:
            got[i].append(y[o:o + q].float().cpu())
            o += q
    return [torch.cat(g).to(F64) for g in got]


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("W,groups", [(77, 1), (77, 7), (96, 2), (96, 8), (90, 3), (2304, 2), (2304, 64), (1024, 256)])
def test_residual_sum_and_group_norm(device, W, groups):
    """x + y, x + fp32 sum, and the mean of two branches that are each normed first; the norm in `groups` parts, also
    with parts that are no multiple of four columns."""
    g = torch.Generator().manual_seed(W + groups)
    T, eps = 9, 1e-5
    x, y1, y2, y3 = (torch.randn(T, W, generator=g).to(F64) * s for s in (3.0, 1.0, 5.0, 2.0))
    w, w1, w2 = (torch.randn(W, generator=g).to(F64) * 0.3 + 1.0 for _ in range(3))
    f = lambda t: t.float().to(device)  # noqa: E731
    for mode in ("one", "fp32", "two"):
        xs = f(x).clone()
        if mode == "one":
            ref_x = x + y1
            n32, n = sq.residual_norm(xs, f(y1), None, None, None, None, f(w), eps, torch.float32, True, groups)
        elif mode == "fp32":
            ref_x = x + y3
            n32, n = sq.residual_norm(xs, None, None, None, f(y3), None, f(w), eps, torch.float32, True, groups)
        else:
            ref_x = x + 0.5 * (orc.unit_rms(y1, eps) * w1 + orc.unit_rms(y2, eps) * w2)
            n32, n = sq.residual_norm(xs, f(y1), None, f(y2), None, None, f(w), eps, torch.float32, True, groups,
                                      branch_w=(f(w1), f(w2)))
        assert float((xs.cpu().to(F64) - ref_x).abs().max()) < 1e-5
        ref_n = orc.group_norm(ref_x, w, groups, eps)
        assert float((n32.cpu().to(F64) - ref_n).abs().max()) < 2e-5 and torch.equal(n32, n)
    # strided branch outputs of an activation dtype (columns of a wider tensor)
    wide = torch.randn(T, 2 * W + 8, generator=g).to(torch.bfloat16)
    xs = f(x).clone()
    ya, yb = wide.to(device)[:, :W], wide.to(device)[:, W + 8:]
    sq.residual_norm(xs, ya, None, yb, None, None, None, eps, None, False, groups, branch_w=(f(w1), f(w2)))
    ref_x = x + 0.5 * (orc.unit_rms(wide[:, :W].to(F64), eps) * w1 + orc.unit_rms(wide[:, W + 8:].to(F64), eps) * w2)
    assert float((xs.cpu().to(F64) - ref_x).abs().max()) < 1e-5


def test_rotation_frequencies_in_all_three_ranges():
    rot = {"base": 5000.0, "dims": 16, "scaling": {"factor": 6.0, "low": 1.0, "high": 8.0, "original": 160}}
    plain = orc.frequencies({"base": 5000.0, "dims": 16})
    scaled = orc.frequencies(rot)
    ratio = (scaled / plain).tolist()
    assert any(abs(r - 1.0) < 1e-12 for r in ratio) and any(abs(r - 1 / 6.0) < 1e-12 for r in ratio)
    assert any(1 / 6.0 + 1e-6 < r < 1.0 - 1e-6 for r in ratio)
    assert torch.allclose(sq.rot_frequencies(16, 5000.0, rot["scaling"]), scaled, rtol=1e-12, atol=0)


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("n,cuts", [(70, [[1, 1, 1, 3, 16, 1, 17, 40, 1, 128, 129, 2, 300], [2, 5, 1, 1, 1, 1, 200, 7, 1, 1, 1, 1, 1]]),
                                    (64, [[400], [1] * 6]), (200, [[17, 130], [131, 16]]),
                                    (130, [[3, 1300, 1, 257], [700, 2, 513, 1]]), (64, [[900, 1, 600], [5, 1, 1]])])
@pytest.mark.parametrize("two_pass", [True, False], ids=["chunks", "one-workgroup"])
def test_minimal_gated_recurrence_over_portions_and_slots(device, n, cuts, two_pass, monkeypatch):
    """Steps of single tokens, short and long portions (every workgroup shape of the scan; the longest ones as chunks
    over the whole grid, in two launches), two sequences sharing steps, a slot with another sequence's leftovers,
    columns of a wider strided row."""
    monkeypatch.setattr(sq, "MINGRU_TWO_PASS", two_pass)
    g = torch.Generator().manual_seed(n)
    W = 24
    cfg = {"width": W, "vocab": 8, "layers": [{"type": "mingru", "mixer": {"width": n}, "mlp": None}]}
    Wt = {k[len("l0.mix."):]: v for k, v in orc.random_weights(cfg, seed=n).items() if k.startswith("l0.mix.")}
    hs = [torch.randn(sum(c), W, generator=g).to(F64) for c in cuts]
    Wo = Wt["o"]
    refs = [orc.mingru(h, Wt, "") for h in hs]
    Wcat = torch.cat([Wt["x"], Wt["g"], Wt["z"]])       # any column order
    state = torch.randn(3, n).to(device)                # stale contents: a new sequence must not see them
    bz, bx = Wt["z.b"].float().to(device), Wt["x.b"].float().to(device)

    def fn(x, sm):
        proj = torch.zeros(x.shape[0], 3 * n + 5, device=device)
        proj[:, 3:3 + 3 * n] = (x.to(F64).cpu() @ Wcat.T).float().to(device)
        y = sq.mingru_scan(proj, 3 + 2 * n, 3, 3 + n, n, bz, bx, state, sm, torch.float32)
        return (y.to(F64).cpu() @ Wo.T).float()
    got = in_portions(device, hs, cuts, [2, 0], fn)
    for a, b in zip(got, refs):
        assert rel_err(a, b) < 1e-4
    # the carried state is the recurrence's own last value
    z = torch.sigmoid(hs[0] @ Wt["z"].T + Wt["z.b"])
    u = hs[0] @ Wt["x"].T + Wt["x.b"]
    c = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    S = torch.zeros(n, dtype=F64)
    for t in range(hs[0].shape[0]):
        S = (1 - z[t]) * S + z[t] * c[t]
    assert float((state[2].cpu().to(F64) - S).abs().max()) < 1e-4


def test_candidate_of_the_minimal_recurrence_on_both_sides_of_zero():
    """z = 1 makes the state equal the candidate: u + 1/2 from zero upward, sigmoid(u) below."""
    u = torch.tensor([[-3.0, -1e-3, 0.0, 1e-3, 2.5]])
    proj = torch.cat([torch.full_like(u, 40.0), u, torch.full_like(u, 30.0)], 1)
    sm = seq_meta("cpu", [(0, 0, 1)], 4, [[0]])
    y = sq.mingru_scan(proj, 0, 5, 10, 5, None, None, torch.zeros(1, 5), sm, torch.float32)
    ref = torch.tensor([[torch.sigmoid(torch.tensor(-3.0)), torch.sigmoid(torch.tensor(-1e-3)), 0.5, 0.501, 3.0]]) * 30.0
    assert torch.allclose(y, ref, rtol=1e-5)


def _attention_case(device, dtype, H, G, dk, dv, bs, T, single, mode, size=0, strong=None, rot=None):
    """Queries of one sequence over scrambled pages against dense formulas. mode "window": sliding window, sink,
    gate per entry, (i, i + n / 2) rotation, value mixing; "sigmoid": causal, unnormalised sigmoid weights with a
    per-head bias, whole-vector norms, (2i, 2i + 1) rotation. `strong` = (query, key): that score stands out."""
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(H * 100 + dk + T + size)
    rnd = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(F64)  # noqa: E731
    q, k, v, vf = rnd(T, H, dk), rnd(T, G, dk), rnd(T, G, dv), rnd(T, G * dv)
    eps, lam = 1e-5, 0.375
    if strong is not None:
        i, j = strong
        k[j] = q[i, ::H // G] * 1.5          # every head's query i lines up with key j
    rd = rot["dims"] if rot else 0
    pos = torch.arange(T)
    scale = 0.4 / dk ** 0.5 * (6.0 if strong is not None else 1.0)
    f32 = lambda t: t.float().to(device)  # noqa: E731
    if mode == "window":
        sink, gate = rnd(H) + 1.0, rnd(T, H * dv + 3)
        qr, kr = (orc.rotate(q, pos, rot, "half"), orc.rotate(k, pos, rot, "half")) if rot else (q, k)
        vm = ((1 - lam) * v.reshape(T, -1) + lam * vf).reshape(T, G, dv)
        ref = torch.zeros(T, H, dv, dtype=F64)
        for i in range(T):
            lo = max(0, i - size + 1)
            for h in range(H):
                c = h // (H // G)
                sc = torch.cat([(kr[lo:i + 1, c] @ qr[i, h]) * scale, sink[h:h + 1]])
                ref[i, h] = torch.softmax(sc, 0)[:-1] @ vm[lo:i + 1, c]
        ref = ref * torch.sigmoid(gate[:, :H * dv]).view(T, H, dv)
    else:
        pb = rnd(H) - 1.0
        wq, wk = rnd(H * dk) * 0.3 + 1.0, rnd(G * dk) * 0.3 + 1.0
        qn = (orc.unit_rms(q.reshape(T, -1), eps) * wq).reshape(T, H, dk)
        kn = (orc.unit_rms(k.reshape(T, -1), eps) * wk).reshape(T, G, dk)
        scale *= 4.0 if strong is not None else 1.0
        qr, kr = (orc.rotate(qn, pos, rot, "pairs"), orc.rotate(kn, pos, rot, "pairs")) if rot else (qn, kn)
        ref = torch.zeros(T, H, dv, dtype=F64)
        for i in range(T):
            for h in range(H):
                c = h // (H // G)
                ref[i, h] = torch.sigmoid((kr[:i + 1, c] @ qr[i, h]) * scale + pb[h]) @ v[:i + 1, c]
    pages = torch.randperm(80, generator=g)[:(T + bs - 1) // bs].tolist()
    kc = torch.randn(80 * bs, G * dk, generator=g).to(dt).to(device)      # stale rows everywhere
    vc = torch.randn(80 * bs, G * dv, generator=g).to(dt).to(device)
    table = sq.build_rot_table(rd, rot["base"], T + 1, device, rot.get("scaling")) if rot else None
    out = []
    steps = [(0, T)] if not single else [(0, T - 6)] + [(T - 6 + i, 1) for i in range(6)]
    for ctx, n in steps:
        sm = seq_meta(device, [(0, ctx, n)], bs, [pages])
        src = torch.cat([q[ctx:ctx + n].reshape(n, -1), k[ctx:ctx + n].reshape(n, -1), v[ctx:ctx + n].reshape(n, -1)], 1)
        src = src.to(dt).to(device)
        if mode == "window":
            qq = sq.head_norm_rope_cache(src, H, G, dk, dv, None, None, 0.0, table, rd, sm, kc, vc, dt, half=True,
                                         v_first=vf[ctx:ctx + n].to(dt).to(device), v_mix=torch.tensor([lam], device=device))
            out.append(sq.masked_attention(qq, kc, vc, H, G, dk, dv, sq.MASK_WINDOW, size, scale, None, f32(sink), bs, sm,
                                           gate=gate[ctx:ctx + n].to(dt).to(device), gate_elem=True))
        else:
            qq = sq.head_norm_rope_cache(src, H, G, dk, dv, f32(wq), f32(wk), eps, table, rd, sm, kc, vc, dt, whole=True)
            out.append(sq.masked_attention(qq, kc, vc, H, G, dk, dv, sq.MASK_CAUSAL, 0, scale, None, None, bs, sm,
                                           weights=sq.W_SIGMOID, score_bias=f32(pb)))
    return torch.cat(out).float().cpu().view(T, H, dv), ref


ROT_A = {"base": 50.0, "dims": 16, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 24}}


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("shape", [(6, 2, 20, 12), (1, 1, 32, 32), (8, 2, 64, 32), (4, 4, 96, 48), (16, 2, 32, 128)],
                         ids=lambda s: "H%dG%dk%dv%d" % s)
@pytest.mark.parametrize("single", [False, True], ids=["prompt", "decoded"])
@pytest.mark.parametrize("mode,size", [("window", 7), ("window", 70), ("sigmoid", 0)])
def test_attention_variants_alone(device, dtype, shape, single, mode, size):
    """Both attention variants with their own rotation layout, for the general and the matrix-core kernels, as a
    prompt portion and as single tokens, windows shorter and longer than a key tile."""
    got, ref = _attention_case(device, dtype, *shape, bs=4, T=75, single=single, mode=mode, size=size, rot=ROT_A)
    assert rel_err(got.reshape(75, -1), ref.reshape(75, -1)) < (1e-4 if dtype == "float32" else 4e-2)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("back", [0, 1, 15, 16, 17, 63, 64, 130, 299, 300])
@pytest.mark.parametrize("single", [False, True], ids=["prompt", "decoded"])
def test_sigmoid_weights_one_standing_out_key(device, dtype, back, single):
    """The last query's score for one key (the first token, a page's first / last row, hundreds of tokens back, the
    query itself) stands out among keys whose weights are near zero: a lost or misplaced key moves the output."""
    T = 301
    got, ref = _attention_case(device, dtype, 4, 2, 32, 16, bs=16, T=T, single=single, mode="sigmoid",
                               strong=(T - 1, T - 1 - back), rot={"base": 1e4, "dims": 32})
    assert rel_err(got[-1].reshape(1, -1), ref[-1].reshape(1, -1)) < (1e-4 if dtype == "float32" else 4e-2)
    assert rel_err(got.reshape(T, -1), ref.reshape(T, -1)) < (1e-4 if dtype == "float32" else 4e-2)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("size", [1, 2, 16, 17, 40, 64, 65])
@pytest.mark.parametrize("edge", ["inside", "outside"])
@pytest.mark.parametrize("single", [False, True], ids=["prompt", "decoded"])
def test_window_edge_one_standing_out_key(device, dtype, size, edge, single):
    """The key that stands out for the last query is the oldest one the window keeps, or the one just before it
    (which must stay unseen: then the sink and the other keys share the weight)."""
    T = 140
    back = size - 1 if edge == "inside" else size
    got, ref = _attention_case(device, dtype, 4, 2, 32, 16, bs=16, T=T, single=single, mode="window", size=size,
                               strong=(T - 1, T - 1 - back), rot=ROT_A)
    assert rel_err(got[-1].reshape(1, -1), ref[-1].reshape(1, -1)) < (1e-4 if dtype == "float32" else 4e-2)
    assert rel_err(got.reshape(T, -1), ref.reshape(T, -1)) < (1e-4 if dtype == "float32" else 4e-2)


@pytest.mark.parametrize("device", OP_CASES)
def test_sink_can_take_all_the_weight(device):
    H, G, dk, dv, T = 2, 1, 16, 8, 9
    g = torch.Generator().manual_seed(3)
    sm = seq_meta(device, [(0, 0, T)], 4, [[2, 0, 1]])
    q = torch.randn(T, H * dk, generator=g).to(device)
    kc, vc = torch.randn(12, G * dk, generator=g).to(device), torch.randn(12, G * dv, generator=g).to(device)
    sink = torch.tensor([60.0, -60.0], device=device)
    o = sq.masked_attention(q, kc, vc, H, G, dk, dv, sq.MASK_WINDOW, 3, 0.1, None, sink, 4, sm).view(T, H, dv)
    assert float(o[:, 0].abs().max()) < 1e-12 and float(o[:, 1].abs().max()) > 1e-2


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("H,dk,dv,tau,rank", [(3, 20, 12, 5.0, 6), (2, 16, 16, 1.0, 1), (1, 6, 70, 16.0, 3), (2, 64, 80, 2.5, 8)])
@pytest.mark.parametrize("lens,cuts", [((29, 11), [[5, 1, 1, 2, 17, 1, 2], [2, 2, 1, 1, 5]]),
                                       ((900, 40), [[3, 600, 1, 257, 39], [20, 1, 2, 1, 16]])], ids=["short", "long"])
@pytest.mark.parametrize("two_pass", [True, False], ids=["chunks", "one-workgroup"])
def test_decayed_linear_attention_over_portions_and_slots(device, H, dk, dv, tau, rank, lens, cuts, two_pass, monkeypatch):
    """Short portions and single tokens, and portions of several hundred tokens (scanned as chunks over the whole grid,
    in two launches, beside another sequence's short portions), on slots with leftovers."""
    monkeypatch.setattr(sq, "SCAN_TWO_PASS", two_pass)
    g = torch.Generator().manual_seed(dk)
    W, eps = 24, 1e-5
    m = {"heads": H, "dim": dk, "vdim": dv, "tau": tau, "decay_rank": rank}
    cfg = {"width": W, "vocab": 8, "layers": [{"type": "parallel", "mlp": None, "mixer": {
        "left": {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 1.0}, "right": m}}]}
    Wt = {k[len("l0.mix.right."):]: v for k, v in orc.random_weights(cfg, seed=dk).items() if k.startswith("l0.mix.right.")}
    hs = [torch.randn(n, W, generator=g).to(F64) for n in lens]
    refs = [orc.decayed_linear_attention(h, Wt, "", m, eps) for h in hs]
    n, nv = H * dk, H * dv
    Wcat = torch.cat([Wt["q"], Wt["k"], Wt["v"], Wt["g"], Wt["a1"]])
    state = torch.randn(3, H, dk, dv).to(device)      # stale contents: a new sequence must not see them
    f = lambda t: t.float().to(device)  # noqa: E731

    def fn(x, sm):
        proj = (x.to(F64).cpu() @ Wcat.T).float().to(device)
        z = (proj[:, 2 * n + 2 * nv:].cpu().to(F64) @ Wt["a2"].T).float().to(device)
        q, fg, k = sq.decay_gates(proj, 0, n, n, dk ** -0.5, z, f(Wt["a2.b"]), tau)
        o = sq.gated_linear_scan(q, fg, k, proj[:, 2 * n:2 * n + nv], state, H, dk, dv, sm)
        y = sq.gated_group_norm(o, proj[:, 2 * n + nv:2 * n + 2 * nv], f(Wt["norm"]), eps, H, torch.float32, gate_after=True)
        return (y.cpu().to(F64) @ Wt["o"].T).float()
    got = in_portions(device, hs, cuts, [1, 2], fn)
    for a, b in zip(got, refs):
        assert rel_err(a, b) < 1e-4


@pytest.mark.parametrize("device", OP_CASES)
def test_decay_of_a_very_negative_logit_stays_finite(device):
    proj = torch.zeros(2, 4, device=device)
    z = torch.tensor([[-200.0, -30.0], [0.0, 50.0]], device=device)
    _, f, _ = sq.decay_gates(proj, 0, 2, 2, 1.0, z, None, 4.0)
    ref = torch.sigmoid(z.cpu().to(F64)).pow(0.25)
    assert torch.isfinite(f).all() and float((f.cpu().to(F64) - ref).abs().max()) < 1e-6


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("T,E,top,K,F_", [(7, 5, 2, 40, 24), (50, 1, 1, 32, 16), (100, 1, 1, 64, 32), (300, 3, 3, 64, 48), (700, 4, 1, 96, 64),
                                          (1300, 4, 2, 128, 32), (64, 12, 1, 24, 10)])
def test_experts_scaled_at_their_input(device, dtype, T, E, top, K, F_):
    """Every grouped-GEMM path (tiles of 16, 32, 64 and 128 rows; matrix-core and general) against the dense form in which
    the routing score multiplies the expert's input; scores far from one, so a weight applied at the output (which the
    squared activation would turn into its square) shows."""
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(T + E)
    mlp = {"router": {"experts": E, "top": top}, "expert": {"ff": F_}}
    w = {"router": torch.randn(E, K, generator=g).to(F64) * 3.0 / math.sqrt(K)}
    for e in range(E):
        w[f"e{e}.up"] = (torch.randn(F_, K, generator=g) / math.sqrt(K)).to(torch.bfloat16).to(F64)
        w[f"e{e}.down"] = (torch.randn(K, F_, generator=g) / math.sqrt(F_)).to(torch.bfloat16).to(F64)
    h = torch.randn(T, K, generator=g).to(torch.bfloat16).to(F64)
    ref = orc.moe(h, w, "", mlp)
    logits = (h @ w["router"].T).float().to(device)
    ids, wts = sq.grouped_router(logits, None, 1, 1, top, 1.0)
    s = torch.sigmoid(h @ w["router"].T)
    assert torch.equal(ids.cpu().long().sort(-1).values, s.topk(top, -1).indices.sort(-1).values)
    up = torch.stack([w[f"e{e}.up"] for e in range(E)]).to(dt).to(device)
    down = torch.stack([w[f"e{e}.down"] for e in range(E)]).to(dt).to(device)
    got = sq.routed_experts(h.to(dt).to(device), up, down, ids, wts, sq.ACT_RELU2, scale_input=True)
    assert rel_err(got, ref) < (1e-4 if dtype == "float32" else 3e-2)
    # the logits formed inside the router kernel (short steps) or by a matrix product (long ones)
    ids2, wts2 = sq.grouped_router(None, None, 1, 1, top, 1.0, rows=h.float().to(device),
                                   router_w=w["router"].float().to(device))
    assert torch.equal(ids2.cpu().long().sort(-1).values, ids.cpu().long().sort(-1).values)
    assert float((wts2.sort(-1).values - wts.sort(-1).values).abs().max()) < 1e-5
    # the sum over a token's choices inside the residual update
    rows = sq.routed_experts(h.to(dt).to(device), up, down, ids, wts, sq.ACT_RELU2, scale_input=True, combine=False)
    x = torch.randn(T, K, generator=g)
    xs = x.clone().to(device)
    nw = (torch.rand(K, generator=g) + 0.5)
    _, n = sq.residual_norm(xs, None, None, None, rows, None, nw.to(device), 1e-5, torch.float32, False, 2)
    assert rel_err(xs, x.to(F64) + ref) < (1e-4 if dtype == "float32" else 3e-2)
    assert rel_err(n, orc.group_norm(x.to(F64) + ref, nw.to(F64), 2, 1e-5)) < (1e-4 if dtype == "float32" else 3e-2)
    # weights applied at the output: the same rows with a weight per choice
    plain = sq.routed_experts(h.to(dt).to(device), up, down, ids, wts, sq.ACT_RELU2)
    rows = sq.routed_experts(h.to(dt).to(device), up, down, ids, wts, sq.ACT_RELU2, combine=False)
    xs = torch.zeros(T, K, device=device)
    sq.residual_norm(xs, None, None, None, rows, None, None, 1e-5)
    assert rel_err(xs, plain.cpu().to(F64)) < 1e-5


# ---------------------------------------------------------------------------------- random configurations
def _random_config(rng):
    W = rng.choice([64, 96, 160])

    def rot(dk):
        rd = rng.choice([0, 2, dk // 2 // 2 * 2, dk // 2 * 2])
        if not rd:
            return None
        r = {"base": rng.choice([100.0, 10000.0]), "dims": rd}
        if rng.random() < 0.6:
            r["scaling"] = {"factor": rng.choice([2.0, 8.0]), "low": 1.0, "high": rng.choice([2.0, 4.0]),
                            "original": rng.choice([16, 64])}
        return r
    vrow = rng.choice([32, 48, 64])     # value rows of the mixing layers

    def att():
        mix = rng.random() < 0.7
        G = rng.choice([1, 2, 4])
        dk = rng.choice([16, 32, 64])
        dv = vrow // G if mix else rng.choice([8, 16, 32])
        m = {"heads": G * rng.choice([1, 2, 4]), "kv_heads": G, "dim": dk, "vdim": dv, "scale": round(dk ** -0.5, 6),
             "v_mix": mix}
        if rng.random() < 0.8:
            m["mask"] = {"size": rng.choice([1, 3, 16, 30, 64, 100])}
        r = rot(dk)
        if r:
            m["rot"] = r
        return m

    def par():
        G, dk = rng.choice([1, 2]), rng.choice([16, 32, 48])
        left = {"heads": G * rng.choice([1, 2, 4]), "kv_heads": G, "dim": dk, "vdim": rng.choice([16, 32, 48]),
                "scale": round(dk ** -0.5, 6)}
        r = rot(dk)
        if r:
            left["rot"] = {"base": r["base"], "dims": r["dims"]}
        return {"left": left, "right": {"heads": rng.choice([1, 2, 4]), "dim": rng.choice([8, 16, 64, 96]),
                                        "vdim": rng.choice([8, 32, 96]), "tau": rng.choice([1.0, 4.0, 16.0]),
                                        "decay_rank": rng.choice([2, 16])}}
    layers = []
    for _ in range(rng.choice([2, 3, 4, 5])):
        t = rng.choice(["attention", "parallel", "mingru"])
        mixer = att() if t == "attention" else par() if t == "parallel" else {"width": rng.choice([40, 64, 200])}
        E = rng.choice([1, 2, 8, 12])
        mlp = None if rng.random() < 0.25 else {"kind": "moe", "expert": {"ff": rng.choice([16, 32, 40])},
                                                "router": {"experts": E, "top": rng.randrange(1, min(E, 3) + 1)}}
        layers.append({"type": t, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Lotelix", "width": W, "vocab": rng.choice([97, 300]),
            "norm": {"eps": rng.choice([1e-5, 1e-6]), "groups": rng.choice([1, 2, 4, 8])},
            "embedding": {"scale": round(W ** 0.5, 4)}, "layers": layers}


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("seed", [3, 14, 15, 92])
def test_random_configurations_through_mixed_schedules(seed, device, dtype, tmp_path):
    import random
    rng = random.Random(seed)
    cfg = _random_config(rng)
    Wt = orc.random_weights(cfg, seed)
    orc.write_checkpoint(str(tmp_path), cfg, Wt)
    lens = [rng.choice([150, 185]), rng.randrange(2, 20), rng.randrange(20, 45), 1]
    toks = [tokens_of(cfg, n, seed + i) for i, n in enumerate(lens)]
    refs = [orc.forward(cfg, Wt, t) for t in toks]
    eng = engine(str(tmp_path), device, dtype, block_size=16, num_blocks=sum((n + 63) // 64 * 64 for n in lens) // 16,
                 max_num_seqs=4, max_model_len=256)
    at, got = [0] * 4, [[] for _ in lens]
    while any(at[i] < lens[i] for i in range(4)):
        entries, who = [], []
        for i in range(4):
            if at[i] >= lens[i] or rng.random() < 0.2:
                continue
            n = min(lens[i] - at[i], rng.choice([1, 1, 2, 3, 17, 40, 140]))
            entries.append(("r%d" % i, toks[i][at[i]:at[i] + n], list(range(n))))
            who.append((i, n))
            at[i] += n
        if not entries:
            continue
        lg = eng.score_step(entries, ["r%d" % i for i, _ in who if at[i] == lens[i]])
        o = 0
        for i, n in who:
            got[i].append(lg[o:o + n])
            o += n
    for i in range(4):
        assert close(torch.cat(got[i], 0), refs[i], dtype), (i, cfg)
    assert eng.sched.num_used_blocks() == 0
