"""Loluzen on the engine against the dense fp64 oracle (tests/loluzen_oracle.py).

Every test runs on the CPU (PyTorch forms of the ops, same scheduler / cache / state code) and,
marked `gpu`, on the HIP kernels in float32 and bfloat16. Configurations and weights are made
here; the oracle shares no code with xgserve.
"""
import copy
import json
import os
import subprocess
import sys

import pytest
import torch

import loluzen_oracle as orc
from xgserve.engine import EngineConfig, LLMEngine, SamplingParams
from xgserve.models import build_model, get_config
from xgserve.models.config import loluzen_config
from xgserve.models.loluzen import ConvRopeAttention
from xgserve.models.seq_cache import LayerCache
from xgserve.ops import seqmix as sq

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
F64 = torch.float64

CASES = [pytest.param("cpu", "float32", id="cpu-f32"),
         pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)]
OP_CASES = [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)]
TOL = {"float32": 2e-4, "bfloat16": 6e-2}


def config_a():
    """Parallel layer first; key sizes unlike value sizes; three query heads per key head; recurrent head with
    dim != vdim; a looped run in the middle, three times; a layer without feed-forward; rotation of a whole head
    without rescaling, and of a part with all three wavelength ranges."""
    a1 = {"heads": 6, "kv_heads": 2, "dim": 20, "vdim": 12, "scale": 0.31, "conv": 2,
          "rot": {"base": 100.0, "dims": 20}}
    a2 = {"heads": 3, "kv_heads": 3, "dim": 24, "vdim": 40, "scale": 0.2, "conv": 5,
          "rot": {"base": 5000.0, "dims": 16, "scaling": {"factor": 6.0, "low": 1.0, "high": 8.0, "original": 160}}}
    par = {"left": {"heads": 6, "kv_heads": 3, "dim": 12, "vdim": 20, "scale": 0.35},
           "right": {"heads": 3, "dim": 20, "vdim": 12}}
    par2 = {"left": {"heads": 2, "kv_heads": 2, "dim": 40, "vdim": 8, "scale": 0.15},
            "right": {"heads": 1, "dim": 6, "vdim": 70}}
    return {"architecture": "Loluzen", "width": 88, "vocab": 150, "norm": {"eps": 1e-5}, "residual_mult": 0.4,
            "embedding": {"scale": 9.0}, "loop": {"start": 1, "stop": 3, "times": 3},
            "layers": [{"type": "parallel", "mixer": par, "mlp": {"kind": "dense", "ff": 72}},
                       {"type": "attention", "mixer": a1, "mlp": None},
                       {"type": "parallel", "mixer": par2, "mlp": {"kind": "dense", "ff": 40}},
                       {"type": "attention", "mixer": a2, "mlp": {"kind": "dense", "ff": 56}}]}


def config_b():
    """One head; one tap (no carried convolution inputs); no rotation; no loop; factors of one; a loop of one
    pass would be the same model."""
    a1 = {"heads": 1, "kv_heads": 1, "dim": 32, "vdim": 32, "scale": 0.2, "conv": 1}
    a2 = {"heads": 4, "kv_heads": 1, "dim": 16, "vdim": 8, "scale": 0.5, "conv": 3,
          "rot": {"base": 10.0, "dims": 2, "scaling": {"factor": 2.0, "low": 1.0, "high": 2.0, "original": 8}}}
    par = {"left": {"heads": 1, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.25},
           "right": {"heads": 2, "dim": 16, "vdim": 16}}
    return {"architecture": "Loluzen", "width": 48, "vocab": 97, "norm": {"eps": 1e-6}, "residual_mult": 1.0,
            "embedding": {"scale": 1.0}, "loop": None,
            "layers": [{"type": "attention", "mixer": a1, "mlp": {"kind": "dense", "ff": 32}},
                       {"type": "parallel", "mixer": par, "mlp": None},
                       {"type": "attention", "mixer": a2, "mlp": {"kind": "dense", "ff": 40}}]}


def config_c():
    """Sizes the matrix-core attention kernels take (key sizes multiples of 32, value sizes of 16); the whole
    model loops twice, the loop reaching the last layer."""
    a1 = {"heads": 4, "kv_heads": 2, "dim": 64, "vdim": 32, "scale": 0.125, "conv": 4,
          "rot": {"base": 10000.0, "dims": 32, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}}
    par = {"left": {"heads": 8, "kv_heads": 2, "dim": 32, "vdim": 16, "scale": 0.18},
           "right": {"heads": 2, "dim": 64, "vdim": 80}}
    return {"architecture": "Loluzen", "width": 128, "vocab": 200, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
            "embedding": {"scale": 11.3}, "loop": {"start": 0, "stop": 2, "times": 2},
            "layers": [{"type": "attention", "mixer": a1, "mlp": {"kind": "dense", "ff": 96}},
                       {"type": "parallel", "mixer": par, "mlp": {"kind": "dense", "ff": 64}}]}


_MADE = {}


def made(name, tmp_path_factory):
    """(config, oracle weights, checkpoint dir) of a test model, written once per session."""
    if name not in _MADE:
        cfg = {"a": config_a, "b": config_b, "c": config_c}[name]()
        Wt = orc.random_weights(cfg, seed={"a": 5, "b": 13, "c": 21}[name])
        path = str(tmp_path_factory.mktemp("loluzen_" + name))
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
    return rel_err(got, ref) < TOL[dtype]


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
    toks = tokens_of(cfg, 45, 1)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype)
    got = eng.score_step([("w", toks, list(range(len(toks))))], ["w"])
    assert close(got, ref, dtype)
    assert eng.sched.num_used_blocks() == 0


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("name", ["a", "c"])
def test_residual_after_every_layer_run(name, device, dtype, tmp_path_factory):
    cfg, Wt, path = made(name, tmp_path_factory)
    toks = tokens_of(cfg, 17, 2)
    res = []
    orc.forward(cfg, Wt, toks, res)
    assert len(res) == len(orc.layer_order(cfg)) > len(cfg["layers"])
    m = build_model(get_config(path), device=device, dtype=getattr(torch, dtype), checkpoint=path)
    eng = LLMEngine(EngineConfig(model=path, device=device, dtype=dtype, block_size=4, num_blocks=16, max_num_seqs=2,
                                 max_model_len=64, use_graphs=False), model=m)
    m.keep_residuals = seen = []
    with_hook = eng.score_step([("x", toks, [0, 16])], ["x"])
    m.keep_residuals = None
    fused = eng.score_step([("y", toks, [0, 16])], ["y"])   # the path that adds the embedding rows inside the kernel
    tol = 1e-4 if dtype == "float32" else 5e-2
    assert len(seen) == len(res)
    for got, ref in zip(seen, res):
        assert float((got.detach().to("cpu", F64) - ref).abs().max()) < tol * float(ref.abs().max())
    assert rel_err(fused, with_hook.cpu()) < (1e-5 if dtype == "float32" else 2e-2)


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
    cfg, Wt, path = made(name, tmp_path_factory)   # positions up to 170: many pages, every rotation range
    toks = tokens_of(cfg, 170, 5)
    ref = orc.forward(cfg, Wt, toks)
    eng = engine(path, device, dtype, num_blocks=48)
    got = run_portions(eng, "l", toks, [9])
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
    for p, o in zip(prompts, outs):
        ref = orc.forward(cfg, Wt, p + o[:-1])
        for i, tok in enumerate(o):
            row = ref[len(p) - 1 + i]
            gap = float(row.max() - row[tok])
            assert gap <= (1e-3 if dtype == "float32" else 0.15) * float(row.std()), (len(p), i, tok, int(row.argmax()))
    assert eng.sched.num_used_blocks() == 0


def test_registered_tiny_model_generates():
    eng = LLMEngine(EngineConfig(model="loluzen-tiny", device="cpu", dtype="float32", block_size=4, num_blocks=32,
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
    m = build_model(get_config("loluzen-tiny"), device="cpu", dtype=torch.float32, seed=3)
    save_checkpoint(m, str(tmp_path / "ck"))
    cfg2 = get_config(str(tmp_path / "ck"))
    assert cfg2.layer_loop == m.cfg.layer_loop and cfg2.embed_scale == m.cfg.embed_scale
    m2 = build_model(cfg2, device="cpu", dtype=torch.float32, checkpoint=str(tmp_path / "ck"))
    for (n1, p1), (n2, p2) in zip(m.named_parameters(), m2.named_parameters()):
        assert n1 == n2 and torch.equal(p1.to(torch.bfloat16).float(), p2), n1


def test_config_rejects_what_the_design_does_not_have():
    cfg = config_a()
    for edit in (lambda L: L[0].__setitem__("type", "something_else"),
                 lambda L: L[1]["mixer"].__setitem__("kv_heads", 4),           # 6 heads do not divide over 4
                 lambda L: L[0]["mixer"]["left"].__setitem__("kv_heads", 4),
                 lambda L: L[1]["mixer"]["rot"].__setitem__("dims", 22),       # more than the head holds
                 lambda L: L[1]["mixer"].__setitem__("conv", 9),
                 lambda L: L[0]["mlp"].__setitem__("kind", "other")):
        bad = copy.deepcopy(cfg["layers"])
        edit(bad)
        with pytest.raises(ValueError):
            loluzen_config("x", 88, 150, bad)
    with pytest.raises(ValueError):
        loluzen_config("x", 88, 150, cfg["layers"], loop={"start": 2, "stop": 2, "times": 2})
    with pytest.raises(ValueError):
        LLMEngine(EngineConfig(model="loluzen-tiny", device="cpu", num_blocks=8, max_num_seqs=2, max_model_len=32,
                               use_graphs=False, draft_model="llama-tiny-draft", num_speculative_tokens=2))


def test_layer_runs_and_their_caches():
    cfg = get_config("loluzen-tiny")
    assert cfg.layer_runs() == [0, 1, 1, 2]
    m = build_model(cfg, device="cpu", dtype=torch.float32, seed=1)
    cache = m.alloc_cache(8, 4, 2)
    assert len(cache.layers) == 4 and cache.layers[1].k.data_ptr() != cache.layers[2].k.data_ptr()
    assert m.pass_starts == {2}


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
        sm = seq_meta(device, rows, block_size, [tables[i] if tables else [0] * 64 for i, _ in who])
        y = fn(torch.cat(parts).to(device), sm)
        o = 0
        for i, q in who:
            got[i].append(y[o:o + q].float().cpu())
            o += q
    return [torch.cat(g).to(F64) for g in got]


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("W", [77, 96, 2304])
def test_post_norm_residual_one_and_two_branches(device, W):
    g = torch.Generator().manual_seed(W)
    T, eps, mult = 9, 1e-5, 0.3
    x, y, y2, extra = (torch.randn(T, W, generator=g) * s for s in (2.0, 3.0, 0.5, 1.0))
    bias, wb, wn, p1, p2 = (torch.randn(W, generator=g) * 0.3 for _ in range(5))
    n0 = lambda v: orc.unit_rms(v.to(F64), eps)  # noqa: E731
    for dual in (False, True):
        for dt in (torch.float32, torch.bfloat16):
            ya, yb = y.to(dt), y2.to(dt)
            u = 0.5 * (n0(ya) * (1 + p1) + n0(yb) * (1 + p2)) if dual else ya.to(F64) + bias
            xr = x.to(F64) + mult * n0(u) * (1 + wb) + extra
            nr = n0(xr) * (1 + wn)
            xd = x.clone().to(device)
            pad = torch.zeros(T, W + 8, dtype=dt, device=device)     # a row-strided branch output
            pad[:, :W] = ya.to(device)
            n = sq.post_norm_residual(xd, pad[:, :W], None if dual else bias.to(device), wb.to(device), mult,
                                      extra.to(device), wn.to(device), eps, torch.float32,
                                      y2=yb.to(device) if dual else None,
                                      pre_w=((1 + p1).to(device), (1 + p2).to(device)) if dual else None)
            assert float((xd.cpu().to(F64) - xr).abs().max()) < 1e-5 * float(xr.abs().max())
            assert float((n.cpu().to(F64) - nr).abs().max()) < 1e-5 * float(nr.abs().max())
    # without a branch: only the extra rows and the norm; without a next weight: only the sum
    xd = x.clone().to(device)
    n = sq.post_norm_residual(xd, None, None, None, 0.0, extra.to(device), wn.to(device), eps, torch.float32)
    assert float((n.cpu().to(F64) - n0(x + extra) * (1 + wn)).abs().max()) < 1e-5
    assert sq.post_norm_residual(xd, y.to(device), None, wb.to(device), mult, None, None, eps) is None


@pytest.mark.parametrize("device", OP_CASES)
def test_embedding_scale_squared_relu_and_head_norm(device):
    g = torch.Generator().manual_seed(3)
    tab = torch.randn(20, 24, generator=g)
    ids = torch.tensor([3, 19, 0, 7], dtype=torch.int32)
    got = sq.embed_rows(ids.to(device), tab.to(device), scale=6.5)
    assert torch.allclose(got.cpu(), tab[ids.long()] * 6.5, atol=1e-6)
    z, b = torch.randn(7, 36, generator=g), torch.randn(36, generator=g)
    assert torch.allclose(sq.relu2(z.to(device), b.to(device)).cpu(), torch.relu(z + b) ** 2, atol=1e-5)
    z2 = torch.randn(5, 9, generator=g)    # a row length the 4-wide path does not take
    assert torch.allclose(sq.relu2(z2.to(device), None).cpu(), torch.relu(z2) ** 2, atol=1e-6)
    y, w = torch.randn(6, 5 * 14, generator=g) * 3, torch.randn(14, generator=g)
    ref = (orc.unit_rms(y.to(F64).view(6, 5, 14), 1e-5) * w).reshape(6, 70)
    got = sq.gated_group_norm(y.to(device), None, w.to(device), 1e-5, 5, torch.float32)
    assert float((got.cpu().to(F64) - ref).abs().max()) < 1e-5


def test_rotation_frequencies_in_all_three_ranges():
    for rot in ({"base": 10000.0, "dims": 64, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 512}},
                {"base": 100.0, "dims": 6, "scaling": {"factor": 3.0, "low": 2.0, "high": 16.0, "original": 200}},
                {"base": 500.0, "dims": 10}):
        ref = orc.rot_frequencies(rot)
        got = sq.rot_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        assert torch.allclose(got, ref, rtol=1e-12)
        if rot.get("scaling"):
            plain = orc.rot_frequencies({"base": rot["base"], "dims": rot["dims"]})
            kinds = {("kept" if a == b else "slowed" if abs(a / b - rot["scaling"]["factor"]) < 1e-9 else "blend")
                     for a, b in zip(plain.tolist(), ref.tolist())}
            assert kinds == {"kept", "slowed", "blend"}


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("taps,rot_dims,G,dk", [(1, 0, 1, 24), (3, 8, 2, 24), (4, 24, 4, 24), (8, 10, 2, 24), (3, 64, 2, 96),
                                                 (2, 40, 1, 160)])
@pytest.mark.parametrize("fused", [True, False], ids=["one-pass", "two-pass"])
def test_conv_norm_rotation_attention_over_portions(device, dtype, taps, rot_dims, G, dk, fused, monkeypatch):
    """The "attention" mixer alone: carried convolution inputs, per-head norms, rotation by the absolute position,
    pages in a scrambled order, two sequences sharing steps, a slot with another sequence's leftovers."""
    monkeypatch.setattr(sq, "CONV_PREP_FUSED", fused)   # convolution inside the norm / rotation kernel, or before it
    dt = getattr(torch, dtype)
    W, H, dv, eps = 40, 4, 12, 1e-5
    m = {"heads": H, "kv_heads": G, "dim": dk, "vdim": dv, "scale": 0.3 * (24 / dk) ** 0.5, "conv": taps}
    if rot_dims:
        m["rot"] = {"base": 50.0, "dims": rot_dims, "scaling": {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 24}}
    cfg = {"width": W, "vocab": 8, "layers": [{"type": "attention", "mixer": m, "mlp": None}]}
    Wt = {k[len("l0.mix."):]: v for k, v in orc.random_weights(cfg, seed=taps).items() if k.startswith("l0.mix.")}
    g = torch.Generator().manual_seed(7)
    hs = [(torch.randn(n, W, generator=g)).to(torch.bfloat16).to(F64) for n in (37, 21)]
    refs = [orc.conv_rope_attention(Wt, "", m, h, eps) for h in hs]
    mod = ConvRopeAttention(W, m, eps, device, dt)
    nq, nk = H * dk, G * dk
    with torch.no_grad():
        mod.in_proj.copy_(torch.cat([Wt["q"], Wt["k"], Wt["v"], Wt["g"]]).to(dt))
        mod.conv_w.copy_(torch.cat([Wt["q.conv"], Wt["k.conv"], Wt["v.conv"]]))
        mod.q_norm.copy_(Wt["q.norm"])
        mod.k_norm.copy_(Wt["k.norm"])
        mod.o.copy_(Wt["o"].to(dt))
    rot = sq.build_rot_table(rot_dims, 50.0, 64, device, m["rot"]["scaling"]) if rot_dims else None
    lc = LayerCache(k=torch.randn(30 * 4, nk, device=device).to(dt), v=torch.randn(30 * 4, G * dv, device=device).to(dt),
                    mix_conv=torch.randn(3, taps - 1, nq + nk + G * dv, device=device))   # stale contents everywhere
    tables = [[7, 3, 22, 5, 11, 0, 19, 2, 28, 9], [1, 14, 4, 27, 8, 6]]
    got = in_portions(device, hs, [[5, 1, 1, 2, 17, 1, 10], [2, 2, 9, 1, 7]], [2, 0],
                      lambda x, sm: mod(x.to(dt), sm, lc, 4, rot), tables)
    for a, b in zip(got, refs):
        assert rel_err(a, b) < (1e-4 if dtype == "float32" else 4e-2)


def _talking_case(device, dtype, H, G, dk, dv, bs, T, single, strong=None):
    """Queries of one sequence over scrambled pages; `strong` = (query, key): that score stands out by design."""
    dt = getattr(torch, dtype)
    g = torch.Generator().manual_seed(H * 100 + dk + T)
    rnd = lambda *s: torch.randn(*s, generator=g).to(torch.bfloat16).to(F64)  # noqa: E731
    q, k, v = rnd(T, H, dk), rnd(T, G, dk), rnd(T, G, dv)
    if strong is not None:
        i, j = strong
        k[j] = q[i, ::H // G] * 1.5          # every head's query i lines up with key j
    r1, r2 = torch.rand(H, generator=g).to(F64) * 2, torch.rand(H, generator=g).to(F64) * 3 + 0.1
    talk = (torch.eye(H) + torch.randn(H, H, generator=g) * 0.5).to(F64)
    gate = rnd(T, H + 3)
    scale = 0.4 / dk ** 0.5 * (6.0 if strong is not None else 1.0)
    P = orc.causal_weights(q, k, scale, r1, r2)
    P = torch.einsum("hg,gij->hij", talk, P)
    ref = torch.stack([P[h] @ v[:, h // (H // G)] for h in range(H)], 1) * torch.sigmoid(gate[:, :H])[:, :, None]
    pages = torch.randperm(80, generator=g)[:(T + bs - 1) // bs].tolist()
    kc = torch.zeros(80 * bs, G * dk, dtype=dt, device=device)
    vc = torch.zeros(80 * bs, G * dv, dtype=dt, device=device)
    f32 = lambda t: t.float().to(device)  # noqa: E731
    out = []
    steps = [(0, T)] if not single else [(0, T - 6)] + [(T - 6 + i, 1) for i in range(6)]
    for ctx, n in steps:
        sm = seq_meta(device, [(0, ctx, n)], bs, [pages])
        rows = sm.slot_mapping.long()
        kc[rows] = k[ctx:ctx + n].reshape(n, -1).to(dt).to(device)
        vc[rows] = v[ctx:ctx + n].reshape(n, -1).to(dt).to(device)
        qq = q[ctx:ctx + n].reshape(n, -1).to(dt).to(device)
        wide = sq.masked_attention(qq, kc, vc, H, G, dk, dv, sq.MASK_CAUSAL, 0, scale, None, None, bs, sm,
                                   dist=(f32(r1), f32(r2)), values=sq.V_ALL)
        per = torch.stack([sq.masked_attention(qq, kc, vc, H, G, dk, dv, sq.MASK_CAUSAL, 0, scale, None, None, bs, sm,
                                               dist=(f32(r1), f32(r2)), values=c).view(n, H, dv) for c in range(G)], 2)
        assert rel_err(per.reshape(n, -1), wide.float().cpu()) < (1e-5 if dtype == "float32" else 3e-2)
        out.append(sq.talk_mix(wide, f32(talk), H, G, dv, gate=gate[ctx:ctx + n].to(dt).to(device)))
    got = torch.cat(out).float().cpu().view(T, H, dv)
    return got, ref


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("shape", [(6, 2, 20, 12), (1, 1, 32, 32), (8, 2, 64, 32), (4, 4, 96, 48), (16, 2, 32, 128)],
                         ids=lambda s: "H%dG%dk%dv%d" % s)
@pytest.mark.parametrize("single", [False, True], ids=["prompt", "decoded"])
def test_distance_penalty_head_mixing_and_gate(device, dtype, shape, single):
    got, ref = _talking_case(device, dtype, *shape, bs=4, T=75, single=single)
    assert rel_err(got.reshape(75, -1), ref.reshape(75, -1)) < (1e-4 if dtype == "float32" else 4e-2)


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("key", [0, 1, 15, 16, 17, 63, 64, 130, 299, 300])
@pytest.mark.parametrize("single", [False, True], ids=["prompt", "decoded"])
def test_one_standing_out_key_far_back_and_at_page_borders(device, dtype, key, single):
    """The last query's score for one key (the first token, a page's first / last row, hundreds of tokens back, the
    query itself) stands out: a lost or misplaced key, or a penalty taken at the wrong distance, moves the output."""
    T = 301
    got, ref = _talking_case(device, dtype, 4, 2, 32, 16, bs=16, T=T, single=single, strong=(T - 1, key))
    assert rel_err(got[-1].reshape(1, -1), ref[-1].reshape(1, -1)) < (1e-4 if dtype == "float32" else 4e-2)
    assert rel_err(got.reshape(T, -1), ref.reshape(T, -1)) < (1e-4 if dtype == "float32" else 4e-2)


@pytest.mark.parametrize("device", OP_CASES)
@pytest.mark.parametrize("H,dk,dv", [(3, 20, 12), (2, 16, 16), (1, 6, 70), (2, 64, 80), (1, 130, 24)])
@pytest.mark.parametrize("cols", [32, 64])
def test_gated_linear_recurrence_over_portions_and_slots(device, H, dk, dv, cols, monkeypatch):
    monkeypatch.setattr(sq, "SCAN_COLS", cols)    # both workgroup shapes of the scan kernel
    g = torch.Generator().manual_seed(dk)
    W, eps = 24, 1e-5
    m = {"heads": H, "dim": dk, "vdim": dv}
    cfg = {"width": W, "vocab": 8, "layers": [{"type": "parallel", "mlp": None, "mixer": {
        "left": {"heads": 1, "kv_heads": 1, "dim": 4, "vdim": 4, "scale": 1.0}, "right": m}}]}
    Wt = {k[len("l0.mix.right."):]: v for k, v in orc.random_weights(cfg, seed=dk).items() if k.startswith("l0.mix.right.")}
    hs = [torch.randn(n, W, generator=g).to(F64) for n in (29, 11)]
    n = H * dk
    Wcat = torch.cat([Wt["q"], Wt["f"], Wt["v"]])
    state = torch.randn(3, H, dk, dv).to(device)      # stale contents: a new sequence must not see them
    state2 = state.clone()
    fb, low = Wt["f.b"].float().to(device), Wt["lower"].float().to(device)

    def fn(x, sm):
        proj = (x.to(F64).cpu() @ Wcat.T).float().to(device)
        q, f = sq.lower_bound_gates(proj, 0, n, n, fb, low)
        o = sq.gated_linear_scan(q, f, None, proj[:, 2 * n:], state, H, dk, dv, sm)
        return sq.gated_group_norm(o, None, Wt["norm"].float().to(device), eps, H, torch.float32)

    def fused(x, sm):   # gates formed inside the scan, from columns of a wider row
        proj = torch.zeros(x.shape[0], Wcat.shape[0] + 5, device=device)
        proj[:, 5:] = (x.to(F64).cpu() @ Wcat.T).float().to(device)
        o = sq.lower_bound_recurrence(proj, 5, 5 + n, 5 + 2 * n, fb, low, state2, H, dk, dv, sm)
        return sq.gated_group_norm(o, None, Wt["norm"].float().to(device), eps, H, torch.float32)
    cuts = [[3, 1, 1, 2, 20, 2], [2, 2, 7]]
    for run, st in ((fn, state), (fused, state2)):
        got = in_portions(device, hs, cuts, [1, 2], run)
        for h, gt, slot in zip(hs, got, (1, 2)):
            states = []
            ref = orc.gated_linear_recurrence(dict(Wt, o=torch.eye(H * dv, dtype=F64)), "", m, h, eps, states)
            assert rel_err(gt, ref) < 2e-4
            assert float((st[slot].cpu().to(F64) - torch.stack(states)).abs().max()) < 1e-4
    # a general write strength k (not 1 - f) goes the same way
    T = 13
    q, f, k = torch.rand(T, n, generator=g), torch.rand(T, n, generator=g), torch.randn(T, n, generator=g)
    v = torch.randn(T, H * dv, generator=g)
    sm = seq_meta(device, [(0, 0, T)], 4, [[0] * 8])
    o = sq.gated_linear_scan(q.to(device), f.to(device), k.to(device), v.to(device), state, H, dk, dv, sm).cpu()
    S = torch.zeros(H, dk, dv, dtype=F64)
    for t in range(T):
        S = f[t].view(H, dk, 1) * S + k[t].view(H, dk, 1).to(F64) * v[t].view(H, 1, dv)
        assert torch.allclose(o[t].to(F64), torch.einsum("hkd,hk->hd", S, q[t].view(H, dk).to(F64)).reshape(-1), atol=1e-4)


# ---------------------------------------------------------------------------------- configurations drawn at random
def _random_config(rng):
    """Sizes, head counts, taps, rotation settings, layer order and loop drawn independently of each other."""
    W = rng.choice([64, 96, 160])

    def att():
        G, rep = rng.choice([1, 2, 3]), rng.choice([1, 2, 5])
        dk, dv = rng.choice([16, 24, 32, 64, 80]), rng.choice([8, 16, 24, 48])
        m = {"heads": G * rep, "kv_heads": G, "dim": dk, "vdim": dv, "scale": round(dk ** -0.5 * rng.choice([0.7, 1.3]), 6),
             "conv": rng.choice([1, 2, 3, 5])}
        rd = rng.choice([0, 2, dk // 4 * 2, dk])
        if rd:
            m["rot"] = {"base": rng.choice([100.0, 10000.0]), "dims": rd}
            if rng.random() < 0.7:
                m["rot"]["scaling"] = {"factor": rng.choice([2.0, 8.0]), "low": 1.0, "high": rng.choice([2.0, 4.0]),
                                       "original": rng.choice([16, 64])}
        return m

    def par():
        G, rep = rng.choice([1, 2, 4]), rng.choice([1, 2, 4])
        dk, dv = rng.choice([16, 32, 48]), rng.choice([16, 32, 48])
        return {"left": {"heads": G * rep, "kv_heads": G, "dim": dk, "vdim": dv, "scale": round(dk ** -0.5, 6)},
                "right": {"heads": rng.choice([1, 2, 4]), "dim": rng.choice([8, 16, 64, 96]), "vdim": rng.choice([8, 32, 96])}}
    n = rng.choice([2, 3, 4])
    layers = []
    for _ in range(n):
        t = rng.choice(["attention", "parallel"])
        layers.append({"type": t, "mixer": att() if t == "attention" else par(),
                       "mlp": None if rng.random() < 0.25 else {"kind": "dense", "ff": rng.choice([64, 100])}})
    a = rng.randrange(0, n)
    loop = {"start": a, "stop": rng.randrange(a + 1, n + 1), "times": rng.choice([1, 2, 3])} if rng.random() < 0.7 else None
    return {"architecture": "Loluzen", "width": W, "vocab": rng.choice([97, 300]), "norm": {"eps": rng.choice([1e-5, 1e-6])},
            "residual_mult": rng.choice([0.3, 1.0]), "embedding": {"scale": round(W ** 0.5, 4)}, "loop": loop, "layers": layers}


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("seed", [3, 14, 15, 92])
def test_random_configurations_through_mixed_schedules(seed, device, dtype, tmp_path):
    import random
    rng = random.Random(seed)
    cfg = _random_config(rng)
    Wt = orc.random_weights(cfg, seed)
    orc.write_checkpoint(str(tmp_path), cfg, Wt)
    lens = [rng.choice([70, 85]), rng.randrange(2, 20), rng.randrange(20, 45), 1]
    toks = [tokens_of(cfg, n, seed + i) for i, n in enumerate(lens)]
    refs = [orc.forward(cfg, Wt, t) for t in toks]
    eng = engine(str(tmp_path), device, dtype, block_size=16, num_blocks=sum((n + 63) // 64 * 64 for n in lens) // 16,
                 max_num_seqs=4)
    at, got = [0] * 4, [[] for _ in lens]
    while any(at[i] < lens[i] for i in range(4)):
        entries, who = [], []
        for i in range(4):
            if at[i] >= lens[i] or rng.random() < 0.2:
                continue
            n = min(lens[i] - at[i], rng.choice([1, 1, 2, 3, 17, 40]))
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
