"""The Gararax decoder through the engine against the plain oracle
(tests/gararax_oracle.py). Every test makes its own small configuration and
random checkpoint, writes it as a model folder, and loads it with
LLMEngine(folder): config reader, safetensors loader, cache manager, batching
and kernels are all the product's. CPU path always; the HIP path (fp32 and
bf16, decode through captured graphs) under the gpu marker."""
import functools

import pytest
import torch

import gararax_oracle as go
from gararax_oracle import attn, make_config, make_weights, moe, rel_err, \
    write_model_dir
from xllm_service_amd.engine.engine import LLMEngine
from xllm_service_amd.engine.sampling import SamplingParams

TARGETS = [("cpu", torch.float32),
           pytest.param(("cuda", torch.float32), marks=pytest.mark.gpu),
           pytest.param(("cuda", torch.bfloat16), marks=pytest.mark.gpu)]
BAND = dict(factor=8.0, low=1.0, high=2.0, original=48)


def _variants():
    return {
        # all three mixers, a dense and two routed feed-forwards, the token
        # side input, layers 1..2 run twice
        "mixed": make_config(loop=(1, 3, 2), layers=[
            attn("attention_2", size=7, keep_first=2),
            attn("attention_3", mlp=moe()),
            attn("attention", dims=8, scaling=BAND, size=6, keep_first=3,
                 mlp=moe(groups=(2, 1), identity=0, shared=0)),
            attn("attention", mlp=9)]),
        # nothing optional: no side input, no loop, multiplier 1, no mask, no
        # turn, no feed-forward in one layer, as many key/value heads as
        # heads, odd widths, experts without groups / identity / shared
        "plain": make_config(width=20, mult=1.0, side=0, layers=[
            attn("attention", heads=3, kv_heads=3, dim=6, vdim=7, dims=0,
                 size=None, mlp=None),
            attn("attention_3", heads=3, kv_heads=1, dim=10, vdim=4, dims=0,
                 mlp=moe(ff=5, experts=3, top=2, identity=0, groups=None,
                         shared=0)),
            attn("attention_2", heads=2, kv_heads=2, dim=6, size=None,
                 mlp=None)]),
        # everything that can be 1: one head, a window of the position itself,
        # one kept key, one pair turned, one expert chosen, one pass, a side
        # input one wide
        "ones": make_config(width=16, side=1, loop=(0, 2, 1), layers=[
            attn("attention", heads=1, kv_heads=1, dim=6, vdim=6, dims=2,
                 size=1, keep_first=1,
                 mlp=moe(ff=4, experts=1, top=1, identity=1, groups=(2, 1),
                         shared=0)),
            attn("attention_2", heads=1, kv_heads=1, dim=4, size=1,
                 keep_first=0, mlp=1),
            attn("attention_3", heads=1, kv_heads=1, dim=4, vdim=8, dims=4,
                 mlp=None)]),
        # the whole stack repeats three times; windows at a page's size and
        # one past it, more kept keys than the window holds
        "looped": make_config(width=32, loop=(0, 3, 3), layers=[
            attn("attention", heads=4, kv_heads=1, dim=8, vdim=4, dims=8,
                 size=16, keep_first=20, mlp=16),
            attn("attention_2", heads=4, kv_heads=2, dim=8, size=17,
                 keep_first=1, mlp=moe(ff=8, experts=6, top=3, identity=2,
                                       groups=(4, 2), shared=8)),
            attn("attention_3", heads=2, kv_heads=2, dim=16, vdim=8, dims=4,
                 mlp=None)]),
        # head widths of the matrix-core attention classes, three query heads
        # per group, windows around tile borders, a wide side input
        "large": make_config(width=128, vocab=200, eps=2e-6, mult=0.25,
                             side=16, loop=(2, 3, 2), layers=[
            attn("attention_2", heads=6, kv_heads=2, dim=64, size=33,
                 keep_first=4, mlp=192),
            attn("attention", heads=2, kv_heads=1, dim=128, vdim=80, dims=64,
                 base=500.0, scaling=BAND, size=40, keep_first=35,
                 mlp=moe(ff=48, experts=9, top=3, identity=3, groups=(4, 2),
                         shared=64)),
            attn("attention_3", heads=4, kv_heads=2, dim=128, vdim=48,
                 dims=32, base=10000.0, mlp=moe(ff=32, experts=5, top=2,
                                                identity=0, groups=None,
                                                shared=16))]),
    }


@functools.lru_cache(maxsize=None)
def _model(name, tmp_root):
    cfg = _variants()[name]
    w = make_weights(cfg, seed=sum(map(ord, name)))
    folder = write_model_dir(f"{tmp_root}/{name}", cfg, w)
    return cfg, w, folder


@pytest.fixture(scope="module")
def root(tmp_path_factory):
    return str(tmp_path_factory.mktemp("gararax_models"))


def _tokens(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


@functools.lru_cache(maxsize=None)
def _oracle(name, tmp_root, n, seed):
    cfg, w, _ = _model(name, tmp_root)
    return go.forward(cfg, w, _tokens(cfg, n, seed))[0]


def _engine(folder, target, blocks=64, slots=4, **kw):
    dev, dt = target
    return LLMEngine(folder, device=dev, dtype=dt, max_num_seqs=slots,
                     max_kv_blocks=blocks, max_model_len=blocks * 16,
                     enable_graphs=dev == "cuda", swap_space_mb=0, **kw)


def _check(got, want, target, what=""):
    """fp32: every row close, but for a rare row where two experts' choice
    scores nearly tie. bf16: rounding-sized error."""
    e = rel_err(got, want)
    if target[1] == torch.float32:
        assert float(e.median()) < 1e-4, (what, float(e.median()))
        assert int((e > 5e-4).sum()) <= len(e) // 40, (what, e)
    else:
        assert float(e.median()) < 0.06, (what, float(e.median()))
        assert float((e > 0.15).float().mean()) <= 0.1, (what, e)


def _run_portions(eng, rid, toks, cuts, end=True):
    """Feed toks in portions of the given sizes; logits at every position."""
    out, at = [], 0
    for n in cuts:
        last = at + n == len(toks)
        out.append(eng.score_step([(rid, toks[at:at + n], list(range(n)))],
                                  finished=[rid] if (last and end) else []))
        at += n
    assert at == len(toks)
    return torch.cat(out)


NAMES = ["mixed", "plain", "ones", "looped", "large"]


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", NAMES)
def test_whole_prompt(root, target, name):
    cfg, w, folder = _model(name, root)
    eng = _engine(folder, target)
    for n, seed in ((1, 1), (2, 2), (67, 3)):   # first tokens, past a page
        toks = _tokens(cfg, n, seed)
        got = _run_portions(eng, f"w{n}", toks, [n])
        _check(got, _oracle(name, root, n, seed), target, (name, n))


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["mixed", "looped"])
def test_residual_after_every_layer_run(root, target, name):
    """Hook the residual after every layer run of one prompt (a looped block
    is seen once per pass)."""
    cfg, w, folder = _model(name, root)
    eng = _engine(folder, target)
    toks = _tokens(cfg, 21, 5)
    seen = []
    hooks = [b.register_forward_hook(lambda m, i, o: seen.append(
        i[0].detach().float().cpu().clone())) for b in eng.model.blocks]
    eng.score_step([("a", toks, [0])], finished=["a"])
    for h in hooks:
        h.remove()
    trail = go.forward(cfg, w, toks)[1]
    assert len(seen) == len(trail) == len(eng.model.runs)
    for i, (a, b) in enumerate(zip(seen, trail)):
        err = (a.double() - b).norm(dim=-1) / b.norm(dim=-1).mean()
        if target[1] == torch.float32:
            assert float(err.max()) < 2e-4, (name, i, float(err.max()))
        else:
            assert float(err.median()) < 0.04, (name, i, float(err.median()))
            assert float((err > 0.15).float().mean()) <= 0.1, (name, i, err)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", NAMES)
def test_prefill_then_token_by_token(root, target, name):
    cfg, w, folder = _model(name, root)
    eng = _engine(folder, target)
    n = 40
    toks = _tokens(cfg, n, 7)
    want = _oracle(name, root, n, 7)
    for first in (1, 2, 15, 16, 17):
        got = _run_portions(eng, f"d{first}", toks, [first] + [1] * (n - first))
        _check(got, want, target, (name, first))


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["mixed", "looped", "large"])
def test_portions_of_many_sizes(root, target, name):
    cfg, w, folder = _model(name, root)
    eng = _engine(folder, target)
    n = 150
    toks = _tokens(cfg, n, 8)
    want = _oracle(name, root, n, 8)
    for cuts in ([2] * 10 + [16, 15, 17, 2, 64, 3, 1, 1, 11],
                 [63, 2, 64, 1, 2, 2, 16],
                 [65, 31, 33, 1, 1, 17, 2]):
        assert sum(cuts) == n
        got = _run_portions(eng, "p", toks, cuts)
        _check(got, want, target, cuts)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["looped", "large"])
def test_long_prompt_and_long_decoding(root, target, name):
    """A prompt of many pages, then decoding across several more: the windows
    slide over decoded tokens while the kept first keys stay, the unmasked
    layers look all the way back."""
    cfg, w, folder = _model(name, root)
    eng = _engine(folder, target)
    n = 330
    toks = _tokens(cfg, n, 9)
    got = _run_portions(eng, "l", toks, [200] + [1] * (n - 200))
    _check(got, _oracle(name, root, n, 9), target)


def test_a_far_kept_key_decides():
    """One attention layer whose first token's key stands far out: with the
    first keys kept the answer at a late position depends on the first
    token, without them it does not (the oracle agrees in both cases)."""
    out = {}
    for keep in (1, 0):
        cfg = make_config(width=16, side=0, mult=1.0, layers=[
            attn("attention_2", heads=2, kv_heads=1, dim=8, size=4,
                 keep_first=keep, mlp=None)])
        w = make_weights(cfg, seed=3)
        w["l0.mix.q"] *= 4.0
        w["l0.mix.k"] *= 4.0
        import tempfile
        eng = _engine(write_model_dir(tempfile.mkdtemp(), cfg, w),
                      ("cpu", torch.float32))
        rows = []
        for first in (1, 2):
            toks = [first] + _tokens(cfg, 59, 4)
            got = _run_portions(eng, f"k{first}", toks, [33] + [1] * 27)
            _check(got, go.forward(cfg, w, toks)[0], ("cpu", torch.float32))
            rows.append(got[-1])
        out[keep] = float((rows[0] - rows[1]).abs().max())
    assert out[1] > 1e-3 and out[0] < 1e-6, out


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["mixed", "looped", "large"])
def test_unequal_batch_with_reused_pages(root, target, name):
    """A pool far smaller than the sum of all requests: requests come and go
    in mixed batches (prompt portions beside single tokens), later ones land
    on freed pages that still hold the earlier ones' keys. Every request
    must match its own run alone."""
    cfg, w, folder = _model(name, root)
    lens = dict(a=70, b=3, c=33, d=50, e=18, f=41)
    toks = {k: _tokens(cfg, n, 20 + i) for i, (k, n) in enumerate(lens.items())}
    want = {k: _oracle(name, root, n, 20 + i)
            for i, (k, n) in enumerate(lens.items())}
    eng = _engine(folder, target, blocks=10, slots=3)   # 160 tokens of pages
    plan = [
        [("a", 30), ("b", 2)],
        [("a", 1), ("b", 1), ("c", 17)],
        [("a", 16), ("c", 16)],                 # b done: its page is free
        [("a", 1), ("d", 2)],                   # d on b's page
        [("a", 22), ("d", 1)],                  # a done (70)
        [("d", 31), ("e", 18)],                 # c done earlier; e on a's pages
        [("d", 1), ("f", 5)],
        [("d", 15), ("f", 1)],
        [("f", 35)],
    ]
    at = {k: 0 for k in lens}
    got = {k: [] for k in lens}
    for step in plan:
        entries, done = [], []
        for k, n in step:
            entries.append((k, toks[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == lens[k]:
                done.append(k)
        out = eng.score_step(entries, finished=done)
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n])
            o += n
    assert at == lens
    assert eng.block_manager.num_free == 10
    for k in lens:
        _check(torch.cat(got[k]), want[k], target, k)


@pytest.mark.parametrize("target", TARGETS)
@pytest.mark.parametrize("name", ["mixed", "large"])
def test_greedy_generation_through_scheduler(root, target, name):
    """generate(): continuous batching with chunked prompts (a 16-token step
    budget), three unequal prompts on two batch rows, greedy sampling. The
    oracle continues each prompt alone; a step whose two best oracle logits
    are closer than the dtype's noise ends the comparison."""
    cfg, w, folder = _model(name, root)
    dev, dt = target
    eng = LLMEngine(folder, device=dev, dtype=dt, max_num_seqs=2,
                    max_kv_blocks=32, max_model_len=256,
                    max_batched_tokens=16, enable_graphs=dev == "cuda",
                    swap_space_mb=0)
    prompts = [_tokens(cfg, n, 40 + n) for n in (37, 5, 20)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=6, ignore_eos=True))
    margin = 1e-3 if dt == torch.float32 else 0.15
    for p, out in zip(prompts, outs):
        assert len(out) == 6
        seq = list(p)
        for tok in out:
            top = go.forward(cfg, w, seq)[0][-1].topk(2)
            if float(top.values[0] - top.values[1]) < margin:
                break
            assert tok == int(top.indices[0])
            seq.append(tok)
    assert eng.block_manager.num_free == 32


def test_preset_generates_through_the_engine():
    """The named preset (random weights; two of its layers run twice and own
    a cache per pass)."""
    eng = LLMEngine("gararax-tiny", device="cpu", max_num_seqs=2,
                    max_kv_blocks=16, max_model_len=128, swap_space_mb=0)
    assert len(eng.model.blocks) == 4 and len(eng.runner.kv_caches) == 6
    k, v = eng.runner.kv_caches[0]
    assert k is v                       # the gated layer reads keys as values
    a = eng.generate([[1, 2, 3, 4, 5, 6, 7], [9, 8]],
                     SamplingParams(max_tokens=4, ignore_eos=True))
    b = eng.generate([[9, 8]], SamplingParams(max_tokens=4, ignore_eos=True))
    assert [len(x) for x in a] == [4, 4] and a[1] == b[0]


def test_trace_replay_command(root, tmp_path):
    """bin/trace_run on a model folder: steps on stdin, logits in files, a
    pool of 128 tokens used by three requests in turn."""
    import json
    import os
    import subprocess
    import sys

    import numpy as np
    cfg, w, folder = _model("mixed", root)
    toks = {k: _tokens(cfg, n, 60 + n) for k, n in (("a", 40), ("b", 9),
                                                     ("c", 30))}
    steps = [
        dict(step=0, entries=[dict(id="a", tokens=toks["a"][:33], want=[0, 32]),
                              dict(id="b", tokens=toks["b"][:8], want=[])],
             end=[]),
        dict(step=1, entries=[dict(id="a", tokens=toks["a"][33:34], want=[0]),
                              dict(id="b", tokens=toks["b"][8:], want=[0])],
             end=["b"]),
        dict(step=2, entries=[dict(id="c", tokens=toks["c"][:2], want=[1])],
             end=[]),
        dict(step=3, entries=[dict(id="a", tokens=toks["a"][34:], want=[5]),
                              dict(id="c", tokens=toks["c"][2:], want=[27])],
             end=["a", "c"]),
    ]
    exe = os.path.join(os.path.dirname(os.path.dirname(
        os.path.abspath(__file__))), "bin", "trace_run")
    out = tmp_path / "out"
    p = subprocess.run(
        [sys.executable, exe, "--model", folder, "--dtype", "float32", "--out",
         str(out), "--max-tokens", "128", "--slots", "2", "--device", "cpu"],
        input="".join(json.dumps(x) + "\n" for x in steps), text=True,
        capture_output=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.split("\n") if l.startswith("done")] == [
        f"done {i}" for i in range(4)]
    full = {k: go.forward(cfg, w, t)[0] for k, t in toks.items()}
    want = {0: [full["a"][0], full["a"][32]], 1: [full["a"][33], full["b"][8]],
            2: [full["c"][1]], 3: [full["a"][39], full["c"][29]]}
    for i, rows in want.items():
        got = torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4")
                               .reshape(len(rows), -1).copy())
        _check(got, torch.stack(rows), ("cpu", torch.float32), i)


def test_config_is_checked(tmp_path):
    bad = make_config()
    bad["layers"][0]["type"] = "something"
    with pytest.raises(ValueError):
        LLMEngine(write_model_dir(str(tmp_path / "t"), bad, {}), device="cpu")
    bad = make_config()
    bad["layers"][0]["mlp"]["kind"] = "other"
    with pytest.raises(ValueError):
        LLMEngine(write_model_dir(str(tmp_path / "k"), bad, {}), device="cpu")
    bad = make_config(loop=(2, 9, 2))
    with pytest.raises(ValueError):
        LLMEngine(write_model_dir(str(tmp_path / "n"), bad, {}), device="cpu")
    ok = make_config()
    w = make_weights(ok)
    del w["l1.mix.temp"]
    with pytest.raises(KeyError):
        LLMEngine(write_model_dir(str(tmp_path / "m"), ok, w), device="cpu")
    w = make_weights(ok)
    w["l0.mix.v"] = torch.zeros(3, 3)
    with pytest.raises(ValueError):
        LLMEngine(write_model_dir(str(tmp_path / "u"), ok, w), device="cpu")
