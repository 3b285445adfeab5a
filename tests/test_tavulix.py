"""Tavulix through the framework (loader, scheduler, block and state-slot bookkeeping, model runner, kernels on the
GPU / reference ops on the CPU) against the plain float64 model of ``tests/tavulix_oracle.py``.

Every test builds its own small configuration and random weights (stored as bfloat16, so the oracle and the framework
read the same numbers).  The schedules go through ``EngineCore.step_forced`` - the replay path of
``bin/trace_run`` - and generation goes through ``LLM.generate``.  The CPU tests run in float32; the GPU tests run the
HIP kernels in float32 (tight tolerance: an index that is one off shows) and in bfloat16.
"""
import json
import os
import types

import numpy as np
import pytest
import torch

import tavulix_oracle as oracle

HAS_GPU = torch.cuda.device_count() > 0


# ------------------------------------------------------------------------------------------------ models
def mixer(heads, kv, dim, vdim, conv, size, keep, v_mix=True, scale=None, softcap=30.0):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale or dim ** -0.5,
            "softcap": softcap, "v_mix": v_mix, "mask": {"size": size, "keep_first": keep}}


def layer(m, ff=None):
    return {"type": "attention", "mixer": m, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def config(layers, width=48, vocab=97, max_positions=512, eps=1e-5, cap=12.0):
    return {"architecture": "Tavulix", "vocab": vocab, "width": width, "max_positions": max_positions,
            "norm": {"eps": eps}, "logit_softcap": cap, "layers": layers}


CONFIGS = {
    # windows of a few tokens, every layer of another shape, a layer without feed-forward, one outside the value mix
    "varied": config([layer(mixer(4, 2, 16, 8, 3, 9, 2), 80), layer(mixer(6, 3, 8, 24, 4, 5, 0, v_mix=False)),
                      layer(mixer(4, 2, 32, 8, 2, 17, 3), 64), layer(mixer(4, 2, 24, 8, 5, 3, 1), 40)]),
    # values a model can make equal or one: one head, kv heads = heads, vdim = dim, one tap, window of one token,
    # nothing kept, a window wider than any test sequence, no value mixing anywhere
    "degenerate": config([layer(mixer(1, 1, 16, 16, 1, 1, 0, v_mix=False), 32),
                          layer(mixer(3, 3, 8, 8, 2, 400, 0, v_mix=False), 32),
                          layer(mixer(2, 2, 16, 16, 3, 6, 6, v_mix=False))], width=32, vocab=50),
    # a window that spans pages of 16 tokens and a kept prefix longer than a page
    "paged": config([layer(mixer(4, 1, 32, 16, 3, 37, 19), 96), layer(mixer(4, 1, 16, 16, 3, 70, 1), 96)], width=64),
}


def random_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)

    def rnd(*shape, lo=-1.0, hi=1.0):
        return lo + (hi - lo) * torch.rand(shape, generator=g)

    w = {"embed": rnd(cfg["vocab"], cfg["width"]), "pos": rnd(cfg["max_positions"], cfg["width"], lo=-0.5, hi=0.5),
         "final.norm": rnd(lo=0.8, hi=1.3), "head": rnd(cfg["vocab"], cfg["width"]) * (3.0 / cfg["width"]) ** 0.5}
    for i, spec in enumerate(cfg["layers"]):
        m, p, width = spec["mixer"], f"l{i}.", cfg["width"]
        for n in ("norm1", "norm1b", "norm2", "norm2b"):
            w[p + n] = rnd(lo=0.7, hi=1.4)
        for n, rows in (("q", m["heads"] * m["dim"]), ("k", m["kv_heads"] * m["dim"]), ("v", m["kv_heads"] * m["vdim"])):
            w[p + f"mix.{n}"] = rnd(rows, width) * (3.0 / width) ** 0.5
            w[p + f"mix.{n}.conv"] = rnd(rows, m["conv"])
        w[p + "mix.q.norm"], w[p + "mix.k.norm"] = rnd(m["dim"], lo=0.5, hi=1.5), rnd(m["dim"], lo=0.5, hi=1.5)
        w[p + "mix.vmix"] = rnd(lo=0.2, hi=0.7)
        w[p + "mix.r1"], w[p + "mix.r2"] = rnd(m["heads"], lo=0.1, hi=1.0), rnd(m["heads"], lo=0.05, hi=0.8)
        w[p + "mix.sink"] = rnd(m["heads"], lo=-1.0, hi=2.0)
        w[p + "mix.g"] = rnd(m["heads"], width) * (3.0 / width) ** 0.5
        w[p + "mix.o"] = rnd(width, m["heads"] * m["vdim"]) * (3.0 / (m["heads"] * m["vdim"])) ** 0.5
        if spec["mlp"]:
            ff = spec["mlp"]["ff"]
            w[p + "mlp.up"] = rnd(ff, width) * (3.0 / width) ** 0.5
            w[p + "mlp.down"] = rnd(width, ff) * (3.0 / ff) ** 0.5
            w[p + "mlp.act"] = rnd(4)
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


_MODELS = {}


def model_dir(name, tmp_path_factory):
    if name not in _MODELS:
        from safetensors.torch import save_file
        cfg = CONFIGS[name]
        w = random_weights(cfg, seed=sum(map(ord, name)))
        d = tmp_path_factory.mktemp("tavulix_" + name)
        save_file({k: v.contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
        (d / "config.json").write_text(json.dumps(cfg))
        _MODELS[name] = (str(d), cfg, w)
    return _MODELS[name]


_ORACLE = {}


def oracle_logits(name, cfg, w, tokens):
    key = (name, tuple(tokens))
    if key not in _ORACLE:
        _ORACLE[key] = oracle.forward(cfg, w, list(tokens)).numpy()
    return _ORACLE[key]


def tokens_for(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], n).tolist()


# ------------------------------------------------------------------------------------------------ replay
def run_schedule(path, steps, dtype, device, max_tokens, block_size=16, max_seqs=4, eager=False, tmp=None):
    """``steps``: list of ``[(request, tokens, want), ...]`` and, optionally, ``{"end": [...]}`` as last element.
    Returns ``{(request, absolute position): logits}``."""
    from vllm_distributed_amd.entrypoints import trace_replay
    args = types.SimpleNamespace(model=path, dtype=dtype, out=str(tmp), max_tokens=max_tokens, max_seqs=max_seqs,
                                 device=device, block_size=block_size, enforce_eager=eager)
    core = trace_replay.make_core(args)
    lines, where, at = [], {}, {}
    try:
        for n, step in enumerate(steps):
            end = []
            if step and isinstance(step[-1], dict):
                end, step = step[-1]["end"], step[:-1]
            entries = []
            for rid, toks, want in step:
                lo = at.get(rid, 0)
                entries.append({"id": rid, "tokens": toks, "want": want})
                where[n] = where.get(n, []) + [(rid, lo + k) for k in want]
                at[rid] = lo + len(toks)
            for rid in end:
                at.pop(rid, None)
            lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
        said = []
        trace_replay.replay(core, lines, str(tmp), say=said.append)
        assert said == [f"done {n}" for n in range(len(steps))]
    finally:
        core.shutdown()
    vocab = core.vllm_config.model_config.vocab_size
    out = {}
    for n, keys in where.items():
        got = np.fromfile(os.path.join(str(tmp), f"{n}.f32"), dtype="<f4").reshape(len(keys), vocab)
        for row, key in zip(got, keys):
            out[key] = row
    return out


def portions(tokens, sizes, rid, want_all=True):
    """Cut ``tokens`` into steps of the given sizes (the last size repeats)."""
    steps, at, i = [], 0, 0
    while at < len(tokens):
        n = min(sizes[min(i, len(sizes) - 1)], len(tokens) - at)
        steps.append([(rid, tokens[at:at + n], list(range(n)) if want_all else [n - 1])])
        at, i = at + n, i + 1
    steps[-1].append({"end": [rid]})
    return steps


def check(got, name, cfg, w, reqs, tol):
    """``reqs``: request -> (oracle key, tokens); every logits row the run produced is compared."""
    assert got
    for (rid, p), row in got.items():
        want = oracle_logits(name, cfg, w, reqs[rid])[p]
        err = np.abs(row - want).max()
        assert err <= tol, (rid, p, float(err))


DEVICES = [pytest.param("cpu", "float32", 2e-4, id="cpu-f32"),
           pytest.param("cuda", "float32", 2e-4, id="gpu-f32", marks=pytest.mark.gpu),
           pytest.param("cuda", "bfloat16", 0.35, id="gpu-bf16", marks=pytest.mark.gpu)]


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("name", ["varied", "degenerate", "paged"])
def test_whole_prompt_and_first_tokens(name, device, dtype, tol, tmp_path_factory, tmp_path):
    path, cfg, w = model_dir(name, tmp_path_factory)
    reqs = {"a": tokens_for(cfg, 90, 1), "b": tokens_for(cfg, 1, 2), "c": tokens_for(cfg, 2, 3)}
    steps = [[(r, t, list(range(len(t)))), {"end": [r]}] for r, t in reqs.items()]
    got = run_schedule(path, steps, dtype, device, max_tokens=128, tmp=tmp_path)
    assert len(got) == 93
    check(got, name, cfg, w, reqs, tol)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("name", ["varied", "paged"])
def test_prefill_then_token_by_token_matches(name, device, dtype, tol, tmp_path_factory, tmp_path):
    """A prompt, then 100 tokens one at a time: far beyond every window and kept prefix, over several pages."""
    path, cfg, w = model_dir(name, tmp_path_factory)
    toks = tokens_for(cfg, 140, 4)
    steps = portions(toks, [40, 1], "r")
    got = run_schedule(path, steps, dtype, device, max_tokens=192, tmp=tmp_path)
    assert len(got) == 140
    check(got, name, cfg, w, {"r": toks}, tol)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7, 1, 16, 17, 2, 2, 31, 5], [1], [64, 2, 1]])
def test_portions_of_any_size(sizes, device, dtype, tol, tmp_path_factory, tmp_path):
    path, cfg, w = model_dir("varied", tmp_path_factory)
    toks = tokens_for(cfg, 75 if sizes != [1] else 40, 5)
    got = run_schedule(path, portions(toks, sizes, "r"), dtype, device, max_tokens=128, tmp=tmp_path)
    assert len(got) == len(toks)
    check(got, "varied", cfg, w, {"r": toks}, tol)


@pytest.mark.parametrize("eager", [False, True])
@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_mixed_batches_reuse_pages_and_slots(device, dtype, tol, eager, tmp_path_factory, tmp_path):
    """Seven unequal requests through three sequence slots and a pool of 10 pages: portions of prompts beside single
    tokens, requests that sit steps out, slots and pages handed on as requests end; every row against the request
    run alone by the oracle."""
    if eager and device == "cpu":
        pytest.skip("graphs exist on the GPU only")
    path, cfg, w = model_dir("paged", tmp_path_factory)
    reqs = {f"q{i}": tokens_for(cfg, n, 10 + i) for i, n in enumerate([50, 33, 1, 47, 20, 48, 9])}
    at = {r: 0 for r in reqs}
    pattern = {"q0": [7, 1, 1, 2, 30, 1], "q1": [2, 16, 1, 1, 1], "q2": [1], "q3": [17, 1, 15, 1], "q4": [1, 1, 5],
               "q5": [30, 2, 1], "q6": [2, 1]}
    waiting, live, steps, turn = list(reqs), [], [], 0
    while waiting or live:
        while waiting and len(live) < 3 and \
                sum(-(-len(reqs[r]) // 64) * 64 for r in live + waiting[:1]) <= 160:
            live.append(waiting.pop(0))
        step, ended = [], []
        for k, r in enumerate(list(live)):
            if (turn + k) % 4 == 3 and len(live) > 1:
                continue                                    # sits this step out
            sizes = pattern[r]
            n = min(sizes[min(at[r] and (turn % len(sizes)), len(sizes) - 1)], len(reqs[r]) - at[r])
            step.append((r, reqs[r][at[r]:at[r] + n], list(range(n))))
            at[r] += n
            if at[r] == len(reqs[r]):
                ended.append(r)
                live.remove(r)
        if step:
            steps.append(step + ([{"end": ended}] if ended else []))
        turn += 1
    got = run_schedule(path, steps, dtype, device, max_tokens=160, max_seqs=3, eager=eager, tmp=tmp_path)
    assert len(got) == sum(len(t) for t in reqs.values())
    check(got, "paged", cfg, w, reqs, tol)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_batch_rows_equal_single_runs(device, dtype, tol, tmp_path_factory, tmp_path):
    """The same rows run alone and inside a batch of unequal neighbours agree beyond what the oracle tolerance needs."""
    path, cfg, w = model_dir("varied", tmp_path_factory)
    a, b, c = tokens_for(cfg, 30, 20), tokens_for(cfg, 11, 21), tokens_for(cfg, 64, 22)
    alone = run_schedule(path, portions(a, [13, 1], "a"), dtype, device, max_tokens=64, tmp=tmp_path / "x")
    steps = [[("c", c[:50], []), ("a", a[:13], list(range(13))), ("b", b[:2], [])]]
    for i in range(13, 30):
        step = [("a", a[i:i + 1], [0])]
        if i < 22:
            step.append(("b", b[i - 11:i - 10], []))
        if i < 27:
            step.insert(0, ("c", c[50 + i - 13:51 + i - 13], []))
        steps.append(step)
    both = run_schedule(path, steps, dtype, device, max_tokens=192, tmp=tmp_path / "y")
    for p in range(30):
        d = np.abs(alone[("a", p)] - both[("a", p)]).max()
        assert d <= (1e-4 if dtype == "float32" else 0.2), (p, float(d))


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_pages_behind_the_window_are_reused_while_the_request_goes_on(device, dtype, tol, tmp_path_factory, tmp_path):
    """A long request leaves its window behind: the pages over the keys no layer sees any more go back to the pool
    (those over the kept first keys stay), short requests that come and go take them, and the long request's own
    later pages come from the same pool.  Its logits, and theirs, stay those of each request alone."""
    from vllm_distributed_amd.entrypoints import trace_replay
    path, cfg, w = model_dir("varied", tmp_path_factory)              # windows 9 / 5 / 17 / 3, kept 2 / 0 / 3 / 1
    long_req, short = tokens_for(cfg, 420, 30), tokens_for(cfg, 40, 31)
    reqs = {"long": long_req}
    steps, at, k = [[("long", long_req[:250], [249])]], 250, 0
    while at < len(long_req):
        step = [("long", long_req[at:at + 1], [0])]
        at += 1
        ended = []
        if at % 20 == 0 and k < 8:
            k += 1
            reqs[f"s{k}"] = short
            step.append((f"s{k}", short, [len(short) - 1, 7]))
            ended.append(f"s{k}")
        if at == len(long_req):
            ended.append("long")
        steps.append(step + ([{"end": ended}] if ended else []))
    released = []
    original = trace_replay.replay

    def spy(core, lines, out_dir, say=print):
        kv = core.scheduler.kv
        real = kv.release_out_of_window
        kv.release_out_of_window = lambda r: released.append(real(r)) or released[-1]
        return original(core, lines, out_dir, say)

    trace_replay.replay = spy
    try:
        # 27 pages of 16 hold the long request alone; a short one beside it lives on pages the window has left
        got = run_schedule(path, steps, dtype, device, max_tokens=448 + 64, tmp=tmp_path)
    finally:
        trace_replay.replay = original
    assert sum(released) > 5
    assert len(got) == 1 + 170 + 16
    check(got, "varied", cfg, w, reqs, tol)


# --------------------------------------------------------------------------- mechanisms alone, made to show
def _attention_case(device, dtype, n, d, dv, bs=16):
    """One sequence of ``n`` keys in shuffled pages; the keys are orthogonal directions so that a query can single
    one out."""
    g = torch.Generator().manual_seed(n)
    dt = getattr(torch, dtype)
    nblocks = -(-n // bs) + 3
    table = torch.randperm(nblocks, generator=g)[:-(-n // bs)].to(torch.int32).view(1, -1)
    keys = torch.randn(n, d, generator=g) * 0.05
    vals = torch.randn(n, dv, generator=g)
    kc, vc = torch.zeros(nblocks, 1, bs, d), torch.zeros(nblocks, 1, bs // 8, dv, 8)
    for j in range(n):
        kc[table[0, j // bs], 0, j % bs], vc[table[0, j // bs], 0, (j % bs) // 8, :, j % 8] = keys[j], vals[j]
    to = lambda t: t.to(device)                                           # noqa: E731
    return keys, vals, to(kc.to(dt)), to(vc.to(dt)), to(table)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_one_key_stands_out_at_every_edge(device, dtype, tol):
    """The query is aimed at ONE key with a large score: the output is that key's value exactly when the key is
    visible - far back among hundreds inside a wide window, at a page border, the last key inside the window, the
    first one outside, the last kept first token, the first one not kept - in a prompt's portion and in a decoded
    row."""
    from vllm_distributed_amd import ops
    n, d, dv, window, keep = 300, 32, 16, 100, 5
    keys, vals, kc, vc, table = _attention_case(device, dtype, n, d, dv)
    dt = getattr(torch, dtype)
    pos = n - 1
    lo = pos - window + 1
    targets = {"far_inside": lo + 3, "window_first_inside": lo, "window_last_outside": lo - 1, "kept_last": keep - 1,
               "not_kept_first": keep, "page_border_a": 255, "page_border_b": 256, "self": pos, "first": 0,
               "middle_outside": 120}
    for rows in (1, 7):                                   # decoded alone / the last row of a portion
        for what, j in targets.items():
            q = torch.zeros(rows, 1, d)
            q[-1, 0] = keys[j] / keys[j].norm() ** 2 * 60.0             # score 60 on key j, small on the others
            positions = torch.arange(pos - rows + 1, pos + 1, dtype=torch.int32)
            out = ops.window_bias_attention(
                q.to(dt).to(device), kc, vc, table, torch.tensor([0, rows], dtype=torch.int32, device=device),
                torch.tensor([n], dtype=torch.int32, device=device),
                torch.zeros(rows, dtype=torch.int32, device=device), positions.to(device),
                1.0, 0.0, window, keep, None, None, None, None, rows)
            seen = oracle.visible(pos, j, window, keep)
            hit = (out[-1, 0].float().cpu() - vals[j].to(dt).float()).abs().max().item()
            assert (hit < 0.05) == seen, (what, rows, hit)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_sink_cap_and_distance_bias_show(device, dtype, tol):
    """With one visible key the weight is exp(s) / (exp(s) + exp(sink)): a missing sink, a sink that is scaled or
    capped, a missing cap or a missing distance bias each change it."""
    from vllm_distributed_amd import ops
    d, dv = 16, 8
    dt = getattr(torch, dtype)
    kc, vc = torch.zeros(2, 1, 16, d), torch.zeros(2, 1, 2, dv, 8)
    kc[1, 0, :, 0] = 1.0
    vc[1] = 1.0
    table = torch.tensor([[1, 0]], dtype=torch.int32, device=device)
    for pos, window, sink, cap, r1, r2, raw in ((0, 4, 0.7, 2.0, 0.5, 0.3, 5.0), (3, 1, -1.5, 0.0, 0.9, 2.0, 1.0),
                                                (3, 1, 30.0, 1.0, 0.0, 0.0, 0.4)):
        q = torch.zeros(1, 1, d)
        q[0, 0, 0] = raw
        out = ops.window_bias_attention(
            q.to(dt).to(device), kc.to(dt).to(device), vc.to(dt).to(device), table,
            torch.tensor([0, 1], dtype=torch.int32, device=device), torch.tensor([pos + 1], dtype=torch.int32, device=device),
            None, torch.tensor([pos], dtype=torch.int32, device=device), 0.5, cap, window, 0,
            torch.tensor([r1], device=device), torch.tensor([r2], device=device), torch.tensor([sink], device=device), None, 1)
        s = raw * 0.5
        s = cap * np.tanh(s / cap) if cap else s          # (one visible key: itself, at distance 0 -> no bias)
        want = np.exp(s) / (np.exp(s) + np.exp(sink))
        assert abs(out[0, 0, 0].item() - want) < (1e-5 if dtype == "float32" else 1e-2), (pos, out[0, 0, 0].item(), want)
    # two visible keys at distances 0 and 1 with equal raw scores: the bias alone decides their weights
    q = torch.zeros(1, 1, d)
    vc2 = vc.clone()
    vc2[1, 0, 0, :, 0] = 0.0                                # key 0 carries value 0, key 1 value 1
    out = ops.window_bias_attention(
        q.to(dt).to(device), kc.to(dt).to(device), vc2.to(dt).to(device), table,
        torch.tensor([0, 1], dtype=torch.int32, device=device), torch.tensor([2], dtype=torch.int32, device=device),
        None, torch.tensor([1], dtype=torch.int32, device=device), 1.0, 0.0, 8, 0,
        torch.tensor([1.3], device=device), torch.tensor([0.6], device=device), None, None, 1)
    far = np.exp(-1.3 * np.log(1 + 0.6))
    assert abs(out[0, 0, 0].item() - 1.0 / (1.0 + far)) < (1e-5 if dtype == "float32" else 1e-2)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_short_convolution_carries_its_tail_across_portions(device, dtype, tol, taps):
    """The convolved rows of a sequence cut into portions (down to one row, and two rows with more taps than rows)
    equal the convolution of the whole, with the slot holding another request's tail beforehand."""
    from vllm_distributed_amd import ops
    h, g, d, dv = 2, 1, 8, 8
    c = h * d + g * (d + dv)
    gen = torch.Generator().manual_seed(taps)
    dt = getattr(torch, dtype)
    x = torch.randn(40, c, generator=gen).to(dt)
    w = torch.randn(c, taps, generator=gen).to(dt)
    want = oracle.causal_taps(x.double(), w.double())
    w = w.t().contiguous()                                  # the op reads the taps tap-major
    state = torch.randn(3, max(taps - 1, 1), c, generator=gen).to(dt).to(device)        # stale tails
    ones = torch.ones(d, device=device)
    got, at = [], 0
    for n in [1, 2, 1, 1, 9, 2, 2, 21, 1]:
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=device)                 # noqa: E731
        q, kept = ops.conv_norm_cache(
            x[at:at + n].to(device), w.to(device), state, i32([1]), i32([0, n]), i32([at + n]), i32([0] * n),
            i32(list(range(at, at + n))), h, g, d, dv, ones, ones, 1e-6, None, None, True, None, None, i32([-1] * n), True)
        got.append(kept.cpu())              # the value columns leave the op convolved and otherwise untouched
        at += n
    err = (torch.cat(got).double() - want[:, h * d + g * d:]).abs().max().item()
    assert err < (1e-4 if dtype == "float32" else 0.1), err


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_norms_and_polynorm(device, dtype, tol):
    from vllm_distributed_amd import ops
    gen = torch.Generator().manual_seed(0)
    dt = getattr(torch, dtype)
    for width in (24, 200):
        x = torch.randn(5, width, generator=gen) * 2
        gain, gain2 = torch.tensor(1.7), torch.tensor(0.6)
        y = (torch.randn(5, width, generator=gen) * 0.3).to(dt)
        r = x.clone().to(device)
        nxt = ops.scalar_norm_residual(y.to(device), gain.to(device), r, gain2.to(device), 1e-5, dt)
        want_r = x.double() + oracle.one_gain_norm(y.double(), 1.7, 1e-5)
        assert (r.cpu().double() - want_r).abs().max() < 1e-5
        assert (nxt.cpu().double() - oracle.one_gain_norm(want_r, 0.6, 1e-5)).abs().max() < (1e-5 if dtype == "float32" else 0.03)
        z = (torch.randn(5, width, generator=gen) * 1.5).to(dt)
        coef = torch.tensor([0.8, -0.5, 0.25, 0.1])
        got = ops.poly_norm(z.to(device), coef.to(device), 1e-5).cpu().double()
        assert (got - oracle.poly_act(z.double(), coef.double(), 1e-5)).abs().max() < (1e-4 if dtype == "float32" else 0.05)


# ------------------------------------------------------------------------------------------ bookkeeping
def test_kept_first_pages_stay_when_the_window_moves_on():
    from vllm_distributed_amd.engine.kv_cache_manager import KVCacheManager
    from vllm_distributed_amd.engine.request import Request
    from vllm_distributed_amd.sampling_params import SamplingParams
    kv = KVCacheManager(64, 16, 4096, enable_caching=False, sliding_window=40, keep_first=19)
    req = Request("r", list(range(600)), SamplingParams(max_tokens=1))
    assert kv.allocate_slots(req, 600) is not None
    req.num_computed_tokens = 600
    released = kv.release_out_of_window(req)
    held = kv.req_blocks["r"]
    assert held[0] is not None and held[1] is not None          # 19 kept tokens: two pages of 16
    assert held[2] is None and released == (600 - 40 - kv.WINDOW_MARGIN) // 16 - 2
    assert all(b is not None for b in held[(600 - 40 - kv.WINDOW_MARGIN) // 16:])
    kv.free(req)
    assert kv.num_free_blocks == 64


def test_forced_steps_use_the_pools_and_refuse_what_does_not_fit(tmp_path_factory, tmp_path):
    from vllm_distributed_amd.entrypoints import trace_replay
    from vllm_distributed_amd.engine.request import Request, RequestStatus
    from vllm_distributed_amd.sampling_params import SamplingParams
    path, cfg, _ = model_dir("varied", tmp_path_factory)
    args = types.SimpleNamespace(model=path, dtype="float32", out=str(tmp_path), max_tokens=128, max_seqs=2,
                                 device="cpu", block_size=16, enforce_eager=True)
    core = trace_replay.make_core(args)
    try:
        sp = SamplingParams(temperature=0.0, max_tokens=None, score_only=True, ignore_eos=True)
        kv = core.scheduler.kv
        assert kv.num_free_blocks == 8 and not kv.enable_caching
        core.add_request(Request("a", tokens_for(cfg, 40, 1), sp))
        core.add_request(Request("b", tokens_for(cfg, 64, 2), sp))
        core.add_request(Request("c", tokens_for(cfg, 5, 3), sp))
        outs, reply = core.step_forced({"a": 40, "b": 10}, {"a": [39]})
        assert not outs and reply.logits["a"].shape == (1, cfg["vocab"]) and kv.num_free_blocks == 8 - 3 - 1
        with pytest.raises(RuntimeError):
            core.scheduler.schedule_forced({"c": 5})                       # both sequence slots are taken
        with pytest.raises(ValueError):
            core.scheduler.schedule_forced({"a": 1})                       # a has no token left to run
        core.extend_request("a", [1, 2, 3])
        core.step_forced({"a": 2, "b": 54})
        assert core.scheduler.requests["a"].num_computed_tokens == 42 and kv.num_free_blocks == 8 - 3 - 4
        core.finish_requests(["b"], RequestStatus.FINISHED_ABORTED)
        assert kv.num_free_blocks == 8 - 3
        _, reply = core.step_forced({"c": 5, "a": 1}, {"c": [4]})           # c takes b's slot and pages
        assert reply.logits["c"].shape == (1, cfg["vocab"])
        rows = core.executor.driver.worker.model_runner.batch.row_of
        assert set(rows) == {"a", "c"} and set(rows.values()) == {0, 1}
    finally:
        core.shutdown()


def test_the_trace_runner_as_a_program(tmp_path_factory, tmp_path):
    """``bin/trace_run`` itself: steps on standard input, one ``done <step>`` per step (also where nothing is
    wanted), logits files only for steps that want some, exit code 0 at the end of the input."""
    import subprocess
    import sys
    path, cfg, w = model_dir("degenerate", tmp_path_factory)
    a, b = tokens_for(cfg, 9, 50), tokens_for(cfg, 5, 51)
    lines = [{"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [0, 5]}, {"id": "b", "tokens": b[:2], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "b", "tokens": b[2:], "want": []}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[6:], "want": [2]}], "end": ["a"]}]
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
    r = subprocess.run([sys.executable, exe, "--model", path, "--dtype", "float32", "--out", str(tmp_path), "--max-tokens", "128",
                        "--device", "cpu"], input="".join(json.dumps(x) + "\n" for x in lines), text=True,
                       capture_output=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert sorted(f for f in os.listdir(tmp_path) if f.endswith(".f32")) == ["0.f32", "2.f32"]
    want = oracle_logits("degenerate", cfg, w, a)
    got0 = np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, cfg["vocab"])
    got2 = np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(1, cfg["vocab"])
    assert np.abs(got0 - want[[0, 5]]).max() < 2e-4 and np.abs(got2 - want[[8]]).max() < 2e-4


# ------------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("device,dtype", [pytest.param("cpu", "float32", id="cpu-f32"),
                                          pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
                                          pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_scheduler(device, dtype, tmp_path_factory):
    """``LLM.generate`` on five prompts with two sequence slots and small prefill chunks: the scheduler's own batching,
    chunking and sampling.  Every generated token is the oracle's argmax given the tokens before it (in bfloat16: or
    its logit is within rounding of the oracle's best)."""
    from vllm_distributed_amd import LLM, SamplingParams
    path, cfg, w = model_dir("varied", tmp_path_factory)
    prompts = [tokens_for(cfg, n, 40 + n) for n in (3, 30, 1, 17, 45)]
    llm = LLM(model=path, device=device, dtype=dtype, max_model_len=128, max_num_seqs=2, max_num_batched_tokens=16,
              block_size=16, load_format="safetensors", enforce_eager=False)
    try:
        outs = llm.generate(prompts, SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True))
    finally:
        llm.shutdown()
    for prompt, o in zip(prompts, outs):
        gen = list(o.outputs[0].token_ids)
        assert len(gen) == 24
        logits = oracle.forward(cfg, w, prompt + gen).numpy()
        for i, tok in enumerate(gen):
            row = logits[len(prompt) + i - 1]
            if dtype == "float32":
                assert tok == int(row.argmax()), (len(prompt), i)
            else:
                assert row.max() - row[tok] < 0.3, (len(prompt), i, float(row.max() - row[tok]))
                if row.max() - row[tok] > 0:              # a near-tie went the other way: later tokens follow another text
                    break


def test_dummy_weights_and_config_keys():
    from vllm_distributed_amd.config import ModelConfig
    from vllm_distributed_amd.models.loader import hf_weight_shapes
    mc = ModelConfig(model="tavulix-tiny", dtype="float32", load_format="dummy")
    assert mc.architecture == "TavulixForCausalLM" and mc.hidden_size == 192 and mc.vocab_size == 512
    assert mc.max_model_len == 1024 and mc.num_hidden_layers == 3
    shapes = hf_weight_shapes(mc)
    assert shapes["l0.mix.q"] == (6 * 32, 192) and shapes["l1.mix.v.conv"] == (16, 2) and "l1.mlp.up" not in shapes
    assert "l0.mix.vmix" not in shapes and shapes["l2.mix.vmix"] == ()
