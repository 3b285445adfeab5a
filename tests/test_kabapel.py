"""Kabapel through the framework (loader, scheduler, block and state-slot bookkeeping, model runner, kernels on the
GPU / reference ops on the CPU) against the plain float64 model of ``tests/kabapel_oracle.py``.

Every test builds its own small configuration and random weights (stored as bfloat16, so the oracle and the framework
read the same numbers).  The schedules go through ``EngineCore.step_forced`` and generation goes through
``LLM.generate``.  The CPU tests run in float32; the GPU tests run the HIP kernels in float32 (tight tolerance: an index
that is one off shows) and in bfloat16 (with routers made decisive, see ``model_dir``).
"""
import json
import os

import numpy as np
import pytest
import torch

import kabapel_oracle as oracle
from test_tavulix import portions, run_schedule, tokens_for

F64 = torch.float64


# ------------------------------------------------------------------------------------------------ models
def rot(dims, scaling=True, base=10000.0):
    r = {"base": base, "dims": dims}
    if scaling:
        r["scaling"] = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0}
    return r


def lightning(heads, dim, vdim, decay, mlp=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, rank, scale, r, mlp=None, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": r}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, identity, top, ff, limit, groups=None, shared=None):
    r = {"experts": experts, "identity": identity, "top": top}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def config(layers, width=48, vocab=97, eps=1e-5, scale=0.7):
    return {"architecture": "Kabapel", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": scale}, "layers": layers}


CONFIGS = {
    # every layer of another shape; a reader of another layer's rows; a layer without feed-forward; routing with
    # groups and identity experts beside routing without either
    "varied": config([
        lightning(3, 8, 16, [0.5, 0.9, 0.99], moe(6, 2, 3, 24, 1.5, groups=(4, 2), shared=(40, 2.0))),
        latent(3, 12, 8, 20, 24, 0.2, rot(8), dense(64)),
        latent(2, 12, 8, 8, 24, 0.3, rot(8), None, kv_from=1),
        lightning(2, 16, 8, [0.97, 0.8], moe(4, 0, 1, 32, 0.8)),
        latent(4, 8, 6, 8, 10, 0.25, rot(4, scaling=False), moe(3, 3, 2, 16, 3.0, groups=(3, 3), shared=(8, 1.0))),
        latent(1, 8, 8, 12, 24, 0.3, rot(8), dense(32), kv_from=1)]),
    # values a model can make equal or one: one head, vdim = dim, top = 1, one group, keep = count, decay 1 and tiny,
    # only identity experts chosen besides one expert, rotation over the whole part without scaling
    "degenerate": config([
        latent(1, 16, 16, 16, 16, 0.25, rot(16, scaling=False, base=100.0), moe(1, 1, 2, 16, 1.0, groups=(1, 1))),
        lightning(1, 16, 16, [1.0], dense(32)),
        lightning(2, 8, 8, [0.05, 0.999], None)], width=32, vocab=50, scale=1.0),
    # no attention layer at all (nothing cached but the state), and no recurrent layer at all
    "recurrent_only": config([lightning(2, 16, 24, [0.9, 0.95], dense(48)), lightning(4, 8, 8, [0.6, 0.7, 0.8, 0.9])], width=32),
    "attention_only": config([latent(2, 16, 8, 16, 32, 0.2, rot(8), dense(48)),
                              latent(3, 8, 8, 8, 32, 0.3, rot(8), moe(4, 2, 2, 16, 1.0, groups=(2, 1)), kv_from=0)], width=32),
    # a latent width the matrix-core kernel is built for (64 + 32): rows and V^T fragments, shared with a reader
    "fragments": config([latent(4, 16, 32, 16, 64, 0.2, rot(32), dense(64)), lightning(2, 32, 32, [0.9, 0.99], dense(48)),
                         latent(3, 8, 32, 24, 64, 0.2, rot(32), moe(4, 1, 2, 32, 1.0), kv_from=0)], width=64),
    # sizes that are multiples of nothing much: a width the grouped expert kernels do not take (the experts then run
    # one after the other, also in bfloat16 on the GPU, and decode steps are not captured)
    "odd": config([lightning(3, 20, 28, [0.6, 0.9, 0.97], moe(5, 1, 2, 12, 1.1, groups=(3, 2), shared=(20, 1.4))),
                   latent(3, 20, 12, 28, 36, 0.18, rot(12), dense(60)),
                   latent(5, 12, 12, 4, 36, 0.25, rot(12), moe(3, 0, 3, 28, 0.7), kv_from=1)], width=100, vocab=333),
    # wider, for pages of 16 tokens
    "paged": config([lightning(4, 16, 16, [0.8, 0.95, 0.99, 0.999], dense(96)),
                     latent(4, 16, 8, 16, 32, 0.2, rot(8), moe(6, 2, 2, 32, 1.0, groups=(4, 3), shared=(32, 1.0))),
                     latent(4, 16, 8, 16, 32, 0.2, rot(8), dense(64), kv_from=1)], width=64),
}


def random_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    width = cfg["width"]

    def rnd(*shape, lo=-1.0, hi=1.0):
        return lo + (hi - lo) * torch.rand(shape, generator=g)

    def proj(rows, cols, gain=1.0):
        return rnd(rows, cols) * gain * (3.0 / cols) ** 0.5

    def norm(name, n):
        w[name], w[name + ".b"] = rnd(n, lo=0.7, hi=1.4), rnd(n, lo=-0.2, hi=0.2)

    w = {"embed": rnd(cfg["vocab"], width), "head": proj(cfg["vocab"], width)}
    norm("final.norm", width)
    for i, spec in enumerate(cfg["layers"]):
        m, p = spec["mixer"], f"l{i}."
        norm(p + "norm1", width)
        heads, dim, vdim = m["heads"], m["dim"], m["vdim"]
        if spec["type"] == "lightning":
            for n, rows in (("q", heads * dim), ("k", heads * dim), ("v", heads * vdim), ("g", heads * vdim)):
                w[p + "mix." + n] = proj(rows, width, 1.5)
            w[p + "mix.norm"] = rnd(heads * vdim, lo=0.6, hi=1.4)
        else:
            w[p + "mix.q"] = proj(heads * (dim + m["rot_dim"]), width, 2.0)
            if m.get("kv_from") is None:
                w[p + "mix.dkv"] = proj(m["kv_rank"] + m["rot_dim"], width, 2.0)
                w[p + "mix.dkv.norm"] = rnd(m["kv_rank"], lo=0.6, hi=1.4)
            w[p + "mix.uk"], w[p + "mix.uv"] = proj(heads * dim, m["kv_rank"], 1.5), proj(heads * vdim, m["kv_rank"])
        w[p + "mix.o"] = proj(width, heads * vdim)
        mlp = spec["mlp"]
        if not mlp:
            continue
        norm(p + "norm2", width)
        if mlp["kind"] == "dense":
            w[p + "mlp.up"], w[p + "mlp.down"] = proj(mlp["ff"], width), proj(width, mlp["ff"])
            continue
        r, ff = mlp["router"], mlp["expert"]["ff"]
        for e in range(r["experts"]):
            q = f"{p}mlp.e{e}."
            w[q + "gate"], w[q + "up"], w[q + "down"] = proj(ff, width, 2.0), proj(ff, width, 2.0), proj(width, ff)
        n = r["experts"] + r["identity"]
        w[p + "mlp.router"], w[p + "mlp.correction"] = proj(n, width, 3.0), rnd(n, lo=-0.3, hi=0.1)
        if mlp.get("shared"):
            sf, q = mlp["shared"]["ff"], p + "mlp.shared."
            w[q + "gate"], w[q + "up"], w[q + "down"], w[q + "sg"] = proj(sf, width, 2.0), proj(sf, width, 2.0), proj(width, sf), proj(1, width)
    return {k: v.to(torch.bfloat16) for k, v in w.items()}


_MODELS = {}


def model_dir(name, tmp_path_factory, dtype="float32"):
    """The model's folder, configuration and weights.  For bfloat16 runs the routers are made decisive: their
    corrections are set two apart in a random order, so that every token chooses the same outputs (identity ones
    among them or not) whatever rounding does to the scores - the weights of the chosen still differ from token to
    token.  In bfloat16 the router's input carries the rounding of every layer before it, and a close call that falls
    the other way swaps a whole expert; the float32 runs keep the free-running routers."""
    decisive = dtype != "float32"
    if (name, decisive) not in _MODELS:
        from safetensors.torch import save_file
        cfg = CONFIGS[name]
        w = random_weights(cfg, seed=sum(map(ord, name)))
        if decisive:
            g = torch.Generator().manual_seed(11)
            for k in [k for k in w if k.endswith(".correction")]:
                w[k] = (torch.randperm(w[k].numel(), generator=g) * 2.0 - w[k].numel()).to(torch.bfloat16)
        d = tmp_path_factory.mktemp("kabapel_" + name)
        save_file({k: v.contiguous() for k, v in w.items()}, str(d / "model.safetensors"))
        (d / "config.json").write_text(json.dumps(cfg))
        _MODELS[(name, decisive)] = (str(d), cfg, w)
    return _MODELS[(name, decisive)]


_ORACLE = {}


def oracle_logits(name, cfg, w, tokens):
    key = (name, id(w), tuple(tokens))
    if key not in _ORACLE:
        _ORACLE[key] = oracle.forward(cfg, w, list(tokens)).numpy()
    return _ORACLE[key]


def check(got, name, cfg, w, reqs, tol, dtype=None):
    """Every row the run produced against the oracle."""
    assert got
    for (rid, p), row in got.items():
        err = np.abs(row - oracle_logits(name, cfg, w, reqs[rid])[p]).max()
        assert err <= tol, (rid, p, float(err))


CLOSE_CALL = 0.06      # (the expert block alone, bfloat16: routing choices made by less than this are left out)


DEVICES = [pytest.param("cpu", "float32", 2e-4, id="cpu-f32"),
           pytest.param("cuda", "float32", 2e-4, id="gpu-f32", marks=pytest.mark.gpu),
           pytest.param("cuda", "bfloat16", 0.35, id="gpu-bf16", marks=pytest.mark.gpu)]


# ------------------------------------------------------------------------------------------------ schedules
@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_and_first_tokens(name, device, dtype, tol, tmp_path_factory, tmp_path):
    path, cfg, w = model_dir(name, tmp_path_factory, dtype)
    reqs = {"a": tokens_for(cfg, 90, 1), "b": tokens_for(cfg, 1, 2), "c": tokens_for(cfg, 2, 3)}
    steps = [[(r, t, list(range(len(t)))), {"end": [r]}] for r, t in reqs.items()]
    got = run_schedule(path, steps, dtype, device, max_tokens=128, tmp=tmp_path)
    assert len(got) == 93
    check(got, name, cfg, w, reqs, tol, dtype)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_residual_stream_after_every_layer(device, dtype, tol, tmp_path_factory):
    """The fp32 residual stream after each layer against the oracle's (float32 only: layer by layer, tightly)."""
    if dtype != "float32":
        pytest.skip("the per-layer comparison is the float32 one")
    from vllm_distributed_amd.entrypoints import trace_replay
    import types
    path, cfg, w = model_dir("varied", tmp_path_factory, dtype)
    toks = tokens_for(cfg, 37, 8)
    args = types.SimpleNamespace(model=path, dtype=dtype, out="", max_tokens=64, max_seqs=2, device=device,
                                 block_size=16, enforce_eager=True)
    core = trace_replay.make_core(args)
    try:
        from vllm_distributed_amd.engine.request import Request
        from vllm_distributed_amd.sampling_params import SamplingParams
        model = core.executor.driver.worker.model_runner.model
        model.trace_residual = []
        core.add_request(Request("r", toks, SamplingParams(temperature=0.0, max_tokens=None, score_only=True, ignore_eos=True)))
        core.step_forced({"r": len(toks)}, {})
        got = [t.cpu().double() for t in model.trace_residual]
    finally:
        core.shutdown()
    want = []
    oracle.forward(cfg, w, toks, want)
    assert len(got) == len(want) == len(cfg["layers"])
    for i, (a, b) in enumerate(zip(got, want)):
        assert (a - b).abs().max().item() <= 1e-4 * max(1.0, b.abs().max().item()), i


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("name", ["varied", "paged", "recurrent_only", "fragments", "odd"])
def test_prefill_then_long_token_by_token_decoding(name, device, dtype, tol, tmp_path_factory, tmp_path):
    """A prompt, then 150 tokens one at a time: the state is carried through 150 single-row steps, the cache grows
    over several pages."""
    path, cfg, w = model_dir(name, tmp_path_factory, dtype)
    toks = tokens_for(cfg, 190, 4)
    got = run_schedule(path, portions(toks, [40, 1], "r"), dtype, device, max_tokens=192, tmp=tmp_path)
    assert len(got) == 190
    check(got, name, cfg, w, {"r": toks}, tol, dtype)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [("float32", 2e-4), ("bfloat16", 0.35)])
@pytest.mark.parametrize("name", ["varied", "fragments"])
def test_pages_of_64_tokens(name, dtype, tol, tmp_path_factory, tmp_path):
    """The page size a GPU engine uses by default: two requests in turn, portions that end inside, at and just
    behind a page's border, then single rows across the next border."""
    path, cfg, w = model_dir(name, tmp_path_factory, dtype)
    a, b = tokens_for(cfg, 150, 60), tokens_for(cfg, 70, 61)
    steps = [[("a", a[:63], [0, 62])], [("a", a[63:64], [0]), ("b", b[:64], [63])], [("a", a[64:66], [0, 1]), ("b", b[64:65], [0])],
             [("a", a[66:127], [60]), ("b", b[65:70], [4]), {"end": ["b"]}]]
    steps += [[("a", a[i:i + 1], [0])] for i in range(127, 150)]
    steps[-1].append({"end": ["a"]})
    got = run_schedule(path, steps, dtype, "cuda", max_tokens=256, block_size=64, tmp=tmp_path)
    assert len(got) == 2 + 1 + 1 + 2 + 1 + 1 + 1 + 23
    check(got, name, cfg, w, {"a": a, "b": b}, tol)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
@pytest.mark.parametrize("sizes", [[2], [3, 2, 7, 1, 16, 17, 2, 2, 31, 5], [1], [64, 2, 1]])
def test_portions_of_any_size(sizes, device, dtype, tol, tmp_path_factory, tmp_path):
    path, cfg, w = model_dir("varied", tmp_path_factory, dtype)
    toks = tokens_for(cfg, 75 if sizes != [1] else 40, 5)
    got = run_schedule(path, portions(toks, sizes, "r"), dtype, device, max_tokens=128, tmp=tmp_path)
    assert len(got) == len(toks)
    check(got, "varied", cfg, w, {"r": toks}, tol, dtype)


@pytest.mark.parametrize("eager", [False, True])
@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_mixed_batches_reuse_pages_and_slots(device, dtype, tol, eager, tmp_path_factory, tmp_path):
    """Seven unequal requests through three sequence slots and a pool of 10 pages: portions of prompts beside single
    tokens, requests that sit steps out, state slots and pages handed on as requests end (a new owner must not see
    what the old one left); every row against the request run alone by the oracle."""
    if eager and device == "cpu":
        pytest.skip("graphs exist on the GPU only")
    path, cfg, w = model_dir("paged", tmp_path_factory, dtype)
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
    check(got, "paged", cfg, w, reqs, tol, dtype)


@pytest.mark.parametrize("device,dtype,tol", DEVICES)
def test_batch_rows_equal_single_runs(device, dtype, tol, tmp_path_factory, tmp_path):
    """The same rows run alone and inside a batch of unequal neighbours agree far inside the oracle tolerance."""
    path, cfg, w = model_dir("varied", tmp_path_factory, dtype)
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
    worst = sorted(float(np.abs(alone[("a", p)] - both[("a", p)]).max()) for p in range(30))
    assert worst[-1 if dtype == "float32" else -2] <= (1e-4 if dtype == "float32" else 0.2), worst[-3:]


# --------------------------------------------------------------------------- mechanisms alone, made to show
OP_DEVICES = [pytest.param("cpu", "float32", id="cpu-f32"),
              pytest.param("cuda", "float32", id="gpu-f32", marks=pytest.mark.gpu),
              pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)]


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
def test_a_far_token_reaches_through_the_recurrence_and_stale_slots_do_not(device, dtype):
    """One head remembers (decay 0.995), one forgets (0.5).  Token 0 writes a large key / value pair, the query 300
    tokens later asks for it: the remembering head returns ``0.995^300`` of it, the forgetting head nothing.  The
    sequence runs in portions of many sizes through a slot that another sequence has used."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    heads, dim, vdim, n = 2, 8, 8, 301
    g = torch.Generator().manual_seed(3)
    q = torch.randn(n, heads, dim, generator=g) * 0.05
    k = torch.randn(n, heads, dim, generator=g) * 0.05
    v = torch.randn(n, heads, vdim, generator=g) * 0.05
    k[0, :, 0], v[0, :, 1], q[n - 1, :, 0] = 6.0, 5.0, 2.0
    x = torch.cat([q.reshape(n, -1), k.reshape(n, -1), v.reshape(n, -1)], 1).to(dt)
    decay = torch.tensor([0.995, 0.5])
    xf = x.double()
    want, _ = oracle.decayed_heads(xf[:, :16].view(n, heads, dim), xf[:, 16:32].view(n, heads, dim),
                                   xf[:, 32:].view(n, heads, vdim), [float(d) for d in decay])
    assert abs(float(want[n - 1, 0, 1]) - 60 * 0.995 ** 300) < 0.5 and abs(float(want[n - 1, 1, 1])) < 0.1
    state = torch.full((3, heads, dim, vdim), 7.0, device=device)                  # what an earlier owner left
    out, at, sizes = [], 0, [1, 2, 64, 17, 1, 1, 100, 3, 2]
    for i in range(100):
        m = min(sizes[i % len(sizes)], n - at)
        if m == 0:
            break
        i32 = dict(dtype=torch.int32, device=device)
        out.append(ops.decay_linear_attention(x[at:at + m].to(device), heads, dim, vdim, decay.to(device), state,
                                              torch.tensor([2], **i32), torch.tensor([0, m], **i32),
                                              torch.tensor([at + m], **i32), False).cpu())
        at += m
    got = torch.cat(out).view(n, heads, vdim).double()
    assert (got - want).abs().max().item() < 2e-4 * 60


@pytest.mark.parametrize("device,dtype", OP_DEVICES)
def test_one_key_stands_out_far_back_and_at_page_borders(device, dtype):
    """Latent rows in shuffled pages of 16; the query is aimed at ONE key: the output is that row's latent part, for
    keys far back among hundreds, on both sides of page borders, the first and the newest key; a key one past the
    row's own position is not seen."""
    from vllm_distributed_amd import ops
    dt = getattr(torch, dtype)
    n, rank, rope, bs, heads = 330, 16, 8, 16, 2
    g = torch.Generator().manual_seed(9)
    nblk = -(-n // bs) + 2
    table = torch.randperm(nblk, generator=g)[:-(-n // bs)].to(torch.int32).view(1, -1)
    rows = torch.randn(n, rank + rope, generator=g) * 0.3
    cache = torch.zeros(nblk, 1, bs, rank + rope)
    for j in range(n):
        cache[table[0, j // bs], 0, j % bs] = rows[j]
    cache, table_d = cache.to(dt).to(device), table.to(device)
    stored = cache.cpu().float()
    for target in (0, 7, 15, 16, 17, 31, 32, 200, 319, 320, 329):
        for pos, seen in ((n - 1, True), (target, True), (target - 1, False)):
            if pos < 0:
                continue
            key = stored[table[0, target // bs], 0, target % bs]
            q = (key * 60 / key.norm() ** 2).view(1, 1, -1).repeat(1, heads, 1).to(dt).to(device)
            i32 = dict(dtype=torch.int32, device=device)
            for token_seq in (None, torch.tensor([0], **i32)):                     # a decoded row / a prompt's row
                o = ops.latent_row_attention(q, cache, table_d, token_seq, torch.tensor([pos + 1], **i32), 1.0, rank)
                hit = (o[0, 0].float().cpu() - key[:rank]).abs().max().item() < 0.05
                assert hit == seen, (target, pos)


@pytest.mark.parametrize("device", [pytest.param("cpu", id="cpu"), pytest.param("cuda", id="gpu", marks=pytest.mark.gpu)])
def test_routing_rules(device):
    """Choice by score + correction, weights without it; a group outside the kept ones is out even when every choice
    score inside the kept groups is negative; identity outputs are chosen like experts; weights sum to one."""
    from vllm_distributed_amd.models.layers.moe import GroupedIdentityMoE
    with torch.device(device):
        m = GroupedIdentityMoE(32, 16, 5, 3, 3, 1.0, torch.float32, groups=4, keep_groups=2)
    corr = torch.tensor([-2.0, -2.1, -2.2, -2.3, 0.5, -9.0, -2.4, -2.5], device=device)
    m.gate.e_score_correction_bias.data.copy_(corr)
    g = torch.Generator().manual_seed(1)
    z = (torch.randn(64, 8, generator=g) * 2).to(device)
    topw, topi = m.route(z)
    idx, wts = oracle.route(z.cpu().double(), corr.cpu(), 3, 4, 2)
    assert torch.equal(topi.cpu().sort(-1).values, idx.sort(-1).values)
    order = topi.cpu().argsort(-1)
    assert (topw.cpu().gather(1, order).double() - wts.gather(1, idx.argsort(-1))).abs().max().item() < 1e-6
    assert (topw.sum(-1) - 1).abs().max().item() < 1e-5
    # group 2 = outputs (4, 5) always wins a place through output 4's correction; output 5 then beats every
    # output of a group that was not kept, although its choice score is about -9
    assert (topi == 4).any(-1).all() and (topi >= 5).any()
    if device == "cuda":
        from vllm_distributed_amd import ops
        w2, i2 = ops.moe_topk_grouped(z, corr, 3, 4, 2, False, False, True, 1.0)
        assert torch.equal(i2.long().sort(-1).values.cpu(), idx.sort(-1).values)
        assert (w2.cpu().gather(1, i2.long().cpu().argsort(-1)).double() - wts.gather(1, idx.argsort(-1))).abs().max().item() < 1e-5


@pytest.mark.parametrize("hidden", [40, 48])
@pytest.mark.parametrize("device,dtype", OP_DEVICES)
def test_expert_block_against_the_oracle(device, dtype, hidden):
    """The whole block - router, clamped experts with inputs beyond the limit, identity share, gated shared expert -
    on sizes that are no multiple of anything."""
    from vllm_distributed_amd.models.layers.moe import GroupedIdentityMoE
    dt = getattr(torch, dtype)
    ff, experts, identity, top = 24, 5, 1, 3
    mlp = {"expert": {"ff": ff, "limit": 0.6}, "router": {"experts": experts, "identity": identity, "top": top,
                                                         "groups": {"count": 3, "keep": 2}}, "shared": {"ff": 16, "limit": 0.9}}
    g = torch.Generator().manual_seed(2)
    w = {"router": torch.randn(6, hidden, generator=g) * 0.5, "correction": torch.randn(6, generator=g) * 0.2,
         "shared.gate": torch.randn(16, hidden, generator=g) * 0.4, "shared.up": torch.randn(16, hidden, generator=g) * 0.4,
         "shared.down": torch.randn(hidden, 16, generator=g) * 0.3, "shared.sg": torch.randn(1, hidden, generator=g) * 0.3}
    for e in range(experts):
        w[f"e{e}.gate"], w[f"e{e}.up"] = torch.randn(ff, hidden, generator=g) * 0.4, torch.randn(ff, hidden, generator=g) * 0.4
        w[f"e{e}.down"] = torch.randn(hidden, ff, generator=g) * 0.3
    w = {k: v.to(torch.bfloat16) for k, v in w.items()}
    with torch.device(device):
        m = GroupedIdentityMoE(hidden, ff, experts, identity, top, 0.6, dt, groups=3, keep_groups=2, shared_inter=16,
                               shared_limit=0.9)
    m.gate.weight.data.copy_(w["router"])
    m.gate.e_score_correction_bias.data.copy_(w["correction"])
    for e in range(experts):
        m.w13.weight_loader(m.w13, w[f"e{e}.gate"], (e, 0))
        m.w13.weight_loader(m.w13, w[f"e{e}.up"], (e, 1))
        m.w2.weight_loader(m.w2, w[f"e{e}.down"], (e, None))
    m.shared.w13.weight_loader(m.shared.w13, w["shared.gate"], 0)
    m.shared.w13.weight_loader(m.shared.w13, w["shared.up"], 1)
    m.shared.w2.data.copy_(w["shared.down"])
    m.shared_gate.weight.data.copy_(w["shared.sg"])
    x = (torch.randn(50, hidden, generator=g) * 1.5).to(dt)
    margins = []
    want = oracle.moe(x.double(), {"p." + k: v for k, v in w.items()}, "p.", mlp, margins)
    got = m(x.to(device)).cpu().double()
    err = (got - want).abs().max(-1).values
    if dtype != "float32":
        err = err[margins[0] >= CLOSE_CALL]
        assert len(err) > 20
    assert err.max().item() <= (1e-4 if dtype == "float32" else 0.08), err.max().item()


def test_rotary_frequencies_and_partial_rotation():
    from vllm_distributed_amd.models.layers.attention import rotary_frequencies
    from vllm_distributed_amd.ops import torch_ref
    for r in (rot(8), rot(16, scaling=False, base=1e6), {"base": 5e5, "dims": 32, "scaling": {"factor": 8.0, "original": 128, "fast": 32.0, "slow": 2.0}}):
        f, s = rotary_frequencies(r["dims"], r["base"], r.get("scaling"))
        wf, ws = oracle.rotary_frequencies(r)
        assert (f.double() - wf).abs().max().item() < 1e-7 and abs(s - ws) < 1e-12
    # rotation over the first 4 of 6 values: the last two pass unchanged
    r = rot(4, scaling=False)
    f, s = rotary_frequencies(4, r["base"], None)
    x = torch.randn(5, 3, 6, dtype=F64)
    pos = torch.tensor([0, 1, 7, 100, 1000])
    got = torch_ref.rotate_half_first(x.float(), pos, f, s).double()
    want = oracle.rotate(x, pos, r)
    assert (got - want).abs().max().item() < 1e-5 and torch.equal(got[..., 4:], x.float().double()[..., 4:])


def test_norms_and_activations_against_the_oracle():
    from vllm_distributed_amd.ops import torch_ref
    g = torch.Generator().manual_seed(4)
    x = torch.randn(6, 40, generator=g) * 3 + 1
    w, b = torch.rand(40, generator=g) + 0.5, torch.randn(40, generator=g) * 0.2
    assert (torch_ref.layer_norm_to(x, w, b, 1e-5, torch.float32).double() - oracle.layer_norm(x.double(), w, b, 1e-5)).abs().max() < 1e-5
    gate = torch.randn(6, 40, generator=g)
    want = oracle.unit_rms(x.double(), 1e-5) * w.double() * oracle.sigmoid(gate.double())
    assert (torch_ref.gated_rms_norm(x, w, gate, 1e-5, torch.float32).double() - want).abs().max() < 1e-5
    h = torch.randn(6, 32, generator=g) * 3                                       # well beyond the limit on both sides
    gg, uu = h[:, :16].double().clamp(max=1.2), h[:, 16:].double().clamp(-1.2, 1.2)
    assert (torch_ref.clamped_glu(h, 1.2, 1.702).double() - gg * oracle.sigmoid(1.702 * gg) * (uu + 1)).abs().max() < 1e-5


# ------------------------------------------------------------------------------------------- bookkeeping
def test_rows_are_shared_and_state_is_fp32(tmp_path_factory):
    """A reader of another layer's rows owns no cache; the recurrent layers' state tensors are fp32 with one spare
    slot; only owners are counted in what a cached token costs."""
    from vllm_distributed_amd.entrypoints import trace_replay
    import types
    path, cfg, w = model_dir("varied", tmp_path_factory)
    args = types.SimpleNamespace(model=path, dtype="bfloat16", out="", max_tokens=64, max_seqs=3, device="cpu",
                                 block_size=16, enforce_eager=True)
    core = trace_replay.make_core(args)
    try:
        mr = core.executor.driver.worker.model_runner
        model = mr.model
        owners = model.attention_layers()
        assert [a.layer_idx for a in owners] == [1, 4]
        assert model.layers[2].mix.attn.rows is model.layers[1].mix.attn.k_cache
        assert model.layers[5].mix.attn.rows is model.layers[1].mix.attn.k_cache
        assert model.layers[2].mix.attn.k_cache is None
        spec = mr.get_kv_cache_spec()
        assert spec.bytes_per_token == ((24 + 8) + (10 + 6)) * 2
        assert [tuple(s.shape) for s in mr.state_tensors] == [(4, 3, 8, 16), (4, 2, 16, 8)]
        assert all(s.dtype == torch.float32 for s in mr.state_tensors)
        assert spec.state_bytes_per_request == (3 * 8 * 16 + 2 * 16 * 8) * 4
    finally:
        core.shutdown()


def test_config_errors():
    from vllm_distributed_amd.models.kabapel import KabapelLayer
    f32 = torch.float32
    with pytest.raises(ValueError):                                               # reads its own rows
        KabapelLayer(48, latent(2, 8, 8, 8, 16, 0.3, rot(8), None, kv_from=0), 1e-5, 0, f32, [])
    first = KabapelLayer(48, latent(2, 8, 8, 8, 16, 0.3, rot(8)), 1e-5, 0, f32, [])
    reader = KabapelLayer(48, latent(3, 4, 8, 8, 16, 0.3, rot(8), kv_from=0), 1e-5, 1, f32, [first])
    assert reader.mix.attn.source is first.mix.attn
    with pytest.raises(ValueError):                                               # rows of another rank
        KabapelLayer(48, latent(2, 8, 8, 8, 24, 0.3, rot(8), kv_from=0), 1e-5, 1, f32, [first])
    with pytest.raises(ValueError):                                               # rows rotated otherwise
        KabapelLayer(48, latent(2, 8, 8, 8, 16, 0.3, rot(8, scaling=False), kv_from=0), 1e-5, 1, f32, [first])
    with pytest.raises(ValueError):                                               # a reader is no source
        KabapelLayer(48, latent(2, 8, 8, 8, 16, 0.3, rot(8), kv_from=1), 1e-5, 2, f32, [first, reader])
    with pytest.raises(ValueError):
        KabapelLayer(48, {"type": "convolution", "mixer": {}, "mlp": None}, 1e-5, 0, f32, [])


def test_dummy_weights_and_config_keys():
    from vllm_distributed_amd.config import ModelConfig
    from vllm_distributed_amd.models.loader import hf_weight_shapes
    mc = ModelConfig(model="kabapel-tiny", dtype="float32", load_format="dummy")
    assert mc.architecture == "KabapelForCausalLM" and mc.hidden_size == 192 and mc.vocab_size == 512
    assert mc.num_hidden_layers == 3
    shapes = hf_weight_shapes(mc)
    assert shapes["l0.mix.g"] == (4 * 48, 192) and shapes["l1.mix.dkv"] == (48 + 16, 192)
    assert "l2.mix.dkv" not in shapes and "l2.norm2" not in shapes and shapes["l1.mlp.router"] == (8, 192)
    assert shapes["l1.mlp.e5.down"] == (192, 96) and "l1.mlp.e6.down" not in shapes and shapes["l1.mlp.shared.sg"] == (1, 192)


def test_the_trace_runner_as_a_program(tmp_path_factory, tmp_path):
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
    want = oracle_logits("degenerate", cfg, w, a)
    got0 = np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, cfg["vocab"])
    got2 = np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(1, cfg["vocab"])
    assert np.abs(got0 - want[[0, 5]]).max() < 2e-4 and np.abs(got2 - want[[8]]).max() < 2e-4


# ------------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("device,dtype", OP_DEVICES)
def test_greedy_generation_through_the_scheduler(device, dtype, tmp_path_factory):
    """``LLM.generate`` on five prompts with two sequence slots and small prefill chunks: the scheduler's own batching,
    chunking and sampling.  Every generated token is the oracle's argmax given the tokens before it (in bfloat16: or
    its logit is within rounding of the oracle's best)."""
    from vllm_distributed_amd import LLM, SamplingParams
    path, cfg, w = model_dir("varied", tmp_path_factory, dtype)
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
