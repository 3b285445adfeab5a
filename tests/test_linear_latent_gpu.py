"""HIP kernels of ``csrc/linear_latent.hip`` against the plain PyTorch fp32 form of the same op (``ops/torch_ref.py``)."""
import pytest
import torch

pytestmark = pytest.mark.gpu

from vllm_distributed_amd.ops import torch_ref  # noqa: E402


def _hip():
    from vllm_distributed_amd.ops import hip
    hip.load()
    return hip


def _close(a, b, dtype, scale=1.0):
    tol = 3e-5 if dtype == torch.float32 else 1.2e-2
    err = (a.float() - b.float()).abs().max().item()
    assert err <= tol * scale, err


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("h", [24, 384, 1000, 4096])
def test_embed_and_layer_norms(dtype, h):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(h)
    emb = torch.randn(50, h, device="cuda", generator=g).to(dtype)
    ids = torch.tensor([3, 49, 0, 17, 3], dtype=torch.int32, device="cuda")
    _close(hip.embed_scaled(ids, emb, 0.37), torch_ref.embed_scaled(ids, emb, 0.37), torch.float32)
    x = torch.randn(7, h, device="cuda", generator=g) * 3 + 0.5
    w = torch.rand(h, device="cuda", generator=g) + 0.5
    b = torch.randn(h, device="cuda", generator=g) * 0.1
    _close(hip.layer_norm_to(x, w, b, 1e-5, dtype), torch_ref.layer_norm_to(x, w, b, 1e-5, dtype), dtype, 4)
    _close(hip.layer_norm_to(x, w, None, 1e-5, dtype), torch_ref.layer_norm_to(x, w, None, 1e-5, dtype), dtype, 4)
    wide = torch.randn(7, h + 8, device="cuda", generator=g).to(dtype)
    y = wide[:, :h]                                                   # a strided view, as a fused projection gives
    r1, r2 = x.clone(), x.clone()
    o1 = hip.add_layer_norm(y, r1, w, b, 1e-5, dtype)
    o2 = torch_ref.add_layer_norm(y, r2, w, b, 1e-5, dtype)
    _close(r1, r2, torch.float32, 4)
    _close(o1, o2, dtype, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("n", [24, 384, 2050])
def test_gated_norm_and_activations(dtype, n):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(n)
    o = torch.randn(5, n, device="cuda", generator=g) * 2
    w = torch.rand(n, device="cuda", generator=g) + 0.5
    wide = torch.randn(5, 3 * n, device="cuda", generator=g).to(dtype)
    gate = wide[:, 2 * n:]
    _close(hip.gated_rms_norm(o, w, gate, 1e-5, dtype), torch_ref.gated_rms_norm(o, w, gate, 1e-5, dtype), dtype, 4)
    h = (torch.randn(6, 2 * n, device="cuda", generator=g) * 2).to(dtype)
    _close(hip.clamped_glu(h, 1.25, 1.702), torch_ref.clamped_glu(h, 1.25, 1.702), dtype, 4)
    want = torch.relu(h.float()).square()
    _close(hip.relu_squared(h), want, dtype, max(1.0, want.max().item()))          # (one rounding step of the largest)


def _linear_case(dtype, heads, dim, vdim, chunks, seed, silu=True):
    """Sequences as (tokens already run, tokens in this step); slots handed out in reverse so none is its index."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    n_rows = sum(n for _, n in chunks)
    c = heads * (2 * dim + vdim)
    x = (torch.randn(n_rows, c + heads * vdim, device="cuda", generator=gen) * 0.8).to(dtype)
    b = len(chunks)
    slots = torch.tensor([b - i for i in range(b)], dtype=torch.int32, device="cuda")
    state = torch.randn(b + 2, heads, dim, vdim, device="cuda", generator=gen)          # stale contents everywhere
    decay = torch.rand(heads, device="cuda", generator=gen) * 0.5 + 0.5
    ends, acc = [0], 0
    for _, n in chunks:
        acc += n
        ends.append(acc)
    qsl = torch.tensor(ends, dtype=torch.int32, device="cuda")
    lens = torch.tensor([a + n for a, n in chunks], dtype=torch.int32, device="cuda")
    return x, decay, state, slots, qsl, lens


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("heads,dim,vdim", [(3, 8, 16), (5, 64, 48), (2, 128, 128), (2, 40, 72), (1, 200, 130)])
def test_decay_linear_attention(dtype, heads, dim, vdim):
    hip = _hip()
    chunks = [(0, 1), (5, 1), (0, 37), (64, 2), (3, 70), (0, 0), (9, 1)]
    x, decay, state, slots, qsl, lens = _linear_case(dtype, heads, dim, vdim, chunks, seed=dim + vdim)
    s1, s2 = state.clone(), state.clone()
    got = hip.decay_linear_attention(x, heads, dim, vdim, decay, s1, slots, qsl, lens, True)
    want = torch_ref.decay_linear_attention(x, heads, dim, vdim, decay, s2, slots, qsl, lens, True)
    scale = max(1.0, want.abs().max().item())
    _close(got, want, torch.float32, 8 * scale)
    _close(s1, s2, torch.float32, 8 * max(1.0, s2.abs().max().item()))
    # a second step from the states the first left
    x2, _, _, _, qsl2, lens2 = _linear_case(dtype, heads, dim, vdim, [(a + n, 3) for a, n in chunks], seed=7)
    got = hip.decay_linear_attention(x2, heads, dim, vdim, decay, s1, slots, qsl2, lens2, False)
    want = torch_ref.decay_linear_attention(x2, heads, dim, vdim, decay, s2, slots, qsl2, lens2, False)
    _close(got, want, torch.float32, 8 * max(1.0, want.abs().max().item()))


def _latent_case(dtype, heads, rank, rope, half, lens_new, seed, bs=16):
    """``lens_new``: (tokens already cached, tokens in this step) per sequence; blocks handed out scattered."""
    from vllm_distributed_amd.models.layers.attention import rotary_frequencies
    gen = torch.Generator(device="cuda").manual_seed(seed)
    dk = rank + rope
    nope = 12
    b = len(lens_new)
    total = [a + n for a, n in lens_new]
    nblk = [-(-t // bs) for t in total]
    perm = torch.randperm(sum(nblk) + 3, generator=torch.Generator().manual_seed(seed)).tolist()
    table = torch.zeros(b, max(nblk), dtype=torch.int32)
    k = 0
    for i, nb in enumerate(nblk):
        for j in range(nb):
            table[i, j] = perm[k]
            k += 1
    cache = (torch.randn(sum(nblk) + 3, 1, bs, dk, device="cuda", generator=gen) * 0.5).to(dtype)
    rows, pos, slot = [], [], []
    for i, (a, n) in enumerate(lens_new):
        for p in range(a, a + n):
            rows.append(i)
            pos.append(p)
            slot.append(int(table[i, p // bs]) * bs + p % bs)
    t = len(rows)
    freq, rs = rotary_frequencies(2 * half, 10000.0, {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0})
    dev = dict(device="cuda")
    return dict(q=(torch.randn(t, heads, nope + rope, generator=gen, **dev)).to(dtype), nope=nope,
                q_lat=(torch.randn(heads, t, rank, generator=gen, **dev) * 0.3).to(dtype),
                latent=torch.randn(t, dk + 4, generator=gen, **dev).to(dtype)[:, :dk],
                norm_w=torch.rand(rank, generator=gen, **dev) + 0.5, freq=freq.cuda(), rs=rs,
                pos=torch.tensor(pos, dtype=torch.int32, **dev), slot=torch.tensor(slot, dtype=torch.int32, **dev),
                rows=torch.tensor(rows, dtype=torch.int32, **dev), cache=cache, table=table.cuda(),
                lens=torch.tensor([p + 1 for p in pos], dtype=torch.int32, **dev))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("heads,rank,rope,half", [(3, 24, 8, 4), (7, 48, 16, 8), (5, 20, 6, 2), (16, 512, 64, 32), (2, 130, 10, 5)])
def test_latent_prep_and_attention(dtype, heads, rank, rope, half):
    hip = _hip()
    c = _latent_case(dtype, heads, rank, rope, half, [(0, 1), (40, 1), (0, 33), (17, 20), (63, 2)], seed=rank + rope)
    c1, c2 = c["cache"].clone(), c["cache"].clone()
    q1 = hip.latent_prep(c["q"], c["nope"], c["q_lat"], c["latent"], c["norm_w"], 1e-5, c["freq"], c["rs"], c["pos"], c1, c["slot"])
    q2 = torch_ref.latent_prep(c["q"], c["nope"], c["q_lat"], c["latent"], c["norm_w"], 1e-5, c["freq"], c["rs"], c["pos"], c2, c["slot"])
    _close(q1, q2, dtype, 8)
    _close(c1, c2, dtype, 8)
    # a reader of another layer's rows: query only, cache untouched
    q3 = hip.latent_prep(c["q"], c["nope"], c["q_lat"], None, None, 1e-5, c["freq"], c["rs"], c["pos"], None, None)
    _close(q3, q2, dtype, 8)
    o1 = hip.latent_row_attention(q2, c2, c["table"], c["rows"], c["lens"], 0.21, rank)
    o2 = torch_ref.latent_row_attention(q2, c2, c["table"], c["rows"], c["lens"], 0.21, rank)
    _close(o1, o2, dtype, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_latent_attention_decode_rows_and_one_far_key(dtype):
    """A pure decode batch (row t is sequence t) whose query is aimed at ONE key far back: the output is that row."""
    hip = _hip()
    heads, rank, rope = 4, 32, 8
    c = _latent_case(dtype, heads, rank, rope, 4, [(300, 1), (0, 1), (129, 1)], seed=5)
    cache, table = c["cache"], c["table"]
    lens = torch.tensor([301, 1, 130], dtype=torch.int32, device="cuda")
    q = torch.zeros(3, heads, rank + rope, device="cuda", dtype=dtype)
    far = 7
    key = cache[int(table[0, far // 16]), 0, far % 16].float()
    q[0] = (key * 40).to(dtype)
    o = hip.latent_row_attention(q, cache, table, None, lens, 1.0, rank)
    ref = torch_ref.latent_row_attention(q, cache, table, None, lens, 1.0, rank)
    _close(o, ref, dtype, 4)
    assert (o[0, 0].float() - key[:rank]).abs().max().item() < 0.05
    # zero-length rows (the padding of a captured batch) give zeros
    lens0 = torch.tensor([0, 1, 0], dtype=torch.int32, device="cuda")
    o = hip.latent_row_attention(q, cache, table, None, lens0, 1.0, rank)
    assert torch.isfinite(o.float()).all() and o[0].float().abs().max().item() == 0.0


@pytest.mark.parametrize("heads,rank,rope", [(6, 64, 32), (16, 512, 64), (20, 256, 64)])
def test_fragment_cache_and_precise_matrix_core_attention(heads, rank, rope):
    """Widths the matrix-core latent kernel is built for: ``latent_prep`` also writes the V^T fragments, and the
    kernel with fp32-precise softmax weights agrees with the fp32 reference more closely than 8-bit weights could."""
    hip = _hip()
    from vllm_distributed_amd import ops
    dtype = torch.bfloat16
    c = _latent_case(dtype, heads, rank, rope, rope // 2, [(0, 1), (40, 1), (0, 33), (17, 20), (200, 4)], seed=rank)
    nb, bs = c["cache"].shape[0], c["cache"].shape[2]
    k1, k2 = c["cache"].clone(), c["cache"].clone()
    v1 = torch.zeros(ops.v_cache_shape(nb, 1, rank, bs), dtype=dtype, device="cuda")
    # the fragments of what is already cached
    old = c["cache"][:, 0, :, :rank]                                            # [blocks, bs, rank]
    v1[:, 0] = old.reshape(nb, bs // 8, 8, rank // 16, 16).permute(0, 3, 1, 4, 2)
    v2 = v1.clone()
    q1 = hip.latent_prep(c["q"], c["nope"], c["q_lat"], c["latent"], c["norm_w"], 1e-5, c["freq"], c["rs"], c["pos"], k1, c["slot"], v1)
    q2 = torch_ref.latent_prep(c["q"], c["nope"], c["q_lat"], c["latent"], c["norm_w"], 1e-5, c["freq"], c["rs"], c["pos"], k2, c["slot"], v2)
    _close(q1, q2, dtype, 8)
    _close(k1, k2, dtype, 8)
    _close(v1, v2, dtype, 8)
    assert torch.equal(v2[:, 0].permute(0, 2, 4, 1, 3).reshape(nb, bs, rank), k2[:, 0, :, :rank])
    qs = (q2.float() * 3).to(dtype)                                             # peaky softmax: weights near 1 matter
    want = torch_ref.latent_row_attention(qs.float(), k2.float(), c["table"], c["rows"], c["lens"], 0.21, rank)
    fine = hip.mla_attention(qs, k2, v2, c["table"], c["rows"], c["lens"], 0.21, 256, precise=True).float()
    coarse = hip.mla_attention(qs, k2, v2, c["table"], c["rows"], c["lens"], 0.21, 256).float()
    e_fine, e_coarse = (fine - want).abs().max().item(), (coarse - want).abs().max().item()
    assert e_fine <= 6e-3 * max(1.0, want.abs().max().item()), (e_fine, e_coarse)      # (the output's own 8 bits)
    assert e_fine <= e_coarse + 1e-6
    dec = hip.mla_attention(qs[:2], k2, v2, c["table"], None, torch.tensor([1, 41], dtype=torch.int32, device="cuda"),
                            0.21, 64, precise=True).float()
    _close(dec, want[:2], dtype, 1)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("h", [40, 336, 2048])
def test_expert_epilogue(dtype, h):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(h)
    t, k = 9, 3
    routed = torch.randn(t, h, device="cuda", generator=g).to(dtype)
    x = torch.randn(t, h + 8, device="cuda", generator=g).to(dtype)[:, :h]
    shared = torch.randn(t, h, device="cuda", generator=g).to(dtype)
    gate = torch.randn(t, 1, device="cuda", generator=g).to(dtype)
    topw = torch.rand(t, k, device="cuda", generator=g)
    topi = torch.randint(0, 8, (t, k), device="cuda", generator=g).to(torch.int32)
    for args in ((topw, topi, 5, shared, gate), (None, None, 5, shared, gate), (topw, topi, 5, None, None),
                 (topw, topi, 8, shared, gate)):
        _close(hip.expert_epilogue(routed, x, *args), torch_ref.expert_epilogue(routed, x, *args), dtype, 4)
