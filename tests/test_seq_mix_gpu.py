"""HIP kernels of ``csrc/seq_mix.hip`` against the plain PyTorch fp32 form of the same op (``ops/torch_ref.py``)."""
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
@pytest.mark.parametrize("h", [24, 192, 1000, 4096])
def test_scalar_norms(dtype, h):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(h)
    x = torch.randn(7, h, device="cuda", generator=g) * 3
    gain = torch.tensor(1.3, device="cuda")
    got = hip.scalar_rms_norm(x, gain, 1e-5, dtype)
    _close(got, torch_ref.scalar_rms_norm(x, gain, 1e-5, dtype), dtype, 4)
    y = (torch.randn(7, h, device="cuda", generator=g) * 0.2).to(dtype)
    r1, r2 = x.clone(), x.clone()
    g2 = torch.tensor(0.7, device="cuda")
    o1 = hip.scalar_norm_residual(y, gain, r1, g2, 1e-5, dtype)
    o2 = torch_ref.scalar_norm_residual(y, gain, r2, g2, 1e-5, dtype)
    _close(r1, r2, torch.float32, 10)
    _close(o1, o2, dtype, 4)
    assert hip.scalar_norm_residual(y, gain, r1, None, 1e-5, dtype) is None
    torch_ref.scalar_norm_residual(y, gain, r2, None, 1e-5, dtype)
    _close(r1, r2, torch.float32, 10)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("f", [40, 384, 5000])
def test_poly_norm(dtype, f):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(f)
    z = (torch.randn(5, f, device="cuda", generator=g) * 1.5).to(dtype)
    coef = torch.tensor([0.8, -0.4, 0.3, 0.1], device="cuda")
    _close(hip.poly_norm(z, coef, 1e-5), torch_ref.poly_norm(z, coef, 1e-5), dtype, 8)


def _conv_case(dtype, h, g, d, dv, taps, chunks, seed, nblocks=64):
    """Sequences given as (tokens already run, tokens in this step); rows in batch order."""
    gen = torch.Generator(device="cuda").manual_seed(seed)
    c = h * d + g * (d + dv)
    bs = 16
    b = len(chunks)
    n_rows = sum(n for _, n in chunks)
    x = torch.randn(n_rows, c + (8 if seed % 2 else h), device="cuda", generator=gen).to(dtype)
    w = torch.randn(taps, c, device="cuda", generator=gen).to(dtype)
    state = torch.randn(b + 2, max(taps - 1, 1), c, device="cuda", generator=gen).to(dtype)
    slots = torch.randperm(b + 2, device="cuda", generator=gen)[:b].to(torch.int32)
    qsl = torch.tensor([0] + list(torch.tensor([n for _, n in chunks]).cumsum(0)), dtype=torch.int32, device="cuda")
    seq_lens = torch.tensor([a + n for a, n in chunks], dtype=torch.int32, device="cuda")
    pos = torch.cat([torch.arange(a, a + n) for a, n in chunks]).to(torch.int32).cuda()
    tok_seq = torch.cat([torch.full((n,), i) for i, (_, n) in enumerate(chunks)]).to(torch.int32).cuda()
    table = torch.randperm(nblocks, device="cuda", generator=gen).to(torch.int32).view(b, -1)
    slot_map = torch.stack([table[s, p // bs] * bs + p % bs for s, p in zip(tok_seq.tolist(), pos.tolist())]).to(torch.int32)
    kc = torch.zeros(nblocks, g, bs, d, device="cuda", dtype=dtype)
    vc = torch.zeros(nblocks, g, bs // 8, dv, 8, device="cuda", dtype=dtype)
    qn = torch.rand(d, device="cuda", generator=gen) + 0.5
    kn = torch.rand(d, device="cuda", generator=gen) + 0.5
    vf = torch.randn(n_rows, g * dv, device="cuda", generator=gen)
    lam = torch.tensor(0.3, device="cuda")
    return dict(x=x, w=w, state=state, slots=slots, qsl=qsl, seq_lens=seq_lens, pos=pos, tok_seq=tok_seq, kc=kc, vc=vc,
                slot_map=slot_map, qn=qn, kn=kn, vf=vf, lam=lam, table=table)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(4, 2, 32, 16, 3), (6, 3, 64, 48, 4), (2, 1, 24, 8, 2), (3, 3, 128, 128, 1),
                                   (2, 2, 72, 40, 5), (2, 1, 20, 12, 3), (3, 1, 7, 5, 9)])
@pytest.mark.parametrize("mix", [False, True])
def test_conv_norm_cache(dtype, shape, mix):
    hip = _hip()
    h, g, d, dv, taps = shape
    # fresh prompts (one shorter than the taps), continuations of 1, 2 and many rows, a decode row at position 1
    chunks = [(0, 1), (0, 9), (1, 1), (5, 2), (17, 1), (3, 30), (0, 2), (40, 1)]
    c = _conv_case(dtype, h, g, d, dv, taps, chunks, seed=sum(shape))
    s1, s2 = c["state"].clone(), c["state"].clone()
    k1, v1, k2, v2 = c["kc"].clone(), c["vc"].clone(), c["kc"].clone(), c["vc"].clone()
    args = (h, g, d, dv, c["qn"], c["kn"], 1e-5, c["vf"] if mix else None, c["lam"] if mix else None, not mix)
    q1, kept1 = hip.conv_norm_cache(c["x"], c["w"], s1, c["slots"], c["qsl"], c["seq_lens"], c["tok_seq"], c["pos"],
                                    *args, k1, v1, c["slot_map"], True)
    q2, kept2 = torch_ref.conv_norm_cache(c["x"], c["w"], s2, c["slots"], c["qsl"], c["seq_lens"], *args, k2, v2,
                                          c["slot_map"])
    _close(q1, q2, dtype, 4)
    _close(k1, k2, dtype, 4)
    _close(v1, v2, dtype, 8)
    for i, (a, n) in enumerate(chunks):                  # copies of the inputs: exact (rows that lie before the
        first = max(0, (taps - 1) - (a + n))             # sequence's start are never read, whatever they hold)
        slot = int(c["slots"][i])
        if taps > 1:
            _close(s1[slot, first:], s2[slot, first:], dtype, 1e-6)
    if not mix:
        _close(kept1, kept2, torch.float32, 400 if dtype != torch.float32 else 10)


def test_conv_decode_rows_own_their_state():
    """A pure decode batch (no row map): every row moves its own slot on."""
    hip = _hip()
    dtype, (h, g, d, dv, taps) = torch.bfloat16, (4, 2, 32, 16, 4)
    chunks = [(7, 1), (0, 1), (2, 1), (130, 1)]
    c = _conv_case(dtype, h, g, d, dv, taps, chunks, seed=5)
    s1, s2 = c["state"].clone(), c["state"].clone()
    k1, v1, k2, v2 = c["kc"].clone(), c["vc"].clone(), c["kc"].clone(), c["vc"].clone()
    args = (h, g, d, dv, c["qn"], c["kn"], 1e-5, None, None, False)
    q1, _ = hip.conv_norm_cache(c["x"], c["w"], s1, c["slots"], c["qsl"], c["seq_lens"], None, c["pos"], *args, k1, v1,
                                c["slot_map"], False)
    q2, _ = torch_ref.conv_norm_cache(c["x"], c["w"], s2, c["slots"], c["qsl"], c["seq_lens"], *args, k2, v2, c["slot_map"])
    _close(q1, q2, dtype, 4)
    _close(s1[c["slots"].long()], s2[c["slots"].long()], dtype, 1e-6)
    _close(k1, k2, dtype, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [(12, 3, 64, 32), (6, 3, 32, 48), (4, 1, 16, 16), (4, 4, 128, 128), (2, 2, 72, 8),
                                   (40, 2, 64, 64), (2, 2, 20, 12), (3, 1, 7, 5)])
@pytest.mark.parametrize("window,keep", [(0, 0), (20, 0), (20, 3), (200, 7), (1, 2), (40, 70)])
@pytest.mark.parametrize("mfma", [True, False])
def test_window_bias_attention(dtype, shape, window, keep, mfma, monkeypatch):
    hip = _hip()
    if not mfma and dtype != torch.bfloat16:
        pytest.skip("the plain kernel is the only one for fp32")
    monkeypatch.setattr(hip, "WINDOW_ATTENTION_MFMA", mfma)
    h, g, d, dv = shape
    gen = torch.Generator(device="cuda").manual_seed(h * 131 + window)
    bs, nblocks = 16, 40
    chunks = [(0, 1), (0, 70), (33, 1), (60, 12), (149, 1), (5, 2)]
    b = len(chunks)
    n_rows = sum(n for _, n in chunks)
    kc = torch.randn(nblocks, g, bs, d, device="cuda", generator=gen).to(dtype)
    vc = torch.randn(nblocks, g, bs // 8, dv, 8, device="cuda", generator=gen).to(dtype)
    q = torch.randn(n_rows, h, d, device="cuda", generator=gen).to(dtype)
    gate = torch.randn(n_rows, h + 5, device="cuda", generator=gen).to(dtype)[:, 5:]
    table = torch.randint(0, nblocks, (b, 10), device="cuda", generator=gen, dtype=torch.int32)
    qsl = torch.tensor([0] + list(torch.tensor([n for _, n in chunks]).cumsum(0)), dtype=torch.int32, device="cuda")
    seq_lens = torch.tensor([a + n for a, n in chunks], dtype=torch.int32, device="cuda")
    pos = torch.cat([torch.arange(a, a + n) for a, n in chunks]).to(torch.int32).cuda()
    tok_seq = torch.cat([torch.full((n,), i) for i, (_, n) in enumerate(chunks)]).to(torch.int32).cuda()
    r1 = torch.rand(h, device="cuda", generator=gen)
    r2 = torch.rand(h, device="cuda", generator=gen)
    sink = torch.randn(h, device="cuda", generator=gen)
    for use_bias, use_sink, use_gate, cap in ((True, True, True, 7.0), (False, False, False, 0.0)):
        got = hip.window_bias_attention(q, kc, vc, table, qsl, seq_lens, tok_seq, pos, 0.2, cap, window, keep,
                                        r1 if use_bias else None, r2 if use_bias else None,
                                        sink if use_sink else None, gate if use_gate else None, 70)
        want = torch_ref.window_bias_attention(q, kc, vc, table, qsl, seq_lens, 0.2, cap, window, keep,
                                               r1 if use_bias else None, r2 if use_bias else None,
                                               sink if use_sink else None, gate if use_gate else None)
        _close(got, want, dtype, 4)


@pytest.mark.parametrize("shape", [(12, 3, 64, 32), (4, 4, 128, 128), (40, 2, 64, 64), (6, 3, 32, 16), (16, 1, 256, 128)])
@pytest.mark.parametrize("window,keep", [(0, 0), (33, 5), (700, 40)])
def test_window_bias_attention_decode_rows(shape, window, keep):
    """One row per sequence (no row map, the waves of a block share the keys), contexts from 1 to 900 keys."""
    hip = _hip()
    h, g, d, dv = shape
    dtype = torch.bfloat16
    gen = torch.Generator(device="cuda").manual_seed(h + window)
    bs, nblocks = 16, 80
    lens = [1, 2, 31, 32, 33, 64, 257, 900]
    b = len(lens)
    kc = torch.randn(nblocks, g, bs, d, device="cuda", generator=gen).to(dtype)
    vc = torch.randn(nblocks, g, bs // 8, dv, 8, device="cuda", generator=gen).to(dtype)
    q = torch.randn(b, h, d, device="cuda", generator=gen).to(dtype)
    gate = torch.randn(b, h, device="cuda", generator=gen).to(dtype)
    table = torch.randint(0, nblocks, (b, 60), device="cuda", generator=gen, dtype=torch.int32)
    qsl = torch.arange(b + 1, dtype=torch.int32, device="cuda")
    seq_lens = torch.tensor(lens, dtype=torch.int32, device="cuda")
    pos = seq_lens - 1
    r1 = torch.rand(h, device="cuda", generator=gen)
    r2 = torch.rand(h, device="cuda", generator=gen)
    sink = torch.randn(h, device="cuda", generator=gen)
    got = hip.window_bias_attention(q, kc, vc, table, qsl, seq_lens, None, pos, 0.2, 9.0, window, keep, r1, r2, sink, gate, 1)
    want = torch_ref.window_bias_attention(q, kc, vc, table, qsl, seq_lens, 0.2, 9.0, window, keep, r1, r2, sink, gate)
    _close(got, want, dtype, 4)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("h", [8, 37, 256])
def test_embed_positions(dtype, h):
    hip = _hip()
    g = torch.Generator(device="cuda").manual_seed(h)
    emb = torch.randn(50, h, device="cuda", generator=g).to(dtype)
    pos = torch.randn(30, h, device="cuda", generator=g).to(dtype)
    ids = torch.randint(0, 50, (40,), device="cuda", generator=g, dtype=torch.int32)
    ps = torch.randint(0, 30, (40,), device="cuda", generator=g, dtype=torch.int32)
    got = hip.embed_positions(ids, ps, emb, pos)
    assert got.dtype == torch.float32
    assert torch.equal(got, emb[ids.long()].float() + pos[ps.long()].float())


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_conv_norm_cache_long_chunks(dtype):
    """Thousands of rows in one launch (a wave then takes several consecutive rows), chunk borders inside a wave's
    rows, a decode row and a two-row chunk between the long ones."""
    hip = _hip()
    h, g, d, dv, taps = 4, 2, 64, 32, 4
    chunks = [(0, 2999), (5, 1501), (7, 1), (0, 2), (100, 700)]
    c = _conv_case(dtype, h, g, d, dv, taps, chunks, seed=11, nblocks=5 * 200)
    s1, s2 = c["state"].clone(), c["state"].clone()
    k1, v1, k2, v2 = c["kc"].clone(), c["vc"].clone(), c["kc"].clone(), c["vc"].clone()
    args = (h, g, d, dv, c["qn"], c["kn"], 1e-5, c["vf"], c["lam"], False)
    q1, _ = hip.conv_norm_cache(c["x"], c["w"], s1, c["slots"], c["qsl"], c["seq_lens"], c["tok_seq"], c["pos"], *args,
                                k1, v1, c["slot_map"], True)
    q2, _ = torch_ref.conv_norm_cache(c["x"], c["w"], s2, c["slots"], c["qsl"], c["seq_lens"], *args, k2, v2, c["slot_map"])
    _close(q1, q2, dtype, 4)
    _close(k1, k2, dtype, 4)
    _close(v1, v2, dtype, 8)
    for i, (a, n) in enumerate(chunks):
        first = max(0, (taps - 1) - (a + n))
        _close(s1[int(c["slots"][i]), first:], s2[int(c["slots"][i]), first:], dtype, 1e-6)
