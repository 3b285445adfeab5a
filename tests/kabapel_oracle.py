"""Kabapel in float64, written from the equations: one function per mechanism, loops over positions where the model
is a recurrence, whole ``[T, T]`` score matrices where it is attention.  Shares no code with the package; the tests
compare the framework against it.

Weights: a dict of tensors under the checkpoint's names (any float type; used as float64).
"""
import math

import torch

F64 = torch.float64


def f64(t):
    return t.to(F64)


def layer_norm(x, w, b, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * f64(w) + f64(b)


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x / (1 + torch.exp(-x))


def sigmoid(x):
    return 1 / (1 + torch.exp(-x))


# ------------------------------------------------------------------------------------------------ lightning mixer
def decayed_heads(q, k, v, decay, state=None):
    """``q, k [T, H, dk]``, ``v [T, H, dv]``: the recurrence token by token.  Returns (o ``[T, H, dv]``, final state)."""
    t, h, dk = q.shape
    dv = v.shape[2]
    o = torch.zeros(t, h, dv, dtype=F64)
    s = torch.zeros(h, dk, dv, dtype=F64) if state is None else state.clone()
    for i in range(t):
        for hh in range(h):
            s[hh] = decay[hh] * s[hh] + torch.outer(k[i, hh], v[i, hh])
            o[i, hh] = s[hh].T @ q[i, hh]
    return o, s


def lightning_mixer(h, w, p, m, eps):
    t = h.shape[0]
    heads, dk, dv = m["heads"], m["dim"], m.get("vdim") or m["dim"]
    q = silu(h @ f64(w[p + "q"]).T).view(t, heads, dk)
    k = silu(h @ f64(w[p + "k"]).T).view(t, heads, dk)
    v = silu(h @ f64(w[p + "v"]).T).view(t, heads, dv)
    # decays as the 32-bit numbers the recurrence multiplies by
    decay = [float(torch.tensor(d, dtype=torch.float32)) for d in m["decay"]]
    o, _ = decayed_heads(q, k, v, decay)
    o = unit_rms(o.reshape(t, heads * dv), eps) * f64(w[p + "norm"])
    return (o * sigmoid(h @ f64(w[p + "g"]).T)) @ f64(w[p + "o"]).T


# ------------------------------------------------------------------------------------------------ latent attention
def rotary_frequencies(rot):
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2 * i / dims)
    mult = 1.0
    sc = rot.get("scaling")
    if sc:
        def index(turns):
            return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
        lo = max(math.floor(index(sc["fast"])), 0)
        hi = min(math.ceil(index(sc["slow"])), dims - 1)
        ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0, 1)
        f = f / sc["factor"] * ramp + f * (1 - ramp)
        mult = 0.1 * math.log(sc["factor"]) + 1
    return f, mult


def rotate(x, positions, rot):
    """``x [T, ..., n]``: the first ``rot.dims`` values of the last axis rotated, pairs half of that apart."""
    f, mult = rotary_frequencies(rot)
    half = rot["dims"] // 2
    # the 32-bit frequencies and angles of the definition
    f32 = f.to(torch.float32)
    a = (positions.to(torch.float32).view(-1, *([1] * (x.dim() - 1))) * f32).to(F64)
    c, s = torch.cos(a) * mult, torch.sin(a) * mult
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half:]], -1)


def latent_rows(h, w, p, m, eps, positions):
    """The latent ``c [T, kv_rank]`` and the rotated shared key part ``[T, rot_dim]`` of a layer with a ``dkv``."""
    r = m["kv_rank"]
    y = h @ f64(w[p + "dkv"]).T
    return unit_rms(y[:, :r], eps) * f64(w[p + "dkv.norm"]), rotate(y[:, r:], positions, m["rot"])


def latent_mixer(h, w, p, m, rows, positions):
    """``rows``: (c, rotated key part) of this layer or of the layer ``kv_from`` names."""
    t = h.shape[0]
    heads, dn, dr, dv = m["heads"], m["dim"], m["rot_dim"], m.get("vdim") or m["dim"]
    c, kr = rows
    q = (h @ f64(w[p + "q"]).T).view(t, heads, dn + dr)
    qn, qr = q[..., :dn], rotate(q[..., dn:], positions, m["rot"])
    kn = (c @ f64(w[p + "uk"]).T).view(t, heads, dn)
    v = (c @ f64(w[p + "uv"]).T).view(t, heads, dv)
    out = torch.zeros(t, heads, dv, dtype=F64)
    for hh in range(heads):
        s = (qn[:, hh] @ kn[:, hh].T + qr[:, hh] @ kr.T) * m["scale"]
        s = s.masked_fill(torch.triu(torch.ones(t, t, dtype=torch.bool), 1), -math.inf)
        out[:, hh] = torch.softmax(s, -1) @ v[:, hh]
    return out.reshape(t, heads * dv) @ f64(w[p + "o"]).T


# ------------------------------------------------------------------------------------------------ feed-forwards
def glu_expert(h, w, p, limit, alpha=1.702):
    g = torch.clamp(h @ f64(w[p + "gate"]).T, max=limit)
    u = torch.clamp(h @ f64(w[p + "up"]).T, -limit, limit)
    return (g * sigmoid(alpha * g) * (u + 1)) @ f64(w[p + "down"]).T


def route(z, correction, top, groups, keep, margins=None):
    """Router logits ``z [T, n]`` -> (chosen outputs ``[T, top]``, their weights).  ``margins`` (a list) receives, per
    token, by how much the choice was made: the gap between the last chosen and the first rejected choice score, and
    between the last kept and the first dropped group."""
    n = z.shape[1]
    s = torch.softmax(z, -1)
    choice = s + f64(correction)
    margin = torch.full((z.shape[0],), math.inf, dtype=F64)
    if groups > 1 and keep < groups:
        size = n // groups
        for t in range(z.shape[0]):
            score = [float(choice[t, g * size:(g + 1) * size].max()) for g in range(groups)]
            best = sorted(range(groups), key=lambda g: -score[g])
            margin[t] = score[best[keep - 1]] - score[best[keep]]
            for g in best[keep:]:
                choice[t, g * size:(g + 1) * size] = -math.inf
    ranked = torch.sort(choice, -1, descending=True).values
    if top < n:
        margin = torch.minimum(margin, ranked[:, top - 1] - ranked[:, top])
    if margins is not None:
        margins.append(margin)
    idx = torch.topk(choice, top, -1).indices
    wts = s.gather(1, idx)
    return idx, wts / (wts.sum(-1, keepdim=True) + 1e-20)


def moe(h, w, p, mlp, margins=None):
    r = mlp["router"]
    experts, top = r["experts"], r["top"]
    g = r.get("groups") or {}
    idx, wts = route(h @ f64(w[p + "router"]).T, w[p + "correction"], top, g.get("count", 1),
                     g.get("keep", g.get("count", 1)), margins)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            y = h[t] if e >= experts else glu_expert(h[t:t + 1], w, f"{p}e{e}.", mlp["expert"]["limit"])[0]
            out[t] += wts[t, j] * y
    if mlp.get("shared"):
        out = out + sigmoid(h @ f64(w[p + "shared.sg"]).T) * glu_expert(h, w, p + "shared.", mlp["shared"]["limit"])
    return out


def dense(h, w, p):
    return (torch.relu(h @ f64(w[p + "up"]).T) ** 2) @ f64(w[p + "down"]).T


# ------------------------------------------------------------------------------------------------ the model
def forward(cfg, w, tokens, residuals=None, margins=None):
    """Logits ``[T, vocab]`` of one sequence from position 0; ``residuals`` (a list) collects the stream after every
    layer, ``margins`` (a list) one tensor per routed layer: see ``route``."""
    eps = cfg["norm"]["eps"]
    positions = torch.arange(len(tokens))
    x = f64(w["embed"])[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    rows = {}
    for i, spec in enumerate(cfg["layers"]):
        p, m = f"l{i}.", spec["mixer"]
        h = layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps)
        if spec["type"] == "lightning":
            x = x + lightning_mixer(h, w, p + "mix.", m, eps)
        else:
            if m.get("kv_from") is None:
                rows[i] = latent_rows(h, w, p + "mix.", m, eps, positions)
            x = x + latent_mixer(h, w, p + "mix.", m, rows[i if m.get("kv_from") is None else m["kv_from"]], positions)
        if spec.get("mlp"):
            h = layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps)
            x = x + (dense(h, w, p + "mlp.") if spec["mlp"].get("kind", "dense") == "dense" else moe(h, w, p + "mlp.", spec["mlp"], margins))
        if residuals is not None:
            residuals.append(x.clone())
    return layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ f64(w["head"]).T
