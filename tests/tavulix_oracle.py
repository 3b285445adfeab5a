"""A plain, slow Tavulix in float64: one function per mechanism, written from the model's equations and sharing no
code with the package.  Notation: ``T`` tokens, ``W`` width, ``H`` query heads, ``G`` key/value heads, ``D`` / ``Dv``
key / value sizes, ``p`` absolute position."""
import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def one_gain_norm(x, gain, eps):
    return unit_rms(x, eps) * gain


def causal_taps(u, w):
    """``u[T, C]``, ``w[C, K]``: ``y[t] = sum_j w[:, j] * u[t - (K - 1) + j]``, rows before 0 are zero."""
    t_len, k = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for t in range(t_len):
        for j in range(k):
            src = t - (k - 1) + j
            if src >= 0:
                y[t] += w[:, j] * u[src]
    return y


def visible(i, j, size, keep_first):
    return j <= i and (i - j < size or j < keep_first)


def attend(q, k, v, scale, cap, r1, r2, sink, size, keep_first):
    """``q[T, H, D]``, ``k[T, G, D]``, ``v[T, G, Dv]`` of one sequence from position 0 -> ``[T, H, Dv]``."""
    t_len, h, _ = q.shape
    g = k.shape[1]
    out = torch.zeros(t_len, h, v.shape[2], dtype=F64)
    for i in range(t_len):
        for a in range(h):
            kv = a // (h // g)
            js = [j for j in range(i + 1) if visible(i, j, size, keep_first)]
            s = torch.stack([(q[i, a] * k[j, kv]).sum() * scale for j in js])
            if cap:
                s = cap * torch.tanh(s / cap)
            dist = torch.tensor([float(i - j) for j in js], dtype=F64)
            s = s - r1[a] * torch.log(1.0 + r2[a] * dist)
            top = max(float(s.max()), float(sink[a]))
            e = torch.exp(s - top)
            den = e.sum() + math.exp(float(sink[a]) - top)
            for n, j in enumerate(js):
                out[i, a] += e[n] / den * v[j, kv]
    return out


def poly_act(z, coef, eps):
    return coef[0] * unit_rms(z, eps) + coef[1] * unit_rms(z ** 2, eps) + coef[2] * unit_rms(z ** 3, eps) + coef[3]


def forward(cfg, w, tokens, residuals=None):
    """Logits ``[T, vocab]`` of one sequence; ``w``: checkpoint name -> tensor."""
    g = lambda name: w[name].to(F64)                                    # noqa: E731
    eps = cfg["norm"]["eps"]
    n = len(tokens)
    x = g("embed")[torch.tensor(tokens)] + g("pos")[:n]
    v_first = None
    for li, spec in enumerate(cfg["layers"]):
        p, m = f"l{li}.", spec["mixer"]
        h = one_gain_norm(x, g(p + "norm1"), eps)
        hq, hk, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        q = causal_taps(h @ g(p + "mix.q").T, g(p + "mix.q.conv")).view(n, hq, d)
        k = causal_taps(h @ g(p + "mix.k").T, g(p + "mix.k.conv")).view(n, hk, d)
        v = causal_taps(h @ g(p + "mix.v").T, g(p + "mix.v.conv")).view(n, hk, dv)
        q = unit_rms(q, eps) * g(p + "mix.q.norm")
        k = unit_rms(k, eps) * g(p + "mix.k.norm")
        if m.get("v_mix"):
            if v_first is None:
                v_first = v
            else:
                lam = g(p + "mix.vmix")
                v = (1 - lam) * v + lam * v_first
        o = attend(q, k, v, m["scale"], m.get("softcap"), g(p + "mix.r1"), g(p + "mix.r2"), g(p + "mix.sink"),
                   m["mask"]["size"], m["mask"]["keep_first"])
        o = o * torch.sigmoid(h @ g(p + "mix.g").T).unsqueeze(-1)
        x = x + one_gain_norm(o.reshape(n, hq * dv) @ g(p + "mix.o").T, g(p + "norm1b"), eps)
        if spec.get("mlp"):
            h = one_gain_norm(x, g(p + "norm2"), eps)
            y = poly_act(h @ g(p + "mlp.up").T, g(p + "mlp.act"), eps) @ g(p + "mlp.down").T
            x = x + one_gain_norm(y, g(p + "norm2b"), eps)
        if residuals is not None:
            residuals.append(x.clone())
    logits = one_gain_norm(x, g("final.norm"), eps) @ g("head").T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
