"""Kabapel: a decoder-only model that alternates two kinds of sequence mixers around an fp32 residual stream.

``x = embed[token] * scale``; per layer ``x <- x + mixer(LN1(x))`` and, when the layer has a feed-forward,
``x <- x + ff(LN2(x))`` with layer norms that carry weight and bias; a final layer norm and the head give fp32 logits.
``config.json`` lists the layers one by one (``layers[i] = {type, mixer{...}, mlp{...} | null}``), so order, heads and
sizes differ from layer to layer and from model to model.

Mixers
  * ``lightning`` - ``layers.linear_attention.DecayLinearAttention``: q, k, v = SiLU of one fused projection
    ``[q | k | v | g]``, a recurrence ``S <- decay[h] S + k v^T``, ``o = S^T q`` per head with the fp32 state kept per
    request; the heads side by side go through one RMS norm, times ``sigmoid(g)``, into the output projection.
  * ``latent_attention`` - ``layers.attention.RowLatentAttention``: causal softmax attention whose keys and values
    are expanded from one cached latent row per token, ``[RMS-normed c (kv_rank) | rotated shared key part
    (rot_dim)]``.  The per-head expansions ``W_uk`` / ``W_uv`` are folded into the query and the output
    (``q_lat = W_uk^T q_unrotated``, ``out = W_uv o_lat``), so every head attends over the shared rows.  Rotation
    with YaRN-blended frequencies computed from the configuration.  A layer with ``kv_from: j`` has no
    down-projection: it reads the rows layer ``j`` cached, with its own queries and expansions.

Feed-forwards
  * ``dense`` - ``down(relu(up(h))^2)``.
  * ``moe`` - ``layers.moe.GroupedIdentityMoE``: clamped-GLU experts, softmax router with a choice-only correction,
    expert groups, identity experts, a gated shared expert.

Tensor and pipeline parallelism are not implemented for this family (the norms reduce over whole rows and the recurrent
state is not sharded).
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Tuple

import torch
import torch.nn as nn

from .. import ops
from ..config import VllmConfig
from ..parallel.state import get_pp_group, get_tensor_model_parallel_world_size
from .layers.attention import Attention, ResidualLayerNorm, RowLatentAttention, rotary_frequencies
from .layers.linear import ColumnParallelLinear, RowParallelLinear, VocabParallelEmbedding
from .layers.linear_attention import DecayLinearAttention
from .layers.moe import GroupedIdentityMoE
from .utils import IntermediateTensors, materialize

GLU_ALPHA = 1.702


def _f32(*shape: int) -> nn.Parameter:
    return nn.Parameter(torch.zeros(shape, dtype=torch.float32), requires_grad=False)


class LightningMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, layer_idx: int, dtype: torch.dtype):
        super().__init__()
        self.heads, self.dim, self.vdim = int(m["heads"]), int(m["dim"]), int(m.get("vdim") or m["dim"])
        qs, vs = self.heads * self.dim, self.heads * self.vdim
        self.gate_offset, self.eps, self.dtype = 2 * qs + vs, eps, dtype
        self.proj = ColumnParallelLinear(width, [qs, qs, vs, vs], False, dtype)
        self.attn = DecayLinearAttention(self.heads, self.dim, self.vdim, m["decay"], layer_idx)
        self.norm = _f32(vs)
        self.o = RowParallelLinear(vs, width, False, dtype)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        x = self.proj(h)
        o = self.attn(x)
        return self.o(ops.gated_rms_norm(o, self.norm, x[:, self.gate_offset:], self.eps, self.dtype))


class LatentMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, layer_idx: int, dtype: torch.dtype,
                 source: Optional["LatentMixer"]):
        super().__init__()
        self.heads, self.nope, self.rope = int(m["heads"]), int(m["dim"]), int(m["rot_dim"])
        self.vdim, self.rank = int(m.get("vdim") or m["dim"]), int(m["kv_rank"])
        self.eps, self.dtype = eps, dtype
        rot = m.get("rot") or {}
        dims = int(rot.get("dims") or self.rope)
        if dims > self.rope or dims % 2:
            raise ValueError(f"layer {layer_idx}: {dims} rotated dimensions in a part of {self.rope}")
        freq, self.rot_scale = rotary_frequencies(dims, float(rot.get("base", 10000.0)), rot.get("scaling"))
        self.register_buffer("inv_freq", freq, persistent=False)
        if source is not None and not torch.equal(source.inv_freq.cpu(), freq.cpu()):
            raise ValueError(f"layer {layer_idx} reads the rows of layer {source.attn.layer_idx}, which are rotated otherwise")
        qd = self.heads * (self.nope + self.rope)
        self.own_rows = source is None
        self.proj = ColumnParallelLinear(width, [qd, self.rank + self.rope] if self.own_rows else [qd], False, dtype)
        self.q_cols = qd
        self.dkv_norm = _f32(self.rank) if self.own_rows else None
        self.uk = nn.Parameter(torch.empty(self.heads * self.nope, self.rank, dtype=dtype), requires_grad=False)
        self.uv = nn.Parameter(torch.empty(self.heads * self.vdim, self.rank, dtype=dtype), requires_grad=False)
        self.attn = RowLatentAttention(self.heads, self.rank, self.rope, float(m["scale"]), layer_idx,
                                       source=None if source is None else source.attn, dtype=dtype)
        self.o = RowParallelLinear(self.heads * self.vdim, width, False, dtype)
        self._folded = None

    def _folded_weights(self):
        """``uk`` as ``[H, nope, rank]`` (multiplied into the query) and ``uv`` as ``[H, rank, vdim]`` (applied to
        the attention output)."""
        if self._folded is None:
            self._folded = (self.uk.data.view(self.heads, self.nope, self.rank),
                            self.uv.data.view(self.heads, self.vdim, self.rank).transpose(1, 2).contiguous())
        return self._folded

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        t = h.shape[0]
        x = self.proj(h)
        q = x[:, :self.q_cols].view(t, self.heads, self.nope + self.rope)
        latent = x[:, self.q_cols:] if self.own_rows else None
        w_uk, w_uv_t = self._folded_weights()
        q_lat = torch.bmm(q[..., :self.nope].transpose(0, 1), w_uk)                    # [H, T, rank]
        o_lat = self.attn.forward_latent(q, self.nope, q_lat, latent, self.dkv_norm, self.eps, self.inv_freq,
                                         self.rot_scale)
        o = torch.bmm(o_lat.transpose(0, 1), w_uv_t).transpose(0, 1).reshape(t, self.heads * self.vdim)
        return self.o(o)


class SquaredReluMLP(nn.Module):
    def __init__(self, width: int, ff: int, dtype: torch.dtype):
        super().__init__()
        self.up = ColumnParallelLinear(width, [ff], False, dtype)
        self.down = RowParallelLinear(ff, width, False, dtype)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(ops.relu_squared(self.up(h)))


def _make_mlp(width: int, mlp: dict, layer_idx: int, dtype: torch.dtype) -> nn.Module:
    kind = mlp.get("kind", "dense")
    if kind == "dense":
        return SquaredReluMLP(width, int(mlp["ff"]), dtype)
    if kind != "moe":
        raise ValueError(f"layer {layer_idx}: unknown feed-forward kind {kind!r}")
    r, e, s = mlp["router"], mlp["expert"], mlp.get("shared")
    g = r.get("groups") or {}
    return GroupedIdentityMoE(width, int(e["ff"]), int(r["experts"]), int(r.get("identity") or 0), int(r["top"]),
                              float(e["limit"]), dtype, groups=int(g.get("count") or 1),
                              keep_groups=int(g.get("keep") or g.get("count") or 1), alpha=GLU_ALPHA,
                              shared_inter=int(s["ff"]) if s else 0,
                              shared_limit=float(s["limit"]) if s else None)


class KabapelLayer(nn.Module):
    def __init__(self, width: int, spec: dict, eps: float, layer_idx: int, dtype: torch.dtype,
                 earlier: List["KabapelLayer"]):
        super().__init__()
        self.norm1 = ResidualLayerNorm(width, eps, dtype)
        kind, m = spec.get("type"), spec["mixer"]
        if kind == "lightning":
            self.mix = LightningMixer(width, m, eps, layer_idx, dtype)
        elif kind == "latent_attention":
            source = None
            if m.get("kv_from") is not None:
                j = int(m["kv_from"])
                if not 0 <= j < layer_idx or not isinstance(earlier[j].mix, LatentMixer) or not earlier[j].mix.own_rows:
                    raise ValueError(f"layer {layer_idx}: kv_from {j} names no earlier layer with latent rows of its own")
                source = earlier[j].mix
            self.mix = LatentMixer(width, m, eps, layer_idx, dtype, source)
        else:
            raise ValueError(f"layer {layer_idx}: unknown mixer type {kind!r}")
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            self.norm2 = ResidualLayerNorm(width, eps, dtype)
            self.mlp = _make_mlp(width, mlp, layer_idx, dtype)

    def forward(self, x: torch.Tensor, h: torch.Tensor, then: ResidualLayerNorm) -> torch.Tensor:
        """``x``: fp32 residual stream (updated in place), ``h = norm1(x)``; returns ``then(x)`` after this layer.
        Every residual add and the norm that follows it are one launch."""
        y = self.mix(h)
        if self.mlp is None:
            return then.add(y, x)
        return then.add(self.mlp(self.norm2.add(y, x)), x)


class KabapelForCausalLM(nn.Module):
    has_request_state = True          # the recurrent layers remember a state per request: no prefix reuse
    residual_dtype = torch.float32

    def __init__(self, vllm_config: VllmConfig):
        super().__init__()
        mc = vllm_config.model_config
        cfg, dtype = mc.hf_config, mc.torch_dtype
        self.cfg, self.dtype = cfg, dtype
        if get_tensor_model_parallel_world_size() > 1 or get_pp_group().world_size > 1:
            raise NotImplementedError("Kabapel runs on one device: its norms reduce over whole rows and its recurrent "
                                      "state is not sharded")
        self.is_first = self.is_last = True
        width, eps = int(cfg["width"]), float((cfg.get("norm") or {}).get("eps", 1e-5))
        self.embed_scale = float((cfg.get("embedding") or {}).get("scale", 1.0))
        specs = cfg["layers"]
        self.start_layer, self.end_layer = 0, len(specs)
        self.embed = VocabParallelEmbedding(int(cfg["vocab"]), width, dtype)
        layers: List[KabapelLayer] = []
        for i, s in enumerate(specs):
            layers.append(KabapelLayer(width, s, eps, i, dtype, layers))
        self.layers = nn.ModuleList(layers)
        self.final_norm = ResidualLayerNorm(width, eps, dtype)
        self.head = ColumnParallelLinear(width, [int(cfg["vocab"])], False, dtype)
        self.trace_residual: Optional[List[torch.Tensor]] = None      # tests: the residual stream after every layer

    def rebind_buffers(self) -> None:
        return None

    def attention_layers(self) -> List[Attention]:
        """The layers that own cache rows (a layer that reads another's rows owns none)."""
        return [l.mix.attn for l in self.layers if isinstance(l.mix, LatentMixer) and l.mix.own_rows]

    def state_layers(self) -> List[DecayLinearAttention]:
        return [l.mix.attn for l in self.layers if isinstance(l.mix, LightningMixer)]

    def decode_capturable(self) -> bool:
        return all(l.mlp.decode_capturable(self.dtype) for l in self.layers if isinstance(l.mlp, GroupedIdentityMoE))

    def forward(self, input_ids, positions, intermediate: Optional[IntermediateTensors] = None):
        x = ops.embed_scaled(input_ids, self.embed.weight, self.embed_scale)
        n = len(self.layers)
        if not n:
            return self.final_norm(x)
        h = self.layers[0].norm1(x)
        for i, layer in enumerate(self.layers):
            h = layer(x, h, self.layers[i + 1].norm1 if i + 1 < n else self.final_norm)
            if self.trace_residual is not None:
                self.trace_residual.append(x.clone())
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return ops.linear_f32(hidden, self.head.weight)[..., :int(self.cfg["vocab"])]

    # ------------------------------------------------------------ weights
    _LIGHTNING = {"q": ("proj.weight", 0), "k": ("proj.weight", 1), "v": ("proj.weight", 2), "g": ("proj.weight", 3),
                  "norm": ("norm", None), "o": ("o.weight", None)}
    _LATENT = {"q": ("proj.weight", 0), "dkv": ("proj.weight", 1), "dkv.norm": ("dkv_norm", None),
               "uk": ("uk", None), "uv": ("uv", None), "o": ("o.weight", None)}

    def _target(self, name: str):
        """Checkpoint tensor name -> (parameter name, shard of a fused parameter)."""
        top = {"embed": "embed.weight", "final.norm": "final_norm.weight", "final.norm.b": "final_norm.bias",
               "head": "head.weight"}
        if name in top:
            return top[name], None
        if not name.startswith("l"):
            return None
        idx, _, rest = name[1:].partition(".")
        if not idx.isdigit() or int(idx) >= len(self.layers):
            return None
        layer, base = self.layers[int(idx)], f"layers.{idx}."
        norms = {"norm1": "norm1.weight", "norm1.b": "norm1.bias", "norm2": "norm2.weight", "norm2.b": "norm2.bias"}
        if rest in norms:
            return base + norms[rest], None
        kind, _, leaf = rest.partition(".")
        if kind == "mix":
            table = self._LIGHTNING if isinstance(layer.mix, LightningMixer) else self._LATENT
            if leaf not in table:
                return None
            p, shard = table[leaf]
            return base + "mix." + p, shard
        if kind != "mlp" or layer.mlp is None:
            return None
        if isinstance(layer.mlp, SquaredReluMLP):
            return (base + f"mlp.{leaf}.weight", None) if leaf in ("up", "down") else None
        flat = {"router": "gate.weight", "correction": "gate.e_score_correction_bias", "shared.down": "shared.w2",
                "shared.sg": "shared_gate.weight"}
        if leaf in flat:
            return base + "mlp." + flat[leaf], None
        if leaf in ("shared.gate", "shared.up"):
            return base + "mlp.shared.w13", ("gate", "up").index(leaf[7:])
        e, _, part = leaf.partition(".")
        if e[:1] == "e" and e[1:].isdigit() and int(e[1:]) < layer.mlp.real_experts and part in ("gate", "up", "down"):
            if part == "down":
                return base + "mlp.w2", (int(e[1:]), None)
            return base + "mlp.w13", (int(e[1:]), ("gate", "up").index(part))
        return None

    def map_weight_name(self, name: str) -> Optional[str]:
        t = self._target(name)
        return None if t is None else t[0]

    def _owns_layer(self, name: str) -> bool:
        return True

    def load_weights(self, weights: Iterable[Tuple[str, torch.Tensor]]) -> List[str]:
        params: Dict[str, nn.Parameter] = dict(self.named_parameters())
        loaded = []
        for name, w in weights:
            t = self._target(name)
            if t is None or t[0] not in params:
                continue
            p, shard = params[t[0]], t[1]
            loader = getattr(p, "weight_loader", None)
            if loader is not None:
                loader(p, w, shard)
            else:
                w = materialize(w)
                assert w.numel() == p.numel(), (name, tuple(w.shape), tuple(p.shape))
                p.data.copy_(w.reshape(p.shape))
            loaded.append(name)
        return loaded


def weight_shapes(c: dict) -> Dict[str, Tuple[int, ...]]:
    """Checkpoint tensor names and shapes of a Kabapel config (for the random-weight loader)."""
    width, vocab = int(c["width"]), int(c["vocab"])
    out: Dict[str, Tuple[int, ...]] = {"embed": (vocab, width)}
    for i, spec in enumerate(c["layers"]):
        m, p = spec["mixer"], f"l{i}."
        for n in ("norm1",) + (("norm2",) if spec.get("mlp") else ()):
            out[p + n], out[p + n + ".b"] = (width,), (width,)
        heads, dim, vdim = int(m["heads"]), int(m["dim"]), int(m.get("vdim") or m["dim"])
        if spec["type"] == "lightning":
            for n, rows in (("q", heads * dim), ("k", heads * dim), ("v", heads * vdim), ("g", heads * vdim)):
                out[p + "mix." + n] = (rows, width)
            out[p + "mix.norm"] = (heads * vdim,)
        else:
            rank, rope = int(m["kv_rank"]), int(m["rot_dim"])
            out[p + "mix.q"] = (heads * (dim + rope), width)
            if m.get("kv_from") is None:
                out[p + "mix.dkv"], out[p + "mix.dkv.norm"] = (rank + rope, width), (rank,)
            out[p + "mix.uk"], out[p + "mix.uv"] = (heads * dim, rank), (heads * vdim, rank)
        out[p + "mix.o"] = (width, heads * vdim)
        mlp = spec.get("mlp")
        if not mlp:
            continue
        if mlp.get("kind", "dense") == "dense":
            out[p + "mlp.up"], out[p + "mlp.down"] = (int(mlp["ff"]), width), (width, int(mlp["ff"]))
            continue
        r, ff = mlp["router"], int(mlp["expert"]["ff"])
        for e in range(int(r["experts"])):
            q = f"{p}mlp.e{e}."
            out[q + "gate"], out[q + "up"], out[q + "down"] = (ff, width), (ff, width), (width, ff)
        outputs = int(r["experts"]) + int(r.get("identity") or 0)
        out[p + "mlp.router"], out[p + "mlp.correction"] = (outputs, width), (outputs,)
        if mlp.get("shared"):
            sf, q = int(mlp["shared"]["ff"]), p + "mlp.shared."
            out[q + "gate"], out[q + "up"], out[q + "down"], out[q + "sg"] = (sf, width), (sf, width), (width, sf), (1, width)
    out["final.norm"], out["final.norm.b"], out["head"] = (width,), (width,), (vocab, width)
    return out


def random_weight(name: str, shape: Tuple[int, ...], gen: torch.Generator, device, dtype) -> torch.Tensor:
    """A plausible random value for a checkpoint tensor (projections that keep the variance, gains near one, small
    biases and corrections)."""
    def uni(lo: float, hi: float) -> torch.Tensor:
        return lo + (hi - lo) * torch.rand(shape, generator=gen, device=device, dtype=torch.float32)
    leaf = name.rsplit(".", 1)[-1]
    if leaf in ("norm1", "norm2", "norm") or name == "final.norm":
        w = uni(0.8, 1.2)
    elif leaf == "b":
        w = uni(-0.1, 0.1)
    elif leaf == "correction":
        w = uni(-0.05, 0.05)
    elif name == "embed":
        w = uni(-1.0, 1.0)
    else:
        s = (3.0 / shape[-1]) ** 0.5
        w = uni(-s, s)
    return w.to(dtype)
