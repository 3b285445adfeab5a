"""Tavulix: a decoder-only model with learned absolute positions, single-gain RMS norms on both sides of every
sublayer, and attention whose q / k / v pass through a short causal convolution over time.

Per layer ``x <- x + norm1b(mixer(norm1(x)))`` then, when the layer has one, ``x <- x + norm2b(ff(norm2(x)))``.
The residual stream ``x`` is fp32 in every dtype; the norms run in fp32 and hand the projections their input in the
model dtype.  The mixer is ``layers.attention.WindowBiasAttention`` behind ``layers.short_conv.ShortConv``: one fused
projection ``[q | k | v | gate]``, convolution + per-head q / k norm + value mixing + cache write in one op
(``ops.conv_norm_cache``), attention with a window that keeps the first keys, a logarithmic distance bias, a sink and
a per-head sigmoid gate, then the output projection.  Layers that mix values blend their v with the v the first such
layer computed for the same token (handed down the layer loop, never stored).  The feed-forward is ``down(PolyNorm(
up(h)))`` (``ops.poly_norm``).  Logits are capped with a tanh.

``config.json`` lists the layers one by one (``layers[i] = {type, mixer{...}, mlp{...} | null}``), so heads, sizes,
windows and the presence of a feed-forward may differ from layer to layer; ``config.normalize_hf_config`` adds the
keys the rest of the framework reads (``hidden_size`` ...).  Tensor parallelism is not implemented for this family
(PolyNorm and the single-gain norms reduce over whole rows).
"""
from __future__ import annotations

from typing import Dict, Iterable, List, Optional, Tuple

import torch
import torch.nn as nn

from .. import ops
from ..config import VllmConfig
from ..parallel.state import get_pp_group, get_tensor_model_parallel_world_size
from .layers.attention import Attention, ScalarRMSNorm, WindowBiasAttention, get_forward_context
from .layers.linear import ColumnParallelLinear, RowParallelLinear, VocabParallelEmbedding
from .layers.short_conv import ShortConv
from .utils import IntermediateTensors, materialize


def _f32(*shape: int) -> nn.Parameter:
    return nn.Parameter(torch.zeros(shape, dtype=torch.float32), requires_grad=False)


class ConvAttentionMixer(nn.Module):
    def __init__(self, width: int, m: dict, eps: float, layer_idx: int, dtype: torch.dtype):
        super().__init__()
        self.heads, self.kv_heads = int(m["heads"]), int(m.get("kv_heads") or m["heads"])
        self.dim, self.vdim = int(m["dim"]), int(m.get("vdim") or m["dim"])
        if self.heads % self.kv_heads:
            raise ValueError(f"layer {layer_idx}: {self.heads} query heads do not divide over {self.kv_heads} kv heads")
        if not m.get("conv"):
            raise ValueError(f"layer {layer_idx}: the mixer names no convolution length")
        self.eps = eps
        qs, ks, vs = self.heads * self.dim, self.kv_heads * self.dim, self.kv_heads * self.vdim
        self.channels = qs + ks + vs
        self.proj = ColumnParallelLinear(width, [qs, ks, vs, self.heads], False, dtype)
        self.conv = ShortConv([qs, ks, vs], int(m["conv"]), dtype)
        self.q_norm, self.k_norm = _f32(self.dim), _f32(self.dim)
        self.v_mix = bool(m.get("v_mix"))
        self.vmix = _f32() if self.v_mix else None
        mask = m.get("mask") or {}
        self.attn = WindowBiasAttention(self.heads, self.dim, self.vdim, self.kv_heads, float(m["scale"]), layer_idx,
                                        window=int(mask.get("size") or 0), keep_first=int(mask.get("keep_first") or 0),
                                        softcap=m.get("softcap"))
        self.o = RowParallelLinear(self.heads * self.vdim, width, False, dtype)

    def forward(self, h: torch.Tensor, v_first: Optional[torch.Tensor], provide_v: bool):
        """``h[T, W]`` normed input -> (mixer output ``[T, W]``, this layer's unmixed fp32 v if ``provide_v``)."""
        ctx = get_forward_context()
        md = ctx.attn_metadata
        x = self.proj(h)
        if md is None:                    # memory-profiling pass: no cache, no state
            o = x.new_zeros((x.shape[0], self.heads * self.vdim))
            kept = x.new_zeros((x.shape[0], self.kv_heads * self.vdim), dtype=torch.float32) if provide_v else None
            return self.o(o), kept
        rows = None if md.num_prefills == 0 else md.token_rows(ctx.positions)[0]
        q, kept = ops.conv_norm_cache(
            x, self.conv.weight_t, self.conv.state, md.state_slots, md.query_start_loc, md.seq_lens, rows, ctx.positions,
            self.heads, self.kv_heads, self.dim, self.vdim, self.q_norm, self.k_norm, self.eps,
            v_first, self.vmix if v_first is not None else None, provide_v,
            self.attn.k_cache, self.attn.v_cache, md.slot_mapping, md.num_prefills > 0)
        o = self.attn.forward_cached(q, x[:, self.channels:])
        return self.o(o), kept


class PolyNormMLP(nn.Module):
    def __init__(self, width: int, ff: int, eps: float, dtype: torch.dtype):
        super().__init__()
        self.up = ColumnParallelLinear(width, [ff], False, dtype)
        self.down = RowParallelLinear(ff, width, False, dtype)
        self.act = _f32(4)
        self.eps = eps

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.down(ops.poly_norm(self.up(h), self.act, self.eps))


class TavulixLayer(nn.Module):
    def __init__(self, width: int, spec: dict, eps: float, layer_idx: int, dtype: torch.dtype):
        super().__init__()
        if spec.get("type") != "attention":
            raise ValueError(f"layer {layer_idx}: unknown mixer type {spec.get('type')!r}")
        self.norm1, self.norm1b = ScalarRMSNorm(eps, dtype), ScalarRMSNorm(eps, dtype)
        self.mix = ConvAttentionMixer(width, spec["mixer"], eps, layer_idx, dtype)
        mlp = spec.get("mlp")
        self.mlp = None
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {layer_idx}: unknown feed-forward kind {mlp.get('kind')!r}")
            self.norm2, self.norm2b = ScalarRMSNorm(eps, dtype), ScalarRMSNorm(eps, dtype)
            self.mlp = PolyNormMLP(width, int(mlp["ff"]), eps, dtype)

    def forward(self, x: torch.Tensor, h: torch.Tensor, v_first: Optional[torch.Tensor], provide_v: bool,
                then: ScalarRMSNorm):
        """``x``: fp32 residual stream (updated in place), ``h = norm1(x)``; returns (``then(x)`` after this layer,
        the v this layer provides).  Every post-norm + residual add + next pre-norm is one launch."""
        y, kept = self.mix(h, v_first, provide_v)
        if self.mlp is None:
            return self.norm1b.residual_add(y, x, then), kept
        h = self.norm1b.residual_add(y, x, self.norm2)
        return self.norm2b.residual_add(self.mlp(h), x, then), kept


class TavulixForCausalLM(nn.Module):
    has_request_state = True          # the convolutions remember projected rows per request: no prefix reuse
    residual_dtype = torch.float32

    def __init__(self, vllm_config: VllmConfig):
        super().__init__()
        mc = vllm_config.model_config
        cfg, dtype = mc.hf_config, mc.torch_dtype
        self.cfg, self.dtype = cfg, dtype
        if get_tensor_model_parallel_world_size() > 1 or get_pp_group().world_size > 1:
            raise NotImplementedError("Tavulix runs on one device: its norms and PolyNorm reduce over whole rows")
        self.is_first = self.is_last = True
        width, eps = int(cfg["width"]), float((cfg.get("norm") or {}).get("eps", 1e-6))
        specs = cfg["layers"]
        self.start_layer, self.end_layer = 0, len(specs)
        self.embed = VocabParallelEmbedding(int(cfg["vocab"]), width, dtype)
        self.pos = nn.Embedding(int(cfg["max_positions"]), width, dtype=dtype)
        self.pos.weight.requires_grad_(False)
        self.layers = nn.ModuleList(TavulixLayer(width, s, eps, i, dtype) for i, s in enumerate(specs))
        mixing = [i for i, l in enumerate(self.layers) if l.mix.v_mix]
        self.v_provider = mixing[0] if mixing else -1
        for i in mixing[1:]:
            a, b = self.layers[mixing[0]].mix, self.layers[i].mix
            if (a.kv_heads, a.vdim) != (b.kv_heads, b.vdim):
                raise ValueError(f"layer {i} mixes values of another shape than layer {mixing[0]} provides")
        self.final_norm = ScalarRMSNorm(eps, dtype)
        self.head = ColumnParallelLinear(width, [int(cfg["vocab"])], False, dtype)
        self.logit_softcap = float(cfg.get("logit_softcap") or 0.0)
        self.trace_residual: Optional[List[torch.Tensor]] = None      # tests: the residual stream after every layer

    def rebind_buffers(self) -> None:
        return None

    def attention_layers(self) -> List[Attention]:
        return [l.mix.attn for l in self.layers]

    def state_layers(self) -> List[ShortConv]:
        return [l.mix.conv for l in self.layers]

    def forward(self, input_ids, positions, intermediate: Optional[IntermediateTensors] = None):
        x = ops.embed_positions(input_ids, positions, self.embed.weight, self.pos.weight)
        n = len(self.layers)
        h = self.layers[0].norm1(x) if n else None
        v_first = None
        for i, layer in enumerate(self.layers):
            then = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            provide = i == self.v_provider
            h, kept = layer(x, h, v_first if layer.mix.v_mix and not provide else None, provide, then)
            if provide:
                v_first = kept
            if self.trace_residual is not None:
                self.trace_residual.append(x.clone())
        return h if n else self.final_norm(x)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        y = ops.linear_f32(hidden, self.head.weight)[..., :int(self.cfg["vocab"])]
        if self.logit_softcap > 0:
            y = torch.tanh(y / self.logit_softcap) * self.logit_softcap
        return y

    # ------------------------------------------------------------ weights
    _MIX = {"q": ("proj.weight", 0), "k": ("proj.weight", 1), "v": ("proj.weight", 2), "g": ("proj.weight", 3),
            "q.conv": ("conv.weight", 0), "k.conv": ("conv.weight", 1), "v.conv": ("conv.weight", 2),
            "q.norm": ("q_norm", None), "k.norm": ("k_norm", None), "vmix": ("vmix", None),
            "r1": ("attn.bias_scale", None), "r2": ("attn.bias_rate", None), "sink": ("attn.sink", None),
            "o": ("o.weight", None)}
    _MLP = {"up": "up.weight", "down": "down.weight", "act": "act"}

    def _target(self, name: str) -> Optional[Tuple[str, Optional[int]]]:
        """Checkpoint tensor name -> (parameter name, shard of a fused parameter)."""
        top = {"embed": "embed.weight", "pos": "pos.weight", "final.norm": "final_norm.weight", "head": "head.weight"}
        if name in top:
            return top[name], None
        if not name.startswith("l"):
            return None
        layer, _, rest = name[1:].partition(".")
        if not layer.isdigit():
            return None
        base = f"layers.{layer}."
        if rest in ("norm1", "norm1b", "norm2", "norm2b"):
            return base + rest + ".weight", None
        kind, _, leaf = rest.partition(".")
        if kind == "mix" and leaf in self._MIX:
            if leaf == "vmix" and not self.layers[int(layer)].mix.v_mix:
                return None
            p, shard = self._MIX[leaf]
            return base + "mix." + p, shard
        if kind == "mlp" and leaf in self._MLP:
            return base + "mlp." + self._MLP[leaf], None
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
    """Checkpoint tensor names and shapes of a Tavulix config (for the random-weight loader)."""
    width, vocab = int(c["width"]), int(c["vocab"])
    out: Dict[str, Tuple[int, ...]] = {"embed": (vocab, width), "pos": (int(c["max_positions"]), width)}
    for i, spec in enumerate(c["layers"]):
        m, p = spec["mixer"], f"l{i}."
        heads, kvh = int(m["heads"]), int(m.get("kv_heads") or m["heads"])
        dim, vdim, taps = int(m["dim"]), int(m.get("vdim") or m["dim"]), int(m["conv"])
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if spec.get("mlp") else ()):
            out[p + n] = ()
        for n, rows in (("q", heads * dim), ("k", kvh * dim), ("v", kvh * vdim)):
            out[p + "mix." + n] = (rows, width)
            out[p + "mix." + n + ".conv"] = (rows, taps)
        out[p + "mix.q.norm"], out[p + "mix.k.norm"] = (dim,), (dim,)
        if m.get("v_mix"):
            out[p + "mix.vmix"] = ()
        for n in ("r1", "r2", "sink"):
            out[p + "mix." + n] = (heads,)
        out[p + "mix.g"], out[p + "mix.o"] = (heads, width), (width, heads * vdim)
        if spec.get("mlp"):
            ff = int(spec["mlp"]["ff"])
            out[p + "mlp.up"], out[p + "mlp.down"], out[p + "mlp.act"] = (ff, width), (width, ff), (4,)
    out["final.norm"], out["head"] = (), (vocab, width)
    return out


def random_weight(name: str, shape: Tuple[int, ...], gen: torch.Generator, device, dtype) -> torch.Tensor:
    """A plausible random value for a checkpoint tensor (unit-variance-preserving projections, gains near one,
    small positive bias constants)."""
    def uni(lo: float, hi: float) -> torch.Tensor:
        return lo + (hi - lo) * torch.rand(shape, generator=gen, device=device, dtype=torch.float32)
    leaf = name.rsplit(".", 1)[-1]
    if leaf in ("norm1", "norm2", "norm1b", "norm2b") or name in ("final.norm",) or name.endswith((".q.norm", ".k.norm")):
        w = uni(0.8, 1.2)
    elif leaf == "conv":
        w = uni(-0.5, 0.5) + (torch.arange(shape[1], device=device) == shape[1] - 1).float()
    elif leaf == "vmix":
        w = uni(0.2, 0.6)
    elif leaf == "r1":
        w = uni(0.1, 1.0)
    elif leaf == "r2":
        w = uni(0.05, 0.5)
    elif leaf == "sink":
        w = uni(-1.0, 1.0)
    elif leaf == "act":
        w = uni(-1.0, 1.0)
    elif name in ("embed", "pos"):
        w = uni(-1.0, 1.0)
    else:
        s = (3.0 / shape[-1]) ** 0.5
        w = uni(-s, s)
    return w.to(dtype)
