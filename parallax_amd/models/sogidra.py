"""Sogidra: a decoder whose config lists its layers one by one, like Vurizen's,
with these pieces:

* token embedding plus a learned position vector per absolute position;
* mixers 'attention' (differential softmax attention with a query
  temperature, row_attention.DifferentialAttention) and 'attention_2'
  (QK-normed sliding-window attention with pooled blocks and a tanh soft cap,
  row_attention.PooledWindowAttention); an 'attention' layer may read an
  earlier layer's cache rows (`kv_from`);
* a dense feed-forward W_down xielu(W_up h) with two learned activation
  numbers per layer (or no feed-forward);
* RMS norms with weights stored around zero (x / rms * (1 + w)) BEFORE and
  AFTER every branch: x += norm_b(branch(norm_a(x)));
* depth-weighted averaging: with X_0 the embedding output and X_(i+1) the
  result of layer i, the stream handed on by layer i is sum_j dwa_i[j] X_j,
  j <= i + 1;
* logits from the embedding table after a final norm.

The residual stream, the per-layer outputs X_j and all norms are fp32 whatever
the activation dtype; each residual step (branch norm, add, history store,
averaging, next norm) is ONE kernel, ops.sandwich_rmsnorm. Every size and
constant comes from the config or a tensor's shape.

Checkpoint tensor names: 'embed', 'pos', 'l<i>.norm1', 'l<i>.norm1b',
'l<i>.norm2', 'l<i>.norm2b', 'l<i>.dwa', 'l<i>.mix.{q,k,v}[.b]',
'l<i>.mix.{lq1,lk1,lq2,lk2,o}', 'l<i>.mlp.{up,down,act}', 'final.norm'.
"""

from __future__ import annotations

import math
from typing import Callable, List, Optional

import torch
import torch.nn as nn

from .. import ops
from ..parallel.comm import get_comm
from ..parallel.layers import ColumnParallelLinear, RowParallelLinear, VocabEmbedding
from .config import ModelConfig
from .forward_meta import ForwardMeta
from .registry import register_model
from .row_attention import DifferentialAttention, PooledWindowAttention


def _softplus(x: float) -> float:
    return x + math.log1p(math.exp(-x)) if x > 0 else math.log1p(math.exp(x))


class XieluMLP(nn.Module):
    """W_down xielu(W_up h); the activation's two numbers are stored before
    their softplus."""

    def __init__(self, hidden_size: int, ff: int):
        super().__init__()
        self.intermediate_size = ff
        self.up = ColumnParallelLinear(hidden_size, ff)
        self.down = RowParallelLinear(ff, hidden_size)
        self.act = nn.Parameter(torch.empty(2), requires_grad=False)
        self._ab = None

    def invalidate_constants(self) -> None:
        self._ab = None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if self._ab is None:
            p, q = self.act.double().tolist()
            self._ab = (_softplus(p), _softplus(q))
        return self.down(ops.xielu(self.up(x), *self._ab))


class SogidraLayer(nn.Module):
    def __init__(self, cfg: ModelConfig, spec: dict, mixer: nn.Module, n_hist: int):
        super().__init__()
        W = cfg.hidden_size
        self.kind = spec["type"]
        self.mixer = mixer
        self.norm1 = nn.Parameter(torch.empty(W), requires_grad=False)
        self.norm1b = nn.Parameter(torch.empty(W), requires_grad=False)
        self.mlp = None
        mlp = spec.get("mlp")
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"feed-forward kind {mlp.get('kind')!r} is "
                                 "not part of this design")
            self.mlp = XieluMLP(W, int(mlp["ff"]))
            self.norm2 = nn.Parameter(torch.empty(W), requires_grad=False)
            self.norm2b = nn.Parameter(torch.empty(W), requires_grad=False)
        # weights over X_0 .. X_(i+1)
        self.dwa = nn.Parameter(torch.empty(n_hist), requires_grad=False)


@register_model("Sogidra")
class SogidraShardModel(nn.Module):
    """The whole stack on one shard: the depth average of every layer reads
    the outputs of ALL earlier layers, so a layer range cannot be cut out
    without shipping that history between stages."""

    hidden_dtype = torch.float32
    graph_safe = True
    norm_offset = 1.0   # norm weights are stored around zero

    def __init__(self, cfg: ModelConfig, start_layer: int = 0,
                 end_layer: Optional[int] = None):
        super().__init__()
        if cfg.layer_specs is None:
            raise ValueError("Sogidra needs a config with a 'layers' list")
        end_layer = cfg.num_layers if end_layer is None else end_layer
        if start_layer != 0 or end_layer != cfg.num_layers:
            raise NotImplementedError(
                "Sogidra runs as one shard: depth-weighted averaging needs "
                "every earlier layer's output")
        if get_comm().tp_size != 1:
            raise NotImplementedError(
                "tensor parallelism inside a layer is not wired up for Sogidra")
        self.cfg = cfg
        self.start_layer, self.end_layer = 0, cfg.num_layers
        self.is_first = self.is_last = True
        self.eps = cfg.rms_norm_eps
        W = cfg.hidden_size
        self.embed_tokens = VocabEmbedding(cfg.vocab_size, W)
        self.pos_embed = nn.Parameter(
            torch.empty(cfg.max_position_embeddings, W), requires_grad=False)
        self.layers = nn.ModuleList(self._build_layers(cfg))
        self.norm = nn.Parameter(torch.empty(W), requires_grad=False)
        self.rope_cache = None
        self._dwa32: Optional[List[torch.Tensor]] = None
        # debugging aid: called with (layer index, fp32 stream after that
        # layer's averaging) when set
        self.tap: Optional[Callable[[int, torch.Tensor], None]] = None

    def _build_layers(self, cfg: ModelConfig) -> List[SogidraLayer]:
        layers, cache_of = [], {}
        W, eps = cfg.hidden_size, cfg.rms_norm_eps
        for g, spec in enumerate(cfg.layer_specs):
            mx = spec["mixer"]
            src = mx.get("kv_from")
            owns = src is None
            if owns:
                cache_of[g] = len(cache_of)
                idx = cache_of[g]
            else:
                owner = cfg.layer_specs[int(src)] if 0 <= int(src) < g else None
                if owner is None or int(src) not in cache_of \
                        or owner["type"] != spec["type"]:
                    raise ValueError(
                        f"layer {g} reads the cache of layer {src}, which is "
                        "not an earlier cache-owning layer of its kind")
                idx = cache_of[int(src)]
            if spec["type"] == "attention":
                temp = mx.get("q_temp") or {}
                mixer = DifferentialAttention(
                    W, int(mx["heads"]), int(mx.get("kv_heads", mx["heads"])), int(mx["dim"]),
                    int(mx["vdim"]), float(mx["scale"]), float(mx.get("diff", 0.0)),
                    float(temp.get("coef", 0.0)), int(temp.get("every", 0)),
                    eps, idx, owns,
                )
            elif spec["type"] == "attention_2":
                mask = mx.get("mask") or {}
                mixer = PooledWindowAttention(
                    W, int(mx["heads"]), int(mx.get("kv_heads", mx["heads"])), int(mx["dim"]),
                    int(mx.get("vdim", mx["dim"])), float(mx["scale"]),
                    float(mx.get("softcap") or 0.0), int(mask["size"]),
                    int(mask.get("pool", 0)), eps, idx, owns,
                )
            else:
                raise ValueError(f"layer type {spec['type']!r} is not part of "
                                 "this design")
            layers.append(SogidraLayer(cfg, spec, mixer, g + 2))
        return layers

    @property
    def num_local_layers(self) -> int:
        return len(self.layers)

    def embed(self, input_ids: torch.Tensor) -> torch.Tensor:
        return self.embed_tokens(input_ids)

    def _dwa(self, device) -> List[torch.Tensor]:
        if self._dwa32 is None or self._dwa32[0].device != device:
            self._dwa32 = [l.dwa.detach().float().contiguous().to(device)
                           for l in self.layers]
        return self._dwa32

    def forward(self, hidden: torch.Tensor, meta: ForwardMeta) -> torch.Tensor:
        """hidden [T, width]: token embeddings. Returns the final-normed
        activations. `hist` holds X_0 .. X_L (fp32) for the depth averages."""
        x = hidden.float().contiguous()
        T, W = x.shape
        L = len(self.layers)
        dt = self.norm.dtype
        eps, off = self.eps, self.norm_offset
        dwa = self._dwa(x.device)
        hist = torch.empty(L + 1, T, W, dtype=torch.float32, device=x.device)
        first = self.layers[0].norm1 if L else self.norm
        h = ops.sandwich_rmsnorm(x, None, None, hist, 1, None, first, eps, off,
                                 dt, self.pos_embed, meta.positions)
        for i, layer in enumerate(self.layers):
            y, wb = layer.mixer(h, meta), layer.norm1b
            if layer.mlp is not None:
                h = ops.sandwich_rmsnorm(x, y, wb, None, 0, None, layer.norm2,
                                         eps, off, dt)
                y, wb = layer.mlp(h), layer.norm2b
            nxt = self.layers[i + 1].norm1 if i + 1 < L else self.norm
            h = ops.sandwich_rmsnorm(x, y, wb, hist, i + 2, dwa[i], nxt, eps,
                                     off, dt)
            if self.tap is not None:
                self.tap(i, x)
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        w = self.embed_tokens.weight
        return ops.linear(hidden.to(w.dtype).contiguous(), w).float()

    def finalize_weights(self) -> None:
        self._dwa32 = None
        for layer in self.layers:
            layer.mixer.invalidate_constants()
            if layer.mlp is not None:
                layer.mlp.invalidate_constants()

    # -- weight loading ---------------------------------------------------------

    def map_global_layer(self, name: str) -> Optional[str]:
        if name in ("embed", "pos", "final.norm"):
            return name
        if name.startswith("l"):
            first, _, rest = name.partition(".")
            if first[1:].isdigit() and rest and int(first[1:]) < len(self.layers):
                return f"layers.{int(first[1:])}.{rest}"
        return None

    def load_hf_weight(self, name: str, tensor: torch.Tensor) -> bool:
        local = self.map_global_layer(name)
        if local is None:
            return False
        t = tensor.to(torch.bfloat16) if tensor.is_floating_point() else tensor
        if local == "embed":
            self.embed_tokens.weight.data.copy_(t)
            return True
        if local == "pos":
            self.pos_embed.data.copy_(t)
            return True
        if local == "final.norm":
            self.norm.data.copy_(t)
            return True
        parts = local.split(".")
        layer: SogidraLayer = self.layers[int(parts[1])]
        key = ".".join(parts[2:])
        if key in ("norm1", "norm1b", "dwa"):
            getattr(layer, key).data.copy_(t)
        elif key in ("norm2", "norm2b"):
            if layer.mlp is None:
                return False
            getattr(layer, key).data.copy_(t)
        elif parts[2] == "mix":
            return self._load_mixer(layer.mixer, ".".join(parts[3:]), t)
        elif parts[2] == "mlp" and layer.mlp is not None:
            if key == "mlp.up":
                layer.mlp.up.load_full_weight(t)
            elif key == "mlp.down":
                layer.mlp.down.load_full_weight(t)
            elif key == "mlp.act":
                layer.mlp.act.data.copy_(t)
            else:
                return False
        else:
            return False
        return True

    @staticmethod
    def _load_mixer(mixer: nn.Module, key: str, t: torch.Tensor) -> bool:
        slot = {"q": 0, "k": 1, "v": 2}.get(key.split(".")[0])
        if slot is not None and key in ("q", "k", "v", "q.b", "k.b", "v.b"):
            if slot >= len(mixer.in_proj.out_sizes):
                return False   # a layer that reads another layer's rows
            if key.endswith(".b"):
                if mixer.in_proj.bias is None:
                    return False
                mixer.in_proj.load_full_weight_part(slot, None, t)
            else:
                mixer.in_proj.load_full_weight_part(slot, t)
        elif key == "o":
            mixer.o_proj.load_full_weight(t)
        elif key in ("lq1", "lk1", "lq2", "lk2") and hasattr(mixer, key):
            getattr(mixer, key).data.copy_(t)
        else:
            return False
        return True

    @torch.no_grad()
    def init_random(self, seed: int = 1234) -> None:
        """Synthetic weights for benchmarking: projections ~ N(0, 1/fan_in),
        norm weights 0 (= scale 1), biases small, depth averages uniform."""
        g = torch.Generator().manual_seed(seed)
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm", "norm1", "norm1b", "norm2", "norm2b"):
                p.data.zero_()
            elif leaf == "dwa":
                p.data.fill_(1.0 / p.numel())
            elif leaf == "act":
                p.data.fill_(0.5)
            elif leaf in ("lq1", "lk1", "lq2", "lk2", "bias"):
                p.data.copy_(torch.randn(p.shape, generator=g).mul_(0.1).to(p.dtype))
            elif leaf == "pos_embed":
                p.data.copy_(torch.randn(p.shape, generator=g).mul_(0.02).to(p.dtype))
            else:
                p.data.copy_(
                    torch.randn(p.shape, generator=g, dtype=torch.float32)
                    .mul_(1.0 / math.sqrt(p.shape[-1])).to(p.dtype))
        self.finalize_weights()
