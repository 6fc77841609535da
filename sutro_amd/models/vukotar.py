"""Vukotar: a layer-list decoder of parallel layers. One Dynamic-Tanh norm
feeds both branches of a layer, and each branch has a learned per-channel
layer scale:

    h = tanh(alpha * x) * w + b
    x <- x + ls1 * attention(h) + ls2 * experts(h)        (experts optional)

Attention is causal grouped-query softmax attention with split key / value
sizes, no positional signal in the scores and a silent sink in the softmax;
the feed-forward is a mixture of squared-ReLU experts under a sigmoid router
with group-limited choice. A layer may use another layer's parameters while
keeping key/value pages of its own. Embedding: scale * token row + sinusoid of
the position. Output: Dynamic-Tanh norm, logits from the embedding table,
soft-capped.

The residual stream is fp32. Per layer: one merged q/k/v GEMM, the attention
kernels, the output GEMM; the router GEMM in fp32, one routing and one
dispatch kernel, two expert GEMMs over per-expert segments; and ONE kernel
that gathers a token's expert rows with their weights, applies both layer
scales, adds to the stream and emits the next layer's normed input.
"""

from __future__ import annotations

import math
import zlib
from typing import Dict, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..engine.batch import ForwardBatch
from ..engine.kv_cache import PagedKVCache
from ..ops import hybrid as hops
from ..parallel.tp import TPContext
from .hybrid_spec import AttnMixerSpec, HybridLayerSpec, HybridSpec
from .layers import LocalAttention, RoutedExperts, SectionedLinear, _pad


class DynamicTanh(nn.Module):
    """tanh(alpha * x) * weight + bias: a norm without statistics."""

    def __init__(self, width: int):
        super().__init__()
        f32 = torch.float32
        self.alpha = nn.Parameter(torch.ones((), dtype=f32))
        self.weight = nn.Parameter(torch.ones(width, dtype=f32))
        self.bias = nn.Parameter(torch.zeros(width, dtype=f32))

    def parts(self) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        return self.alpha, self.weight, self.bias

    def targets(self, prefix: str, ck: str) -> Dict[str, tuple]:
        W = self.weight.numel()
        return {ck: (prefix + "weight", 0, 0, W, 1.0),
                ck + ".b": (prefix + "bias", 0, 0, W, 1.0),
                ck + ".alpha": (prefix + "alpha", None, 0, 0, 1.0)}


class ParallelBlock(nn.Module):
    """The parameters of one layer (possibly used by several layers): the
    norm, attention with its merged input projection and output projection,
    the routed experts, both layer scales."""

    def __init__(self, spec: HybridSpec, layer: HybridLayerSpec, idx: int,
                 dtype: torch.dtype):
        super().__init__()
        W = spec.hidden_size
        self.idx = idx
        if not isinstance(layer.mixer, AttnMixerSpec):
            raise ValueError(f"layer {idx}: unsupported mixer "
                             f"{type(layer.mixer).__name__}")
        self.norm = DynamicTanh(W)
        self.mixer = LocalAttention(layer.mixer, spec.norm_eps, idx)
        self.in_proj = SectionedLinear(W, self.mixer.in_sections(""), dtype)
        k = _pad(self.mixer.out_width)
        self.out_padded = k != self.mixer.out_width
        self.out_proj = nn.Linear(k, W, bias=False, dtype=dtype)
        self.ls1 = nn.Parameter(torch.ones(W, dtype=torch.float32))
        self.experts: Optional[RoutedExperts] = None
        if layer.moe is not None:
            self.experts = RoutedExperts(layer.moe, W, dtype)
            self.ls2 = nn.Parameter(torch.ones(W, dtype=torch.float32))

    def checkpoint_targets(self, prefix: str) -> Dict[str, tuple]:
        lp = f"l{self.idx}"
        ck = lp + ".mix"
        t = self.norm.targets(prefix + "norm.", lp + ".norm1")
        t.update(self.in_proj.section_targets(
            prefix + "in_proj.", self.mixer.section_names("", ck)))
        t[ck + ".o"] = (prefix + "out_proj.weight", 1, 0,
                        self.mixer.out_width, 1.0)
        W = self.ls1.numel()
        t[lp + ".ls1"] = (prefix + "ls1", 0, 0, W, 1.0)
        if self.experts is not None:
            t.update(self.experts.param_targets(prefix + "experts.",
                                                lp + ".mlp"))
            t[lp + ".ls2"] = (prefix + "ls2", 0, 0, W, 1.0)
        return t

    def forward(self, x: torch.Tensor, h: torch.Tensor, fb: ForwardBatch,
                kv: PagedKVCache, cache_idx: int, next_norm) -> None:
        """x fp32 [T, W]: the stream, updated in place. h [T, W] activation
        type: this layer's normed input, overwritten with the next layer's
        (normed with `next_norm` = (alpha, weight, bias))."""
        T = h.shape[0]
        proj = self.in_proj(h)
        alloc = torch.zeros if self.out_padded else torch.empty
        mix_in = alloc((T, self.out_proj.in_features), dtype=h.dtype,
                       device=h.device)
        self.mixer(proj, self.in_proj.offsets, "", fb, kv, mix_in, 0, 1.0,
                   cache_idx=cache_idx)
        y = self.out_proj(mix_in)
        if self.experts is not None:
            rows, padpos, wts, _ = self.experts(h)
            hops.dyt_residual(x, y, self.ls1, None, self.ls2, rows, padpos,
                              wts, norm=next_norm, h_out=h)
        else:
            hops.dyt_residual(x, y, self.ls1, norm=next_norm, h_out=h)


class VukotarModel(nn.Module):
    """Same engine-facing surface as the other models: forward(fb, kv) ->
    hidden rows, compute_logits(hidden), cache_layout(),
    checkpoint_targets(), init_random_weights()."""

    def __init__(self, spec: HybridSpec, dtype: torch.dtype, max_len: int,
                 tp: Optional[TPContext] = None):
        super().__init__()
        self.spec = spec
        self.tp = tp or TPContext()
        if self.tp.size > 1:
            raise NotImplementedError(
                "layer-list decoders run on one GPU per replica; use data "
                "parallelism")
        W = spec.hidden_size
        self.embed_tokens = nn.Embedding(spec.vocab_size, W, dtype=dtype)
        if spec.pos_base:
            self.register_buffer(
                "pos_inv_freq", hops.sinusoid_inv_freq(W, spec.pos_base),
                persistent=False)
        # one block per layer that owns parameters; `owner[i]` is the block
        # layer i runs (its pages are layer i's own)
        self.blocks = nn.ModuleDict()
        self.owner: List[str] = []
        for i, layer in enumerate(spec.layers):
            own = i if layer.weights_of is None else layer.weights_of
            if spec.layers[own].weights_of is not None:
                raise ValueError(f"layer {i}: weights_of must name a layer "
                                 f"with parameters of its own")
            if str(own) not in self.blocks:
                self.blocks[str(own)] = ParallelBlock(spec, spec.layers[own],
                                                      own, dtype)
            self.owner.append(str(own))
        self.final_norm = DynamicTanh(W)
        self.act_dtype = dtype
        # debugging aid: when set to a list, the fp32 residual stream after
        # every layer is appended to it
        self.layer_taps: Optional[list] = None

    def block_of(self, i: int) -> ParallelBlock:
        return self.blocks[self.owner[i]]

    def cache_layout(self):
        """(per-layer KV shapes, per-layer recurrent state shapes)."""
        n = len(self.owner)
        return ([self.block_of(i).mixer.kv_shape() for i in range(n)],
                [None] * n)

    def checkpoint_targets(self) -> Dict[str, tuple]:
        s = self.spec
        t = {"embed": ("embed_tokens.weight", 0, 0, s.vocab_size, 1.0)}
        t.update(self.final_norm.targets("final_norm.", "final.norm"))
        for key, blk in self.blocks.items():
            t.update(blk.checkpoint_targets(f"blocks.{key}."))
        return t

    @torch.no_grad()
    def forward(self, fb: ForwardBatch, kv: PagedKVCache) -> torch.Tensor:
        fb.aux.clear()
        s = self.spec
        T = fb.input_ids.shape[0]
        dev = fb.input_ids.device
        x = hops.token_embed(
            fb.input_ids, None, fb.positions, self.embed_tokens.weight, None,
            0, 0, 0, self.pos_inv_freq if s.pos_base else None,
            scale=s.embed_scale)
        h = torch.empty((T, s.hidden_size), dtype=self.act_dtype, device=dev)
        n = len(self.owner)
        hops.dyt_residual(x, norm=self.block_of(0).norm.parts(), h_out=h)
        for i in range(n):
            nxt = (self.block_of(i + 1).norm if i + 1 < n
                   else self.final_norm).parts()
            self.block_of(i)(x, h, fb, kv, i, nxt)
            if self.layer_taps is not None:
                self.layer_taps.append(x.clone())
        return h

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = F.linear(hidden, self.embed_tokens.weight)
        if self.spec.logit_softcap:
            return hops.softcap(logits, self.spec.logit_softcap)
        return logits.float()

    @torch.no_grad()
    def init_random_weights(self, seed: int = 0) -> None:
        """Deterministic random init on the parameters' own device, scaled so
        activations and router scores stay in a sane range at any width."""
        for name, p in sorted(self.named_parameters()):
            gen = torch.Generator(device=p.device)
            gen.manual_seed(seed * 1000003 + zlib.crc32(name.encode()))

            def rnd(shape, std):
                return torch.randn(shape, generator=gen, dtype=torch.float32,
                                   device=p.device) * std

            leaf = name.rsplit(".", 1)[-1]
            if leaf == "alpha":
                p.fill_(0.5)
            elif name.endswith("norm.weight"):
                p.copy_(1.0 + rnd(p.shape, 0.05))
            elif name.endswith("norm.bias"):
                p.copy_(rnd(p.shape, 0.02))
            elif leaf in ("ls1", "ls2"):
                p.copy_(0.5 + rnd(p.shape, 0.05))
            elif leaf == "router":
                p.copy_(rnd(p.shape, 2.0 / math.sqrt(p.shape[-1])))
            elif name.startswith("embed_tokens"):
                p.copy_(rnd(p.shape, 1.0).to(p.dtype))
            else:
                p.copy_(rnd(p.shape, 1.0 / math.sqrt(p.shape[-1])).to(p.dtype))
        # padding rows/columns of merged projections stay zero
        for blk in self.blocks.values():
            lin = blk.in_proj
            keep = torch.zeros(lin.out_features, dtype=torch.bool,
                               device=lin.weight.device)
            for sec, o in lin.offsets.items():
                keep[o:o + lin.sizes[sec]] = True
            lin.weight[~keep] = 0
            blk.out_proj.weight[:, blk.mixer.out_width:] = 0
