"""Nosalorn: a layer-list decoder of pre-norm layers,

    x <- x + mixer(n1(x));   x <- x + ff(n2(x))            (ff optional)

with weighted RMS norms. A layer's mixer is softmax attention (biased q/k/v
projections, a partly rotated head with YaRN frequencies, a sliding window
that keeps the first tokens, values blended with those of the first blending
layer), linear attention with a fixed decay per head, or a Mamba-2
state-space mixer. The feed-forward is SwiGLU or a mixture of clamped-GLU
experts under a softmax router with a choice correction, group-limited
choice, identity experts and a gated shared expert. Embedding: scale * token
row. Output: final norm, untied head, logits times a scale.

The residual stream is fp32. Per sublayer: one merged input GEMM, the mixer's
kernels, one output GEMM, and ONE kernel that adds the sublayer's result (for
routed experts: the weighted gather of a token's expert rows, the identity
share of its input and the gated shared expert) to the stream and emits the
next sublayer's normed input.
"""

from __future__ import annotations

import math
import zlib
from typing import Dict, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..engine.batch import ForwardBatch
from ..engine.kv_cache import PagedKVCache
from ..ops import hybrid as hops
from ..parallel.tp import TPContext
from .hybrid_spec import (AttnMixerSpec, DecayAttnMixerSpec, HybridLayerSpec,
                          HybridSpec, SSDMixerSpec)
from .layers import (DecayAttention, LocalAttention, RoutedExperts,
                     SectionedLinear, SSDMixer, _pad)


class PreNormBlock(nn.Module):
    """One layer: norm, merged input projection, mixer, output projection;
    norm, feed-forward (dense gated unit or routed experts)."""

    def __init__(self, spec: HybridSpec, layer: HybridLayerSpec, idx: int,
                 dtype: torch.dtype):
        super().__init__()
        W = spec.hidden_size
        self.idx = idx
        self.eps = spec.norm_eps
        m = layer.mixer
        if isinstance(m, AttnMixerSpec):
            self.mixer = LocalAttention(m, spec.norm_eps, idx)
        elif isinstance(m, DecayAttnMixerSpec):
            self.mixer = DecayAttention(m, spec.norm_eps, idx)
        elif isinstance(m, SSDMixerSpec):
            self.mixer = SSDMixer(m, spec.norm_eps, idx)
        else:
            raise ValueError(f"layer {idx}: unsupported mixer "
                             f"{type(m).__name__}")
        f32 = torch.float32
        self.norm1 = nn.Parameter(torch.ones(W, dtype=f32))
        self.in_proj = SectionedLinear(W, self.mixer.in_sections(""), dtype)
        k = _pad(self.mixer.out_width)
        self.out_padded = k != self.mixer.out_width
        self.out_proj = nn.Linear(k, W, bias=False, dtype=dtype)
        self.ff = layer.ff
        self.experts: Optional[RoutedExperts] = None
        if layer.ff or layer.moe is not None:
            self.norm2 = nn.Parameter(torch.ones(W, dtype=f32))
        if layer.ff:
            self.ff_in = SectionedLinear(
                W, [("gate", layer.ff, False), ("up", layer.ff, False)], dtype)
            self.ff_out = nn.Linear(layer.ff, W, bias=False, dtype=dtype)
        if layer.moe is not None:
            self.experts = RoutedExperts(layer.moe, W, dtype)

    @property
    def has_ff(self) -> bool:
        return bool(self.ff) or self.experts is not None

    def checkpoint_targets(self, prefix: str) -> Dict[str, tuple]:
        lp = f"l{self.idx}"
        ck = lp + ".mix"
        W = self.norm1.numel()
        t = {lp + ".norm1": (prefix + "norm1", 0, 0, W, 1.0)}
        t.update(self.in_proj.section_targets(
            prefix + "in_proj.", self.mixer.section_names("", ck)))
        if hasattr(self.mixer, "param_targets"):
            t.update(self.mixer.param_targets(prefix + "mixer.", ck))
        if isinstance(self.mixer, LocalAttention):
            # a layer that does not blend may still carry the (unused) weight
            t[ck + ".vmix"] = (prefix + "mixer.v_lambda", None, 0, 0, 1.0) \
                if self.mixer.spec.v_mix else None
        t[ck + ".o"] = (prefix + "out_proj.weight", 1, 0,
                        self.mixer.out_width, 1.0)
        if self.has_ff:
            t[lp + ".norm2"] = (prefix + "norm2", 0, 0, W, 1.0)
        if self.ff:
            t.update(self.ff_in.section_targets(
                prefix + "ff_in.", {"gate": lp + ".mlp.gate",
                                    "up": lp + ".mlp.up"}))
            t[lp + ".mlp.down"] = (prefix + "ff_out.weight", 1, 0, self.ff, 1.0)
        if self.experts is not None:
            t.update(self.experts.param_targets(prefix + "experts.",
                                                lp + ".mlp"))
        return t

    def forward(self, x: torch.Tensor, h: torch.Tensor, fb: ForwardBatch,
                kv: PagedKVCache, next_norm: torch.Tensor) -> None:
        """x fp32 [T, W]: the stream, updated in place. h [T, W] activation
        type: this layer's normed input, overwritten with the next layer's
        (normed with the weight `next_norm`)."""
        T = h.shape[0]
        proj = self.in_proj(h)
        alloc = torch.zeros if self.out_padded else torch.empty
        mix_in = alloc((T, self.out_proj.in_features), dtype=h.dtype,
                       device=h.device)
        self.mixer(proj, self.in_proj.offsets, "", fb, kv, mix_in, 0, 1.0)
        y = self.out_proj(mix_in)
        if not self.has_ff:
            hops.add_rmsnorm(x, y, norm_w=next_norm, eps=self.eps, h_out=h)
            return
        hops.add_rmsnorm(x, y, norm_w=self.norm2, eps=self.eps, h_out=h)
        if self.ff:
            proj = self.ff_in(h)
            off = self.ff_in.offsets
            act = hops.glu_mul(proj, off["gate"], off["up"], self.ff,
                               hops.GLU_SILU)
            hops.add_rmsnorm(x, self.ff_out(act), norm_w=next_norm,
                             eps=self.eps, h_out=h)
            return
        ex = self.experts
        rows, padpos, wts, idw = ex(h)
        y2 = proj2 = None
        sg = -1
        if ex.spec.shared_ff:
            y2, proj2, sg = ex.shared_forward(h)
        # h is read (identity experts) and rewritten row by row in one kernel
        hops.add_rmsnorm(x, None, rows, padpos, wts, idw,
                         h if idw is not None else None, y2, proj2, sg,
                         next_norm, self.eps, h)


class NosalornModel(nn.Module):
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
                "layer-list decoders run on one GPU per replica (the "
                "recurrent state is not sharded); use data parallelism")
        W = spec.hidden_size
        self.embed_tokens = nn.Embedding(spec.vocab_size, W, dtype=dtype)
        self.layers = nn.ModuleList(
            [PreNormBlock(spec, layer, i, dtype)
             for i, layer in enumerate(spec.layers)])
        self.final_norm = nn.Parameter(torch.ones(W, dtype=torch.float32))
        self.lm_head = nn.Linear(W, spec.vocab_size, bias=False, dtype=dtype)
        self.act_dtype = dtype
        # debugging aid: when set to a list, the fp32 residual stream after
        # every layer is appended to it
        self.layer_taps: Optional[list] = None

    def cache_layout(self):
        """(per-layer KV shapes, per-layer recurrent state shapes)."""
        return ([blk.mixer.kv_shape() for blk in self.layers],
                [blk.mixer.state_shape() for blk in self.layers])

    def checkpoint_targets(self) -> Dict[str, tuple]:
        s = self.spec
        t = {"embed": ("embed_tokens.weight", 0, 0, s.vocab_size, 1.0),
             "head": ("lm_head.weight", 0, 0, s.vocab_size, 1.0),
             "final.norm": ("final_norm", 0, 0, s.hidden_size, 1.0)}
        for i, blk in enumerate(self.layers):
            t.update(blk.checkpoint_targets(f"layers.{i}."))
        return t

    @torch.no_grad()
    def forward(self, fb: ForwardBatch, kv: PagedKVCache) -> torch.Tensor:
        # per-step scratch (rotation tables, the first blending layer's
        # values) is rebuilt on every pass
        fb.aux.clear()
        s = self.spec
        T = fb.input_ids.shape[0]
        x = hops.token_embed(fb.input_ids, None, fb.positions,
                             self.embed_tokens.weight, None, 0, 0, 0, None,
                             scale=s.embed_scale)
        h = torch.empty((T, s.hidden_size), dtype=self.act_dtype,
                        device=x.device)
        n = len(self.layers)
        hops.add_rmsnorm(x, norm_w=self.layers[0].norm1 if n
                         else self.final_norm, eps=s.norm_eps, h_out=h)
        for i, blk in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            blk(x, h, fb, kv, nxt)
            if self.layer_taps is not None:
                self.layer_taps.append(x.clone())
        return h

    @torch.no_grad()
    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = self.lm_head(hidden).float()
        if self.spec.logit_scale != 1.0:
            logits = logits * self.spec.logit_scale
        return logits

    @torch.no_grad()
    def init_random_weights(self, seed: int = 0) -> None:
        """Deterministic random init on the parameters' own device, scaled so
        activations, decays and router scores stay in a sane range at any
        width."""
        for name, p in sorted(self.named_parameters()):
            gen = torch.Generator(device=p.device)
            gen.manual_seed(seed * 1000003 + zlib.crc32(name.encode()))

            def rnd(shape, std):
                return torch.randn(shape, generator=gen, dtype=torch.float32,
                                   device=p.device) * std

            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "norm2", "final_norm", "norm_w"):
                p.copy_(1.0 + rnd(p.shape, 0.05))
            elif leaf == "v_lambda":
                p.fill_(0.3)
            elif leaf == "a_log":
                p.copy_(rnd(p.shape, 0.3) - 0.5)
            elif leaf == "dt_bias":
                p.copy_(rnd(p.shape, 0.5) - 1.0)
            elif leaf == "skip":
                p.copy_(1.0 + rnd(p.shape, 0.1))
            elif leaf == "conv_w":
                p.copy_(rnd(p.shape, 0.4))
            elif leaf in ("conv_b", "correction"):
                p.copy_(rnd(p.shape, 0.02))
            elif leaf == "bias":
                p.copy_(rnd(p.shape, 0.02).to(p.dtype))
            elif leaf == "router":
                p.copy_(rnd(p.shape, 2.0 / math.sqrt(p.shape[-1])))
            elif name.startswith("embed_tokens"):
                p.copy_(rnd(p.shape, 1.0).to(p.dtype))
            else:
                p.copy_(rnd(p.shape, 1.0 / math.sqrt(p.shape[-1])).to(p.dtype))
        # padding rows/columns of merged projections stay zero
        for blk in self.layers:
            lins = [blk.in_proj]
            if blk.ff:
                lins.append(blk.ff_in)
            if blk.experts is not None and blk.experts.spec.shared_ff:
                lins.append(blk.experts.shared_in)
            for lin in lins:
                keep = torch.zeros(lin.out_features, dtype=torch.bool,
                                   device=lin.weight.device)
                for sec, o in lin.offsets.items():
                    keep[o:o + lin.sizes[sec]] = True
                lin.weight[~keep] = 0
                if lin.bias is not None:
                    lin.bias[~keep] = 0
            blk.out_proj.weight[:, blk.mixer.out_width:] = 0
