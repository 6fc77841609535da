"""Reusable building blocks of layer-list decoders.

Every sublayer reads its input once: all projections that consume that input
(query/key/value of each mixer, low-rank gate inputs, the residual gate) are
rows of ONE merged weight, so a sublayer costs one input GEMM, a handful of
fused HIP kernels and one output GEMM. The kernels address their operands as
column sections of the merged GEMM output.
"""

from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from ..engine.batch import ForwardBatch
from ..engine.kv_cache import PagedKVCache
from ..ops import hybrid as hops
from .hybrid_spec import (AttnMixerSpec, DecayAttnMixerSpec, DeltaMixerSpec,
                          LatentAttnMixerSpec, MLSTMMixerSpec,
                          RoutedExpertsSpec, SSDMixerSpec, TiedAttnMixerSpec)

_ALIGN = 8  # section starts are multiples of 8 columns (16 B in bf16)


def _pad(n: int) -> int:
    return (n + _ALIGN - 1) // _ALIGN * _ALIGN


class SectionedLinear(nn.Module):
    """One Linear whose output columns are named sections (each section a
    separate tensor in the checkpoint). Sections start on 8-column boundaries;
    padding rows are zero. A bias exists if any section has one (zero for the
    others)."""

    def __init__(self, in_features: int,
                 sections: Sequence[Tuple[str, int, bool]],
                 dtype: torch.dtype):
        super().__init__()
        self.offsets: Dict[str, int] = {}
        self.sizes: Dict[str, int] = {}
        self.biased: List[str] = []
        off = 0
        for name, rows, has_bias in sections:
            self.offsets[name] = off
            self.sizes[name] = rows
            if has_bias:
                self.biased.append(name)
            off += _pad(rows)
        self.out_features = off
        self.weight = nn.Parameter(torch.zeros(off, in_features, dtype=dtype))
        self.bias = (nn.Parameter(torch.zeros(off, dtype=dtype))
                     if self.biased else None)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return F.linear(x, self.weight, self.bias)

    def section_targets(self, prefix: str, names: Dict[str, str]):
        """Checkpoint tensor -> (parameter, dim, start, length, scale) for the
        loader. `names` maps section name -> checkpoint tensor name."""
        out = {}
        for sec, ck in names.items():
            o, n = self.offsets[sec], self.sizes[sec]
            out[ck] = (prefix + "weight", 0, o, n, 1.0)
            if sec in self.biased:
                out[ck + ".b"] = (prefix + "bias", 0, o, n, 1.0)
        return out


class LocalAttention(nn.Module):
    """Grouped-query softmax attention under a chunk and/or window mask, with
    per-head q/k RMS norm, rotation of a prefix of each head, split key and
    value sizes, a per-head sigmoid output gate and an optional silent sink
    in the softmax (each part can be switched off by the spec); the window may
    keep the first tokens, the rotation may use YaRN frequencies, and the
    values may be blended with those of the first blending layer of the step
    (which leaves them in `fb.aux`). Owns no
    projection: it works on sections of the sublayer's merged projection and
    writes its gated heads into a slice of the merged output-projection input.
    `cache_idx` in forward names the layer whose pages are used when several
    layers share this module's parameters."""

    def __init__(self, spec: AttnMixerSpec, eps: float, layer_idx: int):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.layer_idx = layer_idx
        if spec.heads % spec.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        if spec.rot_dims % 2 or spec.rot_dims > spec.dim:
            raise ValueError("rot_dims must be even and at most dim")
        if spec.qk_norm:
            self.q_norm = nn.Parameter(torch.ones(spec.dim, dtype=torch.float32))
            self.k_norm = nn.Parameter(torch.ones(spec.dim, dtype=torch.float32))
        inv_freq, self.rot_amp = hops.yarn_inv_freq(
            spec.rot_dims, spec.rot_base, spec.rot_scaling)
        self.register_buffer("inv_freq", inv_freq, persistent=False)
        if spec.v_mix:
            self.v_lambda = nn.Parameter(torch.zeros((), dtype=torch.float32))

    def in_sections(self, tag: str):
        s = self.spec
        secs = [(tag + "q", s.heads * s.dim, s.bias),
                (tag + "k", s.kv_heads * s.dim, s.bias),
                (tag + "v", s.kv_heads * s.vdim, s.bias)]
        if s.out_gate:
            secs.append((tag + "g", s.heads, False))
        return secs

    @property
    def out_width(self) -> int:
        return self.spec.heads * self.spec.vdim

    def kv_shape(self):
        return (self.spec.kv_heads, self.spec.dim, self.spec.vdim)

    def state_shape(self):
        return None

    def section_names(self, tag: str, ck: str):
        n = {tag + "q": ck + ".q", tag + "k": ck + ".k", tag + "v": ck + ".v"}
        if self.spec.out_gate:
            n[tag + "g"] = ck + ".g"
        return n

    def forward(self, proj: torch.Tensor, off: Dict[str, int], tag: str,
                fb: ForwardBatch, kv: PagedKVCache, out: torch.Tensor,
                out_off: int, out_scale: float,
                cache_idx: Optional[int] = None) -> None:
        s = self.spec
        ci = self.layer_idx if cache_idx is None else cache_idx
        kc, vc = kv.k_cache[ci], kv.v_cache[ci]
        cos_sin = None
        if proj.is_cuda:
            # one cos/sin table per step and kind of rotation, shared by layers
            key = ("rope", s.rot_dims, s.rot_base, s.rot_scaling)
            cos_sin = fb.aux.get(key)
            if cos_sin is None:
                cos_sin = fb.aux[key] = hops.rope_table(
                    fb.positions, self.inv_freq, self.rot_amp)
        v_first, v_first_off = None, 0
        if s.v_mix:
            # the first blending layer of a step leaves its value section;
            # later ones blend with it
            first = fb.aux.get("v_first")
            if first is None:
                fb.aux["v_first"] = (proj, off[tag + "v"])
            else:
                v_first, v_first_off = first
        q = hops.attn_prep(
            proj, off[tag + "q"], off[tag + "k"], off[tag + "v"], s.heads,
            s.kv_heads, s.dim, s.vdim,
            self.q_norm if s.qk_norm else None,
            self.k_norm if s.qk_norm else None,
            self.eps, self.inv_freq, fb.positions, fb.slot_mapping, kc, vc,
            cos_sin=cos_sin, rot_amp=self.rot_amp, v_first=v_first,
            v_first_off=v_first_off,
            v_lambda=self.v_lambda if v_first is not None else None)
        hops.local_attention(
            q, kc, vc, fb.block_tables, fb.seq_lens, fb.query_start_locs,
            s.scale, s.chunk, s.window, proj,
            off[tag + "g"] if s.out_gate else -1, out, out_off, out_scale,
            token_seq=fb.token_seq, tile_seq=fb.tile_seq, tile_q0=fb.tile_q0,
            prefill_rows=fb.prefill_token_count, sink=s.sink,
            keep_first=s.keep_first if s.window else 0)


class GatedDeltaRule(nn.Module):
    """Gated delta rule with per-channel decay: short causal filters + silu on
    q/k/v, unit-norm q and k, beta and decay gates in fp32, the token-by-token
    state update, then a per-head RMS norm with a low-rank sigmoid gate. The
    filter history and the memory matrix live in the engine's state cache."""

    def __init__(self, spec: DeltaMixerSpec, eps: float, layer_idx: int):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.layer_idx = layer_idx
        if spec.heads % spec.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        f32 = torch.float32
        ch = 2 * spec.kv_heads * spec.dim + spec.heads * spec.vdim
        self.channels = ch
        # small tensors the kernels read in fp32 (bf16 checkpoint values are
        # held exactly)
        self.conv_w = nn.Parameter(torch.zeros(ch, spec.conv, dtype=f32))
        self.a2 = nn.Parameter(torch.zeros(spec.heads * spec.dim,
                                           spec.decay_rank, dtype=f32))
        self.dt_bias = nn.Parameter(torch.zeros(spec.heads * spec.dim, dtype=f32))
        self.a_log = nn.Parameter(torch.zeros(spec.heads, dtype=f32))
        self.norm_w = nn.Parameter(torch.ones(spec.vdim, dtype=f32))
        self.g2 = nn.Parameter(torch.zeros(spec.heads * spec.vdim,
                                           spec.gate_rank, dtype=f32))
        self._t = None

    def in_sections(self, tag: str):
        s = self.spec
        return [(tag + "q", s.kv_heads * s.dim, False),
                (tag + "k", s.kv_heads * s.dim, False),
                (tag + "v", s.heads * s.vdim, False),
                (tag + "b", s.heads, False),
                (tag + "a1", s.decay_rank, False),
                (tag + "g1", s.gate_rank, False)]

    @property
    def out_width(self) -> int:
        return self.spec.heads * self.spec.vdim

    def state_shape(self):
        s = self.spec
        return (self.channels, s.conv, s.heads, s.dim, s.vdim)

    def param_targets(self, prefix: str, ck: str):
        """Checkpoint tensors of this mixer that are not projections of the
        sublayer input."""
        s = self.spec
        cq = s.kv_heads * s.dim
        return {
            ck + ".q.conv": (prefix + "conv_w", 0, 0, cq, 1.0),
            ck + ".k.conv": (prefix + "conv_w", 0, cq, cq, 1.0),
            ck + ".v.conv": (prefix + "conv_w", 0, 2 * cq, s.heads * s.vdim, 1.0),
            ck + ".a2": (prefix + "a2", 0, 0, s.heads * s.dim, 1.0),
            ck + ".dt_bias": (prefix + "dt_bias", 0, 0, s.heads * s.dim, 1.0),
            ck + ".A_log": (prefix + "a_log", 0, 0, s.heads, 1.0),
            ck + ".norm": (prefix + "norm_w", 0, 0, s.vdim, 1.0),
            ck + ".g2": (prefix + "g2", 0, 0, s.heads * s.vdim, 1.0),
        }

    def forward(self, proj: torch.Tensor, off: Dict[str, int], tag: str,
                fb: ForwardBatch, kv: PagedKVCache, out: torch.Tensor,
                out_off: int, out_scale: float) -> None:
        s = self.spec
        st = kv.state
        if self._t is None or self._t[0].device != proj.device:
            # transposed copies of the low-rank up-projections, made once
            # (before any graph capture: capture is preceded by a warm-up run)
            self._t = (self.a2.detach().t().contiguous(),
                       self.g2.detach().t().contiguous(),
                       self.conv_w.detach().t().contiguous())
        qn, kn, v, decay, beta = hops.delta_prep(
            proj, off[tag + "q"], off[tag + "k"], off[tag + "v"],
            off[tag + "b"], off[tag + "a1"], s.heads, s.kv_heads, s.dim,
            s.vdim, self.conv_w, self.a2, self.dt_bias, self.a_log,
            st.conv[self.layer_idx], fb.state_slots, fb.query_start_locs,
            fb.seq_lens, token_seq=fb.token_seq, a2_t=self._t[0],
            conv_w_t=self._t[2])
        o = hops.delta_scan(qn, kn, v, decay, beta, st.ssm[self.layer_idx],
                            fb.state_slots, fb.query_start_locs, fb.seq_lens)
        hops.delta_out(o, self.norm_w, proj, off[tag + "g1"], self.g2,
                       self.eps, out, out_off, out_scale, g2_t=self._t[1])


class TiedWindowAttention(nn.Module):
    """Windowed grouped-query attention whose values are its raw keys: whole-
    projection q/k RMS norm, position-dependent query temperature, logarithmic
    distance bias per head, no rotation and no value projection. Works on the
    q and k sections of the sublayer's merged projection."""

    def __init__(self, spec: TiedAttnMixerSpec, eps: float, layer_idx: int):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.layer_idx = layer_idx
        if spec.heads % spec.kv_heads:
            raise ValueError("heads must be a multiple of kv_heads")
        f32 = torch.float32
        self.q_norm = nn.Parameter(torch.ones(spec.heads * spec.dim, dtype=f32))
        self.k_norm = nn.Parameter(torch.ones(spec.kv_heads * spec.dim, dtype=f32))
        if spec.dist_bias:
            self.r1 = nn.Parameter(torch.zeros(spec.heads, dtype=f32))
            self.r2 = nn.Parameter(torch.zeros(spec.heads, dtype=f32))

    def in_sections(self, tag: str):
        s = self.spec
        return [(tag + "q", s.heads * s.dim, False),
                (tag + "k", s.kv_heads * s.dim, False)]

    @property
    def out_width(self) -> int:
        return self.spec.heads * self.spec.dim

    def kv_shape(self):
        return (self.spec.kv_heads, self.spec.dim, self.spec.dim)

    def state_shape(self):
        return None

    def param_targets(self, prefix: str, ck: str):
        s = self.spec
        t = {ck + ".q.norm": (prefix + "q_norm", 0, 0, s.heads * s.dim, 1.0),
             ck + ".k.norm": (prefix + "k_norm", 0, 0, s.kv_heads * s.dim, 1.0)}
        if s.dist_bias:
            t[ck + ".r1"] = (prefix + "r1", 0, 0, s.heads, 1.0)
            t[ck + ".r2"] = (prefix + "r2", 0, 0, s.heads, 1.0)
        return t

    def section_names(self, tag: str, ck: str):
        return {tag + "q": ck + ".q", tag + "k": ck + ".k"}

    def forward(self, proj: torch.Tensor, off: Dict[str, int], tag: str,
                fb: ForwardBatch, kv: PagedKVCache, out: torch.Tensor,
                out_off: int, out_scale: float) -> None:
        s = self.spec
        kc, vc = kv.k_cache[self.layer_idx], kv.v_cache[self.layer_idx]
        q = hops.tied_attn_prep(
            proj, off[tag + "q"], off[tag + "k"], s.heads, s.kv_heads, s.dim,
            self.q_norm, self.k_norm, self.eps, fb.positions, s.temp_coef,
            s.temp_every, fb.slot_mapping, kc, vc)
        hops.local_attention(
            q, kc, vc, fb.block_tables, fb.seq_lens, fb.query_start_locs,
            s.scale, 0, s.window, proj, -1, out, out_off, out_scale,
            token_seq=fb.token_seq, tile_seq=fb.tile_seq, tile_q0=fb.tile_q0,
            prefill_rows=fb.prefill_token_count,
            bias_r1=self.r1 if s.dist_bias else None,
            bias_r2=self.r2 if s.dist_bias else None)


class LatentAttention(nn.Module):
    """Attention through low-rank latents without positions. The cache holds
    only the normed key/value latent c [kv_rank] of every token (one "head" of
    a paged K cache; no V pages). Attention runs in latent space: with per-head
    up-projections K_h = U^k_h c and V_h = U^v_h c,
        score = q_h . (U^k_h c) = ((U^k_h)^T q_h) . c,
        out_h = U^v_h (sum_j p_j c_j),
    so queries are folded through U^k once per token, one shared latent serves
    all heads as key and value, and U^v is applied to the attended latent. A
    layer with `kv_from` reads another layer's latent pages and writes none."""

    def __init__(self, spec: LatentAttnMixerSpec, eps: float, layer_idx: int,
                 dtype: torch.dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.layer_idx = layer_idx
        s = spec
        f32 = torch.float32
        self.dq_norm = nn.Parameter(torch.ones(s.q_rank, dtype=f32))
        if s.kv_from is None:
            self.dkv_norm = nn.Parameter(torch.ones(s.kv_rank, dtype=f32))
        self.uq = nn.Parameter(torch.zeros(s.heads * s.dim, s.q_rank, dtype=dtype))
        self.uk = nn.Parameter(torch.zeros(s.heads * s.dim, s.kv_rank, dtype=dtype))
        self.uv = nn.Parameter(torch.zeros(s.heads * s.vdim, s.kv_rank, dtype=dtype))

    def in_sections(self, tag: str):
        s = self.spec
        secs = [(tag + "dq", s.q_rank, False)]
        if s.kv_from is None:
            secs.append((tag + "dkv", s.kv_rank, False))
        secs.append((tag + "g", s.heads * s.vdim, False))
        return secs

    @property
    def out_width(self) -> int:
        return self.spec.heads * self.spec.vdim

    def kv_shape(self):
        # one latent "head" as keys; values are read from the same pages
        return (1, self.spec.kv_rank, 0) if self.spec.kv_from is None else None

    def state_shape(self):
        return None

    def param_targets(self, prefix: str, ck: str):
        s = self.spec
        t = {ck + ".dq.norm": (prefix + "dq_norm", 0, 0, s.q_rank, 1.0),
             ck + ".uq": (prefix + "uq", 0, 0, s.heads * s.dim, 1.0),
             ck + ".uk": (prefix + "uk", 0, 0, s.heads * s.dim, 1.0),
             ck + ".uv": (prefix + "uv", 0, 0, s.heads * s.vdim, 1.0)}
        if s.kv_from is None:
            t[ck + ".dkv.norm"] = (prefix + "dkv_norm", 0, 0, s.kv_rank, 1.0)
        return t

    def section_names(self, tag: str, ck: str):
        n = {tag + "dq": ck + ".dq", tag + "g": ck + ".g"}
        if self.spec.kv_from is None:
            n[tag + "dkv"] = ck + ".dkv"
        return n

    def forward(self, proj: torch.Tensor, off: Dict[str, int], tag: str,
                fb: ForwardBatch, kv: PagedKVCache, out: torch.Tensor,
                out_off: int, out_scale: float) -> None:
        s = self.spec
        T = proj.shape[0]
        H, dk, dv, R = s.heads, s.dim, s.vdim, s.kv_rank
        dev, dt = proj.device, proj.dtype
        cq = torch.empty((T, s.q_rank), dtype=dt, device=dev)
        hops.section_rmsnorm(proj, off[tag + "dq"], s.q_rank, self.dq_norm,
                             self.eps, cq)
        src = self.layer_idx if s.kv_from is None else s.kv_from
        cache = kv.k_cache[src]                    # [blocks, 1, page, R]
        if s.kv_from is None:
            hops.section_rmsnorm(proj, off[tag + "dkv"], R, self.dkv_norm,
                                 self.eps, cache.view(-1, R),
                                 rows=fb.slot_mapping)
        q = F.linear(cq, self.uq)                  # [T, H*dk]
        qa = torch.empty((T, H, R), dtype=dt, device=dev)
        torch.bmm(q.view(T, H, dk).transpose(0, 1), self.uk.view(H, dk, R),
                  out=qa.transpose(0, 1))
        lat = torch.empty((T, H * R), dtype=dt, device=dev)
        hops.local_attention(
            qa, cache, cache, fb.block_tables, fb.seq_lens,
            fb.query_start_locs, s.scale, 0, s.window, proj, -1, lat, 0, 1.0,
            token_seq=fb.token_seq, tile_seq=fb.tile_seq, tile_q0=fb.tile_q0,
            prefill_rows=fb.prefill_token_count)
        sec = out[:, out_off:out_off + H * dv]
        torch.bmm(lat.view(T, H, R).transpose(0, 1),
                  self.uv.view(H, dv, R).transpose(1, 2),
                  out=sec.view(T, H, dv).transpose(0, 1))
        hops.sigmoid_gate_mul(sec, proj, off[tag + "g"])


class MLSTM(nn.Module):
    """mLSTM matrix memory with soft-capped exponential gating; q, k, v, the
    output gate and both gate pre-activations are sections of the sublayer's
    merged projection, the gate biases are added in fp32. The memory (with its
    normaliser as an extra column) and the stabiliser live in the engine's
    state cache."""

    def __init__(self, spec: MLSTMMixerSpec, eps: float, layer_idx: int):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.layer_idx = layer_idx
        f32 = torch.float32
        self.i_bias = nn.Parameter(torch.zeros(spec.heads, dtype=f32))
        self.f_bias = nn.Parameter(torch.zeros(spec.heads, dtype=f32))
        self.norm_w = nn.Parameter(torch.ones(spec.heads * spec.vdim, dtype=f32))

    def in_sections(self, tag: str):
        s = self.spec
        return [(tag + "q", s.heads * s.dim, False),
                (tag + "k", s.heads * s.dim, False),
                (tag + "v", s.heads * s.vdim, False),
                (tag + "g", s.heads * s.vdim, False),
                (tag + "i", s.heads, False),
                (tag + "f", s.heads, False)]

    @property
    def out_width(self) -> int:
        return self.spec.heads * self.spec.vdim

    def kv_shape(self):
        return None

    def state_shape(self):
        s = self.spec
        return {"mem": (s.heads, s.dim, s.vdim + 1), "m": (s.heads,)}

    def param_targets(self, prefix: str, ck: str):
        s = self.spec
        return {ck + ".i.b": (prefix + "i_bias", 0, 0, s.heads, 1.0),
                ck + ".f.b": (prefix + "f_bias", 0, 0, s.heads, 1.0),
                ck + ".norm": (prefix + "norm_w", 0, 0, s.heads * s.vdim, 1.0)}

    def section_names(self, tag: str, ck: str):
        return {tag + k: ck + "." + k for k in ("q", "k", "v", "g", "i", "f")}

    def forward(self, proj: torch.Tensor, off: Dict[str, int], tag: str,
                fb: ForwardBatch, kv: PagedKVCache, out: torch.Tensor,
                out_off: int, out_scale: float) -> None:
        s = self.spec
        st = kv.state.named[self.layer_idx]
        o, em = hops.mlstm_scan(
            proj, off[tag + "q"], off[tag + "k"], off[tag + "v"],
            off[tag + "i"], off[tag + "f"], s.heads, s.dim, s.vdim,
            self.i_bias, self.f_bias, s.gate_cap, st["mem"], st["m"],
            fb.state_slots, fb.query_start_locs, fb.seq_lens)
        hops.mlstm_out(o, em, self.norm_w, proj, off[tag + "g"], self.eps,
                       out, out_off)


class DecayAttention(nn.Module):
    """Linear attention with one fixed decay per head: silu on the q, k, v
    sections of the merged projection, the token-by-token recurrence
    S <- decay S + k v^T, o = S^T q in fp32 (state in the engine's state
    cache), one weighted RMS norm over all heads and an elementwise sigmoid
    gate."""

    def __init__(self, spec: DecayAttnMixerSpec, eps: float, layer_idx: int):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.layer_idx = layer_idx
        f32 = torch.float32
        self.norm_w = nn.Parameter(torch.ones(spec.heads * spec.vdim, dtype=f32))
        self.register_buffer("decay", torch.tensor(spec.decay, dtype=f32),
                             persistent=False)

    def in_sections(self, tag: str):
        s = self.spec
        return [(tag + "q", s.heads * s.dim, False),
                (tag + "k", s.heads * s.dim, False),
                (tag + "v", s.heads * s.vdim, False),
                (tag + "g", s.heads * s.vdim, False)]

    @property
    def out_width(self) -> int:
        return self.spec.heads * self.spec.vdim

    def kv_shape(self):
        return None

    def state_shape(self):
        s = self.spec
        return {"mem": (s.heads, s.dim, s.vdim)}

    def param_targets(self, prefix: str, ck: str):
        s = self.spec
        return {ck + ".norm": (prefix + "norm_w", 0, 0, s.heads * s.vdim, 1.0)}

    def section_names(self, tag: str, ck: str):
        return {tag + k: ck + "." + k for k in ("q", "k", "v", "g")}

    def forward(self, proj: torch.Tensor, off: Dict[str, int], tag: str,
                fb: ForwardBatch, kv: PagedKVCache, out: torch.Tensor,
                out_off: int, out_scale: float = 1.0) -> None:
        s = self.spec
        T = proj.shape[0]
        hk, hv = s.heads * s.dim, s.heads * s.vdim
        q, k, v = hops.silu_sections(
            proj, (off[tag + "q"], off[tag + "k"], off[tag + "v"]),
            (hk, hk, hv))
        o = hops.decay_scan(
            q.view(T, s.heads, s.dim), k.view(T, s.heads, s.dim),
            v.view(T, s.heads, s.vdim), self.decay, None, None,
            kv.state.named[self.layer_idx]["mem"], fb.state_slots,
            fb.query_start_locs, fb.seq_lens)
        hops.gated_group_norm(o, proj, off[tag + "g"], self.norm_w, self.eps,
                              1, False, out, out_off)


class SSDMixer(nn.Module):
    """Mamba-2: the merged projection holds z | x | B | C | dt; x|B|C pass a
    short causal filter (history in the engine's state cache) and silu, the
    step is softplus(dt + bias), and per head S <- exp(-exp(A_log) dt) S +
    dt B x^T, y = S^T C + D x in fp32; y silu(z) is normed in equal parts."""

    def __init__(self, spec: SSDMixerSpec, eps: float, layer_idx: int):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.layer_idx = layer_idx
        f32 = torch.float32
        s = spec
        self.inner = s.heads * s.vdim
        self.channels = self.inner + 2 * s.groups * s.state
        self.conv_w = nn.Parameter(torch.zeros(self.channels, s.conv, dtype=f32))
        self.conv_b = nn.Parameter(torch.zeros(self.channels, dtype=f32))
        self.dt_bias = nn.Parameter(torch.zeros(s.heads, dtype=f32))
        self.a_log = nn.Parameter(torch.zeros(s.heads, dtype=f32))
        self.skip = nn.Parameter(torch.ones(s.heads, dtype=f32))
        self.norm_w = nn.Parameter(torch.ones(self.inner, dtype=f32))
        self._t = None

    def in_sections(self, tag: str):
        # one checkpoint tensor: z | x | B | C | dt stay in its order
        return [(tag + "in", 2 * self.inner + 2 * self.spec.groups
                 * self.spec.state + self.spec.heads, False)]

    @property
    def out_width(self) -> int:
        return self.inner

    def kv_shape(self):
        return None

    def state_shape(self):
        s = self.spec
        return (self.channels, s.conv, s.heads, s.state, s.vdim)

    def param_targets(self, prefix: str, ck: str):
        s = self.spec
        return {ck + ".conv": (prefix + "conv_w", 0, 0, self.channels, 1.0),
                ck + ".conv.b": (prefix + "conv_b", 0, 0, self.channels, 1.0),
                ck + ".dt_bias": (prefix + "dt_bias", 0, 0, s.heads, 1.0),
                ck + ".A_log": (prefix + "a_log", 0, 0, s.heads, 1.0),
                ck + ".D": (prefix + "skip", 0, 0, s.heads, 1.0),
                ck + ".norm": (prefix + "norm_w", 0, 0, self.inner, 1.0)}

    def section_names(self, tag: str, ck: str):
        return {tag + "in": ck + ".in"}

    def forward(self, proj: torch.Tensor, off: Dict[str, int], tag: str,
                fb: ForwardBatch, kv: PagedKVCache, out: torch.Tensor,
                out_off: int, out_scale: float = 1.0) -> None:
        s = self.spec
        st = kv.state
        base = off[tag + "in"]
        if self._t is None or self._t.device != proj.device:
            # made once, before any graph capture (capture follows a warm-up)
            self._t = self.conv_w.detach().t().contiguous()
        x, B, C, decay, dt = hops.ssd_prep(
            proj, base + self.inner, base + self.inner + self.channels,
            s.heads, s.vdim, s.groups, s.state, self.conv_w, self.conv_b,
            self.dt_bias, self.a_log, st.conv[self.layer_idx], fb.state_slots,
            fb.query_start_locs, fb.seq_lens, token_seq=fb.token_seq,
            conv_w_t=self._t)
        y = hops.decay_scan(C, B, x, decay, dt, self.skip,
                            st.ssm[self.layer_idx], fb.state_slots,
                            fb.query_start_locs, fb.seq_lens)
        hops.gated_group_norm(y, proj, base, self.norm_w, self.eps,
                              s.norm_groups, True, out, out_off)


class RoutedExperts(nn.Module):
    """Mixture-of-experts feed-forward. The router runs in fp32: "sigmoid"
    with group-limited choice and normalised weights, or "softmax" with a
    choice correction, identity experts and unnormalised scaled weights.
    Experts are `down act(up h)` ("relu2") or `down glu(gate h, up h)`
    ("clamped_glu"), without biases. The chosen (token, expert) pairs are laid
    out in per-expert segments, the two expert GEMMs run over the segments,
    and the caller folds the weighted sum of a token's rows into its residual
    kernel: forward returns (rows [padded rows, W], padpos [T, top], weights
    [T, top], identity weight [T] or None). A shared expert, if the spec has
    one, is run by `shared_forward`.

    Parameters are stacked [E, N, K] (each expert a torch-Linear matrix), the
    layout the matrix-core expert GEMM reads; gate and up matrices of an
    expert are neighbours ([2E, ff, K], read as [E, 2 ff, K])."""

    def __init__(self, spec: RoutedExpertsSpec, width: int,
                 dtype: torch.dtype):
        super().__init__()
        if (spec.router, spec.act) not in (("sigmoid", "relu2"),
                                           ("softmax", "clamped_glu")):
            raise ValueError("RoutedExperts: unknown router or activation")
        self.spec = spec
        self.width = width
        E, ff = spec.experts, spec.ff
        n = E + spec.identity
        self.router = nn.Parameter(torch.zeros(n, width, dtype=torch.float32))
        if spec.correction:
            self.correction = nn.Parameter(torch.zeros(n, dtype=torch.float32))
        if spec.act == "clamped_glu":
            self.gate_up = nn.Parameter(torch.zeros(2 * E, ff, width, dtype=dtype))
        else:
            self.up = nn.Parameter(torch.zeros(E, ff, width, dtype=dtype))
        self.down = nn.Parameter(torch.zeros(E, width, ff, dtype=dtype))
        if spec.shared_ff:
            self.shared_in = SectionedLinear(
                width, [("gate", spec.shared_ff, False),
                        ("up", spec.shared_ff, False), ("sg", 1, False)], dtype)
            self.shared_down = nn.Linear(spec.shared_ff, width, bias=False,
                                         dtype=dtype)

    def param_targets(self, prefix: str, ck: str):
        s = self.spec
        n = s.experts + s.identity
        t = {ck + ".router": (prefix + "router", 0, 0, n, 1.0)}
        if s.correction:
            t[ck + ".correction"] = (prefix + "correction", 0, 0, n, 1.0)
        for e in range(s.experts):
            if s.act == "clamped_glu":
                t[f"{ck}.e{e}.gate"] = (prefix + "gate_up", 0, 2 * e, 1, 1.0)
                t[f"{ck}.e{e}.up"] = (prefix + "gate_up", 0, 2 * e + 1, 1, 1.0)
            else:
                t[f"{ck}.e{e}.up"] = (prefix + "up", 0, e, 1, 1.0)
            t[f"{ck}.e{e}.down"] = (prefix + "down", 0, e, 1, 1.0)
        if s.shared_ff:
            t.update(self.shared_in.section_targets(
                prefix + "shared_in.",
                {"gate": ck + ".shared.gate", "up": ck + ".shared.up",
                 "sg": ck + ".shared.sg"}))
            t[ck + ".shared.down"] = (prefix + "shared_down.weight", 1, 0,
                                      s.shared_ff, 1.0)
        return t

    def route(self, h: torch.Tensor):
        """(idx, weights, identity weight or None)."""
        s = self.spec
        logits = F.linear(h.float(), self.router)
        if s.router == "softmax":
            return hops.moe_route_softmax(
                logits, self.correction if s.correction else None, s.top,
                s.groups, s.keep, s.experts, s.route_scale)
        idx, wts = hops.moe_route(logits, s.top, s.groups, s.keep,
                                  s.group_rank)
        return idx, wts, None

    def shared_forward(self, h: torch.Tensor):
        """(shared expert result [T, W], its projection buffer, the column
        of the gate logit in it)."""
        s = self.spec
        proj = self.shared_in(h)
        off = self.shared_in.offsets
        act = hops.glu_mul(proj, off["gate"], off["up"], s.shared_ff,
                           hops.GLU_CLAMPED, s.shared_limit)
        return self.shared_down(act), proj, off["sg"]

    def forward(self, h: torch.Tensor):
        s = self.spec
        T = h.shape[0]
        idx, wts, idw = self.route(h)
        glu = s.act == "clamped_glu"
        w1 = self.gate_up.view(s.experts, 2 * s.ff, self.width) if glu \
            else self.up
        bm = hops.expert_gemm_tile(h, w1, T * s.top)
        # chosen identity experts share one segment past the real experts'
        # that no GEMM visits
        segs = s.experts + (1 if s.identity else 0)
        row_tok, tile_off, counts, padpos = hops.moe_dispatch(idx, segs, bm)
        tile_off, counts = tile_off[:s.experts + 1], counts[:s.experts]
        n = row_tok.shape[0]
        act = torch.empty((n, s.ff), dtype=h.dtype, device=h.device)
        if glu:
            hops.expert_gemm(act, h, w1, row_tok, tile_off, counts,
                             hops.ACT_GLU_CLAMPED, bm, s.limit)
        else:
            hops.expert_gemm(act, h, w1, row_tok, tile_off, counts,
                             hops.ACT_RELU2, bm)
        rows = torch.empty((n, self.width), dtype=h.dtype, device=h.device)
        hops.expert_gemm(rows, act, self.down, None, tile_off, counts,
                         hops.ACT_NONE, bm)
        return rows, padpos, wts, idw
