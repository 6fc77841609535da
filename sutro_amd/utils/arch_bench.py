"""Prefill and decode throughput of the layer-list decoders (Vodinex,
Ruludra, Vukotar, Nosalorn) beside the Qwen3 decoder of equal size (same width, layers,
heads, key/value heads, head size and feed-forward width; for Vukotar the
Qwen3 mixture-of-experts decoder with as many experts of the same inner
width and as many choices a token), all with random weights, all through the
engine's own batch path (scheduler, paged cache, state slots, decode
hipGraphs). Used by `bench.py --arch-compare`.

prefill: `seqs` prompts of `prompt` tokens in one engine step, tokens/s.
decode:  `seqs` sequences, each with `prompt` tokens of context, one token a
         step through the captured decode graph, tokens/s.
"""

from __future__ import annotations

import time
from typing import Dict, List

import torch

from ..engine.config import EngineConfig
from ..engine.engine import LLMEngine
from ..models.hybrid_spec import (AttnMixerSpec, DecayAttnMixerSpec,
                                  DeltaMixerSpec, HybridLayerSpec, HybridSpec,
                                  SSDMixerSpec,
                                  LatentAttnMixerSpec, MLSTMMixerSpec,
                                  ParallelMixerSpec, RoutedExpertsSpec,
                                  TiedAttnMixerSpec)
from ..models.registry import ModelSpec

# name -> (width, layers, heads, kv_heads, head size, ff, vocab)
SIZES = {
    "1b": (2048, 4, 16, 4, 128, 8192, 32768),
    "8b": (4096, 4, 32, 8, 128, 12288, 32768),
    "tiny": (192, 2, 3, 1, 64, 384, 320),
}


def hybrid_spec(name: str, chunk: int = 1024) -> HybridSpec:
    W, L, H, G, D, ff, V = SIZES[name]
    left = AttnMixerSpec(heads=H, kv_heads=G, dim=D, vdim=D, scale=D ** -0.5,
                         rot_dims=D // 2, rot_base=10000.0, chunk=chunk)
    right = DeltaMixerSpec(heads=H // 2, kv_heads=H // 2, dim=D, vdim=D, conv=4,
                           decay_rank=32, gate_rank=32)
    solo = DeltaMixerSpec(heads=H, kv_heads=H, dim=D, vdim=D, conv=4,
                          decay_rank=32, gate_rank=32)
    layers: List[HybridLayerSpec] = []
    for i in range(L):
        if i == 0:
            layers.append(HybridLayerSpec("channel_delta", solo, ff=ff))
        else:
            layers.append(HybridLayerSpec(
                "parallel", ParallelMixerSpec(left, right, 0.75, 0.4), ff=ff))
    return HybridSpec(name=f"vodinex-{name}", arch="vodinex", hidden_size=W,
                      vocab_size=V, layers=tuple(layers), norm_eps=1e-6,
                      residual_mult=0.8, max_context=1 << 20)


def sandwich_spec(name: str, window: int = 1024) -> HybridSpec:
    """Ruludra at the same width, depth, heads, head size and feed-forward
    width: tied-value window attention, latent attention (latent 256, query
    latent W/2), an mLSTM layer without feed-forward, and a latent layer that
    reads the first one's cached latent, in turn."""
    W, L, H, G, D, ff, V = SIZES[name]
    rank = min(256, 2 * D)
    attn = TiedAttnMixerSpec(heads=H, kv_heads=G, dim=D, scale=D ** -0.5,
                             window=window, temp_coef=0.2, temp_every=128)
    lat = LatentAttnMixerSpec(heads=H, dim=D, vdim=D, q_rank=W // 2,
                              kv_rank=rank, scale=D ** -0.5, window=window)
    rec = MLSTMMixerSpec(heads=max(1, H // 2), dim=D, vdim=D, gate_cap=10.0)
    layers: List[HybridLayerSpec] = []
    for i in range(L):
        k = i % 4
        if k == 0:
            layers.append(HybridLayerSpec("attention", attn, ff=ff,
                                          ff_kind="poly_norm"))
        elif k == 1:
            layers.append(HybridLayerSpec("latent_attention", lat, ff=ff,
                                          ff_kind="poly_norm"))
        elif k == 2:
            layers.append(HybridLayerSpec("mlstm", rec, ff=0,
                                          ff_kind="poly_norm"))
        else:
            layers.append(HybridLayerSpec(
                "latent_attention",
                LatentAttnMixerSpec(heads=H, dim=D, vdim=D, q_rank=W // 2,
                                    kv_rank=rank, scale=D ** -0.5,
                                    window=window, kv_from=i - 2),
                ff=ff, ff_kind="poly_norm"))
    return HybridSpec(name=f"ruludra-{name}", arch="ruludra", hidden_size=W,
                      vocab_size=V, layers=tuple(layers), norm_eps=1e-6,
                      max_context=1 << 20, bigram=(65521, 131, 7),
                      pos_base=10000.0, logit_scale=0.5)


# routed feed-forwards at a size: experts, choices a token, inner width as a
# fraction of the dense feed-forward width
MOE_EXPERTS, MOE_TOP, MOE_FF_DIV = 32, 4, 4


def parallel_spec(name: str) -> HybridSpec:
    """Vukotar at the same width, depth, heads and head size: every layer a
    sink-softmax attention beside 32 squared-ReLU experts (8 groups of 4, the
    best 4 groups stay, 4 experts a token, inner width ff/4); the second half
    of the layers runs the parameters of the first half again."""
    W, L, H, G, D, ff, V = SIZES[name]
    attn = AttnMixerSpec(heads=H, kv_heads=G, dim=D, vdim=D, scale=D ** -0.5,
                         qk_norm=False, bias=False, out_gate=False, sink=True)
    moe = RoutedExpertsSpec(ff=max(64, ff // MOE_FF_DIV), experts=MOE_EXPERTS,
                            top=MOE_TOP, groups=8, keep=4)
    own = max(1, L // 2)
    layers = [HybridLayerSpec("attention", attn, moe=moe,
                              weights_of=None if i < own else i % own)
              for i in range(L)]
    return HybridSpec(name=f"vukotar-{name}", arch="vukotar", hidden_size=W,
                      vocab_size=V, layers=tuple(layers), norm_eps=1e-6,
                      max_context=1 << 20, pos_base=10000.0, embed_scale=0.7,
                      logit_softcap=25.0, tie_embeddings=True,
                      num_experts=MOE_EXPERTS)


def prenorm_spec(name: str, window: int = 1024) -> HybridSpec:
    """Nosalorn at the same width, depth, heads and head size: a Mamba-2
    layer (state 128) with a dense SwiGLU feed-forward, then window-1024
    rotary attention (64 kept first tokens, YaRN, blended values), fixed-decay
    linear attention and attention again, each beside 28 clamped-GLU experts
    + 4 identity experts (8 groups of 4, the best 4 stay, 4 a token, inner
    width ff/4) and a gated shared expert of the same width."""
    W, L, H, G, D, ff, V = SIZES[name]
    attn = AttnMixerSpec(heads=H, kv_heads=G, dim=D, vdim=D, scale=D ** -0.5,
                         rot_dims=D // 2, rot_base=10000.0, window=window,
                         keep_first=64, rot_scaling=(4.0, 4096.0, 32.0, 1.0),
                         qk_norm=False, bias=True, out_bias=False,
                         out_gate=False, v_mix=True)
    ssd = SSDMixerSpec(heads=H, vdim=D, state=min(128, D), groups=G, conv=4,
                       norm_groups=G)
    lin = DecayAttnMixerSpec(heads=H, dim=D, vdim=D, decay=tuple(
        1.0 - 2.0 ** (-2.0 - 6.0 * i / max(1, H - 1)) for i in range(H)))
    eff = max(64, ff // MOE_FF_DIV)
    moe = RoutedExpertsSpec(ff=eff, experts=MOE_EXPERTS - 4, top=MOE_TOP,
                            groups=8, keep=4, group_rank=1, router="softmax",
                            act="clamped_glu", identity=4, route_scale=2.0,
                            correction=True, limit=7.0, shared_ff=eff,
                            shared_limit=7.0)
    layers: List[HybridLayerSpec] = []
    for i in range(L):
        k = i % 4
        if k == 0:
            layers.append(HybridLayerSpec("mamba2", ssd, ff=ff,
                                          ff_kind="swiglu"))
        elif k == 2:
            layers.append(HybridLayerSpec("lightning", lin, ff_kind="swiglu",
                                          moe=moe))
        else:
            layers.append(HybridLayerSpec("attention", attn, ff_kind="swiglu",
                                          moe=moe))
    return HybridSpec(name=f"nosalorn-{name}", arch="nosalorn", hidden_size=W,
                      vocab_size=V, layers=tuple(layers), norm_eps=1e-6,
                      max_context=1 << 20, embed_scale=4.0, logit_scale=0.5,
                      num_experts=MOE_EXPERTS - 4)


def moe_spec(name: str) -> ModelSpec:
    """The Qwen3 mixture-of-experts decoder with as many experts of the same
    inner width and as many choices a token (softmax router, SwiGLU
    experts)."""
    W, L, H, G, D, ff, V = SIZES[name]
    return ModelSpec(name=f"qwen3moe-{name}", arch="qwen3_moe", hidden_size=W,
                     num_layers=L, num_heads=H, num_kv_heads=G, head_dim=D,
                     intermediate_size=ff, vocab_size=V, max_context=1 << 20,
                     num_experts=MOE_EXPERTS, experts_per_token=MOE_TOP,
                     moe_intermediate_size=max(64, ff // MOE_FF_DIV))


def dense_spec(name: str) -> ModelSpec:
    W, L, H, G, D, ff, V = SIZES[name]
    return ModelSpec(name=f"qwen3-{name}", arch="qwen3", hidden_size=W,
                     num_layers=L, num_heads=H, num_kv_heads=G, head_dim=D,
                     intermediate_size=ff, vocab_size=V, max_context=1 << 20)


def _measure(spec, device: str, seqs: int, prompt: int, steps: int,
             warmup: int) -> Dict[str, float]:
    page = 32
    blocks = seqs * ((prompt + steps + warmup + 2 * page) // page + 1) + 2
    cfg = EngineConfig(spec=spec, device=device, max_model_len=prompt + steps
                       + warmup + 2 * page, max_num_seqs=seqs,
                       num_kv_blocks=blocks,
                       max_tokens_per_step=seqs * prompt + seqs)
    eng = LLMEngine(cfg)
    g = torch.Generator().manual_seed(0)

    def sync():
        if device.startswith("cuda"):
            torch.cuda.synchronize()

    def prompts():
        return [torch.randint(3, spec.vocab_size, (prompt,), generator=g).tolist()
                for _ in range(seqs)]

    def prefill():
        reqs = [eng.new_replay_request() for _ in range(seqs)]
        toks = prompts()
        sync()
        t0 = time.perf_counter()
        eng.replay_step([(r, t, [prompt - 1]) for r, t in zip(reqs, toks)])
        sync()
        return reqs, time.perf_counter() - t0

    # prefill: first pass warms GEMM selection, later ones are timed
    times = []
    reqs = None
    for i in range(3):
        if reqs is not None:
            for r in reqs:
                eng.finish_replay_request(r)
        reqs, dt = prefill()
        if i:
            times.append(dt)
    out = {"prefill_tok_s": seqs * prompt / min(times)}
    # decode: continue the last prefilled batch
    for i in range(warmup + steps):
        if i == warmup:
            sync()
            t0 = time.perf_counter()
        eng.replay_step([(r, [7 + i % 11], [0]) for r in reqs])
    sync()
    out["decode_tok_s"] = seqs * steps / (time.perf_counter() - t0)
    out["decode_graph"] = eng.graph_runner is not None
    return out


MAKERS = {"vodinex": hybrid_spec, "qwen3": dense_spec,
          "ruludra": sandwich_spec, "vukotar": parallel_spec,
          "qwen3moe": moe_spec, "nosalorn": prenorm_spec}


def run_compare(sizes: List[str], device: str, seqs: int, prompt: int,
                steps: int, warmup: int,
                models=("vodinex", "qwen3")) -> List[dict]:
    rows = []
    for name in sizes:
        for kind in models:
            spec = MAKERS[kind](name)
            r = _measure(spec, device, seqs, prompt, steps, warmup)
            r.update(model=spec.name, kind=kind, size=name, seqs=seqs,
                     prompt=prompt, params=spec.param_count())
            rows.append(r)
            if device.startswith("cuda"):
                torch.cuda.empty_cache()
    return rows
