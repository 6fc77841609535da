"""A plain, slow float64 implementation of the Vukotar equations, one function
per mechanism, sharing no code with the package. It works on whole sequences
(no cache, no batching, no portions) and is the yardstick for the engine in
tests/test_vukotar.py. It also makes small configurations and random
checkpoints.

Notation: h [T, W] is a sublayer's input, weights are [out, in], `w` maps
checkpoint tensor names to float64 tensors (already rounded to bf16, which is
how they are stored).

The design: x0 = embed[token] * s + sinusoid(position). A layer reads one
Dynamic-Tanh norm of the stream and adds two branches computed from it,
    x <- x + ls1 * attention(n(x)) + ls2 * experts(n(x)),
where attention is causal grouped-query softmax attention with a silent sink
(a one in the denominator) and no positional signal, and the feed-forward is a
mixture of squared-ReLU experts under a sigmoid router restricted to the best
groups of neighbouring experts. A layer may borrow all tensors of another
layer. Logits come from the embedding table itself and are soft-capped.
"""

import json
import math
import os

import torch

F64 = torch.float64


# ---------------------------------------------------------------- pieces ----

def sinusoid(T, width):
    """[T, width]: column 2i = sin(p / 10000^(2i/width)), column 2i+1 = cos."""
    out = torch.zeros(T, width, dtype=F64)
    for p in range(T):
        for c in range(width):
            ang = p * 10000.0 ** (-2.0 * (c // 2) / width)
            out[p, c] = math.sin(ang) if c % 2 == 0 else math.cos(ang)
    return out


def dynamic_tanh(x, alpha, weight, bias):
    """tanh(alpha * x) * weight + bias; no statistic of x is taken."""
    return torch.tanh(alpha * x) * weight + bias


def sink_attention(q, k, v, scale):
    """One head, causal. q, k [T, dk]; v [T, dv]. The weights of a row are
    exp(s_j) / (1 + sum_j exp(s_j)): a sink of score 0 that carries no value
    takes part in the normalisation."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for i in range(T):
        s = (k[:i + 1] @ q[i]) * scale
        e = torch.exp(s)
        out[i] = (e / (1.0 + e.sum())) @ v[:i + 1]
    return out


def route(z, top, groups, keep, gaps=None):
    """Router of one token. z [E] logits. Returns (chosen experts, weights).
    `gaps`, when a list, gets how far the choice was from another one: the
    distance between the worth of the last kept and the first dropped group,
    and between the last chosen and the first unchosen allowed score.
    Scores are sigmoids. The experts form `groups` equal runs of neighbours; a
    group is worth the sum of its two largest scores (its only score if it has
    one expert); only experts of the `keep` best groups may be chosen; the
    `top` largest of those are, weighted by score / (sum of chosen + 1e-20)."""
    E = z.shape[0]
    s = torch.sigmoid(z)
    size = E // groups
    worth = []
    for g in range(groups):
        part = sorted(s[g * size:(g + 1) * size].tolist(), reverse=True)
        worth.append(sum(part[:2]))
    best = sorted(range(groups), key=lambda g: (-worth[g], g))[:keep]
    allowed = [e for e in range(E) if e // size in best]
    ranked = sorted(allowed, key=lambda e: (-float(s[e]), e))
    chosen = ranked[:top]
    if gaps is not None:
        by_worth = sorted(worth, reverse=True)
        if keep < groups:
            gaps.append(by_worth[keep - 1] - by_worth[keep])
        if top < len(ranked):
            gaps.append(float(s[ranked[top - 1]] - s[ranked[top]]))
    total = sum(float(s[e]) for e in chosen) + 1e-20
    return chosen, [float(s[e]) / total for e in chosen]


def expert(h, up, down):
    """down (relu(up h))^2 for one token or many."""
    a = torch.relu(h @ up.T)
    return (a * a) @ down.T


# ---------------------------------------------------------------- layers ----

def attention_mixer(w, p, mc, h):
    H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    T = h.shape[0]
    q = (h @ w[p + "q"].T).view(T, H, dk)
    k = (h @ w[p + "k"].T).view(T, G, dk)
    v = (h @ w[p + "v"].T).view(T, G, dv)
    heads = []
    for a in range(H):
        g = a // (H // G)
        heads.append(sink_attention(q[:, a], k[:, g], v[:, g], mc["scale"]))
    return torch.cat(heads, dim=1) @ w[p + "o"].T


def moe_feed_forward(w, p, fc, h, picks=None, gaps=None):
    r = fc["router"]
    E, top = r["experts"], r["top"]
    z = h @ w[p + "router"].T
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        chosen, weights = route(z[t], top, r["groups"]["count"],
                                r["groups"]["keep"], gaps)
        if picks is not None:
            picks.append(chosen)
        for e, g in zip(chosen, weights):
            out[t] += g * expert(h[t], w[p + f"e{e}.up"], w[p + f"e{e}.down"])
    return out


def owner(config, i):
    """The layer whose tensors layer i uses."""
    while config["layers"][i].get("weights_of") is not None:
        i = config["layers"][i]["weights_of"]
    return i


def forward(config, w, tokens, streams=None, picks=None, gaps=None):
    """Logits [T, vocab] of one whole sequence. `streams`, when a list, gets
    the residual stream after every layer; `picks` the chosen experts of every
    layer and token; `gaps` how close every routing choice was (see route)."""
    W = config["width"]
    T = len(tokens)
    x = w["embed"][torch.tensor(tokens)] * config["embedding"]["scale"]
    x = x + sinusoid(T, W)
    for i, layer_ in enumerate(config["layers"]):
        lp = f"l{owner(config, i)}."
        h = dynamic_tanh(x, w[lp + "norm1.alpha"], w[lp + "norm1"],
                         w[lp + "norm1.b"])
        add = w[lp + "ls1"] * attention_mixer(w, lp + "mix.", layer_["mixer"], h)
        if layer_.get("mlp") is not None:
            mine = [] if picks is not None else None
            add = add + w[lp + "ls2"] * moe_feed_forward(
                w, lp + "mlp.", layer_["mlp"], h, mine, gaps)
            if picks is not None:
                picks.append(mine)
        x = x + add
        if streams is not None:
            streams.append(x.clone())
    h = dynamic_tanh(x, w["final.norm.alpha"], w["final.norm"],
                     w["final.norm.b"])
    logits = h @ w["embed"].T
    cap = config["logit_softcap"]
    return cap * torch.tanh(logits / cap)


# ------------------------------------------------- configs and checkpoints ----

def attn_cfg(heads, kv_heads, dim, vdim, scale):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "scale": scale}


def moe_cfg(ff, experts, top, groups, keep):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top,
                       "groups": {"count": groups, "keep": keep}}}


def layer(mixer, mlp=None, weights_of=None):
    d = {"type": "attention", "mixer": dict(mixer),
         "mlp": None if mlp is None else json.loads(json.dumps(mlp))}
    if weights_of is not None:
        d["weights_of"] = weights_of
    return d


def make_config(width, vocab, layers, eps=1e-5, embed_scale=0.7, softcap=20.0):
    return {"architecture": "Vukotar", "width": width, "vocab": vocab,
            "norm": {"eps": eps}, "embedding": {"scale": embed_scale},
            "logit_softcap": softcap, "layers": layers}


def make_weights(config, seed=0):
    """Random weights (already rounded to bf16) under checkpoint names."""
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    w = {}

    def rnd(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g) * std + mean

    def lin(out, inn, gain=1.0):
        return rnd(out, inn, std=gain * inn ** -0.5)

    def norm(name):
        w[name] = rnd(W, std=0.2, mean=1.0)
        w[name + ".b"] = rnd(W, std=0.1)
        w[name + ".alpha"] = rnd(1, std=0.05, mean=0.6)[0]

    w["embed"] = rnd(config["vocab"], W)
    norm("final.norm")
    for i, layer_ in enumerate(config["layers"]):
        if layer_.get("weights_of") is not None:
            continue
        lp, mc = f"l{i}.", layer_["mixer"]
        p = lp + "mix."
        norm(lp + "norm1")
        H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
        w[p + "q"], w[p + "k"] = lin(H * dk, W, 2.0), lin(G * dk, W, 2.0)
        w[p + "v"], w[p + "o"] = lin(G * dv, W), lin(W, H * dv)
        w[lp + "ls1"] = rnd(W, std=0.2, mean=0.7)
        fc = layer_.get("mlp")
        if fc is not None:
            ff, E = fc["expert"]["ff"], fc["router"]["experts"]
            for e in range(E):
                w[lp + f"mlp.e{e}.up"] = lin(ff, W, 1.5)
                w[lp + f"mlp.e{e}.down"] = lin(W, ff)
            w[lp + "mlp.router"] = lin(E, W, 3.0)
            w[lp + "ls2"] = rnd(W, std=0.2, mean=0.7)
    return {k: v.to(torch.bfloat16).to(F64) for k, v in w.items()}


def save_checkpoint(path, config, w):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()},
              os.path.join(path, "model.safetensors"))
    return path
