"""A plain, slow float64 implementation of the Nosalorn equations, one function
per mechanism, sharing no code with the package. It works on whole sequences
(no cache, no batching, no portions) and is the yardstick for the engine in
tests/test_nosalorn.py. It also makes small configurations and random
checkpoints.

Notation: h [T, W] is a sublayer's input, weights are [out, in], `w` maps
checkpoint tensor names to float64 tensors (already rounded to bf16, which is
how they are stored).

The design: x0 = embed[token] * s. A layer is pre-norm,
    x <- x + mixer(n1(x));  x <- x + ff(n2(x))          (ff optional),
with weighted RMS norms. The mixer is one of
  * softmax attention with biased projections, a partly rotated head (YaRN
    frequencies), a sliding window that also keeps the first tokens, and
    values blended with the values of the first such layer;
  * linear attention with a fixed decay per head (silu on q, k, v; a norm
    over all heads, a sigmoid gate);
  * a Mamba-2 state-space layer (short causal filter, softplus step, scalar
    decay per head, gate before a grouped norm).
The feed-forward is SwiGLU, or a mixture of clamped-GLU experts under a
softmax router with a choice correction, group-limited choice, identity
experts and a gated shared expert. Logits = head(final norm(x)) * scale.
"""

import json
import math
import os

import torch

F64 = torch.float64


# ---------------------------------------------------------------- pieces ----

def rms_norm(x, weight, eps):
    """x / sqrt(mean(x^2) + eps) * weight over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * weight


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rot_frequencies(rot):
    """(f [dims/2], amplitude) of a rotation config {dims, base, scaling?}."""
    dims, base = rot["dims"], float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    sc = rot.get("scaling")
    if not sc:
        return torch.tensor(f, dtype=F64), 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def turn_dim(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
    out = []
    for i in range(half):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(f[i] / factor * ramp + f[i] * (1.0 - ramp))
    return torch.tensor(out, dtype=F64), 0.1 * math.log(factor) + 1.0


def rotate(x, rot):
    """x [T, dim] of one head at positions 0..T-1: the first rot.dims
    dimensions are rotated in pairs (i, i + dims/2), the rest pass."""
    if not rot or not rot.get("dims"):
        return x
    f, amp = rot_frequencies(rot)
    half = rot["dims"] // 2
    T = x.shape[0]
    ang = torch.arange(T, dtype=F64).unsqueeze(1) * f.unsqueeze(0)
    c, s = torch.cos(ang) * amp, torch.sin(ang) * amp
    u, v = x[:, :half], x[:, half:2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[:, 2 * half:]], dim=1)


def windowed_attention(q, k, v, scale, size, keep_first):
    """One head. Row i sees j <= i with i - j < size or j < keep_first
    (size 0: all j <= i)."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for i in range(T):
        js = [j for j in range(i + 1)
              if size <= 0 or i - j < size or j < keep_first]
        s = (k[js] @ q[i]) * scale
        p = torch.exp(s - s.max())
        out[i] = (p / p.sum()) @ v[js]
    return out


def attention_mixer(h, w, p, mc, v_first):
    """Returns (mixer output [T, W], this layer's raw values [T, G*vdim]).
    `v_first`: the first value-mixing layer's values, or None when this layer
    is that first layer or does not mix."""
    H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
    T = h.shape[0]
    q = h @ w[p + "q"].T + w[p + "q.b"]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    v = h @ w[p + "v"].T + w[p + "v.b"]
    raw_v = v
    if v_first is not None:
        lam = w[p + "vmix"]
        v = (1.0 - lam) * v + lam * v_first
    mask = mc.get("mask") or {}
    heads = []
    for a in range(H):
        g = a // (H // G)
        qa = rotate(q[:, a * dk:(a + 1) * dk], mc.get("rot"))
        kg = rotate(k[:, g * dk:(g + 1) * dk], mc.get("rot"))
        heads.append(windowed_attention(
            qa, kg, v[:, g * dv:(g + 1) * dv], mc["scale"],
            int(mask.get("size", 0)), int(mask.get("keep_first", 0))))
    return torch.cat(heads, dim=1) @ w[p + "o"].T, raw_v


def decay_memory(q, k, v, decay, gain, state=None):
    """One head of a linear recurrence read token by token:
    S_t = decay[t] * S_(t-1) + gain[t] * k_t v_t^T,  o_t = S_t^T q_t."""
    T, dk = k.shape
    S = torch.zeros(dk, v.shape[1], dtype=F64) if state is None else state
    out = torch.zeros(T, v.shape[1], dtype=F64)
    for t in range(T):
        S = decay[t] * S + gain[t] * torch.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out


def lightning_mixer(h, w, p, mc, eps):
    H, dk, dv = mc["heads"], mc["dim"], mc["vdim"]
    T = h.shape[0]
    q, k, v = silu(h @ w[p + "q"].T), silu(h @ w[p + "k"].T), silu(h @ w[p + "v"].T)
    ones = torch.ones(T, dtype=F64)
    heads = [decay_memory(q[:, a * dk:(a + 1) * dk], k[:, a * dk:(a + 1) * dk],
                          v[:, a * dv:(a + 1) * dv],
                          ones * float(mc["decay"][a]), ones)
             for a in range(H)]
    o = rms_norm(torch.cat(heads, dim=1), w[p + "norm"], eps)
    o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


def causal_filter(u, taps_w, bias):
    """u [T, C]; taps_w [C, taps], the last column weighs the current token;
    inputs before the start are zero."""
    T, C = u.shape
    taps = taps_w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        acc = bias.clone()
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                acc = acc + taps_w[:, j] * u[src]
        out[t] = acc
    return out


def mamba2_mixer(h, w, p, mc, eps):
    H, dv, N, G = mc["heads"], mc["vdim"], mc["state"], mc["groups"]
    inner = H * dv
    T = h.shape[0]
    zxbcdt = h @ w[p + "in"].T
    z = zxbcdt[:, :inner]
    xbc = zxbcdt[:, inner:2 * inner + 2 * G * N]
    dt = softplus(zxbcdt[:, 2 * inner + 2 * G * N:] + w[p + "dt_bias"])
    xbc = silu(causal_filter(xbc, w[p + "conv"], w[p + "conv.b"]))
    x, B, C = xbc[:, :inner], xbc[:, inner:inner + G * N], xbc[:, inner + G * N:]
    heads = []
    for a in range(H):
        g = a // (H // G)
        xa = x[:, a * dv:(a + 1) * dv]
        y = decay_memory(C[:, g * N:(g + 1) * N], B[:, g * N:(g + 1) * N], xa,
                         torch.exp(-torch.exp(w[p + "A_log"][a]) * dt[:, a]),
                         dt[:, a])
        heads.append(y + w[p + "D"][a] * xa)
    y = torch.cat(heads, dim=1) * silu(z)
    parts = mc["norm_groups"]
    y = rms_norm(y.view(T, parts, inner // parts),
                 torch.ones((), dtype=F64), eps).reshape(T, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


def dense_ff(h, w, p):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def clamped_expert(h, w, p, limit):
    g = torch.clamp(h @ w[p + "gate"].T, max=limit)
    u = torch.clamp(h @ w[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w[p + "down"].T


def route(z, corr, top, groups, keep, scale, gaps=None):
    """z [n] router logits of one token over experts and identity experts.
    Returns [(index, weight)]. `gaps`, when a list, receives how close the
    choice was (smallest gap between a chosen and a not chosen score, and
    between a kept and a dropped group)."""
    n = z.shape[0]
    s = torch.softmax(z, dim=0)
    c = s + corr
    allowed = [True] * n
    if groups > 1:
        size = n // groups
        worth = [max(float(c[j]) for j in range(g * size, (g + 1) * size))
                 for g in range(groups)]
        order = sorted(range(groups), key=lambda g: (-worth[g], g))
        kept = order[:keep]
        for j in range(n):
            allowed[j] = (j // size) in kept
        if gaps is not None and keep < groups:
            gaps.append(worth[order[keep - 1]] - worth[order[keep]])
    cand = sorted([j for j in range(n) if allowed[j]],
                  key=lambda j: (-float(c[j]), j))
    if gaps is not None and len(cand) > top:
        gaps.append(float(c[cand[top - 1]] - c[cand[top]]))
    return [(j, float(s[j]) * scale) for j in cand[:top]]


def moe_ff(h, w, p, fc, picks=None, gaps=None):
    r = fc["router"]
    E, ident = r["experts"], int(r.get("identity", 0))
    g = r.get("groups") or {"count": 1, "keep": 1}
    T, W = h.shape
    out = torch.zeros(T, W, dtype=F64)
    corr = w.get(p + "correction")
    if corr is None:
        corr = torch.zeros(E + ident, dtype=F64)
    hz = h @ w[p + "router"].T
    for t in range(T):
        chosen = route(hz[t], corr, r["top"], g["count"], g["keep"],
                       float(r.get("scale", 1.0)), gaps)
        if picks is not None:
            picks.append([j for j, _ in chosen])
        for j, wt in chosen:
            if j >= E:
                out[t] += wt * h[t]
            else:
                out[t] += wt * clamped_expert(h[t:t + 1], w, f"{p}e{j}.",
                                              float(fc["expert"]["limit"]))[0]
    sh = fc.get("shared")
    if sh:
        y = clamped_expert(h, w, p + "shared.", float(sh["limit"]))
        out = out + y * torch.sigmoid(h @ w[p + "shared.sg"].T)
    return out


# ----------------------------------------------------------------- model ----

def forward(config, w, tokens, streams=None, picks=None, gaps=None):
    """Logits [T, vocab] of one whole sequence. `streams`, when a list,
    receives the residual stream after every layer."""
    eps = float(config["norm"]["eps"])
    ids = torch.as_tensor(tokens, dtype=torch.long)
    x = w["embed"][ids] * float(config["embedding"]["scale"])
    v_first = None
    for i, layer_ in enumerate(config["layers"]):
        lp, mc, kind = f"l{i}.", layer_["mixer"], layer_["type"]
        h = rms_norm(x, w[lp + "norm1"], eps)
        if kind == "attention":
            mixes = bool(mc.get("v_mix"))
            y, raw_v = attention_mixer(h, w, lp + "mix.", mc,
                                       v_first if mixes else None)
            if mixes and v_first is None:
                v_first = raw_v
        elif kind == "lightning":
            y = lightning_mixer(h, w, lp + "mix.", mc, eps)
        elif kind == "mamba2":
            y = mamba2_mixer(h, w, lp + "mix.", mc, eps)
        else:
            raise ValueError(kind)
        x = x + y
        fc = layer_.get("mlp")
        if fc is not None:
            h = rms_norm(x, w[lp + "norm2"], eps)
            if fc["kind"] == "dense":
                x = x + dense_ff(h, w, lp + "mlp.")
            else:
                x = x + moe_ff(h, w, lp + "mlp.", fc, picks, gaps)
        if streams is not None:
            streams.append(x.clone())
    h = rms_norm(x, w["final.norm"], eps)
    return (h @ w["head"].T) * float(config.get("logit_scale", 1.0))


# ------------------------------------------------- configs and checkpoints ----

def attn_cfg(heads, kv_heads, dim, vdim, scale=None, size=0, keep_first=0,
             rot_dims=0, base=10000.0, scaling=None, v_mix=False):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
         "scale": dim ** -0.5 if scale is None else scale, "v_mix": v_mix,
         "mask": {"size": size, "keep_first": keep_first}}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
        if scaling:
            m["rot"]["scaling"] = dict(scaling)
    return m


def lightning_cfg(heads, dim, vdim, decay):
    return {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}


def mamba2_cfg(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups,
            "conv": conv, "norm_groups": norm_groups}


def dense_cfg(ff):
    return {"kind": "dense", "ff": ff}


def moe_cfg(ff, experts, top, identity=0, groups=1, keep=1, scale=1.0,
            limit=7.0, shared_ff=0, shared_limit=7.0):
    m = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
         "router": {"experts": experts, "top": top, "identity": identity,
                    "scale": scale,
                    "groups": {"count": groups, "keep": keep}}}
    if shared_ff:
        m["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return m


def layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": json.loads(json.dumps(mixer)),
            "mlp": None if mlp is None else json.loads(json.dumps(mlp))}


def make_config(width, vocab, layers, eps=1e-5, embed_scale=4.0,
                logit_scale=0.5):
    return {"architecture": "Nosalorn", "width": width, "vocab": vocab,
            "norm": {"eps": eps}, "embedding": {"scale": embed_scale},
            "logit_scale": logit_scale, "layers": layers}


def make_weights(config, seed=0):
    """Random weights (already rounded to bf16) under checkpoint names."""
    g = torch.Generator().manual_seed(seed)
    W = config["width"]
    w = {}

    def rnd(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=g) * std + mean

    def lin(out, inn, gain=1.0):
        return rnd(out, inn, std=gain * inn ** -0.5)

    def glu(p, ff):
        w[p + "gate"], w[p + "up"] = lin(ff, W, 1.5), lin(ff, W, 1.5)
        w[p + "down"] = lin(W, ff)

    w["embed"] = rnd(config["vocab"], W, std=0.5)
    w["head"] = lin(config["vocab"], W)
    w["final.norm"] = rnd(W, std=0.2, mean=1.0)
    for i, layer_ in enumerate(config["layers"]):
        lp, mc, kind = f"l{i}.", layer_["mixer"], layer_["type"]
        p = lp + "mix."
        w[lp + "norm1"] = rnd(W, std=0.2, mean=1.0)
        if kind == "attention":
            H, G, dk, dv = mc["heads"], mc["kv_heads"], mc["dim"], mc["vdim"]
            w[p + "q"], w[p + "k"] = lin(H * dk, W, 2.0), lin(G * dk, W, 2.0)
            w[p + "v"], w[p + "o"] = lin(G * dv, W), lin(W, H * dv)
            w[p + "q.b"], w[p + "k.b"] = rnd(H * dk, std=0.3), rnd(G * dk, std=0.3)
            w[p + "v.b"] = rnd(G * dv, std=0.3)
            if mc.get("v_mix"):
                w[p + "vmix"] = rnd(1, std=0.1, mean=0.4)[0]
        elif kind == "lightning":
            H, dk, dv = mc["heads"], mc["dim"], mc["vdim"]
            w[p + "q"], w[p + "k"] = lin(H * dk, W, 1.5), lin(H * dk, W, 1.5)
            w[p + "v"], w[p + "g"] = lin(H * dv, W, 1.5), lin(H * dv, W, 1.5)
            w[p + "norm"] = rnd(H * dv, std=0.2, mean=1.0)
            w[p + "o"] = lin(W, H * dv)
        elif kind == "mamba2":
            H, dv, N, G = mc["heads"], mc["vdim"], mc["state"], mc["groups"]
            inner, ch = H * dv, H * dv + 2 * G * N
            w[p + "in"] = lin(2 * inner + 2 * G * N + H, W, 1.5)
            w[p + "conv"] = rnd(ch, mc["conv"], std=mc["conv"] ** -0.5)
            w[p + "conv.b"] = rnd(ch, std=0.2)
            w[p + "dt_bias"] = rnd(H, std=0.5, mean=-1.0)
            w[p + "A_log"] = rnd(H, std=0.7, mean=-1.0)
            w[p + "D"] = rnd(H, std=0.5, mean=1.0)
            w[p + "norm"] = rnd(inner, std=0.2, mean=1.0)
            w[p + "o"] = lin(W, inner)
        fc = layer_.get("mlp")
        if fc is None:
            continue
        w[lp + "norm2"] = rnd(W, std=0.2, mean=1.0)
        if fc["kind"] == "dense":
            glu(lp + "mlp.", fc["ff"])
            continue
        r = fc["router"]
        n = r["experts"] + int(r.get("identity", 0))
        for e in range(r["experts"]):
            glu(lp + f"mlp.e{e}.", fc["expert"]["ff"])
        w[lp + "mlp.router"] = lin(n, W, 3.0)
        w[lp + "mlp.correction"] = rnd(n, std=0.05)
        if fc.get("shared"):
            glu(lp + "mlp.shared.", fc["shared"]["ff"])
            w[lp + "mlp.shared.sg"] = lin(1, W, 2.0)
    return {k: v.to(torch.bfloat16).to(F64) for k, v in w.items()}


def save_checkpoint(path, config, w):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(config, f)
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in w.items()},
              os.path.join(path, "model.safetensors"))
    return path
