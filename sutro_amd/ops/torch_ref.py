"""Pure-PyTorch reference implementations of every engine op.

These are the CPU execution path AND the numerics oracle for the CDNA4 HIP
kernels (GPU tests compare the HIP kernels against these in fp32).
All reductions accumulate in fp32.
"""

from __future__ import annotations

import torch


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    y = xf * torch.rsqrt(var + eps)
    return (y * weight.float()).to(x.dtype)


def fused_add_rmsnorm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
):
    """residual += x; return (rmsnorm(residual), residual)."""
    res = (residual.float() + x.float())
    y = rmsnorm(res, weight, eps)
    return y, res.to(x.dtype)


def silu_mul(x: torch.Tensor) -> torch.Tensor:
    gate, up = x.chunk(2, dim=-1)
    return (torch.nn.functional.silu(gate.float()) * up.float()).to(x.dtype)


def rope_cos_sin(max_len: int, head_dim: int, theta: float) -> torch.Tensor:
    """[max_len, head_dim] fp32 table: first half cos, second half sin (NeoX)."""
    half = head_dim // 2
    inv_freq = 1.0 / (theta ** (torch.arange(half, dtype=torch.float64) / half))
    t = torch.arange(max_len, dtype=torch.float64)
    freqs = torch.outer(t, inv_freq)
    return torch.cat([freqs.cos(), freqs.sin()], dim=-1).float()


def apply_rope(q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor,
               cos_sin: torch.Tensor):
    """NeoX rotate-half RoPE. q: [T, Hq, D], k: [T, Hk, D], positions: [T]."""
    d = q.shape[-1]
    half = d // 2
    cs = cos_sin[positions]              # [T, D]
    cos = cs[:, :half].unsqueeze(1)      # [T, 1, half]
    sin = cs[:, half:].unsqueeze(1)

    def rot(x: torch.Tensor) -> torch.Tensor:
        xf = x.float()
        x1, x2 = xf[..., :half], xf[..., half:]
        return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).to(x.dtype)

    return rot(q), rot(k)


def write_kv_cache(
    k: torch.Tensor, v: torch.Tensor,
    k_cache: torch.Tensor, v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    """k/v: [T, Hk, D]; caches: [num_blocks, Hk, block_size, D]; slots: [T]."""
    nb, hk, bs, d = k_cache.shape
    blk = slot_mapping // bs
    off = slot_mapping % bs
    k_cache[blk, :, off] = k.to(k_cache.dtype)
    v_cache[blk, :, off] = v.to(v_cache.dtype)


def paged_attention(
    q: torch.Tensor,                 # [T, Hq, D] (new tokens, flat over seqs)
    k_cache: torch.Tensor,           # [num_blocks, Hk, bs, D]
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,      # [S, max_blocks] int32
    seq_lens: torch.Tensor,          # [S] total length incl. this step's tokens
    query_start_locs: torch.Tensor,  # [S+1] cu-seqlens of new tokens
    scale: float,
) -> torch.Tensor:
    """Causal attention of each seq's new tokens against its full cached KV.

    New tokens MUST already be written to the cache (write_kv_cache first).
    """
    T, hq, d = q.shape
    nb, hk, bs, _ = k_cache.shape
    group = hq // hk
    out = torch.empty_like(q)
    S = seq_lens.numel()
    for s in range(S):
        q0, q1 = int(query_start_locs[s]), int(query_start_locs[s + 1])
        nq = q1 - q0
        if nq == 0:
            continue
        L = int(seq_lens[s])
        nblk = (L + bs - 1) // bs
        blocks = block_tables[s, :nblk].long()
        keys = k_cache[blocks].transpose(0, 1).reshape(hk, nblk * bs, d)[:, :L].float()
        vals = v_cache[blocks].transpose(0, 1).reshape(hk, nblk * bs, d)[:, :L].float()
        qs = q[q0:q1].float()  # [nq, hq, d]
        # head-major: [hq, nq, d]
        qs = qs.transpose(0, 1)
        kh = keys.repeat_interleave(group, dim=0)   # [hq, L, d]
        vh = vals.repeat_interleave(group, dim=0)
        scores = torch.einsum("hqd,hkd->hqk", qs, kh) * scale
        # causal mask: new token i (absolute pos L-nq+i) sees keys <= its pos
        kpos = torch.arange(L, device=q.device)
        qpos = torch.arange(L - nq, L, device=q.device)
        mask = kpos.unsqueeze(0) > qpos.unsqueeze(1)  # [nq, L]
        scores.masked_fill_(mask.unsqueeze(0), float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        o = torch.einsum("hqk,hkd->hqd", probs, vh)   # [hq, nq, d]
        out[q0:q1] = o.transpose(0, 1).to(out.dtype)
    return out


def mean_pool_normalize(
    hidden: torch.Tensor,            # [T, H] flat hidden states
    query_start_locs: torch.Tensor,  # [S+1]
) -> torch.Tensor:
    """Per-sequence mean pool over tokens + L2 normalize -> [S, H]."""
    S = query_start_locs.numel() - 1
    out = torch.empty((S, hidden.shape[-1]), dtype=torch.float32, device=hidden.device)
    for s in range(S):
        a, b = int(query_start_locs[s]), int(query_start_locs[s + 1])
        m = hidden[a:b].float().mean(dim=0)
        out[s] = m / (m.norm() + 1e-12)
    return out


def topk_softmax_router(
    logits: torch.Tensor, top_k: int
):
    """MoE router: softmax over experts then top-k, renormalized.
    Returns (weights [T,k] fp32, indices [T,k] int64)."""
    probs = torch.softmax(logits.float(), dim=-1)
    w, idx = probs.topk(top_k, dim=-1)
    w = w / w.sum(dim=-1, keepdim=True)
    return w, idx


def grouped_gemm(out, a, w, row_tok, tile_off, counts, max_tiles, gate_silu,
                 bm: int = 64):
    """Reference for csrc/grouped_gemm.hip: per-expert segments padded to the
    bm tile; gate_silu (True or 1) fuses silu(gate)*up over the two N-halves
    of w; gate_silu == 2 squares relu of the single product (rows are still
    gathered through row_tok).
    Padding rows of `out` are left untouched (the kernel writes deterministic
    garbage there; consumers must ignore them either way)."""
    E, N, K = w.shape
    relu2 = int(gate_silu) == 2
    gate_silu = int(gate_silu) == 1
    n_cols = N // 2 if gate_silu else N
    for e in range(E):
        c = int(counts[e])
        if c == 0:
            continue
        s0 = int(tile_off[e]) * bm
        if row_tok is not None:
            toks = row_tok[s0:s0 + c].long().clamp(min=0)
            rows = a[toks].float()
        else:
            rows = a[s0:s0 + c].float()
        if gate_silu:
            g = rows @ w[e, :n_cols].T.float()
            u = rows @ w[e, n_cols:].T.float()
            out[s0:s0 + c] = (torch.nn.functional.silu(g) * u).to(out.dtype)
        elif relu2:
            z = torch.relu(rows @ w[e].T.float())
            out[s0:s0 + c] = (z * z).to(out.dtype)
        else:
            out[s0:s0 + c] = (rows @ w[e].T.float()).to(out.dtype)
    return out


# --------------------------------------------------------------------------
# Layer-list ("hybrid") decoders: scalar-gain norms, gated residuals, local
# (chunked / windowed) attention with split key/value sizes, and the gated
# delta rule. Projections of one sublayer arrive merged in one [T, N] buffer
# (`proj`); ops address their sections by column offset.
# --------------------------------------------------------------------------


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))


def gelu_tanh_mul(proj: torch.Tensor, gate_off: int, up_off: int, ff: int) -> torch.Tensor:
    g = proj[:, gate_off:gate_off + ff].float()
    u = proj[:, up_off:up_off + ff].float()
    return (gelu_tanh(g) * u).to(proj.dtype)


def gated_norm_residual(x: torch.Tensor, y: torch.Tensor, proj: torch.Tensor,
                        gate_off: int, gain: torch.Tensor, eps: float,
                        mult: float, h_out=None) -> None:
    """x (fp32, in place) += mult * gain * n(y * sigmoid(gate)), with
    n(z) = z / sqrt(mean(z^2) + eps) and one scalar gain for all channels;
    h_out, when given, receives the new x in its own dtype."""
    W = x.shape[-1]
    z = y.float() * torch.sigmoid(proj[:, gate_off:gate_off + W].float())
    z = z * torch.rsqrt(z.pow(2).mean(-1, keepdim=True) + eps)
    x.add_(z * (mult * gain.float()))
    if h_out is not None:
        h_out.copy_(x.to(h_out.dtype))


def scalar_rmsnorm(x: torch.Tensor, gain: torch.Tensor, eps: float,
                   out_dtype: torch.dtype) -> torch.Tensor:
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)
            * gain.float()).to(out_dtype)


def rope_inv_freq(rot_dims: int, base: float) -> torch.Tensor:
    """fp32 [rot_dims/2]: f_i = base^(-2i/rot_dims), rounded once from fp64."""
    half = rot_dims // 2
    i = torch.arange(half, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / max(1, rot_dims))).float()


def attn_prep(proj, q_off, k_off, v_off, H, G, dk, dv, q_norm_w, k_norm_w,
              eps, inv_freq, positions, slot_mapping, k_cache, v_cache,
              rot_amp: float = 1.0, v_first=None, v_first_off: int = 0,
              v_lambda=None):
    """Split q/k/v sections out of `proj`, per-head RMS norm on q and k
    (weights may be None), rotate the first 2*len(inv_freq) dims of each q/k
    head (rotate-half pairing, fp32 angles = position * inv_freq, cos and sin
    times `rot_amp`), write k and v into their paged caches and return q
    [T, H, dk]. With `v_first` (a buffer whose columns v_first_off.. hold
    another layer's values of the same tokens) and `v_lambda` (0-d fp32) the
    cached values are (1 - lambda) v + lambda v_first."""
    T = proj.shape[0]
    q = proj[:, q_off:q_off + H * dk].float().reshape(T, H, dk)
    k = proj[:, k_off:k_off + G * dk].float().reshape(T, G, dk)
    v = proj[:, v_off:v_off + G * dv].reshape(T, G, dv)
    if v_first is not None:
        lam = v_lambda.float()
        v = ((1.0 - lam) * v.float() + lam * v_first[
            :, v_first_off:v_first_off + G * dv].float().reshape(T, G, dv))

    def norm(x, w):
        if w is None:
            return x
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()

    q, k = norm(q, q_norm_w), norm(k, k_norm_w)
    half = inv_freq.numel()
    if half:
        ang = positions.to(torch.float32).unsqueeze(1) * inv_freq.float().unsqueeze(0)
        c, s = ang.cos().unsqueeze(1), ang.sin().unsqueeze(1)
        if rot_amp != 1.0:
            c, s = c * rot_amp, s * rot_amp

        def rot(x):
            a, b, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
            return torch.cat([a * c - b * s, b * c + a * s, rest], -1)

        q, k = rot(q), rot(k)
    bs = k_cache.shape[2]
    blk = slot_mapping // bs
    off = slot_mapping % bs
    k_cache[blk, :, off] = k.to(k_cache.dtype)
    v_cache[blk, :, off] = v.to(v_cache.dtype)
    return q.to(proj.dtype)


def local_attention(q, k_cache, v_cache, block_tables, seq_lens,
                    query_start_locs, scale, chunk, window, proj, gate_off,
                    out, out_off, out_scale, bias_r1=None, bias_r2=None,
                    sink=False, keep_first: int = 0):
    """Softmax attention of each sequence's new tokens over its cached keys
    under a local mask: query at position i sees j <= i with
    j >= (i // chunk) * chunk (chunk > 0) and j > i - window (window > 0);
    keys j < keep_first stay visible whatever the window says.
    Head h's result is multiplied by out_scale * sigmoid(proj[t, gate_off+h])
    (gate_off < 0: no gate) and written to out[t, out_off + h*dv : ...].
    With bias_r1 / bias_r2 (fp32 [H]) the score of query i and key j is
    lowered by r1[h] * ln(1 + r2[h] * (i - j)). With `sink` a key of score 0
    that carries no value joins the normalisation."""
    T, H, dk = q.shape
    G, bs, dv = v_cache.shape[1], v_cache.shape[2], v_cache.shape[3]
    rep = H // G
    S = seq_lens.numel()
    for s in range(S):
        q0, q1 = int(query_start_locs[s]), int(query_start_locs[s + 1])
        nq = q1 - q0
        if nq == 0:
            continue
        L = int(seq_lens[s])
        nblk = (L + bs - 1) // bs
        blocks = block_tables[s, :nblk].long()
        keys = k_cache[blocks].transpose(0, 1).reshape(G, nblk * bs, dk)[:, :L].float()
        vals = v_cache[blocks].transpose(0, 1).reshape(G, nblk * bs, dv)[:, :L].float()
        qs = q[q0:q1].float().transpose(0, 1)                  # [H, nq, dk]
        kh = keys.repeat_interleave(rep, dim=0)
        vh = vals.repeat_interleave(rep, dim=0)
        scores = torch.einsum("hqd,hkd->hqk", qs, kh) * scale
        kpos = torch.arange(L, device=q.device).unsqueeze(0)
        qpos = torch.arange(L - nq, L, device=q.device).unsqueeze(1)
        hidden = kpos > qpos
        if bias_r1 is not None:
            d = (qpos - kpos).clamp(min=0).to(torch.float32).unsqueeze(0)
            scores = scores - bias_r1.float().view(H, 1, 1) * torch.log(
                1.0 + bias_r2.float().view(H, 1, 1) * d)
        if chunk > 0:
            hidden = hidden | (kpos < (qpos // chunk) * chunk)
        if window > 0:
            hidden = hidden | ((kpos <= qpos - window) & (kpos >= keep_first))
        scores.masked_fill_(hidden.unsqueeze(0), float("-inf"))
        if sink:
            zero = torch.zeros(H, nq, 1, dtype=scores.dtype, device=q.device)
            pr = torch.softmax(torch.cat([scores, zero], -1), dim=-1)[..., :L]
        else:
            pr = torch.softmax(scores, dim=-1)
        o = torch.einsum("hqk,hkd->hqd", pr, vh)
        o = o.transpose(0, 1) * out_scale                      # [nq, H, dv]
        if gate_off >= 0:
            o = o * torch.sigmoid(proj[q0:q1, gate_off:gate_off + H].float()).unsqueeze(-1)
        out[q0:q1, out_off:out_off + H * dv] = o.reshape(nq, H * dv).to(out.dtype)


def delta_prep(proj, q_off, k_off, v_off, b_off, a1_off, H, G, dk, dv,
               conv_w, a2, dt_bias, a_log, conv_state, state_slots,
               query_start_locs, seq_lens):
    """Inputs of the gated delta rule for every new token.

    q/k/v sections of `proj` pass a causal depthwise filter (`conv_w`
    [C, taps] over channels ordered q|k|v, last tap = current token; inputs
    before the sequence start are zero; the filter's history for a sequence
    that continues comes from conv_state[slot] = its last taps-1 raw inputs,
    time-major) and silu; q and k become unit vectors per head (q also times
    dk^-1/2). beta = sigmoid(b section). decay = exp(-exp(a_log[h]) *
    softplus(a2 @ a1 + dt_bias)) per head and key channel. conv_state is
    brought up to date. Returns fp32 (q [T,G,dk], k [T,G,dk], v [T,H,dv],
    decay [T,H,dk], beta [T,H])."""
    T = proj.shape[0]
    Cq, Cv = G * dk, H * dv
    C = 2 * Cq + Cv
    taps = conv_w.shape[1]
    raw = torch.cat([proj[:, q_off:q_off + Cq], proj[:, k_off:k_off + Cq],
                     proj[:, v_off:v_off + Cv]], dim=1).float()
    y = torch.empty_like(raw)
    S = seq_lens.numel()
    wf = conv_w.float()
    for s in range(S):
        a, b = int(query_start_locs[s]), int(query_start_locs[s + 1])
        n = b - a
        if n == 0:
            continue
        start = int(seq_lens[s]) - n
        slot = int(state_slots[s])
        if taps > 1:
            hist = (conv_state[slot].float() if start > 0
                    else torch.zeros(taps - 1, C, dtype=torch.float32, device=proj.device))
            ext = torch.cat([hist, raw[a:b]], dim=0)          # [taps-1+n, C]
            conv_state[slot] = ext[-(taps - 1):].to(conv_state.dtype)
        else:
            ext = raw[a:b]
        acc = torch.zeros(n, C, dtype=torch.float32, device=proj.device)
        for j in range(taps):
            acc = acc + ext[j:j + n] * wf[:, j]
        y[a:b] = acc * torch.sigmoid(acc)
    qn = y[:, :Cq].reshape(T, G, dk)
    kn = y[:, Cq:2 * Cq].reshape(T, G, dk)
    v = y[:, 2 * Cq:].reshape(T, H, dv).contiguous()
    qn = qn * torch.rsqrt(qn.pow(2).sum(-1, keepdim=True) + 1e-6) * (float(dk) ** -0.5)
    kn = kn * torch.rsqrt(kn.pow(2).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(proj[:, b_off:b_off + H].float())
    r = a2.shape[1]
    a = proj[:, a1_off:a1_off + r].float() @ a2.float().T + dt_bias.float()
    decay = torch.exp(-torch.exp(a_log.float()).view(1, H, 1)
                      * torch.nn.functional.softplus(a).view(T, H, dk))
    return qn.contiguous(), kn.contiguous(), v, decay.contiguous(), beta.contiguous()


def delta_scan(qn, kn, v, decay, beta, ssm_state, state_slots,
               query_start_locs, seq_lens):
    """Token-by-token gated delta rule per sequence and head, state
    ssm_state[slot] = S [H, dk, dv] (fp32, zero at a sequence's start):
        S <- decay[:, None] * S;  u = beta * (v - S^T k);
        S <- S + k u^T;           o = S^T q.
    Returns o [T, H, dv] fp32 and leaves the new state in ssm_state."""
    T, H, dv = v.shape
    G = kn.shape[1]
    rep = H // G
    o = torch.empty(T, H, dv, dtype=torch.float32, device=v.device)
    S_n = seq_lens.numel()
    for s in range(S_n):
        a, b = int(query_start_locs[s]), int(query_start_locs[s + 1])
        n = b - a
        if n == 0:
            continue
        start = int(seq_lens[s]) - n
        slot = int(state_slots[s])
        St = (ssm_state[slot].clone() if start > 0
              else torch.zeros_like(ssm_state[slot]))
        for t in range(a, b):
            kt = kn[t].repeat_interleave(rep, dim=0)           # [H, dk]
            qt = qn[t].repeat_interleave(rep, dim=0)
            St = St * decay[t].unsqueeze(-1)
            u = beta[t].unsqueeze(-1) * (v[t] - torch.einsum("hkv,hk->hv", St, kt))
            St = St + kt.unsqueeze(-1) * u.unsqueeze(1)
            o[t] = torch.einsum("hkv,hk->hv", St, qt)
        ssm_state[slot] = St
    return o


def delta_out(o, norm_w, proj, g1_off, g2, eps, out, out_off, out_scale):
    """out[t, out_off + h*dv + j] = out_scale * n(o[t,h])_j * norm_w[j] *
    sigmoid(g2 @ g1)[h*dv + j], n = divide by the root mean square over dv."""
    T, H, dv = o.shape
    r = g2.shape[1]
    gate = torch.sigmoid(proj[:, g1_off:g1_off + r].float() @ g2.float().T).view(T, H, dv)
    y = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    out[:, out_off:out_off + H * dv] = (y * gate * out_scale).reshape(T, H * dv).to(out.dtype)


# --------------------------------------------------------------------------
# More mechanisms of layer-list decoders: hashed-bigram + sinusoid embedding,
# weighted RMS norms around a sublayer with a depth-weighted sum of all earlier
# layer results, PolyNorm, windowed attention with whole-projection q/k norm /
# position-dependent query temperature / logarithmic distance bias, latent
# attention helpers, and the mLSTM matrix memory.
# --------------------------------------------------------------------------


def sinusoid_inv_freq(width: int, base: float) -> torch.Tensor:
    """fp32 [ceil(width/2)]: base^(-2i/width), rounded once from fp64."""
    i = torch.arange((width + 1) // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / width)).float()


def token_embed(ids, prev_ids, positions, embed_w, bigram_w, buckets: int,
                mul_prev: int, mul_cur: int, inv_freq, scale: float = 1.0):
    """fp32 [T, W]: scale * embed[id] (+ bigram[(prev*mul_prev + id*mul_cur) mod
    buckets], row `buckets` where prev < 0) (+ the sinusoid of the position:
    column 2i = sin(p * inv_freq[i]), column 2i+1 = cos of the same fp32
    angle)."""
    x = embed_w[ids].float()
    if scale != 1.0:
        x = x * scale
    if bigram_w is not None:
        row = (prev_ids * mul_prev + ids * mul_cur) % buckets
        row = torch.where(prev_ids < 0, torch.full_like(row, buckets), row)
        x = x + bigram_w[row].float()
    if inv_freq is not None:
        ang = positions.to(torch.float32).unsqueeze(1) * inv_freq.unsqueeze(0)
        x = x + torch.stack([ang.sin(), ang.cos()],
                            dim=-1).reshape(x.shape[0], -1)[:, :x.shape[1]]
    return x


def _unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def weighted_rmsnorm(x, w, eps: float, out_dtype: torch.dtype):
    return (_unit_rms(x.float(), eps) * w.float()).to(out_dtype)


def norm_residual(x_in, y, w_post, eps: float, x_out, stack=None,
                  depth_w=None, mix_out=None, next_w=None, h_out=None) -> None:
    """r = x_in + n(y) * w_post -> x_out (fp32; may be x_in itself). With
    `depth_w` [n]: z = sum_j depth_w[j] * stack[j] over the first n entries of
    `stack` [*, T, W], whose entry n-1 is x_out, -> mix_out; else z = r. With
    `next_w`: h_out = n(z) * next_w in h_out's dtype. n divides a row by its
    root mean square (eps inside the root)."""
    r = x_in + _unit_rms(y.float(), eps) * w_post.float()
    x_out.copy_(r)
    z = r
    if depth_w is not None:
        n = depth_w.numel()
        z = (depth_w.float().view(n, 1, 1) * stack[:n]).sum(0)
        mix_out.copy_(z)
    if next_w is not None:
        h_out.copy_((_unit_rms(z, eps) * next_w.float()).to(h_out.dtype))


def poly_act(z, coef, eps: float):
    """coef[0] n(z) + coef[1] n(z^2) + coef[2] n(z^3) + coef[3], powers taken
    element by element, n as above over the row."""
    zf = z.float()
    c = coef.float()
    z2 = zf * zf
    z3 = z2 * zf
    y = (c[0] * _unit_rms(zf, eps) + c[1] * _unit_rms(z2, eps)
         + c[2] * _unit_rms(z3, eps) + c[3])
    return y.to(z.dtype)


def tied_attn_prep(proj, q_off, k_off, H, G, dk, q_w, k_w, eps, positions,
                   temp_coef: float, temp_every: int, slot_mapping, k_cache,
                   v_cache):
    """Queries and keys of attention whose values are its raw keys: the q and
    k sections of `proj` are each RMS-normed over the WHOLE section (all heads
    at once) with weights q_w / k_w; q is then scaled by 1 + temp_coef *
    ln(floor((p + 1) / temp_every) + 1) at position p (temp_every <= 0: no
    scaling). The normed k goes to k_cache, the raw k section to v_cache.
    Returns q [T, H, dk]."""
    T = proj.shape[0]
    q = proj[:, q_off:q_off + H * dk].float()
    k = proj[:, k_off:k_off + G * dk]
    q = _unit_rms(q, eps) * q_w.float()
    kn = _unit_rms(k.float(), eps) * k_w.float()
    if temp_every > 0:
        steps = torch.div(positions + 1, temp_every, rounding_mode="floor")
        q = q * (1.0 + temp_coef * torch.log(
            steps.to(torch.float32) + 1.0)).unsqueeze(1)
    bs = k_cache.shape[2]
    blk = slot_mapping // bs
    off = slot_mapping % bs
    k_cache[blk, :, off] = kn.reshape(T, G, dk).to(k_cache.dtype)
    v_cache[blk, :, off] = k.reshape(T, G, dk).to(v_cache.dtype)
    return q.reshape(T, H, dk).to(proj.dtype)


def section_rmsnorm(proj, off: int, n: int, w, eps: float, out, rows=None):
    """out[rows[t] or t] = n(proj[t, off:off+n]) * w; `out` is [N, n]."""
    y = (_unit_rms(proj[:, off:off + n].float(), eps) * w.float()).to(out.dtype)
    if rows is None:
        out.copy_(y)
    else:
        out[rows] = y


def sigmoid_gate_mul(v, proj, g_off: int) -> None:
    """v [T, N] *= sigmoid(proj[:, g_off:g_off+N]), in place."""
    N = v.shape[1]
    v.copy_((v.float() * torch.sigmoid(proj[:, g_off:g_off + N].float())).to(v.dtype))


def mlstm_scan(proj, q_off, k_off, v_off, i_off, f_off, H, dk, dv, i_bias,
               f_bias, cap: float, mem, mstate, state_slots, query_start_locs,
               seq_lens):
    """mLSTM matrix memory over every sequence's new tokens.

    Per head, with log gates i = cap*tanh((a_i + b_i)/cap) and f =
    logsigmoid(cap*tanh((a_f + b_f)/cap)) (a_* = the i/f sections of `proj`)
    and the running maximum m (0 at a sequence's start):
        m' = max(f + m, i);  C <- exp(f + m - m') C + exp(i - m') k [v, 1]^T
    where C [dk, dv+1] carries the normaliser n as its last column
    (mem[slot, h]), m lives in mstate[slot, h], q is scaled by dk^-1/2.
    Returns (C^T q [T, H, dv+1] fp32, exp(-m') [T, H] fp32)."""
    T = proj.shape[0]
    q = proj[:, q_off:q_off + H * dk].float().reshape(T, H, dk) * (float(dk) ** -0.5)
    k = proj[:, k_off:k_off + H * dk].float().reshape(T, H, dk)
    v = proj[:, v_off:v_off + H * dv].float().reshape(T, H, dv)
    v1 = torch.cat([v, torch.ones(T, H, 1, dtype=torch.float32, device=v.device)], -1)
    ig = cap * torch.tanh((proj[:, i_off:i_off + H].float() + i_bias.float()) / cap)
    fg = torch.nn.functional.logsigmoid(
        cap * torch.tanh((proj[:, f_off:f_off + H].float() + f_bias.float()) / cap))
    o = torch.empty(T, H, dv + 1, dtype=torch.float32, device=proj.device)
    em = torch.empty(T, H, dtype=torch.float32, device=proj.device)
    for s in range(seq_lens.numel()):
        a, b = int(query_start_locs[s]), int(query_start_locs[s + 1])
        n = b - a
        if n == 0:
            continue
        start = int(seq_lens[s]) - n
        slot = int(state_slots[s])
        if start > 0:
            C, m = mem[slot].clone(), mstate[slot].clone()
        else:
            C, m = torch.zeros_like(mem[slot]), torch.zeros_like(mstate[slot])
        for t in range(a, b):
            mn = torch.maximum(fg[t] + m, ig[t])
            fa = torch.exp(fg[t] + m - mn)
            ib = torch.exp(ig[t] - mn)
            C = fa.view(H, 1, 1) * C + (ib.view(H, 1) * k[t]).unsqueeze(-1) * v1[t].unsqueeze(1)
            m = mn
            o[t] = torch.einsum("hkv,hk->hv", C, q[t])
            em[t] = torch.exp(-m)
        mem[slot] = C
        mstate[slot] = m
    return o, em


def mlstm_out(o, em, norm_w, proj, g_off: int, eps: float, out, out_off: int):
    """h = o[..., :dv] / (max(|o[..., dv]|, em) + 1e-6); each head of h divided
    by its root mean square; times norm_w [H*dv] and sigmoid of the gate
    section of `proj`; written to out[:, out_off : out_off + H*dv]."""
    T, H, dv1 = o.shape
    dv = dv1 - 1
    den = torch.maximum(o[..., dv].abs(), em) + 1e-6
    h = o[..., :dv] / den.unsqueeze(-1)
    h = _unit_rms(h, eps).reshape(T, H * dv) * norm_w.float()
    h = h * torch.sigmoid(proj[:, g_off:g_off + H * dv].float())
    out[:, out_off:out_off + H * dv] = h.to(out.dtype)


# --------------------------------------------------------------------------
# Parallel layers under one Dynamic-Tanh norm, layer scales, routed experts.
# --------------------------------------------------------------------------


def moe_combine_rows(rows, padpos, w):
    """fp32 [T, W]: sum_j w[t, j] * rows[padpos[t, j]]."""
    return (rows[padpos.long()].float() * w.unsqueeze(-1)).sum(dim=1)


def dyt_residual(x, y1, ls1, y2, ls2, rows, padpos, wts, alpha, nw, nb,
                 h_out):
    """x (fp32, in place) += ls1 * y1 + ls2 * y2, where the second branch is
    either y2 [T, W] or the weighted sum of expert rows
    sum_j wts[t, j] * rows[padpos[t, j]] (both None: one branch; y1 None: no
    update). Then, unless h_out is None, h_out = tanh(alpha * x) * nw + nb
    (alpha a 0-d tensor) in h_out's type."""
    if y1 is not None:
        add = y1.float() * ls1
        if y2 is not None:
            add = add + y2.float() * ls2
        elif rows is not None:
            add = add + moe_combine_rows(rows, padpos, wts) * ls2
        x.add_(add)
    if h_out is not None:
        h_out.copy_((torch.tanh(alpha * x) * nw + nb).to(h_out.dtype))


def moe_route(logits, top: int, groups: int, keep: int, group_rank: int = 2):
    """Sigmoid router with group-limited choice. logits fp32 [T, E]. Returns
    (idx int32 [T, top], weights fp32 [T, top]): the `top` largest sigmoid
    scores among the experts of the `keep` groups (equal runs of neighbours)
    whose `group_rank` largest scores sum highest, each divided by the sum of
    the chosen scores + 1e-20. Ties go to the lower index."""
    T, E = logits.shape
    s = torch.sigmoid(logits.float())
    if groups > 1:
        size = E // groups
        per = s.view(T, groups, size)
        worth = per.topk(min(group_rank, size), dim=-1).values.sum(-1)
        # stable descending order: ties keep the lower group
        order = torch.sort(worth, dim=-1, descending=True, stable=True).indices
        allow = torch.zeros(T, groups, dtype=torch.bool, device=s.device)
        allow.scatter_(1, order[:, :keep], True)
        masked = torch.where(allow.unsqueeze(-1), per,
                             torch.full_like(per, -1.0)).reshape(T, E)
    else:
        masked = s
    idx = torch.sort(masked, dim=-1, descending=True,
                     stable=True).indices[:, :top]
    w = s.gather(1, idx)
    w = w / (w.sum(-1, keepdim=True) + 1e-20)
    return idx.to(torch.int32), w


def moe_dispatch(idx, experts: int, bm: int):
    """Lay the (token, choice) pairs of idx [T, k] out in per-expert segments
    padded to `bm` rows. Returns (row_tok int32 [(ceil(T*k / bm) + experts) *
    bm], a whole number of tiles that holds every padded segment: the token
    of every padded row, -1 for padding; tile_off int32 [experts+1]: segment
    starts in tiles; counts int32 [experts]; padpos int32 [T, k]: the padded
    row of every pair)."""
    T, k = idx.shape
    dev = idx.device
    flat = idx.reshape(-1).long()
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=experts)
    padded = (counts + bm - 1) // bm * bm
    pad_off = torch.zeros(experts + 1, dtype=torch.long, device=dev)
    pad_off[1:] = torch.cumsum(padded, 0)
    first = torch.zeros(experts + 1, dtype=torch.long, device=dev)
    first[1:] = torch.cumsum(counts, 0)
    se = flat[order]
    pos = torch.arange(T * k, device=dev) - first[se]
    where = pad_off[se] + pos
    row_tok = torch.full((((T * k + bm - 1) // bm + experts) * bm,), -1,
                         dtype=torch.int32, device=dev)
    row_tok[where] = (order // k).to(torch.int32)
    padpos = torch.empty(T * k, dtype=torch.int32, device=dev)
    padpos[order] = where.to(torch.int32)
    return (row_tok, (pad_off // bm).to(torch.int32), counts.to(torch.int32),
            padpos.view(T, k))


def softcap(logits, cap: float):
    """cap * tanh(logits / cap) in fp32."""
    return cap * torch.tanh(logits.float() / cap)


# --------------------------------------------------------------------------
# Pre-norm layers with a fused residual + routed-experts gather, YaRN
# frequencies, gated linear units, a softmax router with identity experts,
# and decay recurrences (fixed-decay linear attention, Mamba-2).
# --------------------------------------------------------------------------

GLU_GELU_TANH, GLU_SILU, GLU_CLAMPED = 0, 1, 2


def yarn_inv_freq(rot_dims: int, base: float, scaling=None):
    """(fp32 [rot_dims/2] frequencies, amplitude of cos / sin). `scaling` =
    (factor, original length, fast turns, slow turns): with
    d(t) = rot_dims ln(original / (2 pi t)) / (2 ln base), lo = max(floor(
    d(fast)), 0), hi = min(ceil(d(slow)), rot_dims - 1) and ramp_i =
    clamp((i - lo) / max(hi - lo, 0.001), 0, 1), pair i turns at
    f_i / factor * ramp_i + f_i (1 - ramp_i); amplitude 0.1 ln(factor) + 1.
    Computed in fp64 and rounded once."""
    import math

    half = rot_dims // 2
    i = torch.arange(half, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / max(1, rot_dims))
    if not scaling:
        return f.float(), 1.0
    factor, orig, fast, slow = (float(z) for z in scaling)

    def d(turns: float) -> float:
        return rot_dims * math.log(orig / (2.0 * math.pi * turns)) / (
            2.0 * math.log(float(base)))

    lo = max(math.floor(d(fast)), 0)
    hi = min(math.ceil(d(slow)), rot_dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    f = f / factor * ramp + f * (1.0 - ramp)
    return f.float(), 0.1 * math.log(factor) + 1.0


def glu_mul(proj, gate_off: int, up_off: int, ff: int, act: int,
            limit: float = 0.0):
    """act(gate) * up over two sections of `proj`: GLU_GELU_TANH, GLU_SILU,
    or GLU_CLAMPED: g = min(gate, limit), u = clamp(up, -limit, limit),
    g sigmoid(1.702 g) (u + 1)."""
    g = proj[:, gate_off:gate_off + ff].float()
    u = proj[:, up_off:up_off + ff].float()
    if act == GLU_GELU_TANH:
        y = gelu_tanh(g) * u
    elif act == GLU_SILU:
        y = g * torch.sigmoid(g) * u
    else:
        g = g.clamp(max=limit)
        y = g * torch.sigmoid(1.702 * g) * (u.clamp(-limit, limit) + 1.0)
    return y.to(proj.dtype)


def add_rmsnorm(x, y, rows, padpos, wts, idw, h_in, y2, proj2, sg_off,
                norm_w, eps: float, h_out):
    """x (fp32 [T, W], in place) += y (optional) + sum_j wts[t, j] *
    rows[padpos[t, j]] over the pairs with wts != 0 (optional) + idw[t] *
    h_in[t] (optional) + sigmoid(proj2[t, sg_off]) * y2[t] (optional; sg_off
    < 0: no gate). Then h_out = x / sqrt(mean(x^2) + eps) * norm_w, unless
    h_out is None."""
    add = None

    def acc(a, b):
        return b if a is None else a + b

    if y is not None:
        add = acc(add, y.float())
    if rows is not None:
        live = (wts != 0).unsqueeze(-1)
        r = torch.where(live, rows[padpos.long().clamp(min=0)].float(),
                        torch.zeros((), dtype=torch.float32, device=x.device))
        add = acc(add, (r * wts.unsqueeze(-1)).sum(dim=1))
    if idw is not None:
        add = acc(add, idw.float().unsqueeze(-1) * h_in.float())
    if y2 is not None:
        z = y2.float()
        if sg_off >= 0:
            z = z * torch.sigmoid(proj2[:, sg_off:sg_off + 1].float())
        add = acc(add, z)
    if add is not None:
        x.add_(add)
    if h_out is not None:
        h_out.copy_((x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
                     * norm_w.float()).to(h_out.dtype))


def moe_route_softmax(logits, corr, top: int, groups: int, keep: int,
                      n_real: int, scale: float):
    """Softmax router over fp32 logits [T, n] (n = n_real experts + identity
    experts). Choice scores are softmax + corr (corr may be None); the
    outputs form `groups` equal runs of neighbours, a run is worth its
    largest choice score, only members of the `keep` best runs can be chosen
    (ties to the lower index), and the `top` largest choice scores among them
    are. Returns (idx int32 [T, top], w fp32 [T, top], idw fp32 [T]): a chosen
    expert has its softmax score times `scale` as weight; chosen identity
    experts appear as index n_real with weight 0, and the sum of their
    weights is idw."""
    T, n = logits.shape
    s = torch.softmax(logits.float(), dim=-1)
    c = s if corr is None else s + corr.float()
    if groups > 1:
        size = n // groups
        per = c.view(T, groups, size)
        worth = per.max(dim=-1).values
        order = torch.sort(worth, dim=-1, descending=True, stable=True).indices
        allow = torch.zeros(T, groups, dtype=torch.bool, device=s.device)
        allow.scatter_(1, order[:, :keep], True)
        c = torch.where(allow.unsqueeze(-1), per,
                        torch.full_like(per, float("-inf"))).reshape(T, n)
    idx = torch.sort(c, dim=-1, descending=True, stable=True).indices[:, :top]
    w = s.gather(1, idx) * scale
    ident = idx >= n_real
    idw = torch.where(ident, w, torch.zeros_like(w)).sum(-1)
    w = torch.where(ident, torch.zeros_like(w), w)
    idx = torch.where(ident, torch.full_like(idx, n_real), idx)
    return idx.to(torch.int32), w, idw


def glu_grouped_gemm(out, a, w, row_tok, tile_off, counts, bm: int,
                     limit: float):
    """Per-expert segments like `grouped_gemm`, gathered rows, w [E, 2*ff, K]
    holding gate rows then up rows; out[r] = g sigmoid(1.702 g) (u + 1) with
    g = min(gate, limit), u = clamp(up, -limit, limit)."""
    E, N, K = w.shape
    ff = N // 2
    for e in range(E):
        c = int(counts[e])
        if c == 0:
            continue
        s0 = int(tile_off[e]) * bm
        rows = a[row_tok[s0:s0 + c].long().clamp(min=0)].float()
        g = (rows @ w[e, :ff].T.float()).clamp(max=limit)
        u = (rows @ w[e, ff:].T.float()).clamp(-limit, limit)
        out[s0:s0 + c] = (g * torch.sigmoid(1.702 * g) * (u + 1.0)).to(out.dtype)
    return out


def silu_sections(proj, offs, sizes):
    """fp32 silu of column sections of `proj`: one [T, size] tensor each."""
    outs = []
    for o, n in zip(offs, sizes):
        z = proj[:, o:o + n].float()
        outs.append((z * torch.sigmoid(z)).contiguous())
    return outs


def ssd_prep(proj, xbc_off: int, dt_off: int, H: int, dv: int, G: int, N: int,
             conv_w, conv_b, dt_bias, a_log, conv_state, state_slots,
             query_start_locs, seq_lens):
    """Inputs of the Mamba-2 recurrence for every new token. The x|B|C
    section of `proj` (H*dv + 2*G*N channels) passes a causal depthwise
    filter (`conv_w` [C, taps], last tap = current token, bias `conv_b`;
    inputs before a sequence's start are zero; a continuing sequence's
    history is conv_state[slot] = its last taps-1 raw inputs, time-major,
    which is brought up to date) and silu. dt = softplus(dt section +
    dt_bias), decay = exp(-exp(a_log) dt). Returns fp32 (x [T,H,dv],
    B [T,G,N], C [T,G,N], decay [T,H], dt [T,H])."""
    T = proj.shape[0]
    inner = H * dv
    Cn = inner + 2 * G * N
    taps = conv_w.shape[1]
    raw = proj[:, xbc_off:xbc_off + Cn].float()
    y = torch.empty_like(raw)
    wf = conv_w.float()
    for s in range(seq_lens.numel()):
        a, b = int(query_start_locs[s]), int(query_start_locs[s + 1])
        n = b - a
        if n == 0:
            continue
        start = int(seq_lens[s]) - n
        slot = int(state_slots[s])
        if taps > 1:
            hist = (conv_state[slot].float() if start > 0
                    else torch.zeros(taps - 1, Cn, dtype=torch.float32,
                                     device=proj.device))
            ext = torch.cat([hist, raw[a:b]], dim=0)
            conv_state[slot] = ext[-(taps - 1):].to(conv_state.dtype)
        else:
            ext = raw[a:b]
        acc = conv_b.float().unsqueeze(0).expand(n, Cn).clone()
        for j in range(taps):
            acc = acc + ext[j:j + n] * wf[:, j]
        y[a:b] = acc * torch.sigmoid(acc)
    x = y[:, :inner].reshape(T, H, dv).contiguous()
    B = y[:, inner:inner + G * N].reshape(T, G, N).contiguous()
    C = y[:, inner + G * N:].reshape(T, G, N).contiguous()
    dt = torch.nn.functional.softplus(
        proj[:, dt_off:dt_off + H].float() + dt_bias.float())
    decay = torch.exp(-torch.exp(a_log.float()) * dt)
    return x, B, C, decay.contiguous(), dt.contiguous()


def decay_scan(q, k, v, decay, gain, skip, state, state_slots,
               query_start_locs, seq_lens):
    """Token-by-token decay recurrence per sequence and head, state[slot] =
    S [H, dk, dv] (fp32, zero at a sequence's start):
        S <- decay * S + gain * k v^T;   o = S^T q + skip * v.
    q, k fp32 [T, G, dk] (head h reads group h // (H/G)); v fp32 [T, H, dv];
    decay fp32 [T, H] or [H] (the same at every token); gain fp32 [T, H] or
    None (1); skip fp32 [H] or None (0). Returns o [T, H, dv] fp32 and leaves
    the new state in `state`."""
    T, H, dv = v.shape
    G = k.shape[1]
    rep = H // G
    o = torch.empty(T, H, dv, dtype=torch.float32, device=v.device)
    for s in range(seq_lens.numel()):
        a, b = int(query_start_locs[s]), int(query_start_locs[s + 1])
        n = b - a
        if n == 0:
            continue
        start = int(seq_lens[s]) - n
        slot = int(state_slots[s])
        St = (state[slot].clone() if start > 0
              else torch.zeros_like(state[slot]))
        for t in range(a, b):
            kt = k[t].repeat_interleave(rep, dim=0)
            qt = q[t].repeat_interleave(rep, dim=0)
            d = decay if decay.dim() == 1 else decay[t]
            kv = kt.unsqueeze(-1) * v[t].unsqueeze(1)
            if gain is not None:
                kv = kv * gain[t].view(H, 1, 1)
            St = St * d.view(H, 1, 1) + kv
            o[t] = torch.einsum("hkv,hk->hv", St, qt)
            if skip is not None:
                o[t] += skip.view(H, 1) * v[t]
        state[slot] = St
    return o


def gated_group_norm(o, proj, g_off: int, norm_w, eps: float, groups: int,
                     gate_first: bool, out, out_off: int):
    """o fp32 [T, n] (any trailing shape), gate = the n columns of `proj` from
    g_off. gate_first: y = o * silu(gate), then each of `groups` equal parts
    of y divided by its root mean square, times norm_w. Otherwise: parts of o
    normed, times norm_w, times sigmoid(gate). Written to
    out[:, out_off : out_off + n]."""
    T = o.shape[0]
    y = o.reshape(T, -1)
    n = y.shape[1]
    g = proj[:, g_off:g_off + n].float()
    if gate_first:
        y = y * (g * torch.sigmoid(g))
    y = _unit_rms(y.view(T, groups, n // groups), eps).reshape(T, n) * norm_w.float()
    if not gate_first:
        y = y * torch.sigmoid(g)
    out[:, out_off:out_off + n] = y.to(out.dtype)
