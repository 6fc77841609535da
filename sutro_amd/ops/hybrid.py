"""Ops of layer-list ("hybrid") decoders: scalar-gain norms with gated
residuals, tanh-GELU gating, local (chunked / windowed) paged attention with
split key/value sizes, partial rotation and an optional distance bias, the
gated delta rule; hashed-bigram + sinusoid embedding, weighted norms around a
sublayer with depth-weighted sums of all layer results, PolyNorm, tied-value
attention prep, latent norms and gates, the mLSTM; Dynamic-Tanh norms fused
with layer-scaled parallel residuals, and routed experts (sigmoid router with
group-limited choice, dispatch into per-expert segments, expert GEMMs);
weighted RMS norms fused with the residual sum and the gather of expert rows,
YaRN rotation tables, gated linear units, a softmax router with identity
experts, and decay recurrences (fixed-decay linear attention, Mamba-2).

GPU tensors run the HIP kernels of the `sutro_amd._C_mix` extension
(csrc/mix_*.hip), templated on the activation type: bf16 when the engine
serves in bf16, fp32 when it serves in fp32. CPU tensors run the torch
reference. A GPU tensor without the built extension raises.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import torch_ref

_M = None
_M_ERR: Optional[str] = None
try:
    from sutro_amd import _C_mix as _M  # type: ignore
except Exception as e:  # pragma: no cover - only without the built extension
    _M_ERR = f"{type(e).__name__}: {e}"


def mix_available() -> bool:
    return _M is not None


def _mix():
    global _M, _M_ERR
    if _M is None:  # the extension may have been built after this import
        try:
            import importlib

            _M = importlib.import_module("sutro_amd._C_mix")
        except Exception as e:
            _M_ERR = f"{type(e).__name__}: {e}"
    if _M is None:
        raise RuntimeError(
            "sutro_amd HIP extension (_C_mix) is not built but a GPU tensor "
            "was passed. Build it with `python setup.py build_ext --inplace` "
            f"(import error: {_M_ERR})")
    return _M


rope_inv_freq = torch_ref.rope_inv_freq


def gelu_tanh_mul(proj: torch.Tensor, gate_off: int, up_off: int,
                  ff: int) -> torch.Tensor:
    if proj.is_cuda:
        out = torch.empty((proj.shape[0], ff), dtype=proj.dtype,
                          device=proj.device)
        _mix().gelu_tanh_mul(out, proj, gate_off, up_off)
        return out
    return torch_ref.gelu_tanh_mul(proj, gate_off, up_off, ff)


def gated_norm_residual(x, y, proj, gate_off: int, gain, eps: float,
                        mult: float, h_out=None) -> None:
    if x.is_cuda:
        _mix().gated_norm_residual(x, y, proj, gate_off, gain, eps, mult,
                                   h_out)
        return
    torch_ref.gated_norm_residual(x, y, proj, gate_off, gain, eps, mult, h_out)


def scalar_rmsnorm(x, gain, eps: float, out_dtype: torch.dtype):
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _mix().scalar_rmsnorm(out, x, gain, eps)
        return out
    return torch_ref.scalar_rmsnorm(x, gain, eps, out_dtype)


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor,
               amp: float = 1.0) -> torch.Tensor:
    """fp32 [T, 2*half]: cos | sin of the fp32 angle position * inv_freq,
    times `amp`. One table serves every layer of a step that rotates alike."""
    ang = positions.to(torch.float32).unsqueeze(1) * inv_freq.unsqueeze(0)
    tab = torch.cat([ang.cos(), ang.sin()], dim=1)
    if amp != 1.0:
        tab = tab * amp
    return tab.contiguous()


def attn_prep(proj, q_off, k_off, v_off, H, G, dk, dv, q_norm_w, k_norm_w,
              eps, inv_freq, positions, slot_mapping, k_cache, v_cache,
              cos_sin=None, rot_amp: float = 1.0, v_first=None,
              v_first_off: int = 0, v_lambda=None):
    """`rot_amp` multiplies cos and sin (a table passed as `cos_sin` already
    carries it). `v_first` / `v_first_off` / `v_lambda`: the cached values
    become (1 - lambda) v + lambda * v_first[:, v_first_off : ...]."""
    if proj.is_cuda:
        q = torch.empty((proj.shape[0], H, dk), dtype=proj.dtype,
                        device=proj.device)
        if cos_sin is None:
            cos_sin = rope_table(positions, inv_freq, rot_amp)
        _mix().attn_prep(q, proj, q_off, k_off, v_off, q_norm_w, k_norm_w,
                         eps, cos_sin, slot_mapping, k_cache, v_cache,
                         v_first, v_first_off, v_lambda)
        return q
    return torch_ref.attn_prep(proj, q_off, k_off, v_off, H, G, dk, dv,
                               q_norm_w, k_norm_w, eps, inv_freq, positions,
                               slot_mapping, k_cache, v_cache,
                               rot_amp=rot_amp, v_first=v_first,
                               v_first_off=v_first_off, v_lambda=v_lambda)


def local_attention(q, k_cache, v_cache, block_tables, seq_lens,
                    query_start_locs, scale: float, chunk: int, window: int,
                    proj, gate_off: int, out, out_off: int, out_scale: float,
                    token_seq=None, tile_seq=None, tile_q0=None,
                    prefill_rows: int = 0, bias_r1=None, bias_r2=None,
                    sink: bool = False, keep_first: int = 0):
    """`tile_seq`/`tile_q0` (int32, 32 query rows a tile) cover the first
    `prefill_rows` rows: on the GPU in bf16 those rows run on the MFMA kernel
    when page size and head sizes allow it; the remaining (single-token) rows
    and all other cases run on the generic one-wave-per-row kernel.
    `bias_r1` / `bias_r2` (fp32 [H]): r1[h] * ln(1 + r2[h] * (i - j)) is taken
    off the score of query i and key j. `sink`: a key of score 0 without a
    value joins every row's normalisation (a one in the denominator).
    `keep_first`: keys at positions below it stay visible past the window."""
    if q.is_cuda:
        if tile_seq is None or tile_seq.numel() == 0:
            tile_seq = tile_q0 = None
            prefill_rows = 0
        _mix().local_attention(out, out_off, q, k_cache, v_cache,
                               block_tables, seq_lens, query_start_locs,
                               token_seq, scale, chunk, window, proj,
                               gate_off, out_scale, tile_seq, tile_q0,
                               prefill_rows, bias_r1, bias_r2, sink,
                               keep_first)
        return
    torch_ref.local_attention(q, k_cache, v_cache, block_tables, seq_lens,
                              query_start_locs, scale, chunk, window, proj,
                              gate_off, out, out_off, out_scale,
                              bias_r1=bias_r1, bias_r2=bias_r2, sink=sink,
                              keep_first=keep_first)


def delta_prep(proj, q_off, k_off, v_off, b_off, a1_off, H, G, dk, dv,
               conv_w, a2, dt_bias, a_log, conv_state, state_slots,
               query_start_locs, seq_lens, token_seq=None, a2_t=None,
               conv_w_t=None):
    """`a2_t`, `conv_w_t`: a2 and conv_w transposed and contiguous ([rank,
    H*dk] and [taps, C], what the kernels read); made on the fly when the
    caller does not keep them."""
    if proj.is_cuda:
        if a2_t is None:
            a2_t = a2.t().contiguous()
        if conv_w_t is None:
            conv_w_t = conv_w.t().contiguous()
        T = proj.shape[0]
        f32 = dict(dtype=torch.float32, device=proj.device)
        qn = torch.empty((T, G, dk), **f32)
        kn = torch.empty((T, G, dk), **f32)
        v = torch.empty((T, H, dv), **f32)
        decay = torch.empty((T, H, dk), **f32)
        beta = torch.empty((T, H), **f32)
        _mix().delta_prep(qn, kn, v, decay, beta, proj, q_off, k_off, v_off,
                          b_off, a1_off, conv_w, a2_t, dt_bias, a_log,
                          conv_state, state_slots, query_start_locs, seq_lens,
                          token_seq, conv_w_t)
        return qn, kn, v, decay, beta
    return torch_ref.delta_prep(proj, q_off, k_off, v_off, b_off, a1_off, H,
                                G, dk, dv, conv_w, a2, dt_bias, a_log,
                                conv_state, state_slots, query_start_locs,
                                seq_lens)


def delta_scan(qn, kn, v, decay, beta, ssm_state, state_slots,
               query_start_locs, seq_lens):
    if v.is_cuda:
        o = torch.empty_like(v)
        _mix().delta_scan(o, qn, kn, v, decay, beta, ssm_state, state_slots,
                          query_start_locs, seq_lens)
        return o
    return torch_ref.delta_scan(qn, kn, v, decay, beta, ssm_state,
                                state_slots, query_start_locs, seq_lens)


def delta_out(o, norm_w, proj, g1_off: int, g2, eps: float, out,
              out_off: int, out_scale: float, g2_t=None) -> None:
    if o.is_cuda:
        if g2_t is None:
            g2_t = g2.t().contiguous()
        _mix().delta_out(out, out_off, o, norm_w, proj, g1_off, g2_t, eps,
                         out_scale)
        return
    torch_ref.delta_out(o, norm_w, proj, g1_off, g2, eps, out, out_off,
                        out_scale)


# ---- hashed-bigram / sinusoid embedding, sandwich norms with depth-weighted
# ---- sums, PolyNorm, tied-value attention prep, latent helpers, mLSTM ----

sinusoid_inv_freq = torch_ref.sinusoid_inv_freq


def token_embed(ids, prev_ids, positions, embed_w, bigram_w, buckets: int,
                mul_prev: int, mul_cur: int, inv_freq, out=None,
                scale: float = 1.0):
    """fp32 [T, W] sum of `scale` times the token row, the hashed bigram row
    (row `buckets` where prev_ids < 0) and the sinusoid of the position."""
    if out is None:
        out = torch.empty((ids.shape[0], embed_w.shape[1]),
                          dtype=torch.float32, device=ids.device)
    if ids.is_cuda:
        _mix().token_embed(out, ids, prev_ids, positions, embed_w, bigram_w,
                           buckets, mul_prev, mul_cur, inv_freq, scale)
    else:
        out.copy_(torch_ref.token_embed(ids, prev_ids, positions, embed_w,
                                        bigram_w, buckets, mul_prev, mul_cur,
                                        inv_freq, scale))
    return out


def weighted_rmsnorm(x, w, eps: float, out_dtype: torch.dtype):
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
        _mix().weighted_rmsnorm(out, x, w, eps)
        return out
    return torch_ref.weighted_rmsnorm(x, w, eps, out_dtype)


def norm_residual(x_in, y, w_post, eps: float, x_out, stack=None,
                  depth_w=None, mix_out=None, next_w=None, h_out=None) -> None:
    """x_out = x_in + n(y) * w_post; optionally the depth-weighted sum of the
    first len(depth_w) entries of `stack` (the last of which is x_out) into
    mix_out, and the next sublayer's normed input into h_out. One kernel."""
    if x_in.is_cuda:
        _mix().norm_residual(x_in, y, w_post, eps, x_out, stack, depth_w,
                             mix_out, next_w, h_out)
        return
    torch_ref.norm_residual(x_in, y, w_post, eps, x_out, stack, depth_w,
                            mix_out, next_w, h_out)


def poly_act(z, coef, eps: float):
    if z.is_cuda:
        out = torch.empty_like(z)
        _mix().poly_act(out, z, coef, eps)
        return out
    return torch_ref.poly_act(z, coef, eps)


def tied_attn_prep(proj, q_off, k_off, H, G, dk, q_w, k_w, eps, positions,
                   temp_coef: float, temp_every: int, slot_mapping, k_cache,
                   v_cache):
    if proj.is_cuda:
        q = torch.empty((proj.shape[0], H, dk), dtype=proj.dtype,
                        device=proj.device)
        _mix().tied_attn_prep(q, proj, q_off, k_off, q_w, k_w, eps, positions,
                              temp_coef, temp_every, slot_mapping, k_cache,
                              v_cache)
        return q
    return torch_ref.tied_attn_prep(proj, q_off, k_off, H, G, dk, q_w, k_w,
                                    eps, positions, temp_coef, temp_every,
                                    slot_mapping, k_cache, v_cache)


def section_rmsnorm(proj, off: int, n: int, w, eps: float, out,
                    rows=None) -> None:
    if proj.is_cuda:
        _mix().section_rmsnorm(out, proj, off, w, eps, rows)
        return
    torch_ref.section_rmsnorm(proj, off, n, w, eps, out, rows)


def sigmoid_gate_mul(v, proj, g_off: int) -> None:
    if v.is_cuda:
        _mix().sigmoid_gate_mul(v, proj, g_off)
        return
    torch_ref.sigmoid_gate_mul(v, proj, g_off)


def mlstm_scan(proj, q_off, k_off, v_off, i_off, f_off, H, dk, dv, i_bias,
               f_bias, cap: float, mem, mstate, state_slots, query_start_locs,
               seq_lens):
    if proj.is_cuda:
        T = proj.shape[0]
        o = torch.empty((T, H, dv + 1), dtype=torch.float32,
                        device=proj.device)
        em = torch.empty((T, H), dtype=torch.float32, device=proj.device)
        _mix().mlstm_scan(o, em, proj, q_off, k_off, v_off, i_off, f_off,
                          i_bias, f_bias, cap, mem, mstate, state_slots,
                          query_start_locs, seq_lens)
        return o, em
    return torch_ref.mlstm_scan(proj, q_off, k_off, v_off, i_off, f_off, H,
                                dk, dv, i_bias, f_bias, cap, mem, mstate,
                                state_slots, query_start_locs, seq_lens)


def mlstm_out(o, em, norm_w, proj, g_off: int, eps: float, out,
              out_off: int) -> None:
    if o.is_cuda:
        _mix().mlstm_out(out, out_off, o, em, norm_w, proj, g_off, eps)
        return
    torch_ref.mlstm_out(o, em, norm_w, proj, g_off, eps, out, out_off)


# ---- Dynamic-Tanh norm with layer-scaled parallel residuals, routed
# ---- experts, logit soft cap ----

ACT_NONE, ACT_SILU_GATE, ACT_RELU2, ACT_GLU_CLAMPED = 0, 1, 2, 3


def dyt_residual(x, y1=None, ls1=None, y2=None, ls2=None, rows=None,
                 padpos=None, wts=None, norm=None, h_out=None) -> None:
    """x (fp32 [T, W], in place) += ls1 * y1 + ls2 * y2; the second branch is
    y2 [T, W] or, with `rows`, the weighted sum of expert results
    sum_j wts[t, j] * rows[padpos[t, j]]. Then h_out = tanh(alpha * x) * w + b
    for norm = (alpha, w, b). Every part is optional; one kernel."""
    alpha, nw, nb = norm if norm is not None else (None, None, None)
    if x.is_cuda:
        _mix().dyt_residual(x, y1, ls1, y2, ls2, rows, padpos, wts, alpha, nw,
                            nb, h_out)
        return
    torch_ref.dyt_residual(x, y1, ls1, y2, ls2, rows, padpos, wts, alpha, nw,
                           nb, h_out if norm is not None else None)


def moe_route(logits, top: int, groups: int, keep: int, group_rank: int = 2):
    """Sigmoid router with group-limited choice over fp32 logits [T, E]:
    (idx int32 [T, top], weights fp32 [T, top])."""
    if logits.is_cuda:
        T = logits.shape[0]
        idx = torch.empty((T, top), dtype=torch.int32, device=logits.device)
        w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
        _mix().moe_route(idx, w, logits, groups, keep, group_rank)
        return idx, w
    return torch_ref.moe_route(logits, top, groups, keep, group_rank)


def moe_dispatch(idx, experts: int, bm: int):
    """Per-expert segments padded to `bm` rows for idx int32 [T, k]:
    (row_tok int32 [(ceil(T*k / bm) + experts) * bm], tile_off int32
    [experts+1], counts int32 [experts], padpos int32 [T, k]). One kernel, no
    host round trip."""
    if idx.is_cuda:
        T, k = idx.shape
        dev = idx.device
        row_tok = torch.empty(((T * k + bm - 1) // bm + experts) * bm,
                              dtype=torch.int32, device=dev)
        tile_off = torch.empty(experts + 1, dtype=torch.int32, device=dev)
        counts = torch.empty(experts, dtype=torch.int32, device=dev)
        padpos = torch.empty((T, k), dtype=torch.int32, device=dev)
        _mix().moe_dispatch(row_tok, tile_off, counts, padpos, idx, bm)
        return row_tok, tile_off, counts, padpos
    return torch_ref.moe_dispatch(idx, experts, bm)


def expert_gemm_tile(a, w, n_rows: int) -> int:
    """Segment padding (rows) the expert GEMM of these operands wants: the
    matrix-core kernel takes bf16 with K and N multiples of 64 and pads to
    128 rows when segments are long; everything else runs the plain kernel on
    64-row tiles."""
    E = w.shape[0]
    if a.is_cuda and a.dtype == torch.bfloat16 and n_rows >= E * 256:
        return 128
    return 64


def expert_gemm(out, a, w, row_tok, tile_off, counts, act: int, bm: int,
                limit: float = 0.0):
    """out[r] = act(a[row_tok[r]] @ w[e(r)]^T) over padded per-expert
    segments (row_tok None: a is already laid out in segments). w [E, N, K];
    act: ACT_NONE, ACT_RELU2, or ACT_GLU_CLAMPED (w holds N/2 gate rows then
    N/2 up rows per expert; out is N/2 wide: g sigmoid(1.702 g) (u + 1) with
    g = min(gate, limit), u = clamp(up, -limit, limit))."""
    if out.is_cuda:
        _mix().expert_gemm(out, a, w, row_tok, tile_off, counts, act, bm,
                           limit)
        return out
    if act == ACT_GLU_CLAMPED:
        return torch_ref.glu_grouped_gemm(out, a, w, row_tok, tile_off,
                                          counts, bm, limit)
    return torch_ref.grouped_gemm(out, a, w, row_tok, tile_off, counts,
                                  out.shape[0] // bm, act, bm)


def softcap(logits, cap: float):
    """fp32 cap * tanh(logits / cap)."""
    if logits.is_cuda:
        out = torch.empty(logits.shape, dtype=torch.float32,
                          device=logits.device)
        _mix().softcap(out, logits.contiguous(), cap)
        return out
    return torch_ref.softcap(logits, cap)


# ---- pre-norm layers: residual sum + expert gather + weighted RMS norm in
# ---- one kernel, gated linear units, softmax router, decay recurrences ----

yarn_inv_freq = torch_ref.yarn_inv_freq
GLU_GELU_TANH, GLU_SILU, GLU_CLAMPED = (torch_ref.GLU_GELU_TANH,
                                        torch_ref.GLU_SILU,
                                        torch_ref.GLU_CLAMPED)


def glu_mul(proj, gate_off: int, up_off: int, ff: int, act: int,
            limit: float = 0.0):
    """act(gate) * up over two sections of the merged projection; `act` one
    of GLU_GELU_TANH, GLU_SILU, GLU_CLAMPED (g = min(gate, limit), u =
    clamp(up, -limit, limit), g sigmoid(1.702 g) (u + 1))."""
    if proj.is_cuda:
        out = torch.empty((proj.shape[0], ff), dtype=proj.dtype,
                          device=proj.device)
        _mix().glu_mul(out, proj, gate_off, up_off, act, limit)
        return out
    return torch_ref.glu_mul(proj, gate_off, up_off, ff, act, limit)


def add_rmsnorm(x, y=None, rows=None, padpos=None, wts=None, idw=None,
                h_in=None, y2=None, proj2=None, sg_off: int = -1, norm_w=None,
                eps: float = 1e-6, h_out=None) -> None:
    """x (fp32 [T, W], in place) += y + sum_j wts[t, j] rows[padpos[t, j]]
    (pairs of weight 0 are skipped) + idw[t] h_in[t] + sigmoid(proj2[t,
    sg_off]) y2[t]; then h_out = x / sqrt(mean(x^2) + eps) * norm_w. Every
    part is optional; one kernel."""
    if x.is_cuda:
        _mix().add_rmsnorm(x, y, rows, padpos, wts, idw, h_in, y2, proj2,
                           sg_off, norm_w, eps, h_out)
        return
    torch_ref.add_rmsnorm(x, y, rows, padpos, wts, idw, h_in, y2, proj2,
                          sg_off, norm_w, eps, h_out)


def moe_route_softmax(logits, corr, top: int, groups: int, keep: int,
                      n_real: int, scale: float):
    """Softmax router with a choice correction, group-limited choice (a
    group is worth its largest choice score) and identity experts over fp32
    logits [T, n]: (idx int32 [T, top], weights fp32 [T, top], idw fp32 [T]).
    Identity experts (outputs n_real..n-1) come back as index n_real with
    weight 0; their weights are summed in idw."""
    if logits.is_cuda:
        T = logits.shape[0]
        idx = torch.empty((T, top), dtype=torch.int32, device=logits.device)
        w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
        idw = torch.empty((T,), dtype=torch.float32, device=logits.device)
        _mix().moe_route_softmax(idx, w, idw, logits, corr, groups, keep,
                                 n_real, scale)
        return idx, w, idw
    return torch_ref.moe_route_softmax(logits, corr, top, groups, keep,
                                       n_real, scale)


def silu_sections(proj, offs, sizes):
    """fp32 silu of up to three column sections of `proj`, as views of one
    [T, sum(sizes)] buffer."""
    if proj.is_cuda:
        buf = torch.empty((proj.shape[0], sum(sizes)), dtype=torch.float32,
                          device=proj.device)
        _mix().silu_sections(buf, proj, list(offs), list(sizes))
        outs, c = [], 0
        for n in sizes:
            outs.append(buf[:, c:c + n])
            c += n
        return outs
    return torch_ref.silu_sections(proj, offs, sizes)


def ssd_prep(proj, xbc_off: int, dt_off: int, H: int, dv: int, G: int, N: int,
             conv_w, conv_b, dt_bias, a_log, conv_state, state_slots,
             query_start_locs, seq_lens, token_seq=None, conv_w_t=None):
    """Mamba-2 inputs of every new token: filtered + silu x [T,H,dv],
    B [T,G,N], C [T,G,N] (views of one fp32 buffer), decay [T,H], dt [T,H];
    brings the filter history in `conv_state` up to date."""
    if proj.is_cuda:
        T = proj.shape[0]
        inner, gn = H * dv, G * N
        f32 = dict(dtype=torch.float32, device=proj.device)
        buf = torch.empty((T, inner + 2 * gn), **f32)
        decay = torch.empty((T, H), **f32)
        dt = torch.empty((T, H), **f32)
        if conv_w_t is None:
            conv_w_t = conv_w.t().contiguous()
        _mix().ssd_prep(buf, decay, dt, proj, xbc_off, dt_off, conv_w_t,
                        conv_b, dt_bias, a_log, conv_state, state_slots,
                        query_start_locs, seq_lens, token_seq)
        return (buf[:, :inner].view(T, H, dv),
                buf[:, inner:inner + gn].view(T, G, N),
                buf[:, inner + gn:].view(T, G, N), decay, dt)
    return torch_ref.ssd_prep(proj, xbc_off, dt_off, H, dv, G, N, conv_w,
                              conv_b, dt_bias, a_log, conv_state, state_slots,
                              query_start_locs, seq_lens)


def decay_scan(q, k, v, decay, gain, skip, state, state_slots,
               query_start_locs, seq_lens):
    """S <- decay S + gain k v^T, o = S^T q + skip v per sequence and head
    over the new tokens; q, k [T, G, dk], v [T, H, dv] fp32 (row-strided views
    are fine), decay [T, H] or [H], gain [T, H] or None, skip [H] or None,
    state [slots, H, dk, dv] fp32. Returns o [T, H, dv] fp32."""
    if v.is_cuda:
        T, H, dv = v.shape
        o = torch.empty((T, H, dv), dtype=torch.float32, device=v.device)
        _mix().decay_scan(o, q, k, v, decay, gain, skip, state, state_slots,
                          query_start_locs, seq_lens)
        return o
    return torch_ref.decay_scan(q, k, v, decay, gain, skip, state,
                                state_slots, query_start_locs, seq_lens)


def gated_group_norm(o, proj, g_off: int, norm_w, eps: float, groups: int,
                     gate_first: bool, out, out_off: int) -> None:
    """Read-out o fp32 [T, ...n] against a gate section of `proj`:
    gate_first: o * silu(gate), normed in `groups` equal parts, times norm_w;
    else: normed, times norm_w, times sigmoid(gate). Written into
    out[:, out_off : out_off + n]."""
    if o.is_cuda:
        _mix().gated_group_norm(out, out_off, o, proj, g_off, norm_w, eps,
                                groups, gate_first)
        return
    torch_ref.gated_group_norm(o, proj, g_off, norm_w, eps, groups,
                               gate_first, out, out_off)
