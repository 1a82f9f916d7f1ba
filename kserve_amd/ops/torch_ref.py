"""Plain-PyTorch reference implementations of every custom op.

These are the numerics oracle for the HIP kernels (GPU tests compare the
CDNA4 kernels against these run in fp32) and the CPU execution path for
engine logic tests. They are NOT used on GPU tensors in production — the
dispatcher fails loudly instead (errors.NoNativeExtension).
"""

from __future__ import annotations

import math
from typing import Optional, Tuple

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    dtype = x.dtype
    xf = x.float()
    var = xf.pow(2).mean(dim=-1, keepdim=True)
    out = xf * torch.rsqrt(var + eps)
    return (out * weight.float()).to(dtype)


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Returns (normed, new_residual) where new_residual = x + residual."""
    new_residual = (x.float() + residual.float()).to(x.dtype)
    return rms_norm(new_residual, weight, eps), new_residual


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    """x: [..., 2*d] (gate | up) -> silu(gate) * up."""
    d = x.shape[-1] // 2
    gate, up = x[..., :d], x[..., d:]
    return (torch.nn.functional.silu(gate.float()) * up.float()).to(x.dtype)


def _llama3_scale_inv_freq(inv_freq, rope_scaling: dict):
    """Llama-3.1 rope scaling (HF 'rope_type: llama3'): low-frequency
    components are slowed by `factor`, high-frequency ones kept, with a
    smooth interpolation between the two wavelength thresholds."""
    import math

    factor = rope_scaling.get("factor", 8.0)
    lo = rope_scaling.get("low_freq_factor", 1.0)
    hi = rope_scaling.get("high_freq_factor", 4.0)
    orig = rope_scaling.get("original_max_position_embeddings", 8192)
    low_wl = orig / lo
    high_wl = orig / hi
    out = inv_freq.clone()
    for i, f in enumerate(inv_freq.tolist()):
        wl = 2 * math.pi / f
        if wl < high_wl:
            continue  # high frequency: unscaled
        if wl > low_wl:
            out[i] = f / factor  # low frequency: fully scaled
        else:
            smooth = (orig / wl - lo) / (hi - lo)
            out[i] = (1 - smooth) * f / factor + smooth * f
    return out


def make_cos_sin_cache(
    head_dim: int,
    max_positions: int,
    theta: float = 10000.0,
    dtype: torch.dtype = torch.float32,
    device="cpu",
    rope_scaling: Optional[dict] = None,
) -> torch.Tensor:
    """[max_positions, head_dim] with cos in the first half, sin in the second
    (host-precomputed per CDNA guide Appendix B: no on-device trig).
    rope_scaling: HF dict; 'llama3' rope_type applies 3.1-style frequency
    scaling."""
    inv_freq = 1.0 / (
        theta ** (torch.arange(0, head_dim, 2, dtype=torch.float64) / head_dim)
    )
    if rope_scaling:
        rtype = rope_scaling.get("rope_type", rope_scaling.get("type"))
        if rtype == "llama3":
            inv_freq = _llama3_scale_inv_freq(inv_freq, rope_scaling)
        elif rtype == "linear":
            inv_freq = inv_freq / rope_scaling.get("factor", 1.0)
    t = torch.arange(max_positions, dtype=torch.float64)
    freqs = torch.outer(t, inv_freq)  # [P, head_dim/2]
    cache = torch.cat([freqs.cos(), freqs.sin()], dim=-1).to(dtype).to(device)
    return cache


def rotary_embedding(
    positions: torch.Tensor,  # [num_tokens]
    q: torch.Tensor,  # [num_tokens, num_heads, head_dim]
    k: torch.Tensor,  # [num_tokens, num_kv_heads, head_dim]
    cos_sin_cache: torch.Tensor,  # [max_pos, head_dim]
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Neox-style (rotate half) RoPE, out-of-place reference."""
    head_dim = q.shape[-1]
    half = head_dim // 2
    cs = cos_sin_cache[positions].float()  # [T, head_dim]
    cos = cs[:, :half].unsqueeze(1)  # [T, 1, half]
    sin = cs[:, half:].unsqueeze(1)

    def rot(x):
        xf = x.float()
        x1, x2 = xf[..., :half], xf[..., half:]
        return torch.cat([x1 * cos - x2 * sin, x2 * cos + x1 * sin], dim=-1).to(x.dtype)

    return rot(q), rot(k)


def reshape_and_cache(
    k: torch.Tensor,  # [num_tokens, num_kv_heads, head_dim]
    v: torch.Tensor,
    k_cache: torch.Tensor,  # [num_blocks, num_kv_heads, block_size, head_dim]
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,  # [num_tokens] int64/int32
) -> None:
    block_size = k_cache.shape[2]
    slots = slot_mapping.long()
    blk = slots // block_size
    off = slots % block_size
    # advanced indexing: k_cache[blk[i], h, off[i], :] = k[i, h, :]
    # (fp8 caches need an explicit cast: index_put refuses mixed dtypes)
    k_cache[blk, :, off] = k.to(k_cache.dtype)
    v_cache[blk, :, off] = v.to(v_cache.dtype)


def paged_attention_decode(
    q: torch.Tensor,  # [num_seqs, num_heads, head_dim]
    k_cache: torch.Tensor,  # [num_blocks, num_kv_heads, block_size, head_dim]
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [num_seqs, max_blocks] int32 (padded)
    context_lens: torch.Tensor,  # [num_seqs] int32 — includes current token
    scale: float,
    window: int = 0,
) -> torch.Tensor:
    num_seqs, num_heads, head_dim = q.shape
    num_kv_heads = k_cache.shape[1]
    block_size = k_cache.shape[2]
    group = num_heads // num_kv_heads
    out = torch.empty_like(q)
    for s in range(num_seqs):
        ctx = int(context_lens[s])
        nb = -(-ctx // block_size)
        blocks = block_tables[s, :nb].long()
        # [nb, H_kv, B, D] -> [H_kv, nb*B, D]
        keys = k_cache[blocks].permute(1, 0, 2, 3).reshape(num_kv_heads, -1, head_dim)[
            :, :ctx
        ]
        vals = v_cache[blocks].permute(1, 0, 2, 3).reshape(num_kv_heads, -1, head_dim)[
            :, :ctx
        ]
        qh = q[s].float()  # [H, D]
        scores = torch.einsum(
            "hd,htd->ht", qh, keys.float().repeat_interleave(group, dim=0)
        ) * scale
        if window > 0 and ctx > window:
            scores[:, : ctx - window] = float("-inf")
        probs = torch.softmax(scores, dim=-1)
        o = torch.einsum(
            "ht,htd->hd", probs, vals.float().repeat_interleave(group, dim=0)
        )
        out[s] = o.to(q.dtype)
    return out


def flash_prefill_varlen(
    q: torch.Tensor,  # [total_tokens, num_heads, head_dim]
    k: torch.Tensor,  # [total_tokens, num_kv_heads, head_dim]
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,  # [num_seqs+1] int32
    scale: float,
    causal: bool = True,
    window: int = 0,
) -> torch.Tensor:
    num_heads = q.shape[1]
    num_kv_heads = k.shape[1]
    group = num_heads // num_kv_heads
    out = torch.empty_like(q)
    for s in range(cu_seqlens.numel() - 1):
        a, b = int(cu_seqlens[s]), int(cu_seqlens[s + 1])
        qs = q[a:b].float().transpose(0, 1)  # [H, T, D]
        ks = k[a:b].float().transpose(0, 1).repeat_interleave(group, dim=0)
        vs = v[a:b].float().transpose(0, 1).repeat_interleave(group, dim=0)
        scores = torch.einsum("htd,hsd->hts", qs, ks) * scale
        if causal:
            T = b - a
            mask = torch.triu(
                torch.ones(T, T, dtype=torch.bool, device=q.device), diagonal=1
            )
            if window > 0:
                # sliding window: token i sees only (i-window, i]
                mask |= torch.tril(
                    torch.ones(T, T, dtype=torch.bool, device=q.device),
                    diagonal=-window,
                )
            scores.masked_fill_(mask, float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        o = torch.einsum("hts,hsd->htd", probs, vs)
        out[a:b] = o.transpose(0, 1).to(q.dtype)
    return out


def context_attention_varlen(
    q: torch.Tensor,  # [total_new_tokens, num_heads, head_dim]
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,  # [num_seqs, max_blocks]
    cu_seqlens_q: torch.Tensor,  # [num_seqs+1] new-token offsets
    context_lens: torch.Tensor,  # [num_seqs] total context (incl. new tokens)
    scale: float,
    window: int = 0,
) -> torch.Tensor:
    """Prefill attention against the paged cache (supports chunked prefill:
    new tokens attend to all cached tokens before them, causally)."""
    num_heads = q.shape[1]
    num_kv_heads = k_cache.shape[1]
    head_dim = q.shape[2]
    block_size = k_cache.shape[2]
    group = num_heads // num_kv_heads
    out = torch.empty_like(q)
    for s in range(cu_seqlens_q.numel() - 1):
        a, b = int(cu_seqlens_q[s]), int(cu_seqlens_q[s + 1])
        n_new = b - a
        ctx = int(context_lens[s])
        nb = -(-ctx // block_size)
        blocks = block_tables[s, :nb].long()
        keys = k_cache[blocks].permute(1, 0, 2, 3).reshape(num_kv_heads, -1, head_dim)[
            :, :ctx
        ].float().repeat_interleave(group, dim=0)
        vals = v_cache[blocks].permute(1, 0, 2, 3).reshape(num_kv_heads, -1, head_dim)[
            :, :ctx
        ].float().repeat_interleave(group, dim=0)
        qs = q[a:b].float().transpose(0, 1)  # [H, n_new, D]
        scores = torch.einsum("htd,hsd->hts", qs, keys) * scale
        # causal: new token i (absolute pos ctx - n_new + i) sees pos <= its own
        start = ctx - n_new
        pos_q = torch.arange(start, ctx, device=q.device).unsqueeze(1)
        pos_k = torch.arange(ctx, device=q.device).unsqueeze(0)
        bad = pos_k > pos_q
        if window > 0:
            bad |= pos_k <= pos_q - window
        scores.masked_fill_(bad.unsqueeze(0), float("-inf"))
        probs = torch.softmax(scores, dim=-1)
        o = torch.einsum("hts,hsd->htd", probs, vals)
        out[a:b] = o.transpose(0, 1).to(q.dtype)
    return out


def greedy_sample(logits: torch.Tensor) -> torch.Tensor:
    return logits.argmax(dim=-1).to(torch.int64)


def random_sample(
    logits: torch.Tensor,  # [num_seqs, vocab]
    temperatures: torch.Tensor,  # [num_seqs]
    top_p: torch.Tensor,  # [num_seqs]
    top_k: torch.Tensor,  # [num_seqs] (-1 disables)
    generator: Optional[torch.Generator] = None,
    min_p: Optional[torch.Tensor] = None,  # [num_seqs] (0 disables)
) -> torch.Tensor:
    """Temperature + top-k + top-p + min-p sampling, fp32 reference."""
    lf = logits.float()
    temps = temperatures.clamp_min(1e-5).unsqueeze(-1)
    lf = lf / temps
    vocab = lf.shape[-1]
    # top-k mask
    k_eff = torch.where(top_k > 0, top_k, torch.full_like(top_k, vocab))
    sorted_logits, sorted_idx = lf.sort(dim=-1, descending=True)
    ranks = torch.arange(vocab, device=lf.device).unsqueeze(0)
    mask = ranks >= k_eff.unsqueeze(-1)
    # top-p mask on sorted probs
    probs_sorted = torch.softmax(sorted_logits, dim=-1)
    cumprobs = probs_sorted.cumsum(dim=-1)
    mask |= (cumprobs - probs_sorted) > top_p.unsqueeze(-1)
    if min_p is not None:
        # min-p: keep tokens with prob >= min_p * p_max
        mask |= probs_sorted < (min_p.unsqueeze(-1) * probs_sorted[:, :1])
    sorted_logits = sorted_logits.masked_fill(mask, float("-inf"))
    # degenerate rows (everything masked, e.g. an exhausted guided-decoding
    # machine with EOS disabled): pick rank 0 deterministically instead of
    # feeding NaNs to multinomial — callers discard the token
    dead = torch.isinf(sorted_logits).all(dim=-1)
    if bool(dead.any()):
        sorted_logits[dead, 0] = 0.0
    probs = torch.softmax(sorted_logits, dim=-1)
    choice = torch.multinomial(probs, 1, generator=generator).squeeze(-1)
    return sorted_idx.gather(-1, choice.unsqueeze(-1)).squeeze(-1)


def layer_norm(
    x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, eps: float
) -> torch.Tensor:
    return torch.nn.functional.layer_norm(
        x.float(), (x.shape[-1],), weight.float(), bias.float(), eps
    ).to(x.dtype)


def fused_add_layer_norm(
    x: torch.Tensor,
    residual: torch.Tensor,
    weight: torch.Tensor,
    bias: torch.Tensor,
    eps: float,
) -> torch.Tensor:
    return layer_norm((x.float() + residual.float()).to(x.dtype), weight, bias, eps)


def gelu(x: torch.Tensor) -> torch.Tensor:
    return torch.nn.functional.gelu(x.float()).to(x.dtype)


# ---------------------------------------------------------------------------
# Mechanisms of models with a 32-bit residual stream and recurrent state.
# CPU forms of the kernels in residual_norm_f32.hip / ssm_scan.hip /
# attention_f32.hip; same arguments, same in-place effects on caches/state.
# ---------------------------------------------------------------------------


def sinusoid_inv_freq(width: int, base: float = 10000.0) -> torch.Tensor:
    """inv_freq[i] = base^(-2i/width), rounded once from float64."""
    i = torch.arange((width + 1) // 2, dtype=torch.float64)
    return (base ** (-2.0 * i / width)).to(torch.float32)


def embed_scale_sinpos(table, tokens, positions, inv_freq, scale: float):
    if inv_freq is None:
        return table[tokens].float() * scale
    width = table.shape[1]
    ang = positions.to(torch.float32).unsqueeze(1) * inv_freq.unsqueeze(0)
    pe = torch.stack([torch.sin(ang), torch.cos(ang)], dim=-1).reshape(
        tokens.shape[0], -1
    )[:, :width]
    return table[tokens].float() * scale + pe


def add_rms_norm_f32res(
    residual, weight, eps, w_offset, out_dtype, d0=None, s0=1.0, d1=None, s1=1.0
):
    if d0 is not None:
        residual += s0 * d0.float()
    if d1 is not None:
        residual += s1 * d1.float()
    inv = torch.rsqrt(residual.pow(2).mean(-1, keepdim=True) + eps)
    return (residual * inv * (w_offset + weight)).to(out_dtype)


def gated_group_rms_norm(
    y, z, weight, eps, groups: int, out_dtype, gate_after: bool = False
):
    zf = z.float()
    gate = zf * torch.sigmoid(zf)
    v = y if gate_after else y * gate
    vg = v.reshape(v.shape[0], groups, -1)
    vg = vg * torch.rsqrt(vg.pow(2).mean(-1, keepdim=True) + eps)
    out = vg.reshape(v.shape)
    if weight is not None:
        out = out * weight.repeat(v.shape[1] // weight.numel())
    if gate_after:
        out = out * gate
    return out.to(out_dtype)


def causal_conv_silu(x_in, w, bias, conv_state, positions, cu_seqlens, slots):
    taps = w.shape[1]
    hist = taps - 1
    out = torch.empty(x_in.shape, dtype=torch.float32)
    cu = cu_seqlens.tolist()
    for s, slot in enumerate(slots.tolist()):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        start = int(positions[a])
        prev = conv_state[slot, :hist].float().clone()
        # history rows hold positions start-hist .. start-1; zeros before 0
        for i in range(hist):
            if start - hist + i < 0:
                prev[i] = 0
        full = torch.cat([prev, x_in[a:b].float()], dim=0)
        acc = (
            bias.unsqueeze(0).expand(b - a, -1).clone()
            if bias is not None
            else torch.zeros(b - a, x_in.shape[1])
        )
        for j in range(taps):
            acc = acc + full[j : j + b - a] * w[:, j].unsqueeze(0)
        out[a:b] = acc * torch.sigmoid(acc)
        if hist:
            conv_state[slot, :hist] = full[full.shape[0] - hist :].to(
                conv_state.dtype
            )
    return out


def ssd_scan(
    xbc, dt_raw, dt_bias, a_log, d_skip, state, positions, cu_seqlens, slots,
    groups: int,
):
    _, heads, P, N = state.shape
    inner = heads * P
    T = xbc.shape[0]
    y = torch.empty(T, inner, dtype=torch.float32)
    cu = cu_seqlens.tolist()
    A = -torch.exp(a_log)
    rep = heads // groups
    for s, slot in enumerate(slots.tolist()):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        S = state[slot].clone()  # [heads, P, N]
        if int(positions[a]) == 0:
            S.zero_()
        for t in range(a, b):
            x = xbc[t, :inner].reshape(heads, P)
            B = xbc[t, inner : inner + groups * N].reshape(groups, N)
            C = xbc[t, inner + groups * N :].reshape(groups, N)
            B = B.repeat_interleave(rep, dim=0)
            C = C.repeat_interleave(rep, dim=0)
            v = dt_raw[t].float() + dt_bias
            dt = torch.where(v > 30.0, v, torch.log1p(torch.exp(v)))
            decay = torch.exp(A * dt)
            S = decay[:, None, None] * S + (dt[:, None] * x)[:, :, None] * B[:, None, :]
            y[t] = ((S * C[:, None, :]).sum(-1) + d_skip[:, None] * x).reshape(-1)
        state[slot] = S
    return y


def qk_norm_temp_cache(
    q, k, v, qw, kw, positions, slot_mapping, k_cache, v_cache, eps,
    temp_coef: float, temp_every: int, heads: int,
):
    _, G, bs, D = k_cache.shape
    DV = v_cache.shape[3]
    qf, kf = q.float(), k.float()
    qn = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps) * qw
    kn = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps) * kw
    if temp_every > 0:
        steps = torch.div(positions + 1, temp_every, rounding_mode="floor")
        qn = qn * (1.0 + temp_coef * torch.log(steps.float() + 1.0)).unsqueeze(1)
    slots = slot_mapping.long()
    ok = slots >= 0
    blk, off = slots[ok] // bs, slots[ok] % bs
    k_cache[blk, :, off] = kn[ok].reshape(-1, G, D).to(k_cache.dtype)
    v_cache[blk, :, off] = v[ok].reshape(-1, G, DV).to(v_cache.dtype)
    return qn


def ctx_attention_f32(
    q, k_cache, v_cache, block_tables, cu_q, ctx_lens, scale: float,
    heads: int, gate=None, out_dtype=torch.float32, sink=None, chunk: int = 0,
    out_inv_freq=None, window: int = 0,
):
    _, G, bs, D = k_cache.shape
    DV = v_cache.shape[3]
    T = q.shape[0]
    out = torch.zeros(T, heads, DV, dtype=torch.float32)
    cu = cu_q.tolist()
    rep = heads // G
    for s, ctx in enumerate(ctx_lens.tolist()):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        nb = -(-ctx // bs)
        blocks = block_tables[s, :nb].long()
        K = k_cache[blocks].float().permute(1, 0, 2, 3).reshape(G, nb * bs, D)[:, :ctx]
        V = v_cache[blocks].float().permute(1, 0, 2, 3).reshape(G, nb * bs, DV)[:, :ctx]
        K = K.repeat_interleave(rep, dim=0)
        V = V.repeat_interleave(rep, dim=0)
        qs = q[a:b].reshape(b - a, heads, D).float().transpose(0, 1)
        sc = torch.matmul(qs, K.transpose(1, 2)) * scale  # [heads, n, ctx]
        qpos = torch.arange(ctx - (b - a), ctx).unsqueeze(1)
        kpos = torch.arange(ctx).unsqueeze(0)
        vis = kpos <= qpos
        if chunk > 0:
            vis = vis & (kpos // chunk == qpos // chunk)
        if window > 0:
            vis = vis & (qpos - kpos < window)
        sc = sc.masked_fill(~vis.unsqueeze(0), float("-inf"))
        if sink is None:
            w = torch.softmax(sc, dim=-1)
        else:
            # one more term exp(sink) in the denominator, no key, no value
            sk = sink.float().view(heads, 1, 1)
            m = torch.maximum(sc.max(-1, keepdim=True).values, sk)
            e = torch.exp(sc - m)
            w = e / (e.sum(-1, keepdim=True) + torch.exp(sk - m))
        o = torch.matmul(w, V).transpose(0, 1)  # [n, heads, DV]
        if out_inv_freq is not None:
            # turn every head output back by its own position
            o = rotate_halves(o, qpos.view(-1), out_inv_freq, -1.0)
        out[a:b] = o
    if gate is not None:
        out = out * torch.sigmoid(gate.float()).unsqueeze(-1)
    return out.reshape(T, heads * DV).to(out_dtype)


def rotary_inv_freq(n_rot: int, base: float) -> torch.Tensor:
    """inv_freq[i] = base^(-2i/n_rot), i < n_rot/2, rounded once from float64."""
    i = torch.arange(n_rot // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / n_rot)).to(torch.float32)


def rotate_halves(x, positions, inv_freq, sign: float = 1.0):
    """Rotate the first 2*len(inv_freq) coordinates of the last axis of
    x [T, heads, D] (fp32): coordinate i pairs with i + half, pair i turns by
    sign * position * inv_freq[i]; angles and sin/cos in fp32."""
    half = inv_freq.numel()
    if half == 0:
        return x
    a = positions.to(torch.float32).view(-1, 1, 1) * inv_freq.view(1, 1, -1)
    c, s = torch.cos(a), torch.sin(a) * sign
    u, v = x[..., :half], x[..., half : 2 * half]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., 2 * half :]], dim=-1)


def qk_headnorm_rope_cache(
    q, k, v, qw, kw, positions, slot_mapping, k_cache, v_cache, eps,
    heads: int, qk_inv_freq, v_unit_norm: bool, v_inv_freq,
):
    """Per-head RMS norm of q and k (weights [dim], shared by the heads),
    rotary positions on their first 2*len(qk_inv_freq) coordinates; values
    optionally divided by their per-head RMS and rotated by their position
    over 2*len(v_inv_freq) coordinates; k / v scattered to the pages; q
    returned in fp32."""
    _, G, bs, D = k_cache.shape
    DV = v_cache.shape[3]
    T = q.shape[0]
    qf = q.float().reshape(T, heads, D)
    kf = k.float().reshape(T, G, D)
    vf = v.float().reshape(T, G, DV)
    qn = qf * torch.rsqrt(qf.pow(2).mean(-1, keepdim=True) + eps)
    kn = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps)
    if qw is not None:
        qn = qn * qw
    if kw is not None:
        kn = kn * kw
    if qk_inv_freq is not None:
        qn = rotate_halves(qn, positions, qk_inv_freq)
        kn = rotate_halves(kn, positions, qk_inv_freq)
    if v_unit_norm:
        vf = vf * torch.rsqrt(vf.pow(2).mean(-1, keepdim=True) + eps)
    if v_inv_freq is not None:
        vf = rotate_halves(vf, positions, v_inv_freq)
    slots = slot_mapping.long()
    ok = slots >= 0
    blk, off = slots[ok] // bs, slots[ok] % bs
    k_cache[blk, :, off] = kn[ok].to(k_cache.dtype)
    v_cache[blk, :, off] = vf[ok].to(v_cache.dtype)
    return qn.reshape(T, heads * D)


def post_norm_add_rms_norm(
    residual, delta, post_gain: float, layer_scale, eps: float,
    next_gain: float, out_dtype, add_rows=None, add_vec=None,
    want_out: bool = True,
):
    """residual (fp32, in place) += layer_scale * (delta / rms(delta) *
    post_gain), then += add_rows (per token) and += add_vec (one row for
    all) when given; returns residual / rms(residual) * next_gain in
    ``out_dtype`` (None when ``want_out`` is false). Gains are scalars."""
    if delta is not None:
        d = delta.float()
        d = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * post_gain
        residual += d * layer_scale
    if add_rows is not None:
        residual += add_rows
    if add_vec is not None:
        residual += add_vec
    if not want_out:
        return None
    inv = torch.rsqrt(residual.pow(2).mean(-1, keepdim=True) + eps)
    return (residual * inv * next_gain).to(out_dtype)


def router_topk(
    logits, top: int, softmax: bool = False, renorm: bool = False,
    dense: bool = False, correction=None, renorm_eps: float = 0.0,
    weight_scale: float = 1.0,
):
    """Scores (sigmoid, or softmax over the experts) of fp32 router logits
    [T, E]; the ``top`` largest per token -> (indices int32 [T, top],
    weights fp32 [T, top], and with ``dense`` the same weights as a [T, E]
    matrix that is zero elsewhere), optionally renormalised to sum 1
    (divided by their sum + ``renorm_eps``). With ``correction`` [E] the
    choice goes by score + correction while the weights stay the scores."""
    z = logits.float()
    s = torch.softmax(z, dim=-1) if softmax else torch.sigmoid(z)
    if correction is None:
        w, idx = s.topk(top, dim=-1)
    else:
        idx = (s + correction.float()).topk(top, dim=-1).indices
        w = torch.gather(s, 1, idx)
    if renorm:
        w = w / (w.sum(-1, keepdim=True) + renorm_eps)
    if weight_scale != 1.0:
        w = w * weight_scale
    dw = torch.zeros_like(s).scatter_(1, idx, w) if dense else None
    return idx.to(torch.int32), w, dw


def route_tokens(
    h, router, top: int, softmax: bool = False, renorm: bool = False,
    dense: bool = False, want_logits: bool = False, correction=None,
    renorm_eps: float = 0.0, weight_scale: float = 1.0,
):
    """Router logits h @ router^T in fp32 (h in the activation dtype, router
    fp32 [E, W]) followed by ``router_topk``; returns (indices, weights,
    dense weights or None, logits or None)."""
    logits = torch.nn.functional.linear(h.float(), router.float())
    idx, w, dw = router_topk(
        logits, top, softmax, renorm, dense, correction, renorm_eps,
        weight_scale,
    )
    return idx, w, dw, (logits if want_logits else None)


def gather_scale_rows(x, rows, scales):
    """out[r] = x[rows[r]] * scales[r] (product in fp32, rounded to x's dtype);
    without scales a plain row gather."""
    if scales is None:
        return x[rows.long()].contiguous()
    return (x[rows.long()].float() * scales.float().unsqueeze(1)).to(x.dtype)


def combine_rows(
    y, index, top: int, extra=None, weights=None, scaled=None, scaled_w=None
):
    """out[t] = sum_k weights[t*top + k] * y[index[t*top + k]] (+ extra[t])
    (+ scaled_w[t] * scaled[t]), summed in fp32 in the order k = 0..top-1,
    extra, scaled row; weights default to 1; fp32 result."""
    T = index.numel() // top
    out = torch.zeros(T, y.shape[1], dtype=torch.float32, device=y.device)
    idx = index.long().view(T, top)
    for k in range(top):
        r = y[idx[:, k]].float()
        if weights is not None:
            r = r * weights.float().view(T, top)[:, k : k + 1]
        out += r
    if extra is not None:
        out += extra.float()
    if scaled is not None:
        out += scaled.float() * scaled_w.float().view(T, 1)
    return out


def clamped_swiglu(x, alpha: float, limit: float):
    d = x.shape[-1] // 2
    g = x[..., :d].float().clamp(max=limit)
    u = x[..., d:].float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1.0)).to(x.dtype)


# -- latent attention, post-layer-norm residual, plain feed-forwards ----------

def post_layer_norm_add(
    residual, delta, weight, mult: float, eps: float, out_dtype,
    next_weight=None, want_out: bool = True,
):
    """residual (fp32, in place) += mult * LayerNorm(delta) * weight (mean
    removed, biased variance, no bias term), when ``delta`` is given. Returns
    the new residual in ``out_dtype`` or, with ``next_weight``, its layer
    norm times that weight (None when ``want_out`` is false)."""
    if delta is not None:
        d = delta.float()
        d = d - d.mean(-1, keepdim=True)
        d = d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps)
        residual += mult * (d * weight)
    if not want_out:
        return None
    if next_weight is None:
        return residual.to(out_dtype)
    r = residual - residual.mean(-1, keepdim=True)
    r = r * torch.rsqrt(r.pow(2).mean(-1, keepdim=True) + eps)
    return (r * next_weight).to(out_dtype)


def rotate_pairs(x, positions, inv_freq):
    """Rotate the first 2*len(inv_freq) coordinates of the last axis of
    x [T, ..., n] (fp32): coordinate 2i pairs with 2i+1 and turns by
    position * inv_freq[i]; angles and sin/cos in fp32."""
    half = 0 if inv_freq is None else inv_freq.numel()
    if half == 0:
        return x
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    a = (positions.to(torch.float32).view(-1, 1) * inv_freq.view(1, -1)).view(shape)
    c, s = torch.cos(a), torch.sin(a)
    u, v = x[..., 0 : 2 * half : 2], x[..., 1 : 2 * half : 2]
    out = x.clone()
    out[..., 0 : 2 * half : 2] = u * c - v * s
    out[..., 1 : 2 * half : 2] = v * c + u * s
    return out


def latent_norm_rope_cache(
    proj, q_rank: int, kv_rank: int, rot_dim: int, qw, kw, positions,
    slot_mapping, cache, eps: float, inv_freq,
):
    """proj [T, >= q_rank + kv_rank + rot_dim] = [query latent | kv latent |
    key part to rotate | ...]. Returns the RMS-normed query latent times
    ``qw`` in proj's dtype; writes [normed kv latent * kw | rotated key part]
    into ``cache`` [blocks, 1, block, kv_rank + rot_dim] at the tokens'
    slots (negative slots are skipped). ``cache`` None: the query side only."""
    x = proj[:, :q_rank].float()
    cq = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * qw
    if cache is not None:
        c = proj[:, q_rank : q_rank + kv_rank].float()
        c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * kw
        row = c
        if rot_dim:
            kr = proj[:, q_rank + kv_rank : q_rank + kv_rank + rot_dim].float()
            row = torch.cat([c, rotate_pairs(kr, positions, inv_freq)], dim=-1)
        bs = cache.shape[2]
        slots = slot_mapping[: proj.shape[0]].long()
        ok = slots >= 0
        cache[slots[ok] // bs, 0, slots[ok] % bs] = row[ok].to(cache.dtype)
    return cq.to(proj.dtype)


def head_matmul_rope(
    x, w, heads: int, tail: int, positions, inv_freq, out_dtype
):
    """x [T, heads * (k + tail)], w [heads, n, k] -> [T, heads * (n + tail)]:
    per head the head's matrix times the first k coordinates (fp32 sums),
    followed by the ``tail`` coordinates rotated in pairs by the token's
    position (copied when ``inv_freq`` is None)."""
    T = x.shape[0]
    H, n, k = w.shape
    xh = x.reshape(T, heads, k + tail).float()
    y = torch.einsum("thk,hnk->thn", xh[..., :k], w.float())
    if tail:
        y = torch.cat([y, rotate_pairs(xh[..., k:], positions, inv_freq)], dim=-1)
    return y.reshape(T, heads * (n + tail)).to(out_dtype)


def glu_silu_scale(x, scales=None):
    """x [rows, 2 d] = [gate | up] -> silu(gate) * up (* scales[row]) in x's
    dtype; arithmetic in fp32."""
    d = x.shape[-1] // 2
    g, u = x[..., :d].float(), x[..., d:].float()
    y = g * torch.sigmoid(g) * u
    if scales is not None:
        y = y * scales.float().view(-1, 1)
    return y.to(x.dtype)


def bias_gelu_tanh(x, bias):
    """gelu (tanh form) of x + bias in x's dtype; arithmetic in fp32."""
    z = x.float() + bias.float()
    y = 0.5 * z * (1.0 + torch.tanh(0.7978845608028654 * (z + 0.044715 * z * z * z)))
    return y.to(x.dtype)


def rope_scale_heads(x, positions, inv_freq, heads_a, scale_a, heads_b, scale_b, dim):
    """fp32 copy of x [T, width]; rotary positions (pairs i, i + half) on the
    first heads_a + heads_b heads of ``dim`` columns, the first run times
    scale_a, the second times scale_b; the remaining columns unchanged."""
    T = x.shape[0]
    out = x.float().clone()
    n = (heads_a + heads_b) * dim
    if n:
        xf = out[:, :n].reshape(T, heads_a + heads_b, dim)
        if inv_freq is not None:
            xf = rotate_halves(xf, positions, inv_freq)
        sc = torch.cat(
            [torch.full((heads_a,), float(scale_a)), torch.full((heads_b,), float(scale_b))]
        ).view(1, -1, 1)
        out[:, :n] = (xf * sc).reshape(T, n)
    return out


def unit_norm_heads(x, heads_a, scale_a, heads_b, scale_b, dim, eps):
    """In place: heads of ``dim`` columns become unit vectors
    (x / sqrt(sum x^2 + eps)) times scale_a (first heads_a heads) or scale_b
    (next heads_b)."""
    T = x.shape[0]
    for lo, n, sc in ((0, heads_a, scale_a), (heads_a * dim, heads_b, scale_b)):
        if n:
            part = x[:, lo : lo + n * dim].reshape(T, n, dim)
            part = part * torch.rsqrt(part.pow(2).sum(-1, keepdim=True) + eps) * sc
            x[:, lo : lo + n * dim] = part.reshape(T, n * dim)
    return x


def linear_scan(
    q, k, v, state, positions, cu_seqlens, slots, qk_heads, decay=None,
    a_raw=None, b_raw=None, a_log=None, dt_bias=None,
):
    """Token-by-token form of the decay / gated-delta recurrences; state
    [slots, heads, V, K] fp32 is read (unless the portion starts at position
    0) and written back."""
    _, heads, V, K = state.shape
    T = q.shape[0]
    rep = heads // qk_heads
    o = torch.empty(T, heads * V, dtype=torch.float32)
    cu = cu_seqlens.tolist()
    if decay is None:
        sp = a_raw.float() + dt_bias
        sp = torch.where(sp > 30.0, sp, torch.log1p(torch.exp(sp)))
        g_all = torch.exp(-torch.exp(a_log) * sp)          # [T, heads]
        b_all = torch.sigmoid(b_raw.float())
    for s, slot in enumerate(slots.tolist()):
        a, b = cu[s], cu[s + 1]
        if b <= a:
            continue
        S = state[slot].clone()                              # [heads, V, K]
        if int(positions[a]) == 0:
            S.zero_()
        for t in range(a, b):
            qt = q[t].float().reshape(qk_heads, K).repeat_interleave(rep, dim=0)
            kt = k[t].float().reshape(qk_heads, K).repeat_interleave(rep, dim=0)
            vt = v[t].float().reshape(heads, V)
            if decay is not None:
                S = decay[:, None, None] * S + vt[:, :, None] * kt[:, None, :]
            else:
                S = g_all[t][:, None, None] * S
                u = b_all[t][:, None] * (vt - (S * kt[:, None, :]).sum(-1))
                S = S + u[:, :, None] * kt[:, None, :]
            o[t] = (S * qt[:, None, :]).sum(-1).reshape(-1)
        state[slot] = S
    return o


def relu2_scale(x, scales=None):
    """max(x, 0)^2 (* scales[row]) in x's dtype; arithmetic in fp32."""
    y = torch.relu(x.float()).pow(2)
    if scales is not None:
        y = y * scales.float().view(-1, 1)
    return y.to(x.dtype)


def scale_softcap(x, scale: float, cap: float):
    z = x.float() * scale
    return cap * torch.tanh(z / cap) if cap > 0 else z
