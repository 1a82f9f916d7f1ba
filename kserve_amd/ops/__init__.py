"""Custom op dispatch: CDNA4 HIP kernels on GPU, torch reference on CPU.

Policy: GPU tensors MUST run the native
extension — if ``kserve_amd_C`` is missing on a CUDA/ROCm device the op
raises ``NoNativeExtension`` instead of silently falling back to eager
torch. CPU tensors use the fp32 torch reference (tests, engine logic).
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from kserve_amd.errors import NoNativeExtension
from kserve_amd.ops import torch_ref

_C = None
_IMPORT_ERROR: Optional[str] = None
try:
    import kserve_amd_C as _C  # built in-tree by setup.py (travels to GPU box)
except ImportError as e:  # pragma: no cover - exercised on GPU box
    _IMPORT_ERROR = str(e)


# kernels of the 32-bit-residual / recurrent-state mechanisms (own module so
# a model built from them compiles nothing else); carries the samplers too
_SEQ = None
_SEQ_IMPORT_ERROR: Optional[str] = None
try:
    import kserve_amd_seq_C as _SEQ
except ImportError as e:  # pragma: no cover - exercised on GPU box
    _SEQ_IMPORT_ERROR = str(e)


def has_native() -> bool:
    return _C is not None


def has_native_seq() -> bool:
    return _SEQ is not None


def _native_seq(op: str):
    if _SEQ is None:
        raise NoNativeExtension(op, f"(import error: {_SEQ_IMPORT_ERROR})")
    return _SEQ


def _native_sampling(op: str):
    """The samplers are linked into every extension module."""
    return _C if _C is not None else _native_seq(op)


def _native(op: str):
    if _C is None:
        raise NoNativeExtension(op, f"(import error: {_IMPORT_ERROR})")
    return _C


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    if x.is_cuda:
        out = torch.empty_like(x)
        _native("rms_norm").rms_norm(out, x, weight, eps)
        return out
    return torch_ref.rms_norm(x, weight, eps)


def fused_add_rms_norm(
    x: torch.Tensor, residual: torch.Tensor, weight: torch.Tensor, eps: float
) -> Tuple[torch.Tensor, torch.Tensor]:
    """In-place on GPU: x <- rmsnorm(x+residual), residual <- x+residual."""
    if x.is_cuda:
        _native("fused_add_rms_norm").fused_add_rms_norm(x, residual, weight, eps)
        return x, residual
    return torch_ref.fused_add_rms_norm(x, residual, weight, eps)


def silu_and_mul(x: torch.Tensor) -> torch.Tensor:
    if x.is_cuda:
        d = x.shape[-1] // 2
        out = torch.empty(
            (*x.shape[:-1], d), dtype=x.dtype, device=x.device
        )
        _native("silu_and_mul").silu_and_mul(out, x)
        return out
    return torch_ref.silu_and_mul(x)


def rotary_embedding(
    positions: torch.Tensor,
    q: torch.Tensor,
    k: torch.Tensor,
    cos_sin_cache: torch.Tensor,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Neox-style RoPE. GPU path mutates q/k in place and returns them."""
    if q.is_cuda:
        _native("rotary_embedding").rotary_embedding(positions, q, k, cos_sin_cache)
        return q, k
    return torch_ref.rotary_embedding(positions, q, k, cos_sin_cache)


def reshape_and_cache(
    k: torch.Tensor,
    v: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    slot_mapping: torch.Tensor,
) -> None:
    if k.is_cuda:
        _native("reshape_and_cache").reshape_and_cache(
            k, v, k_cache, v_cache, slot_mapping
        )
        return
    torch_ref.reshape_and_cache(k, v, k_cache, v_cache, slot_mapping)


def paged_attention_decode(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    context_lens: torch.Tensor,
    scale: float,
    out: Optional[torch.Tensor] = None,
    window: int = 0,
) -> torch.Tensor:
    if q.is_cuda:
        if out is None:
            out = torch.empty_like(q)
        _native("paged_attention_decode").paged_attention_decode(
            out, q, k_cache, v_cache, block_tables, context_lens, scale,
            window,
        )
        return out
    return torch_ref.paged_attention_decode(
        q, k_cache, v_cache, block_tables, context_lens, scale,
        window=window,
    )


def flash_prefill_varlen(
    q: torch.Tensor,
    k: torch.Tensor,
    v: torch.Tensor,
    cu_seqlens: torch.Tensor,
    max_seqlen: int,
    scale: float,
    window: int = 0,
) -> torch.Tensor:
    if q.is_cuda:
        out = torch.empty_like(q)
        _native("flash_prefill").flash_prefill_varlen(
            out, q, k, v, cu_seqlens, int(max_seqlen), scale,
            causal=True, window=window,
        )
        return out
    return torch_ref.flash_prefill_varlen(
        q, k, v, cu_seqlens, scale, causal=True, window=window
    )


def context_attention_varlen(
    q: torch.Tensor,
    k_cache: torch.Tensor,
    v_cache: torch.Tensor,
    block_tables: torch.Tensor,
    cu_seqlens_q: torch.Tensor,
    context_lens: torch.Tensor,
    max_q_len: int,
    scale: float,
    window: int = 0,
) -> torch.Tensor:
    """Prefill attention against the paged cache (chunked prefill): the
    chunk's KV must already be written to the cache; queries attend causally
    to the whole per-seq context (bounded below by the sliding window when
    window > 0)."""
    if q.is_cuda:
        out = torch.empty_like(q)
        _native("context_prefill").context_prefill_varlen(
            out, q, k_cache, v_cache, block_tables, context_lens,
            cu_seqlens_q, int(max_q_len), scale, window
        )
        return out
    return torch_ref.context_attention_varlen(
        q, k_cache, v_cache, block_tables, cu_seqlens_q, context_lens, scale,
        window=window,
    )


def greedy_sample(logits: torch.Tensor) -> torch.Tensor:
    if logits.is_cuda:
        if logits.dtype != torch.bfloat16:
            # fp32 engines: the argmax must see every bit of the logits
            return torch.argmax(logits, dim=-1)
        out = torch.empty(
            logits.shape[0], dtype=torch.int64, device=logits.device
        )
        _native_sampling("greedy_sample").greedy_sample(out, logits)
        return out
    return torch_ref.greedy_sample(logits)


def random_sample(
    logits: torch.Tensor,
    temperatures: torch.Tensor,
    top_p: torch.Tensor,
    top_k: torch.Tensor,
    seeds: Optional[torch.Tensor] = None,
    generator: Optional[torch.Generator] = None,
    min_p: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """Temperature/top-k/top-p/min-p sampling.

    GPU: one fused HIP kernel. Plain temperature sampling is Gumbel-max;
    top-k/top-p use a bf16 radix-histogram select (exact k-th value / mass
    threshold, no sort) followed by Gumbel-max over the surviving set.
    min_p (rare) routes to the fp32 sort path.
    """
    has_min_p = min_p is not None and bool((min_p > 0).any())
    if logits.is_cuda and seeds is not None and not has_min_p:
        if logits.dtype != torch.bfloat16:
            logits = logits.to(torch.bfloat16)  # the fused samplers' format
        out = torch.empty(
            logits.shape[0], dtype=torch.int64, device=logits.device
        )
        needs_trunc = bool((top_p < 1.0).any()) or bool((top_k > 0).any())
        if needs_trunc:
            _native_sampling("random_sample").topk_topp_sample(
                out, logits, temperatures, top_p, top_k.to(torch.int32), seeds
            )
        else:
            _native_sampling("random_sample").gumbel_sample(
                out, logits, temperatures, top_k.to(torch.int32), seeds
            )
        return out
    # min-p (or CPU): fp32 sort path
    return torch_ref.random_sample(
        logits, temperatures, top_p, top_k, generator=generator, min_p=min_p
    )


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """GEMM dispatch: custom MFMA skinny-GEMM for decode-sized batches
    (weight-streaming regime where hipBLASLt underperforms ~4x on gfx950 —
    see tools/gemm_bench.py), hipBLASLt via F.linear otherwise."""
    import torch.nn.functional as F

    # measured crossover (tools/gemm_bench.py on MI355X): the custom kernel
    # beats hipBLASLt only for small token batches on qkv/o-sized shapes;
    # hipBLASLt keeps the wide-M / large-K / large-N shapes.
    if (
        _C is not None
        and x.is_cuda
        and bias is None
        and x.dim() == 2
        and 0 < x.shape[0] <= 64
        and weight.shape[0] % 64 == 0
        and weight.shape[0] <= 8192
        and weight.shape[1] % 64 == 0
        and weight.shape[1] <= 8192
        and x.stride(1) == 1
    ):
        out = torch.empty(
            (x.shape[0], weight.shape[0]), dtype=x.dtype, device=x.device
        )
        _C.skinny_gemm(out, x, weight)
        return out
    return F.linear(x, weight, bias)


def layer_norm(x, weight, bias, eps: float):
    if x.is_cuda:
        out = torch.empty_like(x)
        _native("layer_norm").layer_norm(out, x, weight, bias, eps)
        return out
    return torch_ref.layer_norm(x, weight, bias, eps)


def fused_add_layer_norm(x, residual, weight, bias, eps: float):
    if x.is_cuda:
        out = torch.empty_like(x)
        _native("fused_add_layer_norm").fused_add_layer_norm(
            out, x, residual, weight, bias, eps
        )
        return out
    return torch_ref.fused_add_layer_norm(x, residual, weight, bias, eps)


def gelu(x):
    if x.is_cuda:
        out = torch.empty_like(x)
        _native("gelu").gelu(out, x)
        return out
    return torch_ref.gelu(x)


def flash_attn_varlen(q, k, v, cu_seqlens, max_seqlen, scale, causal=True):
    """Bidirectional-capable variant (encoder models)."""
    if q.is_cuda:
        out = torch.empty_like(q)
        _native("flash_prefill").flash_prefill_varlen(
            out, q, k, v, cu_seqlens, int(max_seqlen), scale, causal
        )
        return out
    return torch_ref.flash_prefill_varlen(q, k, v, cu_seqlens, scale, causal=causal)


def topk_topp_sample_into(
    out: torch.Tensor,
    logits: torch.Tensor,
    temperatures: torch.Tensor,
    top_p: torch.Tensor,
    top_k: torch.Tensor,
    seeds: torch.Tensor,
) -> torch.Tensor:
    """Destination-passing form of the fused sampler for hipGraph capture
    (static out buffer, per-row device seeds; see model_runner
    _ensure_sampled_graph). GPU-only."""
    if logits.dtype != torch.bfloat16:
        logits = logits.to(torch.bfloat16)  # the fused samplers' format
    _native_sampling("random_sample").topk_topp_sample(
        out, logits, temperatures, top_p,
        top_k if top_k.dtype == torch.int32 else top_k.to(torch.int32),
        seeds,
    )
    return out


# -- 32-bit residual stream, recurrent state, fp32 attention -----------------

def _f32_like(rows: int, cols: int, ref: torch.Tensor) -> torch.Tensor:
    return torch.empty((rows, cols), dtype=torch.float32, device=ref.device)


def embed_scale_sinpos(table, tokens, positions, inv_freq, scale: float):
    """fp32 [T, width]: table[token] * scale + interleaved sin/cos of
    position * inv_freq (the start of an fp32 residual stream)."""
    if table.is_cuda:
        out = _f32_like(tokens.shape[0], table.shape[1], table)
        # inv_freq None: no positional term
        _native_seq("embed_scale_sinpos").embed_scale_sinpos(
            out, table, tokens, positions, inv_freq, float(scale)
        )
        return out
    return torch_ref.embed_scale_sinpos(table, tokens, positions, inv_freq, scale)


def add_rms_norm_f32res(
    residual, weight, eps: float, w_offset: float, out_dtype,
    d0=None, s0: float = 1.0, d1=None, s1: float = 1.0,
):
    """residual (fp32, in place) += s0*d0 + s1*d1, then RMS norm with weight
    (w_offset + w); returns the normed rows in ``out_dtype``."""
    if residual.is_cuda:
        out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
        _native_seq("add_rms_norm_f32res").add_rms_norm_f32res(
            residual, d0, float(s0), d1, float(s1), weight, float(w_offset),
            float(eps), out,
        )
        return out
    return torch_ref.add_rms_norm_f32res(
        residual, weight, eps, w_offset, out_dtype, d0, s0, d1, s1
    )


def gated_group_rms_norm(
    y, z, weight, eps: float, groups: int, out_dtype, gate_after: bool = False
):
    """RMS norm of fp32 ``y`` in ``groups`` equal parts with a silu(z) gate:
    on the input of the norm, or (``gate_after``) on its output. ``weight``
    may be shorter than a row (it repeats: one vector shared by the groups)
    or None."""
    if y.is_cuda:
        out = torch.empty(y.shape, dtype=out_dtype, device=y.device)
        _native_seq("gated_group_rms_norm").gated_group_rms_norm(
            out, y, z, weight, float(eps), int(groups), bool(gate_after)
        )
        return out
    return torch_ref.gated_group_rms_norm(
        y, z, weight, eps, groups, out_dtype, gate_after
    )


def causal_conv_silu(
    x_in, w, bias, conv_state, positions, seq_of_token, cu_seqlens, slots
):
    """Depthwise causal conv + silu over a flat varlen batch; reads and then
    advances each sequence's conv history in ``conv_state[slot]``."""
    if x_in.is_cuda:
        out = _f32_like(x_in.shape[0], x_in.shape[1], x_in)
        _native_seq("causal_conv_silu").causal_conv_silu(
            out, x_in, w, bias, conv_state, positions, seq_of_token,
            cu_seqlens, slots,
        )
        return out
    return torch_ref.causal_conv_silu(
        x_in, w, bias, conv_state, positions, cu_seqlens, slots
    )


def ssd_scan(
    xbc, dt_raw, dt_bias, a_log, d_skip, state, positions, cu_seqlens, slots,
    groups: int,
):
    """State-space scan; carries ``state[slot]`` ([heads, P, N] fp32)."""
    if xbc.is_cuda:
        heads, P = state.shape[1], state.shape[2]
        y = _f32_like(xbc.shape[0], heads * P, xbc)
        _native_seq("ssd_scan").ssd_scan(
            y, xbc, dt_raw, dt_bias, a_log, d_skip, state, positions,
            cu_seqlens, slots, int(groups),
        )
        return y
    return torch_ref.ssd_scan(
        xbc, dt_raw, dt_bias, a_log, d_skip, state, positions, cu_seqlens,
        slots, groups,
    )


def qk_norm_temp_cache(
    q, k, v, qw, kw, positions, slot_mapping, k_cache, v_cache, eps: float,
    temp_coef: float, temp_every: int, heads: int,
):
    if q.is_cuda:
        q_out = _f32_like(q.shape[0], q.shape[1], q)
        _native_seq("qk_norm_temp_cache").qk_norm_temp_cache(
            q_out, q, k, v, qw, kw, positions, slot_mapping, k_cache, v_cache,
            float(eps), float(temp_coef), int(temp_every), int(heads),
        )
        return q_out
    return torch_ref.qk_norm_temp_cache(
        q, k, v, qw, kw, positions, slot_mapping, k_cache, v_cache, eps,
        temp_coef, temp_every, heads,
    )


def ctx_attention_f32(
    q, k_cache, v_cache, block_tables, cu_q, ctx_lens, scale: float,
    max_q_len: int, heads: int, gate=None, out_dtype=torch.float32,
    sink=None, chunk: int = 0, out_inv_freq=None, window: int = 0,
):
    """Paged causal attention with fp32 scores and weights. Optional parts:
    ``gate`` [T, heads] (output times sigmoid), ``sink`` [heads] fp32 (one
    more term exp(sink) in the softmax denominator), ``chunk`` (a query sees
    only keys of its own block of that many positions), ``window`` (a query
    sees itself and the window-1 positions before it), ``out_inv_freq``
    [vdim/2] fp32 (each head output turned back by its query position).
    ``v_cache`` may be a view of the leading columns of ``k_cache`` (values
    that are a prefix of the keys are stored once)."""
    if q.is_cuda:
        out = torch.empty(
            (q.shape[0], heads * v_cache.shape[3]), dtype=out_dtype,
            device=q.device,
        )
        _native_seq("ctx_attention_f32").ctx_attention_f32(
            out, q, k_cache, v_cache, block_tables, cu_q, ctx_lens, gate,
            float(scale), int(max_q_len), int(heads), sink, int(chunk),
            out_inv_freq, int(window),
        )
        return out
    return torch_ref.ctx_attention_f32(
        q, k_cache, v_cache, block_tables, cu_q, ctx_lens, scale, heads,
        gate, out_dtype, sink, chunk, out_inv_freq, window,
    )


def qk_headnorm_rope_cache(
    q, k, v, qw, kw, positions, slot_mapping, k_cache, v_cache, eps: float,
    heads: int, qk_inv_freq=None, v_unit_norm: bool = False, v_inv_freq=None,
):
    """Per-head q/k RMS norm (weights [dim]) + rotary positions, optional
    unit-norm and rotation of the values, KV page scatter; returns q fp32."""
    if q.is_cuda:
        q_out = _f32_like(q.shape[0], q.shape[1], q)
        _native_seq("qk_headnorm_rope_cache").qk_headnorm_rope_cache(
            q_out, q, k, v, qw, kw, positions, slot_mapping, k_cache, v_cache,
            float(eps), int(heads), qk_inv_freq, bool(v_unit_norm), v_inv_freq,
        )
        return q_out
    return torch_ref.qk_headnorm_rope_cache(
        q, k, v, qw, kw, positions, slot_mapping, k_cache, v_cache, eps,
        heads, qk_inv_freq, v_unit_norm, v_inv_freq,
    )


def post_norm_add_rms_norm(
    residual, delta, post_gain: float, layer_scale, eps: float,
    next_gain: float, out_dtype, add_rows=None, add_vec=None,
    want_out: bool = True,
):
    """Close one sandwich-normed sublayer and open the next in one pass over
    the fp32 residual (in place): += layer_scale * scalar-gain RMS norm of the
    sublayer output, += optional per-token rows and one shared row, then the
    scalar-gain RMS norm of the result in ``out_dtype``."""
    if residual.is_cuda:
        out = (
            torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
            if want_out else None
        )
        _native_seq("post_norm_add_rms_norm").post_norm_add_rms_norm(
            residual, delta, float(post_gain), layer_scale, float(eps),
            float(next_gain), out, add_rows, add_vec,
        )
        return out
    return torch_ref.post_norm_add_rms_norm(
        residual, delta, post_gain, layer_scale, eps, next_gain, out_dtype,
        add_rows, add_vec, want_out,
    )


def router_topk(
    logits, top: int, softmax: bool = False, renorm: bool = False,
    dense: bool = False, correction=None, renorm_eps: float = 0.0,
    weight_scale: float = 1.0,
):
    """fp32 router logits [T, E] -> (expert ids int32 [T, top], weights fp32
    [T, top], dense [T, E] weights or None) by sigmoid (or softmax) score;
    with ``correction`` [E] fp32 the choice goes by score + correction."""
    if logits.is_cuda:
        T, E = logits.shape
        idx = torch.empty((T, top), dtype=torch.int32, device=logits.device)
        w = torch.empty((T, top), dtype=torch.float32, device=logits.device)
        dw = (
            torch.empty((T, E), dtype=torch.float32, device=logits.device)
            if dense else None
        )
        _native_seq("router_topk").router_topk(
            idx, w, dw, logits, bool(softmax), bool(renorm), correction,
            float(renorm_eps), float(weight_scale),
        )
        return idx, w, dw
    return torch_ref.router_topk(
        logits, top, softmax, renorm, dense, correction, renorm_eps,
        weight_scale,
    )


def route_tokens(
    h, router, top: int, softmax: bool = False, renorm: bool = False,
    dense: bool = False, want_logits: bool = False, correction=None,
    renorm_eps: float = 0.0, weight_scale: float = 1.0,
):
    """The router in one kernel: fp32 logits of h [T, W] (activation dtype)
    against fp32 router rows [E, W], scores, the ``top`` experts. Returns
    (expert ids int32 [T, top], weights fp32 [T, top], dense [T, E] weights or
    None, logits fp32 [T, E] or None)."""
    if h.is_cuda:
        T, E = h.shape[0], router.shape[0]
        dev = h.device
        idx = torch.empty((T, top), dtype=torch.int32, device=dev)
        w = torch.empty((T, top), dtype=torch.float32, device=dev)
        dw = torch.empty((T, E), dtype=torch.float32, device=dev) if dense else None
        lg = torch.empty((T, E), dtype=torch.float32, device=dev) if want_logits else None
        _native_seq("route_tokens").route_tokens(
            idx, w, dw, lg, h, router, bool(softmax), bool(renorm), correction,
            float(renorm_eps), float(weight_scale),
        )
        return idx, w, dw, lg
    return torch_ref.route_tokens(
        h, router, top, softmax, renorm, dense, want_logits, correction,
        renorm_eps, weight_scale,
    )


def gather_scale_rows(x, rows, scales=None):
    """out[r] = x[rows[r]] * scales[r] in x's dtype (rows int32, scales fp32
    or None for a plain gather)."""
    if x.is_cuda:
        out = torch.empty((rows.numel(), x.shape[1]), dtype=x.dtype, device=x.device)
        _native_seq("gather_scale_rows").gather_scale_rows(out, x, rows, scales)
        return out
    return torch_ref.gather_scale_rows(x, rows, scales)


def combine_rows(
    y, index, top: int, extra=None, weights=None, scaled=None, scaled_w=None
):
    """fp32 out[t] = sum_k weights[t*top + k] * y[index[t*top + k]]
    (+ extra[t]) (+ scaled_w[t] * scaled[t]); weights (fp32) default to 1."""
    if y.is_cuda:
        out = _f32_like(index.numel() // top, y.shape[1], y)
        _native_seq("combine_rows").combine_rows(
            out, y, index, int(top), extra, weights, scaled, scaled_w
        )
        return out
    return torch_ref.combine_rows(y, index, top, extra, weights, scaled, scaled_w)


def clamped_swiglu(x, alpha: float, limit: float):
    if x.is_cuda:
        out = torch.empty(
            (*x.shape[:-1], x.shape[-1] // 2), dtype=x.dtype, device=x.device
        )
        _native_seq("clamped_swiglu").clamped_swiglu(
            out, x, float(alpha), float(limit)
        )
        return out
    return torch_ref.clamped_swiglu(x, alpha, limit)


# -- latent attention, post-layer-norm residual, plain feed-forwards ----------

def post_layer_norm_add(
    residual, delta, weight, mult: float, eps: float, out_dtype,
    next_weight=None, want_out: bool = True,
):
    """fp32 residual (in place) += mult * LayerNorm(delta) * weight (no bias)
    when ``delta`` is given; returns the new residual in ``out_dtype`` or,
    with ``next_weight``, its layer norm times that weight."""
    if residual.is_cuda:
        out = (
            torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
            if want_out else None
        )
        _native_seq("post_layer_norm_add").post_layer_norm_add(
            residual, delta, weight, float(mult), float(eps), out, next_weight
        )
        return out
    return torch_ref.post_layer_norm_add(
        residual, delta, weight, mult, eps, out_dtype, next_weight, want_out
    )


def latent_norm_rope_cache(
    proj, q_rank: int, kv_rank: int, rot_dim: int, qw, kw, positions,
    slot_mapping, cache, eps: float, inv_freq,
):
    """Rows [query latent | kv latent | key part | ...] -> the RMS-normed
    query latent (returned, activation dtype) and, when ``cache`` is given,
    [normed kv latent | key part rotated in pairs (2i, 2i+1)] scattered into
    the paged cache [blocks, 1, block, kv_rank + rot_dim]."""
    if proj.is_cuda:
        cq = torch.empty((proj.shape[0], q_rank), dtype=proj.dtype, device=proj.device)
        _native_seq("latent_norm_rope_cache").latent_norm_rope_cache(
            cq, proj, int(q_rank), int(kv_rank), int(rot_dim), qw, kw,
            positions, slot_mapping, cache, float(eps), inv_freq,
        )
        return cq
    return torch_ref.latent_norm_rope_cache(
        proj, q_rank, kv_rank, rot_dim, qw, kw, positions, slot_mapping,
        cache, eps, inv_freq,
    )


def head_matmul_rope(
    x, w, heads: int, tail: int = 0, positions=None, inv_freq=None,
    out_dtype=None,
):
    """Per-head matrix product with an optional rotated tail:
    x [T, heads*(k + tail)], w [heads, n, k] -> [T, heads*(n + tail)], the
    tail coordinates turned in pairs by the token's position."""
    out_dtype = out_dtype or x.dtype
    if x.is_cuda:
        n = w.shape[1]
        out = torch.empty(
            (x.shape[0], heads * (n + tail)), dtype=out_dtype, device=x.device
        )
        _native_seq("head_matmul_rope").head_matmul_rope(
            out, x, w, int(heads), int(tail), positions, inv_freq
        )
        return out
    return torch_ref.head_matmul_rope(
        x, w, heads, tail, positions, inv_freq, out_dtype
    )


def glu_silu_scale(x, scales=None):
    """[rows, 2 d] = [gate | up] -> silu(gate) * up (* scales[row])."""
    if x.is_cuda:
        out = torch.empty(
            (x.shape[0], x.shape[1] // 2), dtype=x.dtype, device=x.device
        )
        _native_seq("glu_silu_scale").glu_silu_scale(out, x, scales)
        return out
    return torch_ref.glu_silu_scale(x, scales)


def bias_gelu_tanh(x, bias):
    """gelu (tanh form) of x + bias, in x's dtype."""
    if x.is_cuda:
        out = torch.empty_like(x)
        _native_seq("bias_gelu_tanh").bias_gelu_tanh(out, x, bias)
        return out
    return torch_ref.bias_gelu_tanh(x, bias)


# -- linear-attention recurrences, squared-relu experts, capped logits --------

def rope_scale_heads(
    x, positions, inv_freq, heads_a: int, scale_a: float, heads_b: int,
    scale_b: float, dim: int,
):
    """fp32 copy of rows x [T, width]: the first ``heads_a`` heads of ``dim``
    columns get rotary positions on their first 2*len(inv_freq) coordinates
    (i pairs with i + half) and are multiplied by scale_a, the next
    ``heads_b`` likewise with scale_b; further columns are only widened."""
    if x.is_cuda:
        out = _f32_like(x.shape[0], x.shape[1], x)
        _native_seq("rope_scale_heads").rope_scale_heads(
            out, x, positions, inv_freq, int(heads_a), float(scale_a),
            int(heads_b), float(scale_b), int(dim),
        )
        return out
    return torch_ref.rope_scale_heads(
        x, positions, inv_freq, heads_a, scale_a, heads_b, scale_b, dim
    )


def unit_norm_heads(
    x, heads_a: int, scale_a: float, heads_b: int, scale_b: float, dim: int,
    eps: float,
):
    """In place on fp32 rows: the first ``heads_a`` heads of ``dim`` columns
    become x / sqrt(sum(x^2) + eps) * scale_a, the next ``heads_b`` likewise
    with scale_b; further columns are left alone."""
    if x.is_cuda:
        _native_seq("unit_norm_heads").unit_norm_heads(
            x, int(heads_a), float(scale_a), int(heads_b), float(scale_b),
            int(dim), float(eps),
        )
        return x
    return torch_ref.unit_norm_heads(x, heads_a, scale_a, heads_b, scale_b, dim, eps)


def linear_scan(
    q, k, v, state, positions, cu_seqlens, slots, qk_heads: int,
    decay=None, a_raw=None, b_raw=None, a_log=None, dt_bias=None,
):
    """Linear-attention recurrence over a flat varlen batch; carries
    ``state[slot]`` ([heads, V, K] fp32). q, k [T, qk_heads*K] and
    v [T, heads*V] are fp32 (rows may be strided). With ``decay`` [heads]:
    S <- d S + k v^T. Without: the gated delta rule with
    g = exp(-exp(a_log) softplus(a_raw + dt_bias)), b = sigmoid(b_raw):
    S <- g S; S <- S + k (b (v - S^T k))^T. Output o = S^T q, fp32."""
    if q.is_cuda:
        heads, V = state.shape[1], state.shape[2]
        o = _f32_like(q.shape[0], heads * V, q)
        _native_seq("linear_scan").linear_scan(
            o, q, k, v, decay, a_raw, b_raw, a_log, dt_bias, state, positions,
            cu_seqlens, slots, int(qk_heads),
        )
        return o
    return torch_ref.linear_scan(
        q, k, v, state, positions, cu_seqlens, slots, qk_heads, decay, a_raw,
        b_raw, a_log, dt_bias,
    )


def relu2_scale(x, scales=None):
    """max(x, 0)^2 (* scales[row]) in x's dtype."""
    if x.is_cuda:
        out = torch.empty_like(x)
        _native_seq("relu2_scale").relu2_scale(out, x, scales)
        return out
    return torch_ref.relu2_scale(x, scales)


def scale_softcap(x, scale: float, cap: float):
    """fp32 cap * tanh(x * scale / cap); cap 0 leaves x * scale."""
    if x.is_cuda:
        out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
        _native_seq("scale_softcap").scale_softcap(out, x, float(scale), float(cap))
        return out
    return torch_ref.scale_softcap(x, scale, cap)
