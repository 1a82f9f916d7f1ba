"""Sequence mixers and feed-forwards for models with a 32-bit residual stream.

Each module owns its weights and runs one sublayer on a flat token batch
``[T, width]`` in the activation dtype (bf16 or fp32). Matrix products go to
the vendor GEMM; everything around them is a HIP kernel from ``kserve_amd.ops``
(CPU tensors take the plain torch forms). Small vectors that enter fp32
arithmetic (norm weights, convolution taps, decay and step parameters) are
kept in fp32 regardless of the activation dtype.

Per-step inputs come from ``AttentionMetadata``: besides the paged-KV fields
they need ``cu_seqlens`` / ``seq_of_token`` (flat-batch layout) and
``state_slots`` (one row of the recurrent-state pools per sequence).
"""

from __future__ import annotations

from typing import NamedTuple, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from kserve_amd import ops
from kserve_amd.engine.config import (
    AttentionMixerSpec,
    DeltaMixerSpec,
    GLUSpec,
    LatentAttentionSpec,
    MLPSpec,
    MoESpec,
    RetentionMixerSpec,
    SoftmaxMoESpec,
    SquaredReluMoESpec,
    SSMMixerSpec,
)
from kserve_amd.ops.torch_ref import rotary_inv_freq


class LayerCache(NamedTuple):
    """What one layer keeps between steps; absent parts are None."""

    k: Optional[torch.Tensor] = None      # [blocks, kv_heads, block, dim]
    v: Optional[torch.Tensor] = None      # [blocks, kv_heads, block, vdim];
    #                                       None where values are read from k
    conv: Optional[torch.Tensor] = None   # [slots, taps-1, channels]
    # matrix state of a recurrent layer, fp32: [slots, heads, vdim, state]
    # (state-space scan) or [slots, heads, vdim, dim] (linear attention)
    ssm: Optional[torch.Tensor] = None


def _param(*shape, dtype):
    return nn.Parameter(torch.empty(*shape, dtype=dtype), requires_grad=False)


class SSDMixer(nn.Module):
    """State-space sublayer (Mamba-2 form): in-projection to
    [z | x | B | C | dt], causal conv + silu over x|B|C, the scan, a gated
    grouped RMS norm, out-projection."""

    def __init__(self, width: int, spec: SSMMixerSpec, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.dtype = dtype
        self.in_proj = _param(spec.proj_width, width, dtype=dtype)
        self.conv_w = _param(spec.conv_channels, spec.conv, dtype=torch.float32)
        self.conv_b = _param(spec.conv_channels, dtype=torch.float32)
        self.dt_bias = _param(spec.heads, dtype=torch.float32)
        self.a_log = _param(spec.heads, dtype=torch.float32)
        self.d_skip = _param(spec.heads, dtype=torch.float32)
        self.norm_w = _param(spec.inner, dtype=torch.float32)
        self.o_proj = _param(width, spec.inner, dtype=dtype)

    def state_shapes(self):
        s = self.spec
        return {
            "conv": ((max(s.conv - 1, 1), s.conv_channels), self.dtype),
            "ssm": ((s.heads, s.vdim, s.state), torch.float32),
        }

    def load(self, get, prefix: str):
        self.in_proj.copy_(get(prefix + "in").to(self.dtype))
        self.conv_w.copy_(get(prefix + "conv").float())
        self.conv_b.copy_(get(prefix + "conv.b").float())
        self.dt_bias.copy_(get(prefix + "dt_bias").float())
        self.a_log.copy_(get(prefix + "A_log").float())
        self.d_skip.copy_(get(prefix + "D").float())
        self.norm_w.copy_(get(prefix + "norm").float())
        self.o_proj.copy_(get(prefix + "o").to(self.dtype))

    def mix(self, proj, positions, cache: LayerCache, meta):
        """``proj``: [T, proj_width] rows of this mixer's in-projection (may be
        a column slice of a wider fused projection)."""
        s = self.spec
        z = proj[:, : s.inner]
        xbc_raw = proj[:, s.inner : s.inner + s.conv_channels]
        dt_raw = proj[:, s.inner + s.conv_channels :]
        xbc = ops.causal_conv_silu(
            xbc_raw, self.conv_w, self.conv_b, cache.conv, positions,
            meta.seq_of_token, meta.cu_seqlens, meta.state_slots,
        )
        y = ops.ssd_scan(
            xbc, dt_raw, self.dt_bias, self.a_log, self.d_skip, cache.ssm,
            positions, meta.cu_seqlens, meta.state_slots, s.groups,
        )
        yn = ops.gated_group_rms_norm(
            y, z, self.norm_w, self.eps, s.norm_groups, self.dtype
        )
        return F.linear(yn, self.o_proj)

    def forward(self, h, positions, cache: LayerCache, meta):
        return self.mix(F.linear(h, self.in_proj), positions, cache, meta)


class NormedGatedAttention(nn.Module):
    """Causal softmax attention without rotation: biased q/k/v projections,
    RMS norm over the whole q (and k) projection, a position-dependent query
    temperature, fp32 scores against the paged cache, a sigmoid output gate
    per head read from the sublayer input, out-projection. The q|k|v|gate
    projections are one fused GEMM."""

    def __init__(self, width: int, spec: AttentionMixerSpec, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.dtype = dtype
        self.q_w = spec.heads * spec.dim
        self.k_w = spec.kv_heads * spec.dim
        self.v_w = spec.kv_heads * spec.vdim
        self.proj_width = self.q_w + self.k_w + self.v_w + spec.heads
        self.qkvg = _param(self.proj_width, width, dtype=dtype)
        self.qkvg_bias = _param(self.proj_width, dtype=dtype)
        self.q_norm = _param(self.q_w, dtype=torch.float32)
        self.k_norm = _param(self.k_w, dtype=torch.float32)
        self.o_proj = _param(width, spec.heads * spec.vdim, dtype=dtype)

    def load(self, get, prefix: str):
        dt = self.dtype
        w = torch.cat(
            [get(prefix + n).to(dt) for n in ("q", "k", "v", "g")], dim=0
        )
        b = torch.cat(
            [get(prefix + n + ".b").to(dt) for n in ("q", "k", "v")]
            + [torch.zeros(self.spec.heads, dtype=dt)]
        )
        self.qkvg.copy_(w)
        self.qkvg_bias.copy_(b)
        self.q_norm.copy_(get(prefix + "q.norm").float())
        self.k_norm.copy_(get(prefix + "k.norm").float())
        self.o_proj.copy_(get(prefix + "o").to(dt))

    def mix(self, proj, positions, cache: LayerCache, meta):
        s = self.spec
        a, b, c = self.q_w, self.q_w + self.k_w, self.q_w + self.k_w + self.v_w
        q, k, v, gate = proj[:, :a], proj[:, a:b], proj[:, b:c], proj[:, c:]
        qn = ops.qk_norm_temp_cache(
            q, k, v, self.q_norm, self.k_norm, positions, meta.slot_mapping,
            cache.k, cache.v, self.eps, s.q_temp_coef, s.q_temp_every, s.heads,
        )
        o = ops.ctx_attention_f32(
            qn, cache.k, cache.v, meta.block_tables, meta.cu_seqlens,
            meta.context_lens, s.scale, meta.max_seqlen, s.heads, gate=gate,
            out_dtype=self.dtype,
        )
        return F.linear(o, self.o_proj)

    def forward(self, h, positions, cache: LayerCache, meta):
        return self.mix(
            F.linear(h, self.qkvg, self.qkvg_bias), positions, cache, meta
        )


class RotaryChunkSinkAttention(nn.Module):
    """Softmax attention with per-head q/k RMS norm (weights of size ``dim``
    shared by the heads), rotary positions on the first ``rot_dims``
    coordinates, fp32 scores against the paged cache, and three optional
    parts: a chunk-local causal mask (``spec.chunk``), a learned per-head
    sink term in the softmax denominator (``sink``), and unit-norm values
    that are rotated by their own position over all of ``vdim`` before they
    are cached, with every head output turned back by the query's position
    (``value_unit_norm`` / ``rotate_values``). ``spec.window`` adds a sliding
    window. With ``norm_weights`` off the q/k norm has no weights (it then
    commutes with the rotation, so "rotate, then norm" is the same sublayer).
    No biases, no gate. The q|k|v projections are one fused GEMM."""

    def __init__(
        self, width: int, spec: AttentionMixerSpec, eps: float, dtype,
        sink: bool = True, value_unit_norm: bool = True,
        rotate_values: bool = True, norm_weights: bool = True,
    ):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.dtype = dtype
        self.q_w = spec.heads * spec.dim
        self.k_w = spec.kv_heads * spec.dim
        self.v_w = spec.kv_heads * spec.vdim
        if spec.rot_dims % 2 or spec.rot_dims > spec.dim:
            raise ValueError("rot dims must be even and at most the head size")
        if rotate_values and spec.vdim % 2:
            raise ValueError("rotated values need an even value size")
        self.qkv = _param(self.q_w + self.k_w + self.v_w, width, dtype=dtype)
        self.q_norm = _param(spec.dim, dtype=torch.float32) if norm_weights else None
        self.k_norm = _param(spec.dim, dtype=torch.float32) if norm_weights else None
        self.sink = _param(spec.heads, dtype=torch.float32) if sink else None
        self.o_proj = _param(width, spec.heads * spec.vdim, dtype=dtype)
        self.value_unit_norm = value_unit_norm
        self.register_buffer(
            "qk_inv_freq",
            rotary_inv_freq(spec.rot_dims, spec.rot_base) if spec.rot_dims else None,
            persistent=False,
        )
        self.register_buffer(
            "v_inv_freq",
            rotary_inv_freq(spec.vdim, spec.rot_base) if rotate_values else None,
            persistent=False,
        )

    def load(self, get, prefix: str):
        dt = self.dtype
        self.qkv.copy_(
            torch.cat([get(prefix + n).to(dt) for n in ("q", "k", "v")], dim=0)
        )
        if self.q_norm is not None:
            self.q_norm.copy_(get(prefix + "q.norm").float())
            self.k_norm.copy_(get(prefix + "k.norm").float())
        if self.sink is not None:
            self.sink.copy_(get(prefix + "sink").float())
        self.o_proj.copy_(get(prefix + "o").to(dt))

    def forward(self, h, positions, cache: LayerCache, meta):
        s = self.spec
        proj = F.linear(h, self.qkv)
        a, b = self.q_w, self.q_w + self.k_w
        qn = ops.qk_headnorm_rope_cache(
            proj[:, :a], proj[:, a:b], proj[:, b:], self.q_norm, self.k_norm,
            positions, meta.slot_mapping, cache.k, cache.v, self.eps, s.heads,
            self.qk_inv_freq, self.value_unit_norm, self.v_inv_freq,
        )
        o = ops.ctx_attention_f32(
            qn, cache.k, cache.v, meta.block_tables, meta.cu_seqlens,
            meta.context_lens, s.scale, meta.max_seqlen, s.heads,
            out_dtype=self.dtype, sink=self.sink, chunk=s.chunk,
            out_inv_freq=self.v_inv_freq, window=s.window,
        )
        return F.linear(o, self.o_proj)


class ClampedGLU(nn.Module):
    """y = g * sigmoid(alpha g) * (u + 1), g = min(W_gate h, limit),
    u = clamp(W_up h, -limit, limit); gate|up are one fused GEMM."""

    ALPHA = 1.702

    def __init__(self, width: int, spec: GLUSpec, dtype):
        super().__init__()
        self.spec = spec
        self.gate_up = _param(2 * spec.ff, width, dtype=dtype)
        self.down = _param(width, spec.ff, dtype=dtype)

    def load(self, get, prefix: str):
        dt = self.gate_up.dtype
        self.gate_up.copy_(
            torch.cat([get(prefix + "gate").to(dt), get(prefix + "up").to(dt)], dim=0)
        )
        self.down.copy_(get(prefix + "down").to(dt))

    def forward(self, h):
        act = ops.clamped_swiglu(
            F.linear(h, self.gate_up), self.ALPHA, self.spec.limit
        )
        return F.linear(act, self.down)


class RoutedClampedMoE(nn.Module):
    """Mixture of clamped gated experts. Router logits are fp32; a token runs
    the ``top`` experts with the largest scores (sigmoid, used as they are),
    each on the token's input TIMES its score, and the expert outputs are
    summed in fp32 together with an optional always-on shared expert.

    Expert weights are stacked ([E, 2 ff, width] gate|up and [E, width, ff]).
    Small batches and captured decode graphs run every expert on every token
    (a GEMM pair per expert) with zero input rows for the experts a token did
    not choose (an expert without biases maps zero to zero, so nothing has to
    be masked afterwards): static shapes, no host synchronisation. Larger
    batches sort the (token, expert) pairs by expert and run one GEMM pair
    per expert on its contiguous rows."""

    ALPHA = ClampedGLU.ALPHA
    # the all-experts form does experts/top times the arithmetic of the sorted
    # one; it is used while that factor times the batch stays below this many
    # token-rows (where reading the expert weights dominates anyway)
    DENSE_ROW_BUDGET = 1024

    def __init__(self, width: int, spec: MoESpec, dtype):
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        E = spec.experts
        # batches up to this size take the all-experts form, eager or
        # captured; decode graphs are captured up to it and larger decode
        # batches run eager steps through the sorted form
        self.dense_max_tokens = max(16, self.DENSE_ROW_BUDGET * spec.top // E)
        if not 1 <= spec.top <= E:
            raise ValueError("top must be between 1 and the number of experts")
        self.router = _param(E, width, dtype=torch.float32)
        self.gate_up = _param(E, 2 * spec.ff, width, dtype=dtype)
        self.down = _param(E, width, spec.ff, dtype=dtype)
        self.shared = (
            ClampedGLU(width, spec.shared, dtype) if spec.shared is not None else None
        )

    def load(self, get, prefix: str):
        dt = self.dtype
        self.router.copy_(get(prefix + "router").float())
        for e in range(self.spec.experts):
            p = f"{prefix}e{e}."
            self.gate_up[e].copy_(
                torch.cat([get(p + "gate").to(dt), get(p + "up").to(dt)], dim=0)
            )
            self.down[e].copy_(get(p + "down").to(dt))
        if self.shared is not None:
            self.shared.load(get, prefix + "shared.")

    def _dense(self, h, dense_w, extra):
        E, T = self.spec.experts, h.shape[0]
        ar = torch.arange(T, dtype=torch.int32, device=h.device)
        # row e*T + t = h[t] * weight[t, e] (zero where e was not chosen)
        xb = ops.gather_scale_rows(
            h, ar.repeat(E), dense_w.t().contiguous().view(-1)
        ).view(E, T, -1)
        # one plain GEMM per expert: the same library call every dense layer
        # makes, and as safe inside a captured graph
        gu = torch.empty((E, T, 2 * self.spec.ff), dtype=h.dtype, device=h.device)
        for e in range(E):
            torch.mm(xb[e], self.gate_up[e].t(), out=gu[e])
        act = ops.clamped_swiglu(
            gu.view(E * T, -1), self.ALPHA, self.spec.limit
        ).view(E, T, -1)
        ye = torch.empty((E, T, h.shape[1]), dtype=h.dtype, device=h.device)
        for e in range(E):
            torch.mm(act[e], self.down[e].t(), out=ye[e])
        ye = ye.view(E * T, -1)
        # token t's E rows are e*T + t
        index = (
            ar.view(T, 1) + T * torch.arange(E, dtype=torch.int32, device=h.device)
        ).view(-1)
        return ops.combine_rows(ye, index, E, extra)

    def _sorted(self, h, idx, w, extra):
        E, top = self.spec.experts, self.spec.top
        flat = idx.view(-1).long()
        order = torch.sort(flat, stable=True).indices
        counts = torch.bincount(flat, minlength=E).tolist()  # host sync
        xs = ops.gather_scale_rows(
            h, (order // top).to(torch.int32), w.view(-1)[order]
        )
        n = xs.shape[0]
        gu = torch.empty((n, 2 * self.spec.ff), dtype=h.dtype, device=h.device)
        a = 0
        for e, c in enumerate(counts):
            if c:
                torch.mm(xs[a : a + c], self.gate_up[e].t(), out=gu[a : a + c])
            a += c
        act = ops.clamped_swiglu(gu, self.ALPHA, self.spec.limit)
        ys = torch.empty((n, h.shape[1]), dtype=h.dtype, device=h.device)
        a = 0
        for e, c in enumerate(counts):
            if c:
                torch.mm(act[a : a + c], self.down[e].t(), out=ys[a : a + c])
            a += c
        # pair p = t*top + k sits at sorted row inv[p]
        inv = torch.empty_like(order)
        inv[order] = torch.arange(n, device=h.device)
        return ops.combine_rows(ys, inv.to(torch.int32), top, extra)

    def forward(self, h):
        """[T, width] in the activation dtype -> fp32 [T, width]."""
        T = h.shape[0]
        extra = self.shared(h) if self.shared is not None else None
        dense = T <= self.dense_max_tokens or (
            h.is_cuda and torch.cuda.is_current_stream_capturing()
        )
        idx, w, dense_w, _ = ops.route_tokens(
            h, self.router, self.spec.top, dense=dense
        )
        if dense:
            return self._dense(h, dense_w, extra)
        return self._sorted(h, idx, w, extra)


class LatentAttention(nn.Module):
    """Attention over one cached latent row per token. The sublayer input is
    projected to [query latent | kv latent | key part | gate] in one GEMM;
    both latents are RMS-normed, the key part is rotated in pairs (2i, 2i+1)
    by the position, and [kv latent | rotated key part] is the only thing
    written to the pages (one "kv head" of ``kv_rank + rot_dim`` columns).

    Keys and values are never expanded. With k_h = U_k[h] c and v_h = U_v[h] c
    the score q_h . k_h equals (U_k[h]^T q_h) . c, so every query head is
    folded through its U_k[h] into latent coordinates (fp32) and attention
    runs as multi-query attention against the cached rows, the latent part of
    the row serving as the value; the weighted latent sum is then taken
    through U_v[h] per head. Scores, weights, sink and the output gate
    (a per-head scalar, so it commutes with U_v[h]) stay in the fp32
    attention kernel.

    Options: ``window`` (sliding), ``sink`` (softmax denominator term),
    ``gate``, ``rot_dim`` = 0 (no positions at all), ``kv_from`` (no kv
    projection: the layer attends to the pages of an earlier layer with its
    own U_k / U_v).

    Rows wider than the attention kernel takes (``MAX_CACHE_DIM``) switch the
    layer to the expanded form: every step reads the sequences' cached rows,
    expands them to per-head keys [unrotated | shared rotated part] and values
    in scratch pages, and runs the same kernel as plain multi-head attention.
    That costs a pass over the whole context per step and a host read of the
    context lengths, so such a model decodes without captured graphs; it is
    there so that any size runs."""

    # widest cached row (and widest head) the fp32 attention kernel takes
    MAX_CACHE_DIM = 256

    def __init__(self, width: int, spec: LatentAttentionSpec, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.dtype = dtype
        s = spec
        if s.rot_dims % 2 or s.rot_dims > s.rot_dim:
            raise ValueError("rotated coordinates: even, at most the rotated part")
        self.expanded = s.cache_dim > self.MAX_CACHE_DIM
        if self.expanded and max(s.dim + s.rot_dim, s.vdim) > self.MAX_CACHE_DIM:
            raise NotImplementedError(
                f"heads of {s.dim + s.rot_dim} key / {s.vdim} value columns: "
                f"the attention kernel takes at most {self.MAX_CACHE_DIM}"
            )
        self.own_kv = s.kv_from is None
        self.kv_cols = s.cache_dim if self.own_kv else 0
        self.in_proj = _param(
            s.q_rank + self.kv_cols + (s.heads if s.gate else 0), width, dtype=dtype
        )
        self.q_norm = _param(s.q_rank, dtype=torch.float32)
        self.kv_norm = (
            _param(s.kv_rank, dtype=torch.float32) if self.own_kv else None
        )
        self.uq = _param(s.heads * (s.dim + s.rot_dim), s.q_rank, dtype=dtype)
        # U_k transposed per head, [heads, kv_rank, dim]: it maps a query
        # head into latent coordinates; U_v as stored, [heads, vdim, kv_rank]
        self.uk_t = _param(s.heads, s.kv_rank, s.dim, dtype=dtype)
        self.uv = _param(s.heads, s.vdim, s.kv_rank, dtype=dtype)
        self.sink = _param(s.heads, dtype=torch.float32) if s.sink else None
        self.o_proj = _param(width, s.heads * s.vdim, dtype=dtype)
        self.register_buffer(
            "inv_freq",
            rotary_inv_freq(s.rot_dims, s.rot_base) if s.rot_dims else None,
            persistent=False,
        )

    def load(self, get, prefix: str):
        dt, s = self.dtype, self.spec
        parts = [get(prefix + "dq").to(dt)]
        if self.own_kv:
            parts.append(get(prefix + "dkv").to(dt))
            self.kv_norm.copy_(get(prefix + "dkv.norm").float())
        if s.gate:
            parts.append(get(prefix + "g").to(dt))
        self.in_proj.copy_(torch.cat(parts, dim=0))
        self.q_norm.copy_(get(prefix + "dq.norm").float())
        self.uq.copy_(get(prefix + "uq").to(dt))
        self.uk_t.copy_(
            get(prefix + "uk").to(dt).view(s.heads, s.dim, s.kv_rank).transpose(1, 2)
        )
        self.uv.copy_(get(prefix + "uv").to(dt).view(s.heads, s.vdim, s.kv_rank))
        if self.sink is not None:
            self.sink.copy_(get(prefix + "sink").float())
        self.o_proj.copy_(get(prefix + "o").to(dt))

    def forward(self, h, positions, cache: LayerCache, meta):
        """``cache.k``: this layer's pages, or those of layer ``kv_from``."""
        s = self.spec
        proj = F.linear(h, self.in_proj)
        cq = ops.latent_norm_rope_cache(
            proj, s.q_rank, s.kv_rank if self.own_kv else 0,
            s.rot_dim if self.own_kv else 0, self.q_norm, self.kv_norm,
            positions, meta.slot_mapping, cache.k if self.own_kv else None,
            self.eps, self.inv_freq,
        )
        q = F.linear(cq, self.uq)
        gate = proj[:, s.q_rank + self.kv_cols :] if s.gate else None
        if self.expanded:
            return F.linear(
                self._expanded_attention(q, gate, positions, cache, meta),
                self.o_proj,
            )
        qf = ops.head_matmul_rope(
            q, self.uk_t, s.heads, s.rot_dim, positions, self.inv_freq,
            torch.float32,
        )
        o_lat = ops.ctx_attention_f32(
            qf, cache.k, cache.k[..., : s.kv_rank], meta.block_tables,
            meta.cu_seqlens, meta.context_lens, s.scale, meta.max_seqlen,
            s.heads, gate=gate, out_dtype=self.dtype, sink=self.sink,
            window=s.window,
        )
        o = ops.head_matmul_rope(o_lat, self.uv, s.heads)
        return F.linear(o, self.o_proj)

    def _expanded_attention(self, q, gate, positions, cache: LayerCache, meta):
        """Per-head keys and values of every sequence's whole context, built
        from its cached rows into scratch pages (numbered 0.. in sequence
        order), then plain multi-head attention. -> [T, heads * vdim]."""
        from kserve_amd.ops.torch_ref import rotate_pairs

        s = self.spec
        H, R, rd = s.heads, s.kv_rank, s.rot_dim
        T = q.shape[0]
        q3 = q.view(T, H, s.dim + rd).float()
        if rd:
            q3 = torch.cat(
                [q3[..., : s.dim], rotate_pairs(q3[..., s.dim :], positions, self.inv_freq)],
                dim=-1,
            )
        qf = q3.reshape(T, H * (s.dim + rd)).contiguous()
        n_seq = meta.cu_seqlens.numel() - 1
        ctx = meta.context_lens[:n_seq].tolist()  # host read
        bs = cache.k.shape[2]
        nbs = [-(-c // bs) for c in ctx]
        ids = torch.cat(
            [meta.block_tables[i, :nb] for i, nb in enumerate(nbs)]
        ).long()
        rows = cache.k[ids, 0]                       # [pages, bs, R + rd]
        n_pages = rows.shape[0]
        lat = rows[..., :R].reshape(-1, R)
        keys = torch.matmul(lat, self.uk_t)                                  # [H, n, dim]
        if rd:
            shared = rows[..., R:].reshape(1, -1, rd).expand(H, -1, -1)
            keys = torch.cat([keys, shared], dim=-1)
        vals = torch.matmul(lat, self.uv.transpose(1, 2))                    # [H, n, vdim]
        k_tmp = keys.view(H, n_pages, bs, -1).transpose(0, 1).contiguous()
        v_tmp = vals.view(H, n_pages, bs, -1).transpose(0, 1).contiguous()
        tables = torch.zeros(
            (n_seq, max(nbs)), dtype=torch.int32, device=q.device
        )
        at = 0
        for i, nb in enumerate(nbs):
            tables[i, :nb] = torch.arange(at, at + nb, dtype=torch.int32, device=q.device)
            at += nb
        return ops.ctx_attention_f32(
            qf, k_tmp, v_tmp, tables, meta.cu_seqlens, meta.context_lens,
            s.scale, meta.max_seqlen, H, gate=gate, out_dtype=self.dtype,
            sink=self.sink, window=s.window,
        )


class GeluMLP(nn.Module):
    """down(gelu_tanh(up h + b_up)) + b_down."""

    def __init__(self, width: int, spec: MLPSpec, dtype):
        super().__init__()
        self.spec = spec
        self.up = _param(spec.ff, width, dtype=dtype)
        self.up_b = _param(spec.ff, dtype=torch.float32)
        self.down = _param(width, spec.ff, dtype=dtype)
        self.down_b = _param(width, dtype=dtype)

    def load(self, get, prefix: str):
        dt = self.up.dtype
        self.up.copy_(get(prefix + "up").to(dt))
        self.up_b.copy_(get(prefix + "up.b").float())
        self.down.copy_(get(prefix + "down").to(dt))
        self.down_b.copy_(get(prefix + "down.b").to(dt))

    def forward(self, h):
        a = ops.bias_gelu_tanh(F.linear(h, self.up), self.up_b)
        return F.linear(a, self.down, self.down_b)


class SiluGLU(nn.Module):
    """down(silu(gate h) * (up h)), no biases; gate|up are one GEMM."""

    def __init__(self, width: int, ff: int, dtype):
        super().__init__()
        self.gate_up = _param(2 * ff, width, dtype=dtype)
        self.down = _param(width, ff, dtype=dtype)

    def load(self, get, prefix: str):
        dt = self.gate_up.dtype
        self.gate_up.copy_(
            torch.cat([get(prefix + "gate").to(dt), get(prefix + "up").to(dt)], dim=0)
        )
        self.down.copy_(get(prefix + "down").to(dt))

    def forward(self, h):
        return F.linear(ops.glu_silu_scale(F.linear(h, self.gate_up)), self.down)


class SoftmaxRoutedMoE(nn.Module):
    """Mixture of gated silu experts. fp32 router logits over
    ``experts + identity`` outputs, softmax scores; the ``top`` outputs by
    score + correction are chosen and weighted by their scores renormalised
    to sum 1; the weight multiplies the expert's OUTPUT. An identity expert
    returns the token's input. A shared expert is added for every token.

    Weights: gate|up stacked as [E, 2 ff, width] (also one [E * 2 ff, width]
    matrix), down as [width, E, ff] (also one [width, E * ff] matrix).
    Small batches and captured decode graphs run every expert on every token:
    ONE GEMM against all gate|up rows (the experts share their input), the
    activation scaled by the token's weight for that expert (zero where it
    was not chosen), ONE GEMM against all down columns, which also sums over
    the experts in its fp32 accumulator. Larger batches sort the
    (token, expert) pairs by expert and run a GEMM pair per expert on its
    contiguous rows; the pairs of identity experts sort last and copy their
    input rows."""

    DENSE_ROW_BUDGET = RoutedClampedMoE.DENSE_ROW_BUDGET
    RENORM_EPS = 1e-20

    def __init__(self, width: int, spec: SoftmaxMoESpec, dtype):
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        E, R = spec.experts, spec.router_outputs
        if not 1 <= spec.top <= R:
            raise ValueError("top must be between 1 and the router's outputs")
        self.dense_max_tokens = max(16, self.DENSE_ROW_BUDGET * spec.top // max(E, 1))
        self.router = _param(R, width, dtype=torch.float32)
        self.correction = _param(R, dtype=torch.float32)
        self.gate_up = _param(E, 2 * spec.ff, width, dtype=dtype)
        self.down = _param(width, E, spec.ff, dtype=dtype)
        self.shared = SiluGLU(width, spec.shared_ff, dtype) if spec.shared_ff else None

    def load(self, get, prefix: str):
        dt = self.dtype
        self.router.copy_(get(prefix + "router").float())
        self.correction.copy_(get(prefix + "correction").float())
        for e in range(self.spec.experts):
            p = f"{prefix}e{e}."
            self.gate_up[e].copy_(
                torch.cat([get(p + "gate").to(dt), get(p + "up").to(dt)], dim=0)
            )
            self.down[:, e].copy_(get(p + "down").to(dt))
        if self.shared is not None:
            self.shared.load(get, prefix + "shared.")

    def _dense(self, h, dense_w, extra):
        E, ff = self.spec.experts, self.spec.ff
        T, W = h.shape
        scaled = scaled_w = None
        if self.spec.identity:
            scaled, scaled_w = h, dense_w[:, E:].sum(dim=1)
        ar = torch.arange(T, dtype=torch.int32, device=h.device)
        if E == 0:
            y = torch.zeros((T, W), dtype=h.dtype, device=h.device)
        else:
            gu = F.linear(h, self.gate_up.view(E * 2 * ff, W))
            act = ops.glu_silu_scale(
                gu.view(T * E, 2 * ff), dense_w[:, :E].reshape(-1)
            )
            y = F.linear(act.view(T, E * ff), self.down.view(W, E * ff))
        return ops.combine_rows(y, ar, 1, extra, None, scaled, scaled_w)

    def _sorted(self, h, idx, w, extra):
        E, top = self.spec.experts, self.spec.top
        R = self.spec.router_outputs
        flat = idx.view(-1).long()
        order = torch.sort(flat, stable=True).indices
        counts = torch.bincount(flat, minlength=R).tolist()  # host sync
        xs = ops.gather_scale_rows(h, (order // top).to(torch.int32))
        n = xs.shape[0]
        n_real = sum(counts[:E])
        gu = torch.empty((n_real, 2 * self.spec.ff), dtype=h.dtype, device=h.device)
        a = 0
        for e in range(E):
            c = counts[e]
            if c:
                torch.mm(xs[a : a + c], self.gate_up[e].t(), out=gu[a : a + c])
            a += c
        act = ops.glu_silu_scale(gu)
        # rows of identity experts (sorted last) keep their input
        ys = xs.clone() if n_real < n else torch.empty_like(xs)
        a = 0
        for e in range(E):
            c = counts[e]
            if c:
                torch.mm(act[a : a + c], self.down[:, e].t(), out=ys[a : a + c])
            a += c
        # pair p = t*top + k sits at sorted row inv[p]
        inv = torch.empty_like(order)
        inv[order] = torch.arange(n, device=h.device)
        return ops.combine_rows(ys, inv.to(torch.int32), top, extra, w.view(-1))

    def forward(self, h):
        """[T, width] in the activation dtype -> fp32 [T, width]."""
        T = h.shape[0]
        extra = self.shared(h) if self.shared is not None else None
        dense = T <= self.dense_max_tokens or (
            h.is_cuda and torch.cuda.is_current_stream_capturing()
        )
        idx, w, dense_w, _ = ops.route_tokens(
            h, self.router, self.spec.top, softmax=True, renorm=True,
            dense=dense, correction=self.correction,
            renorm_eps=self.RENORM_EPS,
        )
        if dense:
            return self._dense(h, dense_w, extra)
        return self._sorted(h, idx, w, extra)


class RetentionMixer(nn.Module):
    """Linear attention with a constant decay per head (no softmax, no
    denominator): q, k rotated by their position, k scaled by dim^-1/2, the
    fp32 state S <- decay_h S + k v^T read out as S^T q, every head output
    divided by its RMS (no weight), gated by silu of a projection of the
    sublayer input, out-projection. q|k|v|gate are one fused GEMM."""

    def __init__(self, width: int, spec: RetentionMixerSpec, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.dtype = dtype
        s = spec
        if s.rot_dims % 2 or s.rot_dims > s.dim:
            raise ValueError("rot dims must be even and at most the head size")
        self.qk_w = s.heads * s.dim
        self.v_w = s.heads * s.vdim
        self.qkvg = _param(2 * self.qk_w + 2 * self.v_w, width, dtype=dtype)
        self.o_proj = _param(width, self.v_w, dtype=dtype)
        self.register_buffer(
            "decay", torch.tensor(s.decay, dtype=torch.float32), persistent=False
        )
        self.register_buffer(
            "inv_freq",
            rotary_inv_freq(s.rot_dims, s.rot_base) if s.rot_dims else None,
            persistent=False,
        )

    def state_shapes(self):
        s = self.spec
        return {"ssm": ((s.heads, s.vdim, s.dim), torch.float32)}

    def load(self, get, prefix: str):
        dt = self.dtype
        self.qkvg.copy_(
            torch.cat([get(prefix + n).to(dt) for n in ("q", "k", "v", "g")], dim=0)
        )
        self.o_proj.copy_(get(prefix + "o").to(dt))

    def forward(self, h, positions, cache: LayerCache, meta):
        s = self.spec
        proj = F.linear(h, self.qkvg)
        a, b, c = self.qk_w, 2 * self.qk_w, 2 * self.qk_w + self.v_w
        # q | k | v to fp32 in one pass: q and k rotated, k scaled
        qkv = ops.rope_scale_heads(
            proj[:, :c], positions, self.inv_freq, s.heads, 1.0, s.heads,
            s.dim ** -0.5, s.dim,
        )
        o = ops.linear_scan(
            qkv[:, :a], qkv[:, a:b], qkv[:, b:], cache.ssm, positions,
            meta.cu_seqlens, meta.state_slots, s.heads, decay=self.decay,
        )
        on = ops.gated_group_rms_norm(
            o, proj[:, c:], None, self.eps, s.heads, self.dtype, gate_after=True
        )
        return F.linear(on, self.o_proj)


class GatedDeltaMixer(nn.Module):
    """Gated delta rule: q, k, v go through a short causal convolution + silu
    (history kept per sequence), q and k become unit vectors per head (q also
    times dim^-1/2), and per value head the fp32 state is decayed by
    g = exp(-exp(A_log) softplus(a + dt_bias)), corrected towards the value
    with strength sigmoid(b), S <- S + k (b (v - S^T k))^T, and read as S^T q.
    Head outputs are RMS-normed with one weight vector shared by the heads,
    gated by silu of a projection of the input, then out-projected.
    q|k|v|gate|b|a are one fused GEMM."""

    UNIT_EPS = 1e-6

    def __init__(self, width: int, spec: DeltaMixerSpec, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.eps = eps
        self.dtype = dtype
        s = spec
        self.qk_w = s.kv_heads * s.dim
        self.v_w = s.heads * s.vdim
        self.proj = _param(
            s.conv_channels + self.v_w + 2 * s.heads, width, dtype=dtype
        )
        self.conv_w = _param(s.conv_channels, s.conv, dtype=torch.float32)
        self.a_log = _param(s.heads, dtype=torch.float32)
        self.dt_bias = _param(s.heads, dtype=torch.float32)
        self.norm_w = _param(s.vdim, dtype=torch.float32)
        self.o_proj = _param(width, self.v_w, dtype=dtype)

    def state_shapes(self):
        s = self.spec
        out = {"ssm": ((s.heads, s.vdim, s.dim), torch.float32)}
        if s.conv > 1:
            out["conv"] = ((s.conv - 1, s.conv_channels), self.dtype)
        return out

    def load(self, get, prefix: str):
        dt = self.dtype
        self.proj.copy_(
            torch.cat(
                [get(prefix + n).to(dt) for n in ("q", "k", "v", "g", "b", "a")],
                dim=0,
            )
        )
        self.conv_w.copy_(
            torch.cat([get(prefix + n + ".conv").float() for n in ("q", "k", "v")], dim=0)
        )
        self.a_log.copy_(get(prefix + "A_log").float())
        self.dt_bias.copy_(get(prefix + "dt_bias").float())
        self.norm_w.copy_(get(prefix + "norm").float())
        self.o_proj.copy_(get(prefix + "o").to(dt))

    def forward(self, h, positions, cache: LayerCache, meta):
        s = self.spec
        proj = F.linear(h, self.proj)
        cc = s.conv_channels
        gate = proj[:, cc : cc + self.v_w]
        b_raw = proj[:, cc + self.v_w : cc + self.v_w + s.heads]
        a_raw = proj[:, cc + self.v_w + s.heads :]
        if s.conv > 1:
            qkv = ops.causal_conv_silu(
                proj[:, :cc], self.conv_w, None, cache.conv, positions,
                meta.seq_of_token, meta.cu_seqlens, meta.state_slots,
            )
        else:
            x = proj[:, :cc].float() * self.conv_w[:, 0]
            qkv = x * torch.sigmoid(x)
        ops.unit_norm_heads(
            qkv, s.kv_heads, s.dim ** -0.5, s.kv_heads, 1.0, s.dim, self.UNIT_EPS
        )
        a = self.qk_w
        o = ops.linear_scan(
            qkv[:, :a], qkv[:, a : 2 * a], qkv[:, 2 * a :], cache.ssm, positions,
            meta.cu_seqlens, meta.state_slots, s.kv_heads, a_raw=a_raw,
            b_raw=b_raw, a_log=self.a_log, dt_bias=self.dt_bias,
        )
        on = ops.gated_group_rms_norm(
            o, gate, self.norm_w, self.eps, s.heads, self.dtype, gate_after=True
        )
        return F.linear(on, self.o_proj)


class SquaredReluMoE(nn.Module):
    """Mixture of two-matrix experts down(relu(up h)^2) without biases. fp32
    router logits, sigmoid scores, the ``top`` largest chosen and weighted by
    score / (sum of the chosen scores + 1e-20) * scale; the weight multiplies
    the expert's OUTPUT; the weighted sum is fp32, and ``extra`` (another
    sublayer's output for the same tokens) joins that sum.

    Weights: up stacked as [E, ff, width] (also one [E * ff, width] matrix),
    down as [width, E, ff] (also one [width, E * ff] matrix). Small batches
    and captured decode graphs run every expert on every token: ONE GEMM
    against all up rows, the activation scaled by the token's weight for that
    expert (zero where it was not chosen), ONE GEMM against all down columns,
    which sums over the experts in its fp32 accumulator. Larger batches sort
    the (token, expert) pairs by expert and run a GEMM pair per expert on its
    contiguous rows."""

    DENSE_ROW_BUDGET = RoutedClampedMoE.DENSE_ROW_BUDGET
    RENORM_EPS = 1e-20

    def __init__(self, width: int, spec: SquaredReluMoESpec, dtype):
        super().__init__()
        self.spec = spec
        self.dtype = dtype
        E = spec.experts
        if not 1 <= spec.top <= E:
            raise ValueError("top must be between 1 and the number of experts")
        self.dense_max_tokens = max(16, self.DENSE_ROW_BUDGET * spec.top // E)
        self.router = _param(E, width, dtype=torch.float32)
        self.up = _param(E, spec.ff, width, dtype=dtype)
        self.down = _param(width, E, spec.ff, dtype=dtype)

    def load(self, get, prefix: str):
        dt = self.dtype
        self.router.copy_(get(prefix + "router").float())
        for e in range(self.spec.experts):
            p = f"{prefix}e{e}."
            self.up[e].copy_(get(p + "up").to(dt))
            self.down[:, e].copy_(get(p + "down").to(dt))

    def _dense(self, h, dense_w, extra):
        E, ff = self.spec.experts, self.spec.ff
        T, W = h.shape
        x = F.linear(h, self.up.view(E * ff, W))
        act = ops.relu2_scale(x.view(T * E, ff), dense_w.reshape(-1))
        y = F.linear(act.view(T, E * ff), self.down.view(W, E * ff))
        ar = torch.arange(T, dtype=torch.int32, device=h.device)
        return ops.combine_rows(y, ar, 1, extra)

    def _sorted(self, h, idx, w, extra):
        E, top = self.spec.experts, self.spec.top
        flat = idx.view(-1).long()
        order = torch.sort(flat, stable=True).indices
        counts = torch.bincount(flat, minlength=E).tolist()  # host sync
        xs = ops.gather_scale_rows(h, (order // top).to(torch.int32))
        n = xs.shape[0]
        x = torch.empty((n, self.spec.ff), dtype=h.dtype, device=h.device)
        a = 0
        for e, c in enumerate(counts):
            if c:
                torch.mm(xs[a : a + c], self.up[e].t(), out=x[a : a + c])
            a += c
        act = ops.relu2_scale(x)
        ys = torch.empty_like(xs)
        a = 0
        for e, c in enumerate(counts):
            if c:
                torch.mm(act[a : a + c], self.down[:, e].t(), out=ys[a : a + c])
            a += c
        # pair p = t*top + k sits at sorted row inv[p]
        inv = torch.empty_like(order)
        inv[order] = torch.arange(n, device=h.device)
        return ops.combine_rows(ys, inv.to(torch.int32), top, extra, w.view(-1))

    def forward(self, h, extra=None):
        """[T, width] in the activation dtype -> fp32 [T, width]."""
        T = h.shape[0]
        dense = T <= self.dense_max_tokens or (
            h.is_cuda and torch.cuda.is_current_stream_capturing()
        )
        idx, w, dense_w, _ = ops.route_tokens(
            h, self.router, self.spec.top, renorm=True, dense=dense,
            renorm_eps=self.RENORM_EPS, weight_scale=self.spec.scale,
        )
        if dense:
            return self._dense(h, dense_w, extra)
        return self._sorted(h, idx, w, extra)
