"""Laperax: a decoder whose layers are listed one by one in the config, each
with one of three mixers and an optional mixture of experts beside it.

A layer is parallel: with h = norm1(x), x += mixer(h) + ff(h) — one RMS norm,
both sublayers read its output, and their outputs are summed in fp32 before
they join the stream. Mixers: ``RetentionMixer`` (linear attention with a
constant decay per head), ``GatedDeltaMixer`` (gated delta rule behind short
convolutions) and sliding-window softmax attention with grouped KV heads,
rotary positions on part of each head and a weightless per-head q/k RMS norm
(``RotaryChunkSinkAttention`` without its optional parts). The feed-forward is
``SquaredReluMoE``. The embedding output is RMS-normed before the first
layer; logits are scaled and soft-capped with tanh.

The residual stream is fp32 whatever the activation dtype. "Add the layer's
sublayer sum, norm for the next layer" is one kernel; the experts' combine
kernel adds the mixer's output to the expert sum, so that sum exists once, in
fp32. Attention layers keep KV pages; retention and delta layers keep an fp32
matrix state (and the delta layers a convolution history) per state slot.
"""

from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from kserve_amd import ops
from kserve_amd.engine.config import HybridLayerSpec, HybridModelConfig
from kserve_amd.models.mixers import (
    GatedDeltaMixer,
    RetentionMixer,
    RotaryChunkSinkAttention,
    SquaredReluMoE,
)
from kserve_amd.parallel import comm


def _vec(n: int):
    return nn.Parameter(torch.empty(n, dtype=torch.float32), requires_grad=False)


class LaperaxLayer(nn.Module):
    def __init__(self, width: int, spec: HybridLayerSpec, eps: float, dtype):
        super().__init__()
        self.spec = spec
        self.norm1 = _vec(width)
        if spec.retention is not None:
            self.mix = RetentionMixer(width, spec.retention, eps, dtype)
        elif spec.delta is not None:
            self.mix = GatedDeltaMixer(width, spec.delta, eps, dtype)
        elif spec.attention is not None:
            self.mix = RotaryChunkSinkAttention(
                width, spec.attention, eps, dtype, sink=False,
                value_unit_norm=False, rotate_values=False, norm_weights=False,
            )
        else:
            raise ValueError("a Laperax layer needs a mixer")
        self.mlp = (
            SquaredReluMoE(width, spec.mlp, dtype) if spec.mlp is not None else None
        )

    def forward(self, h, positions, cache, meta):
        """The layer's addend mixer(h) + ff(h): fp32 when there are experts,
        otherwise the mixer's output as it is."""
        m = self.mix(h, positions, cache, meta)
        return m if self.mlp is None else self.mlp(h, extra=m)


class LaperaxForCausalLM(nn.Module):
    # every step attends through the paged cache (no separate un-paged
    # prefill kernel), and steps carry per-sequence state slots
    paged_prefill_only = True
    needs_state_slots = True

    def __init__(
        self,
        config: HybridModelConfig,
        dtype: Optional[torch.dtype] = None,
        device: str = "cpu",
    ):
        super().__init__()
        st = comm.get_state()
        if st.tp_size != 1 or st.pp_size != 1:
            raise NotImplementedError(
                "Laperax runs on one GPU per replica (no tensor/pipeline split)"
            )
        self.config = config
        dtype = dtype or (
            torch.bfloat16 if config.dtype == "bfloat16" else torch.float32
        )
        self.dtype = dtype
        W = config.hidden_size
        self.embed = nn.Parameter(
            torch.empty(config.vocab_size, W, dtype=dtype), requires_grad=False
        )
        self.embed_norm = _vec(W)
        self.layers = nn.ModuleList(
            [LaperaxLayer(W, spec, config.rms_norm_eps, dtype) for spec in config.layers]
        )
        self.num_local_layers = len(self.layers)
        self.final_norm = _vec(W)
        self.head = nn.Parameter(
            torch.empty(config.vocab_size, W, dtype=dtype), requires_grad=False
        )
        self.eps = config.rms_norm_eps
        # largest decode batch worth capturing: above it the experts switch
        # to their sorted form, which synchronises with the host
        caps = [l.mlp.dense_max_tokens for l in self.layers if l.mlp is not None]
        self.decode_graph_max_tokens = min(caps) if caps else None
        # when a list, forward() appends the residual stream after each layer
        self.debug_residuals: Optional[List[torch.Tensor]] = None
        self.to(device)

    # -- cache layout (read by the model runner) ------------------------------
    def cache_layout(self):
        """Per layer: (kv_heads, dim, vdim) or None, and
        {name: (shape_per_slot, dtype)} of recurrent state or {}."""
        out = []
        for layer in self.layers:
            a = layer.spec.attention
            kv = (a.kv_heads, a.dim, a.vdim) if a is not None else None
            state = layer.mix.state_shapes() if a is None else {}
            out.append((kv, state))
        return out

    # -- init -----------------------------------------------------------------
    @torch.no_grad()
    def random_init(self, std: float = 0.02, seed: int = 0):
        dev = self.embed.device
        gen = torch.Generator(device=dev)
        gen.manual_seed(seed)
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf == "conv_w":
                p.normal_(0.0, 0.5, generator=gen)
            elif p.dim() >= 2:
                # keep activations O(1) through the stack
                p.normal_(0.0, p.shape[-1] ** -0.5, generator=gen)
            elif leaf == "a_log":
                p.uniform_(-1.0, 1.0, generator=gen)
            elif leaf == "dt_bias":
                p.uniform_(-3.0, 0.0, generator=gen)
            else:  # norm weights
                p.fill_(1.0)
        return self

    # -- forward --------------------------------------------------------------
    def forward(self, input_ids, positions, caches, meta):
        emb = ops.embed_scale_sinpos(self.embed, input_ids, positions, None, 1.0)
        # the normed embedding starts the fp32 stream
        x = ops.add_rms_norm_f32res(
            emb, self.embed_norm, self.eps, 0.0, torch.float32
        )
        pending = None
        dbg = self.debug_residuals
        for layer, cache in zip(self.layers, caches):
            h = ops.add_rms_norm_f32res(
                x, layer.norm1, self.eps, 0.0, self.dtype, pending
            )
            pending = layer(h, positions, cache, meta)
            if dbg is not None:
                dbg.append(x + pending.float())
        return ops.add_rms_norm_f32res(
            x, self.final_norm, self.eps, 0.0, self.dtype, pending
        )

    def compute_logits(self, hidden):
        return ops.scale_softcap(
            F.linear(hidden, self.head), self.config.logit_scale,
            self.config.logit_softcap,
        )

    # -- weights ----------------------------------------------------------------
    @torch.no_grad()
    def load_hf_state_dict(self, tensors) -> None:
        """Tensor names: embed, embed.norm, l<i>.norm1, l<i>.mix.* (retention:
        q|k|v|g|o; attention: q|k|v|o; delta: q|k|v|g|b|a|o, q.conv|k.conv|
        v.conv, A_log, dt_bias, norm), l<i>.mlp.router, l<i>.mlp.e<j>.up|down,
        final.norm, head."""

        def get(name):
            t = tensors[name]
            return t() if callable(t) else t

        self.embed.copy_(get("embed").to(self.dtype))
        self.embed_norm.copy_(get("embed.norm").float())
        self.head.copy_(get("head").to(self.dtype))
        self.final_norm.copy_(get("final.norm").float())
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            layer.norm1.copy_(get(p + "norm1").float())
            layer.mix.load(get, p + "mix.")
            if layer.mlp is not None:
                layer.mlp.load(get, p + "mlp.")

    def num_parameters(self) -> int:
        return sum(p.numel() for p in self.parameters())
