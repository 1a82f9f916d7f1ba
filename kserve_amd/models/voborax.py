"""Voborax: a decoder of latent-attention layers on an un-normed stream.

The layers are listed one by one in the config. A sublayer reads the residual
stream x itself (no norm in front); its OUTPUT goes through a layer norm
(weight, no bias) and a constant multiplier m before it is added:

    x += m * LN1(mixer(x))
    x += m * LN2(ff(x))          (if the layer has a feed-forward)

The mixer is ``LatentAttention`` in one of two settings: with a rotated key
part, a sliding window and an output gate, or without positions, causal,
with a sink in the softmax. A layer may read the cached rows of an earlier
layer instead of projecting its own (``kv_from``): it then owns no pages.
The feed-forward is ``GeluMLP`` or ``SoftmaxRoutedMoE``. The stream is fp32
whatever the activation dtype; "norm the sublayer output, scale, add, hand
the new stream to the next sublayer in the activation dtype" is one kernel,
and the last one applies the model's final layer norm instead.
"""

from __future__ import annotations

from typing import List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from kserve_amd import ops
from kserve_amd.engine.config import (
    HybridLayerSpec,
    HybridModelConfig,
    MLPSpec,
    SoftmaxMoESpec,
)
from kserve_amd.models.mixers import GeluMLP, LatentAttention, SoftmaxRoutedMoE
from kserve_amd.parallel import comm


def _vec(n: int):
    return nn.Parameter(torch.empty(n, dtype=torch.float32), requires_grad=False)


class VoboraxLayer(nn.Module):
    def __init__(self, width: int, spec: HybridLayerSpec, eps: float, dtype):
        super().__init__()
        if spec.latent is None:
            raise ValueError("a Voborax layer has a latent-attention mixer")
        self.spec = spec
        self.attn = LatentAttention(width, spec.latent, eps, dtype)
        if isinstance(spec.mlp, SoftmaxMoESpec):
            self.mlp = SoftmaxRoutedMoE(width, spec.mlp, dtype)
        elif isinstance(spec.mlp, MLPSpec):
            self.mlp = GeluMLP(width, spec.mlp, dtype)
        elif spec.mlp is None:
            self.mlp = None
        else:
            raise ValueError(f"unsupported feed-forward {type(spec.mlp).__name__}")
        self.norm1 = _vec(width)
        if self.mlp is not None:
            self.norm2 = _vec(width)


class VoboraxForCausalLM(nn.Module):
    # every step attends through the paged cache; no recurrent state
    paged_prefill_only = True
    needs_state_slots = False

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
                "Voborax runs on one GPU per replica (no tensor/pipeline split)"
            )
        self.config = config
        dtype = dtype or (
            torch.bfloat16 if config.dtype == "bfloat16" else torch.float32
        )
        self.dtype = dtype
        W = config.hidden_size
        for i, spec in enumerate(config.layers):
            lt = spec.latent
            if lt is None or lt.kv_from is None:
                continue
            src = config.layers[lt.kv_from].latent if 0 <= lt.kv_from < i else None
            if src is None or src.kv_from is not None:
                raise ValueError(
                    f"layer {i}: kv_from must name an earlier layer with a "
                    "latent projection of its own"
                )
            if (src.kv_rank, src.rot_dim) != (lt.kv_rank, lt.rot_dim):
                raise ValueError(f"layer {i}: cached row differs from layer {lt.kv_from}'s")
        self.embed = nn.Parameter(
            torch.empty(config.vocab_size, W, dtype=dtype), requires_grad=False
        )
        self.layers = nn.ModuleList(
            [VoboraxLayer(W, spec, config.rms_norm_eps, dtype) for spec in config.layers]
        )
        self.num_local_layers = len(self.layers)
        self.final_norm = _vec(W)
        self.head = nn.Parameter(
            torch.empty(config.vocab_size, W, dtype=dtype), requires_grad=False
        )
        self.eps = config.rms_norm_eps
        self.mult = config.residual_mult
        # largest decode batch worth capturing: above it the routed experts
        # switch to their sorted form, which synchronises with the host
        caps = [
            l.mlp.dense_max_tokens for l in self.layers
            if isinstance(l.mlp, SoftmaxRoutedMoE)
        ]
        self.decode_graph_max_tokens = min(caps) if caps else None
        if any(l.attn.expanded for l in self.layers):
            # the expanded form of wide rows reads context lengths on the host
            self.decode_graph_max_tokens = 0
        # when a list, forward() appends the residual stream after each layer
        self.debug_residuals: Optional[List[torch.Tensor]] = None
        self.to(device)

    # -- cache layout (read by the model runner) ------------------------------
    def cache_layout(self):
        """Per layer: one "kv head" of kv_rank + rot_dim columns and no value
        pool (values are the leading columns of the keys); nothing for a
        layer that reads another layer's pages."""
        out = []
        for layer in self.layers:
            lt = layer.spec.latent
            out.append(((1, lt.cache_dim, 0), {}) if lt.kv_from is None else (None, {}))
        return out

    # -- init -----------------------------------------------------------------
    @torch.no_grad()
    def random_init(self, std: float = 0.02, seed: int = 0):
        dev = self.embed.device
        gen = torch.Generator(device=dev)
        gen.manual_seed(seed)
        for name, p in self.named_parameters():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("q_norm", "kv_norm", "norm1", "norm2", "final_norm"):
                p.fill_(1.0)
            elif p.dim() >= 2:
                # keep activations O(1) through the stack
                fan_in = p.shape[-2] if leaf == "uk_t" else p.shape[-1]
                p.normal_(0.0, fan_in ** -0.5, generator=gen)
            else:
                p.normal_(0.0, 0.1, generator=gen)
        return self

    # -- forward --------------------------------------------------------------
    def forward(self, input_ids, positions, caches, meta):
        x = ops.embed_scale_sinpos(
            self.embed, input_ids, positions, None, self.config.embedding_scale
        )
        fp32 = self.dtype == torch.float32
        # the sublayers read the stream itself; in bf16 that is its rounding
        h = x if fp32 else ops.post_layer_norm_add(
            x, None, None, self.mult, self.eps, self.dtype
        )
        dbg = self.debug_residuals
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            src = layer.spec.latent.kv_from
            cache = caches[i if src is None else src]
            d = layer.attn(h, positions, cache, meta)
            last = i == n - 1 and layer.mlp is None
            h = self._add(x, d, layer.norm1, last, fp32)
            if layer.mlp is not None:
                d = layer.mlp(h)
                h = self._add(x, d, layer.norm2, i == n - 1, fp32)
            if dbg is not None:
                dbg.append(x.clone())
        if n == 0:
            h = ops.post_layer_norm_add(
                x, None, None, self.mult, self.eps, self.dtype, self.final_norm
            )
        return h

    def _add(self, x, delta, weight, last: bool, fp32: bool):
        """x += m * LN(delta) * weight; returns what the next sublayer reads
        (or, after the last sublayer, the final layer norm of the stream)."""
        if last:
            return ops.post_layer_norm_add(
                x, delta, weight, self.mult, self.eps, self.dtype, self.final_norm
            )
        if fp32:
            ops.post_layer_norm_add(
                x, delta, weight, self.mult, self.eps, self.dtype, want_out=False
            )
            return x
        return ops.post_layer_norm_add(
            x, delta, weight, self.mult, self.eps, self.dtype
        )

    def compute_logits(self, hidden):
        return F.linear(hidden, self.head)

    # -- weights ----------------------------------------------------------------
    @torch.no_grad()
    def load_hf_state_dict(self, tensors) -> None:
        """Tensor names: embed, l<i>.norm1|norm2,
        l<i>.mix.dq|dq.norm|uq|dkv|dkv.norm|uk|uv|g|sink|o,
        l<i>.mlp.up|up.b|down|down.b (dense) or
        l<i>.mlp.router|correction|e<j>.gate|up|down|shared.gate|up|down,
        final.norm, head."""

        def get(name):
            t = tensors[name]
            return t() if callable(t) else t

        self.embed.copy_(get("embed").to(self.dtype))
        self.head.copy_(get("head").to(self.dtype))
        self.final_norm.copy_(get("final.norm").float())
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            layer.norm1.copy_(get(p + "norm1").float())
            layer.attn.load(get, p + "mix.")
            if layer.mlp is not None:
                layer.norm2.copy_(get(p + "norm2").float())
                layer.mlp.load(get, p + "mlp.")

    def num_parameters(self) -> int:
        return sum(p.numel() for p in self.parameters())
