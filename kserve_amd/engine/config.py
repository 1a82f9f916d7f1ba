"""Engine configuration.

The native LLM engine replaces the reference's delegation to vLLM
(reference: python/huggingfaceserver vllm/vllm_model.py:55-343). Config
surface mirrors the preset flags the control plane renders
(--tensor-parallel-size etc., config-llm-worker-data-parallel.yaml:188-199)
while the internals are MI355X-first: KV sizing against 288 GB HBM3E.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from typing import Optional

from kserve_amd.constants import (
    DEFAULT_GPU_MEMORY_UTILIZATION,
    DEFAULT_KV_BLOCK_SIZE,
    HBM_BYTES_PER_GPU,
)


@dataclass
class ModelConfig:
    """Decoder-only transformer architecture description (Llama family)."""

    vocab_size: int = 128256
    hidden_size: int = 4096
    intermediate_size: int = 14336
    num_layers: int = 32
    num_heads: int = 32
    num_kv_heads: int = 8
    head_dim: Optional[int] = None
    rms_norm_eps: float = 1e-5
    rope_theta: float = 500000.0
    max_position_embeddings: int = 8192
    tie_word_embeddings: bool = False
    dtype: str = "bfloat16"
    model_name: str = "llama"
    # attention bias (Qwen2-style) / mlp bias
    attention_bias: bool = False
    mlp_bias: bool = False
    # mixture-of-experts (Mixtral): 0 experts = dense MLP
    num_local_experts: int = 0
    num_experts_per_tok: int = 2
    # EP: partition experts across the parallel group (full-width weights)
    # instead of TP-sharding every expert
    expert_parallel: bool = False
    # HF rope_scaling dict (Llama-3.1 'llama3' type supported)
    rope_scaling: Optional[dict] = None
    # Mistral-style sliding-window size from the HF config; enforced in
    # all three attention kernels (decode/flash/paged-context) as an
    # absolute-position bound.
    sliding_window: int = None

    def __post_init__(self):
        if self.head_dim is None:
            self.head_dim = self.hidden_size // self.num_heads

    @property
    def kv_bytes_per_token_per_layer(self) -> int:
        # K + V, bf16
        return 2 * self.num_kv_heads * self.head_dim * 2

    @classmethod
    def llama3_8b(cls) -> "ModelConfig":
        return cls(
            vocab_size=128256,
            hidden_size=4096,
            intermediate_size=14336,
            num_layers=32,
            num_heads=32,
            num_kv_heads=8,
            rope_theta=500000.0,
            max_position_embeddings=8192,
            model_name="llama-3-8b",
        )

    @classmethod
    def llama3_70b(cls) -> "ModelConfig":
        return cls(
            vocab_size=128256,
            hidden_size=8192,
            intermediate_size=28672,
            num_layers=80,
            num_heads=64,
            num_kv_heads=8,
            rope_theta=500000.0,
            max_position_embeddings=8192,
            model_name="llama-3-70b",
        )

    @classmethod
    def mistral_7b(cls) -> "ModelConfig":
        return cls(
            vocab_size=32000,
            hidden_size=4096,
            intermediate_size=14336,
            num_layers=32,
            num_heads=32,
            num_kv_heads=8,
            rope_theta=10000.0,
            max_position_embeddings=8192,
            sliding_window=4096,
            model_name="mistral-7b",
        )

    @classmethod
    def mixtral_8x7b(cls) -> "ModelConfig":
        return cls(
            vocab_size=32000,
            hidden_size=4096,
            intermediate_size=14336,
            num_layers=32,
            num_heads=32,
            num_kv_heads=8,
            rope_theta=1e6,
            max_position_embeddings=8192,
            num_local_experts=8,
            num_experts_per_tok=2,
            model_name="mixtral-8x7b",
        )

    @classmethod
    def tiny(cls, vocab_size: int = 256) -> "ModelConfig":
        """Small config for CPU tests."""
        return cls(
            vocab_size=vocab_size,
            hidden_size=64,
            intermediate_size=128,
            num_layers=2,
            num_heads=4,
            num_kv_heads=2,
            max_position_embeddings=512,
            rope_theta=10000.0,
            model_name="tiny-llama",
        )

    @classmethod
    def from_hf_config(cls, config_path: str) -> "ModelConfig":
        """Parse a HuggingFace config.json (model dir contract /mnt/models)."""
        with open(config_path) as f:
            cfg = json.load(f)
        return cls(
            vocab_size=cfg["vocab_size"],
            hidden_size=cfg["hidden_size"],
            intermediate_size=cfg["intermediate_size"],
            num_layers=cfg["num_hidden_layers"],
            num_heads=cfg["num_attention_heads"],
            num_kv_heads=cfg.get("num_key_value_heads", cfg["num_attention_heads"]),
            head_dim=cfg.get("head_dim"),
            rms_norm_eps=cfg.get("rms_norm_eps", 1e-5),
            rope_theta=cfg.get("rope_theta", 10000.0),
            max_position_embeddings=cfg.get("max_position_embeddings", 8192),
            tie_word_embeddings=cfg.get("tie_word_embeddings", False),
            # Qwen2 has qkv bias implicitly (no attention_bias key in HF)
            attention_bias=cfg.get(
                "attention_bias", cfg.get("model_type") == "qwen2"
            ),
            num_local_experts=cfg.get("num_local_experts", 0),
            num_experts_per_tok=cfg.get("num_experts_per_tok", 2),
            sliding_window=cfg.get("sliding_window"),
            rope_scaling=cfg.get("rope_scaling"),
            mlp_bias=cfg.get("mlp_bias", False),
            model_name=cfg.get("_name_or_path", os.path.dirname(config_path) or "model"),
        )


@dataclass
class AttentionMixerSpec:
    """Softmax attention sublayer with grouped KV heads. Independent query/key
    and value head sizes; ``scale`` multiplies q.k; the query temperature
    1 + coef * ln(floor((pos+1)/every) + 1) is off when ``q_temp_every`` is 0."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    q_temp_coef: float = 0.0
    q_temp_every: int = 0
    # rotary positions on the first ``rot_dims`` coordinates of every q/k
    # head (coordinate i pairs with i + rot_dims/2); 0 = no rotation
    rot_dims: int = 0
    rot_base: float = 10000.0
    # chunk-local causal mask: a query sees only keys of its own block of
    # ``chunk`` positions (counted from position 0); 0 = plain causal
    chunk: int = 0
    # sliding window: a query sees itself and the window-1 positions before
    # it; 0 = no window
    window: int = 0

    @classmethod
    def from_dict(cls, d: dict, mask: str = "chunk") -> "AttentionMixerSpec":
        """``mask`` says what the entry's ``mask.size`` means in the design
        that is being read: "chunk" or "window"."""
        qt = d.get("q_temp") or {}
        rot = d.get("rot") or {}
        size = int((d.get("mask") or {}).get("size", 0))
        chunk = size if mask == "chunk" else 0
        window = size if mask == "window" else 0
        return cls(
            heads=int(d["heads"]),
            kv_heads=int(d.get("kv_heads", d["heads"])),
            dim=int(d["dim"]),
            vdim=int(d.get("vdim", d["dim"])),
            scale=float(d["scale"]),
            q_temp_coef=float(qt.get("coef", 0.0)),
            q_temp_every=int(qt.get("every", 0)),
            rot_dims=int(rot.get("dims", 0)),
            rot_base=float(rot.get("base", 10000.0)),
            chunk=chunk,
            window=window,
        )


@dataclass
class RetentionMixerSpec:
    """Linear attention with a constant decay per head and no softmax:
    S <- decay_h S + k v^T, o = S^T q, rotary positions on q and k, keys
    scaled by dim^-1/2, head outputs RMS-normed (no weight) and gated."""

    heads: int
    dim: int
    vdim: int
    decay: list
    rot_dims: int = 0
    rot_base: float = 10000.0

    @classmethod
    def from_dict(cls, d: dict) -> "RetentionMixerSpec":
        rot = d.get("rot") or {}
        decay = [float(x) for x in d["decay"]]
        if len(decay) != int(d["heads"]):
            raise ValueError("one decay per head")
        return cls(
            heads=int(d["heads"]),
            dim=int(d["dim"]),
            vdim=int(d.get("vdim", d["dim"])),
            decay=decay,
            rot_dims=int(rot.get("dims", 0)),
            rot_base=float(rot.get("base", 10000.0)),
        )


@dataclass
class DeltaMixerSpec:
    """Gated delta rule: ``heads`` value heads of ``vdim`` columns, ``kv_heads``
    query/key heads of ``dim`` columns shared by groups of value heads, a
    causal convolution of ``conv`` taps + silu on q, k and v, unit-norm q/k, a
    data-dependent decay and write strength per head."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int = 4

    @property
    def conv_channels(self) -> int:
        return 2 * self.kv_heads * self.dim + self.heads * self.vdim

    @classmethod
    def from_dict(cls, d: dict) -> "DeltaMixerSpec":
        heads = int(d["heads"])
        kv = int(d.get("kv_heads", heads))
        if kv < 1 or heads % kv:
            raise ValueError("heads must be a multiple of kv_heads")
        return cls(
            heads=heads,
            kv_heads=kv,
            dim=int(d["dim"]),
            vdim=int(d.get("vdim", d["dim"])),
            conv=int(d.get("conv", 4)),
        )


@dataclass
class SquaredReluMoESpec:
    """Mixture of two-matrix experts down(relu(up h)^2) routed by sigmoid
    scores: the ``top`` largest are chosen, their scores are divided by their
    sum and multiplied by ``scale``, and the weight multiplies the expert's
    OUTPUT."""

    experts: int
    top: int
    ff: int
    scale: float = 1.0

    @classmethod
    def from_dict(cls, d: dict) -> "SquaredReluMoESpec":
        kind = d.get("kind", "moe")
        if kind != "moe":
            raise ValueError(f"unsupported feed-forward kind {kind!r}")
        r = d["router"]
        return cls(
            experts=int(r["experts"]),
            top=int(r["top"]),
            ff=int(d["expert"]["ff"]),
            scale=float(r.get("scale", 1.0)),
        )


@dataclass
class SSMMixerSpec:
    """State-space (Mamba-2) sublayer: ``heads`` heads of ``vdim`` channels,
    state size ``state`` per channel, B/C shared per ``groups``, a causal
    convolution of ``conv`` taps, and an output norm in ``norm_groups``
    equal parts."""

    heads: int
    vdim: int
    state: int
    groups: int = 1
    conv: int = 4
    norm_groups: int = 1

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    @property
    def proj_width(self) -> int:
        # [z | x | B | C | dt]
        return 2 * self.inner + 2 * self.groups * self.state + self.heads

    @classmethod
    def from_dict(cls, d: dict) -> "SSMMixerSpec":
        return cls(
            heads=int(d["heads"]),
            vdim=int(d["vdim"]),
            state=int(d["state"]),
            groups=int(d.get("groups", 1)),
            conv=int(d.get("conv", 4)),
            norm_groups=int(d.get("norm_groups", 1)),
        )


@dataclass
class GLUSpec:
    """Dense gated feed-forward with clamped branches."""

    ff: int
    limit: float

    @classmethod
    def from_dict(cls, d: dict) -> "GLUSpec":
        kind = d.get("kind", "dense")
        if kind != "dense":
            raise ValueError(f"unsupported feed-forward kind {kind!r}")
        return cls(ff=int(d["ff"]), limit=float(d["limit"]))


@dataclass
class MoESpec:
    """Mixture of clamped gated experts: each token runs the ``top`` experts
    with the largest sigmoid router scores; the (un-normalised) score scales
    the expert's INPUT. An optional shared expert runs for every token."""

    experts: int
    top: int
    ff: int
    limit: float
    shared: Optional[GLUSpec] = None

    @classmethod
    def from_dict(cls, d: dict) -> "MoESpec":
        sh = d.get("shared")
        return cls(
            experts=int(d["router"]["experts"]),
            top=int(d["router"]["top"]),
            ff=int(d["expert"]["ff"]),
            limit=float(d["expert"]["limit"]),
            shared=GLUSpec(ff=int(sh["ff"]), limit=float(sh["limit"])) if sh else None,
        )


@dataclass
class LatentAttentionSpec:
    """Attention whose keys and values are expanded per head from one cached
    latent vector per token: the cache holds ``kv_rank`` normed latent
    coordinates and (with ``rot_dim`` > 0) one rotated key part shared by all
    heads. Queries go through a normed latent of ``q_rank`` coordinates and
    have ``dim`` unrotated + ``rot_dim`` rotated coordinates per head.
    ``window`` > 0: a query sees itself and the window-1 positions before it;
    ``sink``: one more term exp(sink_h) in the softmax denominator; ``gate``:
    head outputs times sigmoid of a projection of the sublayer input;
    ``kv_from``: the layer has no latent projection and reads the cache of
    that earlier layer."""

    heads: int
    dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_dim: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0
    window: int = 0
    sink: bool = False
    gate: bool = False
    kv_from: Optional[int] = None

    @property
    def cache_dim(self) -> int:
        return self.kv_rank + self.rot_dim

    @classmethod
    def from_dict(cls, d: dict, sink: bool, gate: bool) -> "LatentAttentionSpec":
        rot = d.get("rot") or {}
        mask = d.get("mask") or {}
        rot_dim = int(d.get("rot_dim", 0))
        kv_from = d.get("kv_from")
        return cls(
            heads=int(d["heads"]),
            dim=int(d["dim"]),
            vdim=int(d.get("vdim", d["dim"])),
            kv_rank=int(d["kv_rank"]),
            q_rank=int(d["q_rank"]),
            scale=float(d["scale"]),
            rot_dim=rot_dim,
            rot_dims=int(rot.get("dims", rot_dim)) if rot_dim else 0,
            rot_base=float(rot.get("base", 10000.0)),
            window=int(mask.get("size", 0)),
            sink=sink,
            gate=gate,
            kv_from=None if kv_from is None else int(kv_from),
        )


@dataclass
class MLPSpec:
    """Plain two-matrix feed-forward with biases: down(act(up h + b) ) + b,
    act = gelu in its tanh form."""

    ff: int

    @classmethod
    def from_dict(cls, d: dict) -> "MLPSpec":
        return cls(ff=int(d["ff"]))


@dataclass
class SoftmaxMoESpec:
    """Mixture of gated silu experts routed by softmax scores: the ``top``
    experts by score + a per-expert correction are chosen, weighted by their
    (uncorrected) scores renormalised to sum 1, and the weight multiplies the
    expert's OUTPUT. The last ``identity`` router outputs stand for experts
    that return their input; ``experts`` counts the real ones. An optional
    shared expert of the same form runs for every token."""

    experts: int
    top: int
    ff: int
    identity: int = 0
    shared_ff: int = 0

    @property
    def router_outputs(self) -> int:
        return self.experts + self.identity

    @classmethod
    def from_dict(cls, d: dict) -> "SoftmaxMoESpec":
        r = d["router"]
        sh = d.get("shared")
        return cls(
            experts=int(r["experts"]),
            top=int(r["top"]),
            ff=int(d["expert"]["ff"]),
            identity=int(r.get("identity", 0)),
            shared_ff=int(sh["ff"]) if sh else 0,
        )


def voborax_feed_forward_spec(d: Optional[dict]):
    """``mlp`` entry of a Voborax layer -> MLPSpec, SoftmaxMoESpec or None."""
    if not d:
        return None
    if d.get("kind", "moe" if "router" in d else "dense") == "moe":
        return SoftmaxMoESpec.from_dict(d)
    return MLPSpec.from_dict(d)


def feed_forward_spec(d: Optional[dict]):
    """``mlp`` entry of a layer -> GLUSpec, MoESpec or None."""
    if not d:
        return None
    if d.get("kind", "moe" if "router" in d else "dense") == "moe":
        return MoESpec.from_dict(d)
    return GLUSpec.from_dict(d)


def laperax_layer_spec(kind: str, mixer: dict, mlp: Optional[dict]):
    """One Laperax layer: a retention, windowed-attention or delta mixer and
    an optional mixture of squared-relu experts, both reading one norm."""
    ff = SquaredReluMoESpec.from_dict(mlp) if mlp else None
    if kind == "retention":
        return HybridLayerSpec(
            kind, retention=RetentionMixerSpec.from_dict(mixer), mlp=ff
        )
    if kind == "attention":
        return HybridLayerSpec(
            kind, attention=AttentionMixerSpec.from_dict(mixer, mask="window"),
            mlp=ff,
        )
    if kind == "delta":
        return HybridLayerSpec(kind, delta=DeltaMixerSpec.from_dict(mixer), mlp=ff)
    raise ValueError(f"unknown layer type {kind!r}")


@dataclass
class LoopSpec:
    """Layers ``start .. stop-1`` run ``times`` times in a row with the same
    weights (every pass with a cache of its own) before the rest follow."""

    start: int = 0
    stop: int = 0
    times: int = 1


@dataclass
class HybridLayerSpec:
    """One pre-norm layer: a mixer made of an attention branch and/or a
    state-space branch reading the same normed input (outputs summed with
    their scales), then an optional feed-forward."""

    kind: str
    attention: Optional[AttentionMixerSpec] = None
    ssm: Optional[SSMMixerSpec] = None
    latent: Optional[LatentAttentionSpec] = None
    retention: Optional[RetentionMixerSpec] = None
    delta: Optional[DeltaMixerSpec] = None
    attention_scale: float = 1.0
    ssm_scale: float = 1.0
    # GLUSpec, MoESpec, MLPSpec, SoftmaxMoESpec or SquaredReluMoESpec
    mlp: Optional[object] = None


@dataclass
class HybridModelConfig:
    """Decoder made of a per-layer list of mixers (Merulorn design): layers
    may differ in kind and in every size, so nothing here is per-model."""

    vocab_size: int
    hidden_size: int
    layers: list
    rms_norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    dtype: str = "bfloat16"
    model_name: str = "merulorn"
    architecture: str = "Merulorn"
    # fields the engine reads on every model config
    num_local_experts: int = 0
    sliding_window: Optional[int] = None
    loop: Optional[LoopSpec] = None
    # every sublayer output is multiplied by this before it joins the stream
    residual_mult: float = 1.0
    # logits = head x * logit_scale, then cap * tanh(logits / cap) (0: none)
    logit_scale: float = 1.0
    logit_softcap: float = 0.0

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def layer_runs(self) -> list:
        """Execution order as (layer index, pass number or None): a looped
        span appears once per pass. Every run has a cache of its own."""
        n = len(self.layers)
        lp = self.loop
        if lp is None or lp.stop <= lp.start:
            return [(i, None) for i in range(n)]
        runs = [(i, None) for i in range(lp.start)]
        for t in range(lp.times):
            runs += [(i, t) for i in range(lp.start, lp.stop)]
        runs += [(i, None) for i in range(lp.stop, n)]
        return runs

    @property
    def has_recurrent_state(self) -> bool:
        return any(
            l.ssm is not None or l.retention is not None or l.delta is not None
            for l in self.layers
        )

    def kv_bytes_per_block(self, block_size: int, itemsize: int) -> int:
        per_token = 0
        for i, _ in self.layer_runs():
            a, lt = self.layers[i].attention, self.layers[i].latent
            if a is not None:
                per_token += a.kv_heads * (a.dim + a.vdim)
            if lt is not None and lt.kv_from is None:
                # one row per token: latent + shared rotated key part
                per_token += lt.cache_dim
        return per_token * block_size * itemsize

    @classmethod
    def from_dict(cls, cfg: dict, model_name: str = "merulorn") -> "HybridModelConfig":
        layers = []
        arch = cfg.get("architecture", "Merulorn")
        for entry in cfg["layers"]:
            kind = entry["type"]
            mixer = entry["mixer"]
            if arch == "Laperax":
                layers.append(laperax_layer_spec(kind, mixer, entry.get("mlp")))
                continue
            if kind in ("latent_attention", "latent_attention_2"):
                # rotated key part + window + output gate, or none of them
                # and a sink
                first = kind == "latent_attention"
                layers.append(
                    HybridLayerSpec(
                        kind,
                        latent=LatentAttentionSpec.from_dict(
                            mixer, sink=not first, gate=first
                        ),
                        mlp=voborax_feed_forward_spec(entry.get("mlp")),
                    )
                )
                continue
            mlp = feed_forward_spec(entry.get("mlp"))
            if kind == "attention":
                layers.append(
                    HybridLayerSpec(
                        kind, attention=AttentionMixerSpec.from_dict(mixer), mlp=mlp
                    )
                )
            elif kind == "mamba2":
                layers.append(
                    HybridLayerSpec(kind, ssm=SSMMixerSpec.from_dict(mixer), mlp=mlp)
                )
            elif kind == "parallel":
                layers.append(
                    HybridLayerSpec(
                        kind,
                        attention=AttentionMixerSpec.from_dict(mixer["left"]),
                        ssm=SSMMixerSpec.from_dict(mixer["right"]),
                        attention_scale=float(mixer.get("left_scale", 1.0)),
                        ssm_scale=float(mixer.get("right_scale", 1.0)),
                        mlp=mlp,
                    )
                )
            else:
                raise ValueError(f"unknown layer type {kind!r}")
        return cls(
            vocab_size=int(cfg["vocab"]),
            hidden_size=int(cfg["width"]),
            layers=layers,
            rms_norm_eps=float(cfg.get("norm", {}).get("eps", 1e-5)),
            embedding_scale=float(cfg.get("embedding", {}).get("scale", 1.0)),
            model_name=model_name,
            architecture=cfg.get("architecture", "Merulorn"),
            residual_mult=float(cfg.get("residual_mult", 1.0)),
            logit_scale=float(cfg.get("logit_scale", 1.0)),
            logit_softcap=float(cfg.get("logit_softcap", 0.0)),
            loop=(
                LoopSpec(
                    start=int(cfg["loop"].get("start", 0)),
                    stop=int(cfg["loop"].get("stop", 0)),
                    times=int(cfg["loop"].get("times", 1)),
                )
                if cfg.get("loop")
                else None
            ),
        )

    @classmethod
    def from_hf_config(cls, config_path: str) -> "HybridModelConfig":
        with open(config_path) as f:
            cfg = json.load(f)
        return cls.from_dict(
            cfg, model_name=os.path.basename(os.path.dirname(config_path)) or "merulorn"
        )


@dataclass
class CacheConfig:
    """Paged-KV cache sizing. Defaults size the pool from the 288 GB HBM3E
    budget after weights (MI355X-first: large pools, big batches)."""

    block_size: int = DEFAULT_KV_BLOCK_SIZE
    num_gpu_blocks: Optional[int] = None  # None -> derive from memory util
    gpu_memory_utilization: float = DEFAULT_GPU_MEMORY_UTILIZATION
    # host-DRAM offload tier (pinned memory, hipMemcpyAsync side stream)
    num_cpu_blocks: int = 0
    cpu_offload_bytes: int = 0
    # automatic prefix caching: content-addressed full prompt blocks are
    # shared across requests; cache-hit prompts only compute their suffix
    # through the paged-context prefill kernel
    enable_prefix_caching: bool = False
    # "auto" stores KV in the model dtype (bf16). "fp8" stores OCP E4M3
    # bytes (scale 1.0): half the KV bandwidth/capacity; attention math
    # stays fp32/bf16 after in-register conversion. GQA group <= 4, D=128.
    kv_cache_dtype: str = "auto"

    def cache_torch_dtype(self, model_dtype):
        if self.kv_cache_dtype in ("fp8", "fp8_e4m3"):
            import torch

            return torch.float8_e4m3fn
        return model_dtype

    def derive_num_gpu_blocks(
        self, model: ModelConfig, tp_size: int = 1, weight_bytes: Optional[int] = None,
        free_bytes: Optional[int] = None,
    ) -> int:
        if self.num_gpu_blocks is not None:
            return self.num_gpu_blocks
        per_block = (
            model.kv_bytes_per_token_per_layer
            * self.block_size
            * model.num_layers
            // tp_size
        )
        if free_bytes is None:
            total = HBM_BYTES_PER_GPU
            if weight_bytes is None:
                weight_bytes = 0
            free_bytes = int(total * self.gpu_memory_utilization) - weight_bytes
        return max(free_bytes // per_block, 16)


@dataclass
class SchedulerConfig:
    max_num_seqs: int = 256
    max_num_batched_tokens: int = 8192
    max_model_len: int = 8192
    # chunked prefill: cap on prompt tokens scheduled per step
    enable_chunked_prefill: bool = False
    # mixed batches: a step that prefills also carries one decode token of
    # every running request (through the paged-context path), so running
    # requests keep producing while prompts are admitted
    mixed_batches: bool = False
    # multi-step decode: consecutive greedy decode iterations run as pure
    # hipGraph replays (sampled token fed back on-GPU); stop conditions are
    # applied after the window. 1 disables.
    multi_step: int = 8
    # speculative decoding (prompt-lookup/n-gram): max draft tokens verified
    # per step through the paged-context prefill path. 0 disables. When >0 it
    # replaces multi-step windows for greedy batches (exact same outputs —
    # rejected drafts are corrected by the verify forward).
    speculative_ngram: int = 0
    speculative_ngram_min: int = 2
    speculative_ngram_max: int = 3
    # draft-MODEL speculation: tokens proposed per round by the draft
    # model configured in EngineConfig.draft_model. 0 disables.
    speculative_k: int = 0


@dataclass
class ParallelConfig:
    """Mirrors the CRD ParallelismSpec (reference v1alpha2 types :733-759)."""

    tensor_parallel_size: int = 1
    pipeline_parallel_size: int = 1
    data_parallel_size: int = 1
    expert_parallel: bool = False


@dataclass
class EngineConfig:
    model: ModelConfig = field(default_factory=ModelConfig.llama3_8b)
    cache: CacheConfig = field(default_factory=CacheConfig)
    scheduler: SchedulerConfig = field(default_factory=SchedulerConfig)
    parallel: ParallelConfig = field(default_factory=ParallelConfig)
    device: str = "cuda"
    seed: int = 0
    enforce_eager: bool = False  # True disables hipGraph capture
    # weights: path to model dir (safetensors) or None for random init
    model_path: Optional[str] = None
    # draft-model speculation: the small model's config (random-init unless
    # draft_model_path / engine.draft.load_hf_state_dict provides weights);
    # pairs with scheduler.speculative_k
    draft_model: Optional[ModelConfig] = None
    draft_model_path: Optional[str] = None
    eos_token_id: int = 128001
