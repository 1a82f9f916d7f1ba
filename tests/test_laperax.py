"""The Laperax decoder (retention / gated-delta / windowed-attention mixers
beside squared-relu experts) through the engine, against the float64 oracle in
laperax_oracle.py.

Every test builds its own small config and random checkpoint. The same tests
run on the CPU (plain torch forms of the ops, the engine's scheduling, page and
slot logic) and — marked gpu — on the HIP kernels in both activation dtypes.
"""

import json
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import laperax_oracle as O  # noqa: E402

from kserve_amd.engine.config import (  # noqa: E402
    CacheConfig,
    EngineConfig,
    HybridModelConfig,
    SchedulerConfig,
)
from kserve_amd.engine.engine import LLMEngine  # noqa: E402
from kserve_amd.engine.replay import TraceReplayer  # noqa: E402
from kserve_amd.engine.sampling_params import SamplingParams  # noqa: E402
from kserve_amd.models.registry import build_model  # noqa: E402

BACKENDS = [
    pytest.param(("cpu", "float32"), id="cpu-f32"),
    pytest.param(("cuda", "float32"), id="gpu-f32", marks=pytest.mark.gpu),
    pytest.param(("cuda", "bfloat16"), id="gpu-bf16", marks=pytest.mark.gpu),
]


def three_kinds_config(**kw):
    """Every mixer once with experts and once more with other sizes; one
    layer has no feed-forward."""
    return O.make_config(
        layers=[
            O.delta_layer(heads=4, kv_heads=2, dim=8, vdim=12, conv=4, mlp=O.moe()),
            O.retention_layer(heads=2, dim=8, vdim=12, rot_dims=4,
                              mlp=O.moe(experts=5, top=3, ff=16, scale=0.8)),
            O.attention_layer(heads=4, kv_heads=2, dim=8, vdim=12, window=9,
                              mlp=O.moe(experts=3, top=1, ff=40, scale=2.0)),
            O.delta_layer(heads=3, kv_heads=3, dim=20, vdim=4, conv=2),
            O.retention_layer(heads=3, dim=12, vdim=20, rot_dims=12, base=7.0,
                              decay=[0.5, 0.97, 1.0 - 2.0 ** -9], mlp=O.moe(ff=8)),
            O.attention_layer(heads=6, kv_heads=1, dim=16, vdim=8, scale=0.25,
                              window=21, rot_dims=16, base=1000.0, mlp=O.moe()),
        ],
        **kw,
    )


def make_engine(cfg, sd, backend, num_blocks=64, block_size=16, max_seqs=4,
                eager=False, multi_step=1, max_len=1024, batched_tokens=None,
                mixed=False):
    device, dtype = backend
    mc = HybridModelConfig.from_dict(cfg)
    mc.dtype = dtype
    model = build_model(mc, device=device)
    model.load_hf_state_dict(sd)
    ec = EngineConfig(
        model=mc,
        cache=CacheConfig(block_size=block_size, num_gpu_blocks=num_blocks),
        scheduler=SchedulerConfig(
            max_num_seqs=max_seqs,
            max_num_batched_tokens=batched_tokens or max_len,
            max_model_len=max_len, enable_chunked_prefill=True,
            multi_step=multi_step, mixed_batches=mixed,
        ),
        device=device, eos_token_id=-1, enforce_eager=eager,
    )
    return LLMEngine(ec, model=model)


def weights_for(cfg, backend, seed=0):
    """Random checkpoint in the backend's dtype. For bf16 the config is
    changed in place so that every mixture uses all of its experts: with a
    discrete choice, a token whose last chosen and first rejected scores are
    closer than the bf16 rounding of the router's input takes another expert
    than the float64 oracle, and in a recurrent model that one token changes
    every later position. The choice itself is tested in fp32 here and in
    both dtypes on the expert block alone (test_laperax_ops.py)."""
    if backend[1] == "bfloat16":
        for layer in cfg["layers"]:
            # (the router kernel chooses at most 64)
            if layer.get("mlp") and layer["mlp"]["router"]["experts"] <= 64:
                layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    dt = torch.bfloat16 if backend[1] == "bfloat16" else torch.float32
    return O.random_weights(cfg, seed=seed, dtype=dt)


def row_err(got, want):
    """Per position: centered RMS difference over the vocabulary, relative to
    the RMS of the expected logits."""
    got, want = got.double().cpu(), want.double()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    scale = (want - want.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    return d.pow(2).mean(-1).sqrt() / scale


def close(got, want, backend, factor=1.0, most=0.9, worst=0.4):
    """fp32: every position inside the tolerance. bf16: the median well
    inside, nine positions in ten inside, none far outside. A recurrent
    read-out is divided by its own RMS, so where it is small (cancellation
    among the written values) the 8-bit rounding of the GEMM outputs that
    feed it is amplified at that position; cut-independence in bf16 is held
    to a tighter bound by test_alone_equals_batched."""
    e = row_err(got, want)
    if backend[1] == "bfloat16":
        ok = bool(
            e.median() < 3e-2 * factor
            and (e < 8e-2 * factor).float().mean() >= most
            and e.max() < worst * factor
        )
    else:
        ok = bool(e.max() < 2e-4 * factor)
    if not ok:
        print("row errors: median %.3g, 90%% %.3g, max %.3g at %d of %d" % (
            e.median(), e.quantile(0.9), e.max(), e.argmax(), e.numel()))
    return ok


def run_schedule(engine, prompts, schedule):
    """schedule: list of steps, each a list of (request index, count); every
    token's logits are collected. Returns {index: [T, vocab]}."""
    rp = TraceReplayer(engine)
    at = {i: 0 for i in range(len(prompts))}
    got = {i: [] for i in range(len(prompts))}
    for step in schedule:
        entries, end, order = [], [], []
        for i, n in step:
            lo = at[i]
            entries.append(
                {"id": f"r{i}", "tokens": prompts[i][lo : lo + n], "want": list(range(n))}
            )
            order.append((i, n))
            at[i] = lo + n
            if at[i] == len(prompts[i]):
                end.append(f"r{i}")
        logits = rp.step(entries, end)
        off = 0
        for i, n in order:
            got[i].append(logits[off : off + n].float().cpu())
            off += n
    return {i: torch.cat(v) for i, v in got.items() if v}


def random_prompt(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


@pytest.fixture(scope="module", params=BACKENDS)
def backend(request):
    if request.param[0] == "cuda":
        from kserve_amd import ops

        assert ops.has_native_seq(), "kserve_amd_seq_C must be built on a GPU box"
    return request.param


class TestWholePrompts:
    def test_logits_and_residual_stream(self, backend):
        cfg = three_kinds_config()
        sd = weights_for(cfg, backend)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(45, cfg["vocab"], 1)
        res = []
        want = O.forward(cfg, sd, toks, res)
        eng.model.debug_residuals = []
        got = run_schedule(eng, [toks], [[(0, len(toks))]])[0]
        streams = eng.model.debug_residuals
        eng.model.debug_residuals = None
        assert close(got, want, backend)
        assert len(streams) == len(cfg["layers"])
        if backend[1] == "float32":
            for mine, ref in zip(streams, res):
                scale = ref.abs().max().item()
                assert (mine.double().cpu() - ref).abs().max().item() < 1e-3 * scale

    def test_first_tokens(self, backend):
        """Prompts of 1, 2 and 3 tokens: shorter than every convolution and
        window; all history before position 0 is zero."""
        cfg = three_kinds_config()
        sd = weights_for(cfg, backend, seed=3)
        eng = make_engine(cfg, sd, backend)
        for n in (1, 2, 3):
            toks = random_prompt(n, cfg["vocab"], 10 + n)
            got = run_schedule(eng, [toks], [[(0, n)]])[0]
            assert close(got, O.forward(cfg, sd, toks), backend)

    def test_sizes_equal_to_one_and_missing_parts(self, backend):
        """Single heads, one expert, every expert chosen, one tap, a window
        of one, no rotation, no cap, unit scales."""
        cfg = O.make_config(
            vocab=31, width=24, logit_scale=1.0, softcap=0.0,
            layers=[
                O.delta_layer(heads=1, kv_heads=1, dim=8, vdim=8, conv=1,
                              mlp=O.moe(experts=1, top=1, ff=8, scale=1.0)),
                O.retention_layer(heads=1, dim=6, vdim=10, rot_dims=0, decay=[1.0]),
                O.attention_layer(heads=1, kv_heads=1, dim=8, vdim=24, scale=1.0,
                                  window=1, rot_dims=0),
                O.attention_layer(heads=2, kv_heads=2, dim=4, vdim=4, scale=0.5,
                                  window=300, rot_dims=2,
                                  mlp=O.moe(experts=3, top=3, ff=12)),
                O.delta_layer(heads=2, kv_heads=1, dim=17, vdim=5, conv=5),
            ],
        )
        sd = weights_for(cfg, backend, seed=4)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(23, cfg["vocab"], 5)
        got = run_schedule(eng, [toks], [[(0, 12)]] + [[(0, 1)]] * 11)[0]
        assert close(got, O.forward(cfg, sd, toks), backend)

    def test_many_experts_and_wide_heads(self, backend):
        cfg = O.make_config(
            vocab=40, width=48,
            layers=[
                O.retention_layer(heads=2, dim=72, vdim=40, rot_dims=30,
                                  mlp=O.moe(experts=70, top=4, ff=8)),
                O.delta_layer(heads=2, kv_heads=1, dim=40, vdim=72, conv=3),
            ],
        )
        sd = weights_for(cfg, backend, seed=21)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(40, cfg["vocab"], 22)
        got = run_schedule(eng, [toks], [[(0, 33)]] + [[(0, 1)]] * 7)[0]
        # more experts than the all-experts setting of the bf16 runs can
        # cover: there a near-tie in the router may take another expert
        assert close(got, O.forward(cfg, sd, toks), backend, most=0.7, worst=1.0)


class TestSchedules:
    def test_prefill_then_decode(self, backend):
        cfg = three_kinds_config()
        sd = weights_for(cfg, backend, seed=5)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(70, cfg["vocab"], 6)
        want = O.forward(cfg, sd, toks)
        sched = [[(0, 30)]] + [[(0, 1)] for _ in range(40)]
        got = run_schedule(eng, [toks], sched)[0]
        assert close(got, want, backend)

    def test_graphs_equal_eager(self, backend):
        if backend[0] != "cuda":
            pytest.skip("captured graphs are a GPU path")
        cfg = three_kinds_config()
        sd = weights_for(cfg, backend, seed=15)
        toks = random_prompt(50, cfg["vocab"], 16)
        sched = [[(0, 20)]] + [[(0, 1)] for _ in range(30)]
        outs = []
        for eager in (False, True):
            eng = make_engine(cfg, sd, backend, eager=eager)
            outs.append(run_schedule(eng, [toks], sched)[0])
        assert row_err(outs[0], outs[1].double()).max() < 1e-5

    def test_token_by_token_from_the_start(self, backend):
        cfg = three_kinds_config()
        sd = weights_for(cfg, backend, seed=6)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(26, cfg["vocab"], 7)
        got = run_schedule(eng, [toks], [[(0, 1)] for _ in toks])[0]
        assert close(got, O.forward(cfg, sd, toks), backend)

    @pytest.mark.parametrize("sizes", [[2] * 20, [3, 17, 2, 16, 1, 5, 2, 2, 31],
                                       [16, 16, 16, 1, 15, 2, 14], [9, 9, 21, 21, 1, 8]])
    def test_portions(self, backend, sizes):
        """Portions down to two tokens, cut inside pages, windows and
        scan chunks and shorter than the convolutions' history."""
        cfg = three_kinds_config()
        sd = weights_for(cfg, backend, seed=7)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(sum(sizes), cfg["vocab"], 8)
        got = run_schedule(eng, [toks], [[(0, n)] for n in sizes])[0]
        assert close(got, O.forward(cfg, sd, toks), backend)

    def test_mixed_batches_and_reuse(self, backend):
        """Unequal requests side by side — portions next to decode tokens,
        requests skipped for a step — in a pool too small for all of them at
        once, so pages and state slots are handed out again."""
        cfg = three_kinds_config()
        sd = weights_for(cfg, backend, seed=8)
        # 9 usable pages of 16 and 3 slots; six requests
        eng = make_engine(cfg, sd, backend, num_blocks=10, max_seqs=3)
        lens = [40, 23, 9, 33, 17, 48]
        prompts = [random_prompt(n, cfg["vocab"], 20 + i) for i, n in enumerate(lens)]
        sched = [
            [(0, 19), (1, 5)],
            [(0, 1), (1, 16), (2, 2)],
            [(0, 1), (2, 1)],
            [(1, 1), (2, 1), (0, 19)],      # request 0 done
            [(1, 1), (2, 5)],               # requests 1, 2 done
            [(3, 33), (4, 3)],              # request 3 done
            [(4, 1), (5, 20)],
            [(4, 1)],
            [(5, 1), (4, 12)],              # request 4 done
        ] + [[(5, 1)] for _ in range(27)]
        got = run_schedule(eng, prompts, sched)
        for i, toks in enumerate(prompts):
            assert got[i].shape[0] == len(toks)
            assert close(got[i], O.forward(cfg, sd, toks), backend), i
        bm = eng.scheduler.block_manager
        assert bm.num_free_blocks == 9
        assert eng.scheduler.state_slots.num_free == 3

    def test_alone_equals_batched(self, backend):
        cfg = three_kinds_config()
        sd = weights_for(cfg, backend, seed=9)
        prompts = [random_prompt(n, cfg["vocab"], 40 + n) for n in (26, 7, 18)]
        eng = make_engine(cfg, sd, backend)
        together = run_schedule(
            eng, prompts,
            [[(0, 20), (1, 7), (2, 3)], [(0, 1), (2, 15)]] + [[(0, 1)]] * 5,
        )
        for i, toks in enumerate(prompts):
            alone = run_schedule(eng, [toks], [[(0, len(toks))]])[0]
            # same kernels, other batch composition: rounding only
            assert close(together[i], alone.double(), backend, factor=0.25)

    def test_long_decode(self, backend):
        cfg = O.make_config(
            vocab=50, width=32,
            layers=[
                O.retention_layer(heads=2, dim=8, vdim=8, rot_dims=8,
                                  decay=[0.99, 1.0 - 2.0 ** -11]),
                O.delta_layer(heads=2, kv_heads=1, dim=8, vdim=16, conv=3),
                O.attention_layer(heads=2, kv_heads=1, dim=8, vdim=16, window=40),
            ],
        )
        sd = weights_for(cfg, backend, seed=10)
        eng = make_engine(cfg, sd, backend, num_blocks=32)
        toks = random_prompt(300, cfg["vocab"], 11)
        got = run_schedule(eng, [toks], [[(0, 4)]] + [[(0, 1)]] * 296)[0]
        assert close(got, O.forward(cfg, sd, toks), backend)


class TestNeedles:
    """One layer whose weights make a single early token decide the output,
    so that a key lost at a page border, one position off a window's edge or
    dropped from a carried state shows at once.

    Token 1 is the needle. Every other embedding has no component along
    coordinate 0, and all embeddings share a large coordinate 1. Key channel 0
    reads coordinate 0 (non-zero for the needle only), query channel 0 reads
    coordinate 1 (the same for every token); the needle's value is far from
    the others'. Rotation is kept off channel 0."""

    def _setup(self, kind, backend, **kw):
        if kind == "attention":
            layer = O.attention_layer(heads=2, kv_heads=1, dim=8, vdim=8, scale=3.0,
                                      rot_dims=4, **kw)
        elif kind == "retention":
            layer = O.retention_layer(heads=2, dim=8, vdim=8, rot_dims=4,
                                      decay=[1.0 - 2.0 ** -10, 1.0 - 2.0 ** -8])
        else:
            layer = O.delta_layer(heads=2, kv_heads=1, dim=8, vdim=8, conv=2)
        cfg = O.make_config(vocab=40, width=16, layers=[layer], softcap=0.0,
                            logit_scale=1.0)
        sd = weights_for(cfg, backend, seed=12)
        emb = sd["embed"].float()
        emb[:, 0] = 0.0
        emb[1, 0] = 8.0
        emb[:, 1] = 4.0
        sd["embed"] = emb.to(sd["embed"].dtype)
        sd["embed.norm"].fill_(1.0)
        sd["l0.norm1"].fill_(1.0)
        p = "l0.mix."
        ch = 7  # an un-rotated channel of the (only) q/k head group
        for n in ("q", "k"):
            w = sd[p + n].float()
            w[:, :2] = 0.0
            sd[p + n] = w.to(sd[p + n].dtype)
        for head in range(sd[p + "q"].shape[0] // 8):
            sd[p + "q"][head * 8 + ch] = 0.0
            sd[p + "q"][head * 8 + ch, 1] = 3.0
        for head in range(sd[p + "k"].shape[0] // 8):
            sd[p + "k"][head * 8 + ch] = 0.0
            sd[p + "k"][head * 8 + ch, 0] = 3.0
        v = sd[p + "v"].float()
        v[:, 0] = 2.0
        sd[p + "v"] = v.to(sd[p + "v"].dtype)
        if kind == "delta":
            # pass the current token through the convolutions, decay slowly
            for n in ("q", "k", "v"):
                c = sd[p + n + ".conv"]
                c.zero_()
                c[:, -1] = 1.0
            sd[p + "A_log"].fill_(-7.0)
            # unit-norm queries: leave them nothing but the needle's channel,
            # so that the read-out is the needle's row of the state
            q = torch.zeros_like(sd[p + "q"])
            q[ch, 1] = 3.0
            sd[p + "q"] = q
        return cfg, sd

    def _prompt(self, total, needle_at, vocab, seed):
        toks = [2 + t for t in random_prompt(total, vocab - 2, seed)]
        toks[needle_at] = 1
        return toks

    def _check_needle_matters(self, cfg, sd, toks, rows):
        """The oracle's own output changes a lot at ``rows`` when the needle
        is replaced: the test would see it missing."""
        other = list(toks)
        other[toks.index(1)] = 2
        a, b = O.forward(cfg, sd, toks), O.forward(cfg, sd, other)
        assert row_err(a[rows], b[rows]).min() > 0.05

    @pytest.mark.parametrize("window", [33, 48, 64])
    @pytest.mark.parametrize("cut", ["whole", "decode", "portions"])
    def test_window_edges(self, backend, window, cut):
        """The needle just inside and just outside the window, for queries
        in a prompt portion and decoded alone; windows smaller than, equal to
        and no multiple of the 16-token page."""
        cfg, sd = self._setup("attention", backend, window=window)
        needle, total = 5, 5 + window + 6
        toks = self._prompt(total, needle, cfg["vocab"], 13)
        want = O.forward(cfg, sd, toks)
        last_in = needle + window - 1
        self._check_needle_matters(cfg, sd, toks, [last_in - 1, last_in])
        # ... and no longer once it has left the window
        other = list(toks)
        other[needle] = 2
        assert row_err(want[last_in + 1 :], O.forward(cfg, sd, other)[last_in + 1 :]).max() < 1e-9
        eng = make_engine(cfg, sd, backend)
        if cut == "whole":
            sched = [[(0, total)]]
        elif cut == "decode":
            sched = [[(0, last_in - 2)]] + [[(0, 1)]] * (total - last_in + 2)
        else:
            sched = [[(0, last_in)], [(0, 2)], [(0, total - last_in - 2)]]
        got = run_schedule(eng, [toks], sched)[0]
        e = row_err(got, want)
        assert e.max() < (6e-2 if backend[1] == "bfloat16" else 2e-4), e.argmax()

    @pytest.mark.parametrize("kind", ["attention", "retention", "delta"])
    @pytest.mark.parametrize("needle_at", [0, 15, 16, 31])
    def test_far_token_at_page_borders(self, backend, kind, needle_at):
        """The needle 300+ positions back, first and last in a page, read by
        prompt portions and by tokens decoded alone."""
        kw = {"window": 400} if kind == "attention" else {}
        cfg, sd = self._setup(kind, backend, **kw)
        total = 350
        toks = self._prompt(total, needle_at, cfg["vocab"], 14)
        want = O.forward(cfg, sd, toks)
        self._check_needle_matters(cfg, sd, toks, [total - 20, total - 1])
        eng = make_engine(cfg, sd, backend)
        sched = [[(0, 100)], [(0, 37)], [(0, 163)], [(0, 2)], [(0, 16)]] + [[(0, 1)]] * 32
        got = run_schedule(eng, [toks], sched)[0]
        e = row_err(got, want)
        assert e.max() < (6e-2 if backend[1] == "bfloat16" else 2e-4), e.argmax()


class TestGeneration:
    def test_greedy_through_the_engine(self, backend):
        """LLMEngine.generate with its own scheduler, multi-step decode
        windows, mixed batches and a pool that forces preemption equals
        step-by-step argmax of the oracle for every request."""
        cfg = three_kinds_config(softcap=30.0, logit_scale=4.0)
        sd = weights_for(cfg, backend, seed=30)
        prompts = [random_prompt(n, cfg["vocab"], 60 + n) for n in (12, 5, 19, 8)]
        new = 12
        def follows_oracle(prompt, out):
            """Every generated token is the oracle's argmax given what was
            generated before it (or within a hair of it: near-ties)."""
            seq = list(prompt)
            for t in out:
                logits = O.forward(cfg, sd, seq)[-1]
                if (logits.max() - logits[t]).item() > 1e-3:
                    return False
                seq.append(int(t))
            return True

        for kw in (
            dict(multi_step=4),
            dict(multi_step=1, mixed=True, batched_tokens=16),
            dict(multi_step=4, num_blocks=6, max_seqs=2),
        ):
            eng = make_engine(cfg, sd, backend, **kw)
            outs = eng.generate(
                prompts,
                SamplingParams(max_tokens=new, temperature=0.0, ignore_eos=True),
            )
            assert len(outs) == len(prompts)
            got = [list(o.output_token_ids) for o in outs.values()]
            assert all(len(g) == new for g in got)
            if backend[1] == "float32":
                assert all(follows_oracle(p, g) for p, g in zip(prompts, got)), kw
            bm = eng.scheduler.block_manager
            assert bm.num_free_blocks == kw.get("num_blocks", 64) - 1
            assert eng.scheduler.state_slots.num_free == kw.get("max_seqs", 4)


    def test_sampled_generation(self, backend):
        """Temperature sampling through the engine's samplers (on the GPU the
        fused sampler inside captured multi-step windows): the model hands
        over fp32 logits in both activation dtypes."""
        cfg = three_kinds_config()
        sd = weights_for(cfg, backend, seed=31)
        prompts = [random_prompt(n, cfg["vocab"], 80 + n) for n in (9, 4, 15)]
        eng = make_engine(cfg, sd, backend, multi_step=4)
        outs = eng.generate(
            prompts,
            SamplingParams(max_tokens=10, temperature=0.8, top_k=20, top_p=0.9,
                           ignore_eos=True, seed=5),
        )
        assert len(outs) == 3
        for o in outs.values():
            assert len(o.output_token_ids) == 10
            assert all(0 <= t < cfg["vocab"] for t in o.output_token_ids)


class TestPlumbing:
    def test_registry_config_layout_and_loading(self, tmp_path):
        from safetensors.torch import save_file

        from kserve_amd.models.registry import load_model_config, native_modules_for

        cfg = three_kinds_config()
        sd = O.random_weights(cfg, seed=2, dtype=torch.bfloat16)
        d = tmp_path / "model"
        d.mkdir()
        (d / "config.json").write_text(json.dumps(cfg))
        save_file({k: v.contiguous() for k, v in sd.items()}, str(d / "model.safetensors"))
        mc = load_model_config(str(d))
        assert mc.architecture == "Laperax"
        assert native_modules_for(str(d)) == ("kserve_amd_seq_C",)
        assert mc.has_recurrent_state
        assert mc.layers[2].attention.window == 9 and mc.layers[2].attention.chunk == 0
        assert mc.layers[4].retention.decay[0] == 0.5
        assert mc.layers[3].delta.conv == 2 and mc.layers[3].mlp is None
        assert mc.layers[1].mlp.scale == 0.8 and mc.logit_softcap == 8.0
        mc.dtype = "float32"
        model = build_model(mc, device="cpu")
        layout = model.cache_layout()
        assert layout[2][0] == (2, 8, 12) and layout[2][1] == {}
        assert layout[0][0] is None and set(layout[0][1]) == {"ssm", "conv"}
        assert set(layout[1][1]) == {"ssm"}
        assert layout[1][1]["ssm"][0] == (2, 12, 8)

    def test_server_cli_picks_the_engine(self, tmp_path):
        from kserve_amd.runtimes.huggingfaceserver import detect_backend

        (tmp_path / "config.json").write_text(json.dumps(three_kinds_config()))
        assert detect_backend(str(tmp_path)) == "engine"

    def test_unknown_parts_are_refused(self):
        cfg = three_kinds_config()
        cfg["layers"][0]["type"] = "something-else"
        with pytest.raises(ValueError):
            HybridModelConfig.from_dict(cfg)
        cfg = three_kinds_config()
        cfg["layers"][0]["mlp"]["kind"] = "dense"
        with pytest.raises(ValueError):
            HybridModelConfig.from_dict(cfg)
        cfg = three_kinds_config()
        cfg["layers"][1]["mixer"]["decay"] = [0.5]
        with pytest.raises(ValueError):
            HybridModelConfig.from_dict(cfg)

    def test_engine_from_a_model_directory(self, tmp_path):
        from safetensors.torch import save_file

        cfg = three_kinds_config()
        sd = O.random_weights(cfg, seed=2, dtype=torch.float32)
        d = tmp_path / "model"
        d.mkdir()
        (d / "config.json").write_text(json.dumps(cfg))
        save_file({k: v.contiguous() for k, v in sd.items()}, str(d / "model.safetensors"))
        from kserve_amd.engine.replay import engine_config_for_trace

        ec = engine_config_for_trace(str(d), "float32", 128, "cpu", block_size=16)
        eng = LLMEngine(ec)
        toks = random_prompt(30, cfg["vocab"], 3)
        got = run_schedule(eng, [toks], [[(0, 17)], [(0, 13)]])[0]
        assert close(got, O.forward(cfg, sd, toks), ("cpu", "float32"))
