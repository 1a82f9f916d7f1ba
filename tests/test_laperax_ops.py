"""The mechanisms of the Laperax design one at a time, against the float64
functions in laperax_oracle.py: the plain torch form of every op on the CPU,
the HIP kernel under ``-m gpu``.
"""

import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import laperax_oracle as O  # noqa: E402

from kserve_amd import ops  # noqa: E402

DEVICES = [
    pytest.param("cpu", id="cpu"),
    pytest.param("cuda", id="gpu", marks=pytest.mark.gpu),
]


@pytest.fixture(params=DEVICES)
def dev(request):
    if request.param == "cuda":
        assert ops.has_native_seq(), "kserve_amd_seq_C must be built on a GPU box"
    return request.param


def rnd(*shape, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g) * scale


def np64(t):
    return t.detach().double().cpu().numpy()


def maxdiff(got, want):
    return float(np.abs(np64(got) - want).max())


def batch_meta(portions, dev):
    """portions: list of (start position, length, slot) -> positions,
    seq_of_token, cu_seqlens, slots as the step metadata has them."""
    pos, seq, cu = [], [], [0]
    for i, (start, n, _) in enumerate(portions):
        pos += list(range(start, start + n))
        seq += [i] * n
        cu.append(cu[-1] + n)
    return (
        torch.tensor(pos, dtype=torch.int64, device=dev),
        torch.tensor(seq, dtype=torch.int32, device=dev),
        torch.tensor(cu, dtype=torch.int32, device=dev),
        torch.tensor([p[2] for p in portions], dtype=torch.int32, device=dev),
    )


class TestRopeScaleHeads:
    @pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
    @pytest.mark.parametrize("dim,rot", [(8, 8), (12, 6), (5, 0), (64, 20)])
    def test_against_oracle(self, dev, dtype, dim, rot):
        T, ha, hb, tail = 9, 3, 2, 7
        x = rnd(T, 40 + (ha + hb) * dim + tail, seed=1).to(dtype)
        view = x[:, 40:]                           # a column slice of wider rows
        pos = torch.tensor([0, 1, 2, 700, 5, 6, 7, 3001, 9])
        base = 37.0
        inv = O_inv_freq(rot, base)
        got = ops.rope_scale_heads(
            view.to(dev), pos.to(dev), inv.to(dev) if inv is not None else None,
            ha, 1.0, hb, 0.25, dim,
        )
        xv = np64(view)
        want = xv.copy()
        heads = xv[:, : (ha + hb) * dim].reshape(T, ha + hb, dim)
        r = O.rotate(heads, np64(pos), rot, base)
        r[:, ha:] *= 0.25
        want[:, : (ha + hb) * dim] = r.reshape(T, -1)
        assert got.dtype == torch.float32
        assert maxdiff(got, want) < 2e-3  # fp32 angles at positions in the thousands


def O_inv_freq(n, base):
    if not n:
        return None
    i = torch.arange(n // 2, dtype=torch.float64)
    return (float(base) ** (-2.0 * i / n)).to(torch.float32)


class TestUnitNormHeads:
    @pytest.mark.parametrize("dim", [1, 8, 70, 130])
    def test_two_runs_and_untouched_tail(self, dev, dim):
        T, ha, hb = 5, 2, 3
        x = rnd(T, (ha + hb) * dim + 6, seed=2)
        want = np64(x).copy()
        part = want[:, : (ha + hb) * dim].reshape(T, ha + hb, dim)
        part = O.unit(part)
        part[:, :ha] *= 0.5
        part[:, ha:] *= 3.0
        want[:, : (ha + hb) * dim] = part.reshape(T, -1)
        buf = torch.zeros(T, x.shape[1] + 3)
        buf[:, :-3] = x
        xd = buf.to(dev)[:, :-3]                   # rows with a stride
        ops.unit_norm_heads(xd, ha, 0.5, hb, 3.0, dim, 1e-6)
        assert maxdiff(xd, want) < 1e-5


def scan_oracle(q, k, v, qk_heads, decay=None, g=None, beta=None):
    """Whole-sequence recurrence from the oracle's equations. q, k
    [T, G, K], v [T, H, V] -> o [T, H, V]."""
    T, H, V = v.shape
    K = q.shape[2]
    o = np.zeros((T, H, V))
    for a in range(H):
        c = a // (H // qk_heads)
        S = np.zeros((K, V))
        for t in range(T):
            if decay is not None:
                S = decay[a] * S + np.outer(k[t, c], v[t, a])
            else:
                S = g[t, a] * S
                u = beta[t, a] * (v[t, a] - S.T @ k[t, c])
                S = S + np.outer(k[t, c], u)
            o[t, a] = S.T @ q[t, c]
    return o


class TestLinearScan:
    def _inputs(self, T, H, G, K, V, seed):
        q = rnd(T, G * K, seed=seed) * K ** -0.5
        k = rnd(T, G * K, seed=seed + 1) * K ** -0.5
        v = rnd(T, H * V, seed=seed + 2)
        return q, k, v

    def _run(self, dev, q, k, v, state, cuts, slot, G, **kw):
        """One sequence fed in portions ``cuts``; rows are slices of a wider
        buffer."""
        outs, at = [], 0
        wide = torch.cat([q, k, v], dim=1).to(dev)
        a, b = q.shape[1], q.shape[1] + k.shape[1]
        for n in cuts:
            pos, _, cu, slots = batch_meta([(at, n, slot)], dev)
            rows = wide[at : at + n]
            extra = {
                name: t[at : at + n].to(dev) if t.dim() == 2 else t.to(dev)
                for name, t in kw.items()
            }
            outs.append(
                ops.linear_scan(rows[:, :a], rows[:, a:b], rows[:, b:], state, pos,
                                cu, slots, G, **extra)
            )
            at += n
        return torch.cat(outs)

    @pytest.mark.parametrize("H,G,K,V", [(2, 2, 8, 12), (4, 2, 16, 5), (3, 1, 33, 70),
                                         (1, 1, 1, 1), (2, 1, 130, 40), (2, 2, 200, 9)])
    def test_decay_form(self, dev, H, G, K, V):
        T = 45
        q, k, v = self._inputs(T, H, G, K, V, seed=3)
        decay = torch.tensor([1.0 - 2.0 ** -(2 + 3 * i) for i in range(H)])
        want = scan_oracle(np64(q).reshape(T, G, K), np64(k).reshape(T, G, K),
                           np64(v).reshape(T, H, V), G, decay=np64(decay)).reshape(T, -1)
        # junk in every slot: a portion at position 0 must not read it
        state = torch.full((3, H, V, K), 1e6).to(dev)
        for cuts in ([T], [1] * T, [2, 17, 16, 1, 9], [16, 16, 13]):
            got = self._run(dev, q, k, v, state, cuts, 2, G, decay=decay)
            assert maxdiff(got, want) < 1e-4 * max(1.0, np.abs(want).max()), cuts

    @pytest.mark.parametrize("H,G,K,V", [(2, 2, 8, 12), (4, 2, 16, 5), (3, 1, 33, 70),
                                         (1, 1, 1, 1), (2, 1, 130, 40)])
    @pytest.mark.parametrize("ab_dtype", [torch.float32, torch.bfloat16])
    def test_delta_form(self, dev, H, G, K, V, ab_dtype):
        T = 45
        q, k, v = self._inputs(T, H, G, K, V, seed=4)
        qn = O.unit(np64(q).reshape(T, G, K)) * K ** -0.5
        kn = O.unit(np64(k).reshape(T, G, K))
        q = torch.from_numpy(qn.reshape(T, -1)).float()
        k = torch.from_numpy(kn.reshape(T, -1)).float()
        ab = rnd(T, 2 * H + 3, seed=5, scale=2.0).to(ab_dtype)
        a_raw, b_raw = ab[:, 1 : 1 + H], ab[:, 1 + H : 1 + 2 * H]
        a_log = torch.linspace(-2.0, 0.5, H)
        dt_bias = torch.linspace(-1.0, 1.0, H)
        g = np.exp(-np.exp(np64(a_log))[None] * O.softplus(np64(a_raw) + np64(dt_bias)[None]))
        beta = O.sigmoid(np64(b_raw))
        want = scan_oracle(np64(q).reshape(T, G, K), np64(k).reshape(T, G, K),
                           np64(v).reshape(T, H, V), G, g=g, beta=beta).reshape(T, -1)
        state = torch.full((2, H, V, K), -1e6).to(dev)
        for cuts in ([T], [1] * T, [2, 17, 16, 1, 9]):
            got = self._run(dev, q, k, v, state, cuts, 1, G, a_raw=a_raw, b_raw=b_raw,
                            a_log=a_log, dt_bias=dt_bias)
            assert maxdiff(got, want) < 1e-4 * max(1.0, np.abs(want).max()), cuts

    def test_batch_of_unequal_sequences_and_slot_reuse(self, dev):
        """Three sequences in one call (a prompt portion, a single decoded
        token, a portion that continues), slots in any order; then a new
        sequence takes a used slot."""
        H, G, K, V = 2, 1, 16, 8
        lens = [30, 12, 21]
        seqs = [self._inputs(n, H, G, K, V, seed=10 * i) for i, n in enumerate(lens)]
        decay = torch.tensor([0.9, 0.999])
        wants = [
            scan_oracle(np64(q).reshape(n, G, K), np64(k).reshape(n, G, K),
                        np64(v).reshape(n, H, V), G, decay=np64(decay)).reshape(n, -1)
            for (q, k, v), n in zip(seqs, lens)
        ]
        state = torch.full((5, H, V, K), 7.0).to(dev)
        slot = [3, 1, 4]
        got = [[], [], []]

        def step(parts):
            rows = [torch.cat([s[i][lo:hi] for i, lo, hi in parts]) for s in zip(*seqs)]
            # rows[j] concatenates tensor j (q, k or v) of the chosen portions
            q, k, v = [
                torch.cat([seqs[i][j][lo:hi] for i, lo, hi in parts]).to(dev)
                for j in range(3)
            ]
            pos, _, cu, slots = batch_meta([(lo, hi - lo, slot[i]) for i, lo, hi in parts], dev)
            o = ops.linear_scan(q, k, v, state, pos, cu, slots, G, decay=decay.to(dev))
            at = 0
            for i, lo, hi in parts:
                got[i].append(o[at : at + hi - lo].cpu())
                at += hi - lo

        step([(0, 0, 17), (1, 0, 11)])
        step([(1, 11, 12), (0, 17, 18), (2, 0, 2)])
        step([(2, 2, 21), (0, 18, 30)])
        for i in range(3):
            assert maxdiff(torch.cat(got[i]), wants[i]) < 1e-4, i
        # slot 1 (sequence 1 is finished) is handed to a new sequence
        slot[1] = 1
        got[1] = []
        step([(1, 0, 12)])
        assert maxdiff(torch.cat(got[1]), wants[1]) < 1e-4

    def test_far_write_survives_many_tokens(self, dev):
        """One large key/value early on, 700 small ones after it, decay close
        to one: the read-out at the end is the early write."""
        H, G, K, V, T = 1, 1, 8, 4, 720
        q = torch.zeros(T, K)
        q[:, 0] = 1.0
        k = rnd(T, K, seed=6) * 1e-3
        k[:, 0] = 0.0
        k[3, 0] = 5.0
        v = rnd(T, V, seed=7)
        decay = torch.tensor([1.0 - 2.0 ** -12])
        want = scan_oracle(np64(q).reshape(T, 1, K), np64(k).reshape(T, 1, K),
                           np64(v).reshape(T, 1, V), 1, decay=np64(decay)).reshape(T, -1)
        assert abs(want[-1]).max() > 1.0
        state = torch.zeros(2, H, V, K).to(dev)
        got = self._run(dev, q, k, v, state, [300, 37, 363] + [1] * 20, 1, G, decay=decay)
        assert maxdiff(got, want) < 1e-4


class TestNormGate:
    @pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
    @pytest.mark.parametrize("groups,size,weight", [(2, 12, "shared"), (3, 5, None),
                                                    (4, 64, "shared"), (1, 40, "full")])
    def test_gate_after_norm(self, dev, dtype, groups, size, weight):
        T, inner = 6, groups * size
        y = rnd(T, inner, seed=8, scale=3.0)
        z = rnd(T, inner + 4, seed=9).to(dtype)[:, 2 : 2 + inner]
        w = {"shared": 1 + 0.1 * rnd(size, seed=10), "full": 1 + 0.1 * rnd(inner, seed=10),
             None: None}[weight]
        want = O.rms(np64(y).reshape(T, groups, size), 1e-5)
        if weight == "shared":
            want = want * np64(w)[None, None, :]
        want = want.reshape(T, inner)
        if weight == "full":
            want = want * np64(w)[None, :]
        want = want * O.silu(np64(z))
        got = ops.gated_group_rms_norm(
            y.to(dev), z.to(dev), w.to(dev) if w is not None else None, 1e-5, groups,
            dtype, gate_after=True,
        )
        assert got.dtype == dtype
        assert maxdiff(got, want) < (3e-2 if dtype == torch.bfloat16 else 1e-5)

    def test_gate_first_is_unchanged(self, dev):
        T, inner = 4, 24
        y, z, w = rnd(T, inner, seed=1), rnd(T, inner, seed=2), 1 + 0.1 * rnd(inner, seed=3)
        want = O.rms((np64(y) * O.silu(np64(z))).reshape(T, 2, 12), 1e-5).reshape(T, inner) * np64(w)
        got = ops.gated_group_rms_norm(y.to(dev), z.to(dev), w.to(dev), 1e-5, 2, torch.float32)
        assert maxdiff(got, want) < 1e-5


class TestResidualNorm:
    @pytest.mark.parametrize("width", [24, 30, 2048])
    @pytest.mark.parametrize("out_dtype,d_dtype", [(torch.float32, torch.float32),
                                                   (torch.bfloat16, torch.bfloat16),
                                                   (torch.bfloat16, torch.float32)])
    def test_delta_dtype_of_its_own(self, dev, width, out_dtype, d_dtype):
        T = 5
        x, w = rnd(T, width, seed=1), 1 + 0.1 * rnd(width, seed=2)
        d = rnd(T, width, seed=3).to(d_dtype)
        res = x.clone().to(dev)
        got = ops.add_rms_norm_f32res(res, w.to(dev), 1e-5, 0.0, out_dtype, d.to(dev))
        new = np64(x) + np64(d)
        assert maxdiff(res, new) < 1e-6
        assert got.dtype == out_dtype
        assert maxdiff(got, O.rms(new, 1e-5) * np64(w)) < (
            4e-2 if out_dtype == torch.bfloat16 else 1e-5
        )


class TestConvWithoutBias:
    @pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
    @pytest.mark.parametrize("taps,channels", [(2, 8), (3, 20), (4, 64), (6, 5)])
    def test_portions_against_oracle(self, dev, dtype, taps, channels):
        T = 23
        x = rnd(T, channels, seed=4).to(dtype)
        w = rnd(channels, taps, seed=5, scale=0.5)
        want = O.conv_silu(np64(x), np64(w))
        state = torch.full((3, taps - 1, channels), 50.0, dtype=dtype).to(dev)
        for cuts in ([T], [1] * T, [2, 2, 1, 9, 9]):
            outs, at = [], 0
            for n in cuts:
                pos, seq, cu, slots = batch_meta([(at, n, 2)], dev)
                outs.append(ops.causal_conv_silu(x[at : at + n].to(dev), w.to(dev), None,
                                                 state, pos, seq, cu, slots))
                at += n
            assert maxdiff(torch.cat(outs), want) < 1e-5, cuts


class TestActivations:
    @pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
    @pytest.mark.parametrize("d", [8, 13, 64])
    def test_relu2_scale(self, dev, dtype, d):
        x = rnd(7, d, seed=6, scale=2.0).to(dtype)
        sc = torch.tensor([1.0, 0.0, 0.5, 2.0, 0.0, 1.5, 0.25])
        tol = 6e-2 if dtype == torch.bfloat16 else 1e-5
        want = np.maximum(np64(x), 0.0) ** 2
        assert maxdiff(ops.relu2_scale(x.to(dev)), want) < tol * max(1.0, want.max())
        got = ops.relu2_scale(x.to(dev), sc.to(dev))
        assert maxdiff(got, want * np64(sc)[:, None]) < tol * max(1.0, want.max())
        assert float(got[1].abs().max()) == 0.0

    @pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
    def test_scale_softcap(self, dev, dtype):
        x = rnd(5, 33, seed=7, scale=20.0).to(dtype)
        got = ops.scale_softcap(x.to(dev), 0.5, 6.0)
        assert got.dtype == torch.float32
        assert maxdiff(got, 6.0 * np.tanh(np64(x) * 0.5 / 6.0)) < 1e-5
        assert maxdiff(ops.scale_softcap(x.to(dev), 0.5, 0.0), np64(x) * 0.5) < 1e-5


class TestRouterScale:
    @pytest.mark.parametrize("E,top", [(4, 2), (1, 1), (7, 7), (70, 3)])
    def test_weights_and_choice(self, dev, E, top):
        T, W = 11, 24
        h = rnd(T, W, seed=8)
        sd = {"router": rnd(E, W, seed=9, scale=0.5)}
        want = O.route(np64(h), {"router": np64(sd["router"])}, "", {"experts": E, "top": top, "scale": 2.5})
        idx, w, dense, _ = ops.route_tokens(
            h.to(dev), sd["router"].to(dev), top, renorm=True, dense=True,
            renorm_eps=1e-20, weight_scale=2.5,
        )
        for t in range(T):
            assert [int(e) for e in idx[t]] == [e for e, _ in want[t]]
            assert maxdiff(w[t], np.array([x for _, x in want[t]])) < 1e-5
            row = np.zeros(E)
            for e, x in want[t]:
                row[e] = x
            assert maxdiff(dense[t], row) < 1e-5
        assert abs(float(w.sum(-1).mean()) - 2.5) < 1e-4


class TestExperts:
    @pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
    @pytest.mark.parametrize("T", [5, 700])
    def test_both_forms_against_oracle(self, dev, dtype, T):
        """Few tokens take the all-experts form, many the sorted one; the
        mixer's output joins the fp32 sum."""
        from kserve_amd.engine.config import SquaredReluMoESpec
        from kserve_amd.models.mixers import SquaredReluMoE

        W, E, top, ff = 32, 6, 2, 24
        cfg = O.make_config([O.retention_layer(mlp=O.moe(E, top, ff, 1.7))], width=W)
        sd = O.random_weights(cfg, seed=11, dtype=dtype)
        mod = SquaredReluMoE(W, SquaredReluMoESpec(E, top, ff, 1.7), dtype)
        mod.load(lambda n: sd[n], "l0.mlp.")
        mod.to(dev)
        assert (T <= mod.dense_max_tokens) == (T == 5)
        h = rnd(T, W, seed=12).to(dtype)
        extra = rnd(T, W, seed=13).to(dtype)
        Wn = {k: np64(v) for k, v in sd.items()}
        want = O.experts(np64(h), Wn, "l0.mlp.", cfg["layers"][0]["mlp"]) + np64(extra)
        got = mod(h.to(dev), extra=extra.to(dev))
        assert got.dtype == torch.float32
        err = np.abs(np64(got) - want).max(axis=1) / np.abs(want).max()
        if dtype == torch.float32:
            assert err.max() < 1e-4
        else:
            # a near-tie in the router may pick another expert in bf16
            assert np.mean(err < 5e-2) > 0.9


class TestWindowedAttention:
    """Rotate-then-norm without weights, grouped KV heads, a sliding window:
    prompt portions and single decoded tokens through scattered pages."""

    @pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
    @pytest.mark.parametrize("window,bs", [(5, 16), (16, 16), (17, 8), (40, 16), (1, 4)])
    def test_against_oracle(self, dev, dtype, window, bs):
        from kserve_amd.engine.config import AttentionMixerSpec
        from kserve_amd.models.mixers import LayerCache, RotaryChunkSinkAttention

        W, H, G, D, V, T = 24, 4, 2, 8, 12, 70
        layer = O.attention_layer(H, G, D, V, 0.6, window, rot_dims=6, base=11.0)
        cfg = O.make_config([layer], width=W)
        sd = O.random_weights(cfg, seed=14, dtype=dtype)
        spec = AttentionMixerSpec.from_dict(layer["mixer"], mask="window")
        assert spec.window == window and spec.chunk == 0
        mod = RotaryChunkSinkAttention(W, spec, 1e-5, dtype, sink=False,
                                       value_unit_norm=False, rotate_values=False,
                                       norm_weights=False)
        mod.load(lambda n: sd[n], "l0.mix.")
        mod.to(dev)
        h = rnd(T, W, seed=15).to(dtype)
        want = O.attention(np64(h), {k: np64(v) for k, v in sd.items()}, "l0.mix.",
                           layer["mixer"], 1e-5)
        nblocks = -(-T // bs)
        table = torch.randperm(nblocks + 3, generator=torch.Generator().manual_seed(1))[:nblocks] + 1
        cache = LayerCache(
            k=torch.zeros(nblocks + 5, G, bs, D, dtype=dtype, device=dev),
            v=torch.zeros(nblocks + 5, G, bs, V, dtype=dtype, device=dev),
        )
        outs, at = [], 0
        cuts = [window + 3, 2, 9] + [1] * 12
        cuts.append(T - sum(cuts))
        for n in cuts:
            pos = torch.arange(at, at + n)
            meta = _AttnMeta(
                slot_mapping=(table[pos // bs] * bs + pos % bs).to(torch.int32).to(dev),
                block_tables=table.view(1, -1).to(torch.int32).to(dev),
                cu_seqlens=torch.tensor([0, n], dtype=torch.int32, device=dev),
                context_lens=torch.tensor([at + n], dtype=torch.int32, device=dev),
                max_seqlen=n,
            )
            outs.append(mod(h[at : at + n].to(dev), pos.to(dev), cache, meta))
            at += n
        got = torch.cat(outs)
        tol = 4e-2 if dtype == torch.bfloat16 else 1e-4
        assert maxdiff(got, want) < tol * np.abs(want).max()


class _AttnMeta:
    def __init__(self, **kw):
        self.__dict__.update(kw)
