"""Each mechanism of the Voborax design alone: ``kserve_amd.ops`` against the
float64 oracle functions of voborax_oracle.py.

Parametrised over the CPU forms (always) and the HIP kernels in both
activation dtypes (marked gpu). Inputs are rounded to the activation dtype
first, so the oracle and the op see the same numbers.
"""

import math
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import voborax_oracle as O  # noqa: E402

from kserve_amd import ops  # noqa: E402
from kserve_amd.ops.torch_ref import rotary_inv_freq  # noqa: E402

F64 = torch.float64

BACKENDS = [
    pytest.param(("cpu", torch.float32), id="cpu-f32"),
    pytest.param(("cuda", torch.float32), id="gpu-f32", marks=pytest.mark.gpu),
    pytest.param(("cuda", torch.bfloat16), id="gpu-bf16", marks=pytest.mark.gpu),
]


@pytest.fixture(params=BACKENDS)
def be(request):
    if request.param[0] == "cuda":
        assert ops.has_native_seq(), "kserve_amd_seq_C must be built on a GPU box"
    return request.param


def rnd(*shape, seed=0, scale=1.0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(dtype).float()


def act(x, be):
    return x.to(be[1]).to(be[0])


def f32(x, be):
    return x.float().to(be[0])


def i32(v, be):
    return torch.as_tensor(v, dtype=torch.int32).to(be[0])


def i64(v, be):
    return torch.as_tensor(v, dtype=torch.int64).to(be[0])


def close(got, want, be, f32_tol=2e-5, bf16_tol=2e-2):
    tol = bf16_tol if be[1] == torch.bfloat16 else f32_tol
    got, want = got.double().cpu(), want.double()
    scale = max(want.abs().max().item(), 1e-6)
    err = (got - want).abs().max().item() / scale
    assert err < tol, f"relative error {err:.3g} (tolerance {tol})"


class TestPostLayerNorm:
    @pytest.mark.parametrize("width", [16, 50, 192, 1028, 8200])
    @pytest.mark.parametrize("delta_f32", [False, True])
    def test_add_then_cast(self, be, width, delta_f32):
        eps, mult, T = 1e-5, 0.6, 5
        x = rnd(T, width, seed=2, scale=3.0)
        # a large common offset: the norm must remove the mean first
        d = rnd(T, width, seed=3, scale=0.2, dtype=torch.float32 if delta_f32 else be[1]) + 4.0
        d = d.to(torch.float32 if delta_f32 else be[1]).float()
        w = rnd(width, seed=4) * 0.3 + 1.0
        want = x.double() + mult * O.layer_norm(d.double(), w.double(), eps)
        xr = f32(x, be).clone()
        dd = d.to(be[0]) if delta_f32 else act(d, be)
        got = ops.post_layer_norm_add(xr, dd, f32(w, be), mult, eps, be[1])
        assert got.dtype == be[1]
        close(xr, want, be, bf16_tol=3e-3)
        close(got, want, be, bf16_tol=1e-2)

    @pytest.mark.parametrize("width", [24, 130, 2048])
    def test_final_norm_and_no_output(self, be, width):
        eps, mult, T = 1e-6, 1.4, 3
        x = rnd(T, width, seed=5, scale=2.0) - 1.5
        d = rnd(T, width, seed=6, dtype=be[1])
        w, wn = rnd(width, seed=7) + 1.0, rnd(width, seed=8) + 1.0
        new_x = x.double() + mult * O.layer_norm(d.double(), w.double(), eps)
        xr = f32(x, be).clone()
        got = ops.post_layer_norm_add(
            xr, act(d, be), f32(w, be), mult, eps, be[1], f32(wn, be)
        )
        close(xr, new_x, be, bf16_tol=1e-5)
        close(got, O.layer_norm(new_x, wn.double(), eps), be)
        xr2 = f32(x, be).clone()
        assert ops.post_layer_norm_add(
            xr2, act(d, be), f32(w, be), mult, eps, be[1], want_out=False
        ) is None
        close(xr2, new_x, be, bf16_tol=1e-5)
        # no delta: only the cast / the norm of the stream as it is
        xr3 = f32(x, be).clone()
        got = ops.post_layer_norm_add(xr3, None, None, mult, eps, be[1])
        close(got, x.double(), be, bf16_tol=5e-3)
        assert torch.equal(xr3.cpu(), x)
        got = ops.post_layer_norm_add(xr3, None, None, mult, eps, be[1], f32(wn, be))
        close(got, O.layer_norm(x.double(), wn.double(), eps), be)


def make_cache(blocks, bs, cols, be):
    return torch.full((blocks, 1, bs, cols), 7.0, dtype=be[1], device=be[0])


class TestLatentNormRopeCache:
    @pytest.mark.parametrize(
        "q_rank,kv_rank,rot_dim,rot_dims,extra",
        [(24, 16, 8, 8, 3), (100, 72, 20, 12, 0), (64, 40, 0, 0, 5),
         (300, 260, 64, 64, 8), (8, 8, 7, 4, 1)],
    )
    def test_against_oracle(self, be, q_rank, kv_rank, rot_dim, rot_dims, extra):
        eps, base, bs, T = 1e-5, 777.0, 8, 6
        cols = q_rank + kv_rank + rot_dim + extra
        proj = rnd(T, cols, seed=11, scale=2.0, dtype=be[1])
        qw, kw = rnd(q_rank, seed=12) + 1.0, rnd(kv_rank, seed=13) + 1.0
        pos = [0, 1, 2, 500, 31, 7]
        slots = [9, 17, -1, 3, 40, 8]  # scattered; one token is not cached
        inv = rotary_inv_freq(rot_dims, base) if rot_dims else None
        cache = make_cache(6, bs, kv_rank + rot_dim, be)
        got = ops.latent_norm_rope_cache(
            act(proj, be), q_rank, kv_rank, rot_dim, f32(qw, be), f32(kw, be),
            i64(pos, be), i32(slots, be), cache, eps,
            None if inv is None else inv.to(be[0]),
        )
        p = proj.double()
        close(got, O.rms_unit(p[:, :q_rank], eps) * qw.double(), be)
        c = O.rms_unit(p[:, q_rank : q_rank + kv_rank], eps) * kw.double()
        rows = c
        if rot_dim:
            kr = p[:, q_rank + kv_rank : q_rank + kv_rank + rot_dim]
            if rot_dims:
                kr = O.rotate_interleaved(kr, torch.tensor(pos), rot_dims, base)
            rows = torch.cat([c, kr], dim=-1)
        flat = cache.view(-1, kv_rank + rot_dim)
        for t, s in enumerate(slots):
            if s >= 0:
                close(flat[s], rows[t], be)
        untouched = [s for s in range(flat.shape[0]) if s not in slots]
        assert (flat[untouched] == 7.0).all()

    def test_query_side_only(self, be):
        proj = rnd(4, 40, seed=14, dtype=be[1])
        qw = rnd(32, seed=15) + 1.0
        got = ops.latent_norm_rope_cache(
            act(proj, be), 32, 0, 0, f32(qw, be), None, i64([0, 1, 2, 3], be),
            i32([0, 1, 2, 3], be), None, 1e-6, None,
        )
        close(got, O.rms_unit(proj.double()[:, :32], 1e-6) * qw.double(), be)


class TestHeadMatmulRope:
    @pytest.mark.parametrize(
        "T,H,K,N,tail,rot_dims",
        [(5, 3, 16, 24, 8, 8), (70, 2, 40, 300, 0, 0), (33, 5, 64, 96, 32, 32),
         (1, 4, 24, 70, 10, 6), (64, 1, 130, 64, 0, 0), (200, 3, 72, 100, 0, 0),
         (2100, 2, 128, 192, 64, 64), (130, 2, 20, 36, 4, 4), (300, 1, 96, 80, 0, 0)],
    )
    def test_against_oracle(self, be, T, H, K, N, tail, rot_dims):
        base = 5000.0
        x = rnd(T, H * (K + tail), seed=21, dtype=be[1])
        w = rnd(H, N, K, seed=22, scale=K ** -0.5, dtype=be[1])
        pos = torch.arange(T) * 37 % 257   # fp32 angles: keep them small
        inv = rotary_inv_freq(rot_dims, base) if rot_dims else None
        xh = x.double().view(T, H, K + tail)
        want = torch.einsum("thk,hnk->thn", xh[..., :K], w.double())
        if tail:
            tl = xh[..., K:]
            if rot_dims:
                tl = O.rotate_interleaved(
                    tl.transpose(0, 1), pos, rot_dims, base
                ).transpose(0, 1)
            want = torch.cat([want, tl], dim=-1)
        for out_dtype in (torch.float32, be[1]):
            got = ops.head_matmul_rope(
                act(x, be), act(w, be), H, tail, i64(pos, be),
                None if inv is None else inv.to(be[0]), out_dtype,
            )
            assert got.dtype == out_dtype and got.shape == (T, H * (N + tail))
            tol = 2e-2 if out_dtype == torch.bfloat16 else 2e-5
            close(got, want.reshape(T, -1), be, bf16_tol=tol)


def paged_rows(rows_per_seq, bs, be, cols, seed=0):
    """Scatter each sequence's rows over shuffled pages of one pool."""
    nb = [-(-r.shape[0] // bs) for r in rows_per_seq]
    total = sum(nb) + 3
    g = torch.Generator().manual_seed(seed)
    perm = (torch.randperm(total - 1, generator=g) + 1).tolist()
    cache = torch.full((total, 1, bs, cols), float("nan"), dtype=torch.float32)
    tables = torch.zeros(len(rows_per_seq), max(nb), dtype=torch.int32)
    for s, r in enumerate(rows_per_seq):
        for b in range(nb[s]):
            blk = perm.pop()
            tables[s, b] = blk
            part = r[b * bs : (b + 1) * bs]
            cache[blk, 0, : part.shape[0]] = part
    # junk (not NaN: masked lanes multiply by zero weights) in unused places
    cache = torch.where(torch.isnan(cache), torch.full_like(cache, 3.0), cache)
    return cache.to(be[1]).to(be[0]), tables.to(be[0])


def latent_rows_attention(qf, rows, vcols, scale, window, sink, gate, n_q):
    """The last n_q positions of one sequence: fp64 scores of folded queries
    qf [n_q, H, cols] against rows [ctx, cols], values rows[:, :vcols]."""
    ctx = rows.shape[0]
    sc = torch.einsum("thc,jc->htj", qf, rows) * scale
    mask = O.visible(ctx, window)[ctx - n_q :][None].expand(sc.shape)
    sk = None if sink is None else sink[:, None].expand(sc.shape[0], n_q)
    o = O.softmax_sink(sc, mask, sk) @ rows[:, :vcols]          # [H, n_q, vcols]
    if gate is not None:
        o = o * torch.sigmoid(gate).T[:, :, None]
    return o.transpose(0, 1).reshape(n_q, -1)


class TestLatentRowAttention:
    """ctx_attention_f32 as the latent mixers use it: one kv head, values a
    view of the leading columns of the keys."""

    def run(self, be, qs, rows, vcols, scale, window, bs, sink=None, gates=None):
        H = qs[0].shape[1]
        cols = rows[0].shape[1]
        cache, tables = paged_rows(rows, bs, be, cols)
        cu = [0]
        for q in qs:
            cu.append(cu[-1] + q.shape[0])
        qf = torch.cat([q.reshape(q.shape[0], -1) for q in qs])
        gate = None if gates is None else act(torch.cat(gates), be)
        got = ops.ctx_attention_f32(
            f32(qf, be), cache, cache[..., :vcols], tables, i32(cu, be),
            i32([r.shape[0] for r in rows], be), scale,
            max(q.shape[0] for q in qs), H, gate=gate, out_dtype=be[1],
            sink=None if sink is None else f32(sink, be), window=window,
        )
        want = torch.cat([
            latent_rows_attention(
                qs[s].double(), rows[s].to(be[1]).double(), vcols, scale, window,
                None if sink is None else sink.double(),
                None if gates is None else gates[s].to(be[1]).double(),
                qs[s].shape[0],
            )
            for s in range(len(qs))
        ])
        return got, want

    @pytest.mark.parametrize(
        "H,vcols,rot,window,bs",
        [(8, 96, 32, 40, 16), (4, 64, 0, 0, 16), (3, 40, 24, 16, 16),
         (16, 192, 64, 100, 64), (5, 72, 8, 7, 8), (2, 16, 16, 64, 32)],
    )
    def test_prompt_portions_and_decode_batched(self, be, H, vcols, rot, window, bs):
        cols = vcols + rot
        ctxs, nqs = [150, 70, 1, 33, 200], [150, 5, 1, 1, 1]
        rows = [rnd(c, cols, seed=30 + i) for i, c in enumerate(ctxs)]
        qs = [rnd(n, H, cols, seed=40 + i) for i, n in enumerate(nqs)]
        gates = [rnd(n, H, seed=50 + i) for i, n in enumerate(nqs)]
        sink = rnd(H, seed=60) if rot == 0 else None
        got, want = self.run(be, qs, rows, vcols, cols ** -0.5, window, bs, sink, gates)
        close(got, want, be)
        # decode only: one token per sequence
        qs1 = [q[-1:] for q in qs]
        g1 = [g[-1:] for g in gates]
        got, want = self.run(be, qs1, rows, vcols, cols ** -0.5, window, bs, sink, g1)
        close(got, want, be)

    @pytest.mark.parametrize("decode", [False, True])
    @pytest.mark.parametrize("window,bs", [(40, 16), (16, 16), (33, 64), (64, 8)])
    def test_needle_at_the_window_edge(self, be, window, bs, decode):
        """One key stands out by a scaled coordinate; its value is marked.
        The query window-1 positions after it must see it, the next not."""
        H, vcols, rot = 2, 32, 8
        cols, ctx = vcols + rot, 3 * max(window, bs) + 5
        for needle in (ctx - window, ctx - window - 1, 0 if ctx <= window else None):
            if needle is None:
                continue
            rows = rnd(ctx, cols, seed=71, scale=0.1)
            rows[needle, :vcols] = 0.0
            rows[needle, 0] = 5.0
            rows[needle, vcols:] = 3.0
            n_q = 1 if decode else 6
            q = rnd(n_q, H, cols, seed=72, scale=0.1)
            q[:, :, vcols:] = 4.0          # large score with the needle's key part
            got, want = self.run(be, [q], [rows], vcols, 1.0, window, bs)
            close(got, want, be)
            seen = got.float().cpu().view(n_q, H, vcols)[-1, :, 0]
            if needle == ctx - window:
                assert (seen > 4.0).all(), "the last key inside the window was lost"
            else:
                assert (seen.abs() < 1.0).all(), "a key outside the window was seen"

    @pytest.mark.parametrize("decode", [False, True])
    def test_far_key_without_window(self, be, decode):
        H, vcols = 4, 48
        ctx, needle = 1500, 3
        rows = rnd(ctx, vcols, seed=81, scale=0.1)
        rows[needle] = 0.0
        rows[needle, 5] = 6.0
        n_q = 1 if decode else 3
        q = rnd(n_q, H, vcols, seed=82, scale=0.1)
        q[:, :, 5] = 3.0
        sink = torch.tensor([-30.0, 0.0, 2.0, 30.0])
        got, want = self.run(be, [q], [rows], vcols, 1.0, 0, 16, sink)
        close(got, want, be)
        seen = got.float().cpu().view(n_q, H, vcols)[-1, :, 5]
        assert seen[0] > 5.0 and seen[3] < 0.1   # tiny sink / dominating sink

    def test_first_tokens(self, be):
        H, vcols, rot = 3, 24, 8
        for ctx in (1, 2, 3):
            rows = rnd(ctx, vcols + rot, seed=90 + ctx)
            q = rnd(ctx, H, vcols + rot, seed=95 + ctx)
            got, want = self.run(be, [q], [rows], vcols, 0.3, 2, 16)
            close(got, want, be)


class TestRouter:
    @pytest.mark.parametrize("R,top,W", [(6, 2, 32), (18, 2, 100), (70, 4, 64), (3, 3, 16), (5, 1, 48)])
    def test_softmax_with_correction(self, be, R, top, W):
        T = 9
        h = rnd(T, W, seed=101, dtype=be[1])
        router = rnd(R, W, seed=102, scale=W ** -0.5)
        corr = rnd(R, seed=103, scale=0.5)
        wd = {"router": router.double(), "correction": corr.double()}
        idx_w, wt_w = O.route(h.double(), wd, "", {"router": {"top": top}})
        idx, w, dw, lg = ops.route_tokens(
            act(h, be), f32(router, be), top, softmax=True, renorm=True,
            dense=True, want_logits=True, correction=f32(corr, be),
            renorm_eps=1e-20,
        )
        close(lg, h.double() @ router.double().T, be, bf16_tol=1e-5)
        got = {(t, int(e)): float(x) for t in range(T) for e, x in zip(idx[t].cpu(), w[t].cpu())}
        want = {(t, int(e)): float(x) for t in range(T) for e, x in zip(idx_w[t], wt_w[t])}
        assert got.keys() == want.keys()
        for k in want:
            assert abs(got[k] - want[k]) < 1e-5
        dense = torch.zeros(T, R, dtype=F64)
        dense.scatter_(1, idx_w, wt_w)
        close(dw, dense, be, bf16_tol=1e-5)

    def test_correction_changes_the_choice_not_the_weight(self, be):
        # scores favour output 0; the correction lifts output 2 above it
        h = torch.zeros(1, 8)
        h[0, 0] = 1.0
        router = torch.zeros(3, 8)
        router[:, 0] = torch.tensor([2.0, 1.0, 0.0])
        corr = torch.tensor([0.0, 0.0, 5.0])
        idx, w, _, _ = ops.route_tokens(
            act(h, be), f32(router, be), 1, softmax=True, renorm=False,
            correction=f32(corr, be),
        )
        s = torch.softmax(torch.tensor([2.0, 1.0, 0.0], dtype=F64), 0)
        assert int(idx[0, 0]) == 2
        assert abs(float(w[0, 0]) - float(s[2])) < 1e-6
        idx, w, _, _ = ops.route_tokens(
            act(h, be), f32(router, be), 1, softmax=True, renorm=True,
            correction=f32(corr, be), renorm_eps=1e-20,
        )
        assert int(idx[0, 0]) == 2 and abs(float(w[0, 0]) - 1.0) < 1e-6


class TestRows:
    @pytest.mark.parametrize("width", [20, 64, 260])
    def test_weighted_combine_with_scaled_rows(self, be, width):
        T, top = 7, 3
        y = rnd(T * top + 4, width, seed=111, dtype=be[1])
        g = torch.Generator().manual_seed(112)
        index = torch.randperm(T * top + 4, generator=g)[: T * top]
        wts = rnd(T * top, seed=113).abs()
        extra = rnd(T, width, seed=114, dtype=be[1])
        sc = rnd(T, width, seed=115, dtype=be[1])
        scw = rnd(T, seed=116)
        want = (y.double()[index] * wts.double()[:, None]).view(T, top, width).sum(1)
        got = ops.combine_rows(act(y, be), i32(index, be), top, None, f32(wts, be))
        close(got, want, be, bf16_tol=1e-5)
        want = want + extra.double() + sc.double() * scw.double()[:, None]
        got = ops.combine_rows(
            act(y, be), i32(index, be), top, act(extra, be), f32(wts, be),
            act(sc, be), f32(scw, be),
        )
        assert got.dtype == torch.float32
        close(got, want, be, bf16_tol=1e-5)

    def test_plain_gather(self, be):
        x = rnd(9, 50, seed=117, dtype=be[1])
        rows = [8, 0, 0, 3, 5]
        got = ops.gather_scale_rows(act(x, be), i32(rows, be))
        assert torch.equal(got.float().cpu(), x[rows])


class TestActivations:
    @pytest.mark.parametrize("rows,d", [(5, 24), (3, 100), (40, 512), (2, 7)])
    def test_glu_silu_scale(self, be, rows, d):
        x = rnd(rows, 2 * d, seed=121, scale=2.0, dtype=be[1])
        want = O.silu(x.double()[:, :d]) * x.double()[:, d:]
        close(ops.glu_silu_scale(act(x, be)), want, be)
        sc = rnd(rows, seed=122)
        sc[0] = 0.0
        got = ops.glu_silu_scale(act(x, be), f32(sc, be))
        close(got, want * sc.double()[:, None], be)
        assert (got[0] == 0).all()

    @pytest.mark.parametrize("rows,d", [(5, 24), (3, 100), (40, 512), (2, 7)])
    def test_bias_gelu_tanh(self, be, rows, d):
        x = rnd(rows, d, seed=123, scale=3.0, dtype=be[1])
        b = rnd(d, seed=124)
        close(
            ops.bias_gelu_tanh(act(x, be), f32(b, be)),
            O.gelu_tanh(x.double() + b.double()), be,
        )
