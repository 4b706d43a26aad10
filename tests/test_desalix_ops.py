"""Each mechanism of the Desalix design alone: ``kserve_amd.ops`` against the
float64 oracle functions of desalix_oracle.py.

Parametrised over the CPU forms (always) and the HIP kernels in both
activation dtypes (marked gpu). Inputs are rounded to the activation dtype
first, so the oracle and the op see the same numbers.
"""

import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import desalix_oracle as O  # noqa: E402

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
    return torch.tensor(v, dtype=torch.int32, device=be[0])


def i64(v, be):
    return torch.tensor(v, dtype=torch.int64, device=be[0])


def close(got, want, be, f32_tol=2e-5, bf16_tol=2e-2):
    tol = bf16_tol if be[1] == torch.bfloat16 else f32_tol
    got, want = got.double().cpu(), want.double()
    scale = max(want.abs().max().item(), 1e-6)
    err = (got - want).abs().max().item() / scale
    assert err < tol, f"relative error {err:.3g} (tolerance {tol})"


class TestEmbedding:
    @pytest.mark.parametrize("width", [16, 50, 256])
    def test_scaled_embedding_without_positions(self, be, width):
        table = rnd(37, width, seed=1, dtype=be[1])
        toks = [3, 0, 36, 3, 17]
        got = ops.embed_scale_sinpos(
            act(table, be), i64(toks, be), i64([0, 1, 2, 900, 4], be), None, 0.37
        )
        assert got.dtype == torch.float32
        close(got, table.double()[toks] * 0.37, be, bf16_tol=1e-6)


class TestSandwichNorm:
    @pytest.mark.parametrize("width", [16, 50, 192, 1028])
    @pytest.mark.parametrize("delta_f32", [False, True])
    def test_close_and_open(self, be, width, delta_f32):
        eps, gb, gn = 1e-5, 1.3, 0.8
        T = 5
        x = rnd(T, width, seed=2, scale=3.0)
        d = rnd(T, width, seed=3, scale=0.2, dtype=torch.float32 if delta_f32 else be[1])
        ls = rnd(width, seed=4) * 0.3 + 0.5
        rows, vec = rnd(T, width, seed=5), rnd(width, seed=6)
        want_x = (
            x.double()
            + O.scalar_norm(d.double(), torch.tensor(gb), eps) * ls.double()
            + rows.double() + vec.double()
        )
        want_h = O.scalar_norm(want_x, torch.tensor(gn), eps)
        res = f32(x, be).clone()
        dd = f32(d, be) if delta_f32 else act(d, be)
        got = ops.post_norm_add_rms_norm(
            res, dd, gb, f32(ls, be), eps, gn, be[1], f32(rows, be), f32(vec, be)
        )
        assert got.dtype == be[1] and res.dtype == torch.float32
        close(res, want_x, be, bf16_tol=2e-5)  # the stream itself stays fp32
        close(got, want_h, be)

    def test_parts_are_optional(self, be):
        eps = 1e-6
        x = rnd(3, 24, seed=7)
        res = f32(x, be).clone()
        got = ops.post_norm_add_rms_norm(res, None, 1.0, None, eps, 1.7, be[1])
        close(res, x, be, bf16_tol=1e-7)
        close(got, O.scalar_norm(x.double(), torch.tensor(1.7), eps), be)
        d = rnd(3, 24, seed=8, dtype=be[1])
        ls = rnd(24, seed=9)
        none = ops.post_norm_add_rms_norm(
            res, act(d, be), 0.9, f32(ls, be), eps, 1.0, be[1], want_out=False
        )
        assert none is None
        close(res, x.double() + O.scalar_norm(d.double(), torch.tensor(0.9), eps)
              * ls.double(), be, bf16_tol=2e-5)

    def test_tiny_delta_is_still_unit_size(self, be):
        """The post-norm divides by the delta's own RMS: a sublayer output of
        1e-3 adds as much as one of size 1 (eps is far below it)."""
        x = torch.zeros(2, 32)
        d = rnd(2, 32, seed=10, dtype=be[1]) * 1e-3
        d = d.to(be[1]).float()
        res = f32(x, be).clone()
        ops.post_norm_add_rms_norm(
            res, act(d, be), 1.0, f32(torch.ones(32), be), 1e-12, 1.0, be[1],
            want_out=False,
        )
        rms = res.double().cpu().pow(2).mean(-1).sqrt()
        assert (rms - 1.0).abs().max() < 1e-3


class TestRouter:
    @pytest.mark.parametrize("E,top", [(4, 1), (8, 2), (70, 4), (130, 7), (5, 5)])
    def test_sigmoid_scores_as_they_are(self, be, E, top):
        T = 9
        h = rnd(T, 20, seed=11)
        wr = rnd(E, 20, seed=12, scale=0.6)
        idx_w, w_w = O.route(h.double(), wr, top)
        logits = f32(h @ wr.T, be)
        idx, w, dense = ops.router_topk(logits, top, dense=True)
        assert idx.dtype == torch.int32 and w.dtype == torch.float32
        assert torch.equal(idx.cpu().long(), idx_w)
        close(w, w_w, be, bf16_tol=2e-5)
        want_dense = torch.zeros(T, E, dtype=F64).scatter_(1, idx_w, w_w)
        close(dense, want_dense, be, bf16_tol=2e-5)
        assert ops.router_topk(logits, top)[2] is None

    @pytest.mark.parametrize("E,top,W", [(4, 1, 20), (8, 2, 2048), (70, 4, 50),
                                         (130, 7, 260), (1, 1, 8)])
    def test_fused_logits_and_choice(self, be, E, top, W):
        """The router's own matrix product in 32-bit, then the choice."""
        T = 11
        h = rnd(T, W, seed=21, dtype=be[1])
        wr = rnd(E, W, seed=22, scale=2.0 * W ** -0.5)
        idx_w, w_w = O.route(h.double(), wr, top)
        idx, w, dense, logits = ops.route_tokens(
            act(h, be), f32(wr, be), top, dense=True, want_logits=True
        )
        close(logits, h.double() @ wr.double().T, be, bf16_tol=2e-5)
        # inputs are already rounded, so the choice may only differ where two
        # scores are equal to within fp32
        s = torch.sigmoid(h.double() @ wr.double().T)
        picked = s.gather(1, idx.cpu().long())
        assert (picked - w_w).abs().max() < 1e-5
        close(w, w_w, be, bf16_tol=2e-5)
        close(dense.sum(-1), w_w.sum(-1), be, bf16_tol=2e-5)
        out = ops.route_tokens(act(h, be), f32(wr, be), top)
        assert out[2] is None and out[3] is None
        assert torch.equal(out[0].cpu(), idx.cpu())

    def test_softmax_renormalised(self, be):
        z = rnd(6, 10, seed=13, scale=2.0)
        idx, w, _ = ops.router_topk(f32(z, be), 3, softmax=True, renorm=True)
        p = torch.softmax(z.double(), -1)
        pw, pi = p.topk(3, -1)
        assert torch.equal(idx.cpu().long(), pi)
        close(w, pw / pw.sum(-1, keepdim=True), be, bf16_tol=2e-5)


class TestExpertRows:
    def test_gather_scale_and_combine(self, be):
        T, W, top = 7, 40, 3
        h = rnd(T, W, seed=14, dtype=be[1])
        rows = [6, 0, 0, 3, 5, 2]
        sc = rnd(len(rows), seed=15)
        got = ops.gather_scale_rows(act(h, be), i32(rows, be), f32(sc, be))
        assert got.dtype == be[1]
        close(got, h.double()[rows] * sc.double()[:, None], be)
        y = rnd(T * top, W, seed=16, dtype=be[1])
        perm = torch.randperm(T * top, generator=torch.Generator().manual_seed(2))
        extra = rnd(T, W, seed=17, dtype=be[1])
        out = ops.combine_rows(act(y, be), perm.to(torch.int32).to(be[0]), top,
                               act(extra, be))
        want = y.double()[perm].view(T, top, W).sum(1) + extra.double()
        assert out.dtype == torch.float32
        close(out, want, be, bf16_tol=2e-5)
        out = ops.combine_rows(act(y, be), perm.to(torch.int32).to(be[0]), top)
        close(out, want - extra.double(), be, bf16_tol=2e-5)

    def test_clamped_expert_activation(self, be):
        x = rnd(5, 48, seed=18, scale=2.0, dtype=be[1])
        g = x[:, :24].double().clamp(max=0.8)
        u = x[:, 24:].double().clamp(-0.8, 0.8)
        close(ops.clamped_swiglu(act(x, be), 1.702, 0.8),
              g * torch.sigmoid(1.702 * g) * (u + 1.0), be)


def oracle_attention(q, k, v, qw, kw, sink, eps, scale, H, G, D, DV, n_rot, base,
                     chunk):
    """Whole sequence from position 0: q [T, H*D], k [T, G*D], v [T, G*DV]."""
    T = q.shape[0]
    pos = torch.arange(T)
    qn = O.rms_unit(q.double().view(T, H, D), eps) * qw.double()
    kn = O.rms_unit(k.double().view(T, G, D), eps) * kw.double()
    qn = O.rotate_halves(qn, pos, n_rot, base)
    kn = O.rotate_halves(kn, pos, n_rot, base)
    vn = O.rotate_halves(O.rms_unit(v.double().view(T, G, DV), eps), pos, DV, base)
    kn = kn.repeat_interleave(H // G, dim=1)
    vn = vn.repeat_interleave(H // G, dim=1)
    sc = torch.einsum("ihd,jhd->hij", qn, kn) * scale
    vis = O.chunk_visible(T, chunk) if chunk else O.chunk_visible(T, 1 << 30)
    w = O.sink_softmax(sc, vis, sink.double())
    o = torch.einsum("hij,jhd->ihd", w, vn)
    return O.rotate_halves(o, pos, DV, base, sign=-1.0).reshape(T, H * DV)


class PagedAttention:
    """Two-kernel attention sublayer on scattered pages."""

    def __init__(self, be, H, G, D, DV, bs, n_rot, base, chunk, nblocks, tables,
                 eps=1e-5, scale=0.2):
        self.be, self.H, self.G, self.D, self.DV, self.bs = be, H, G, D, DV, bs
        self.eps, self.scale, self.chunk = eps, scale, chunk
        self.kc = torch.zeros(nblocks, G, bs, D).to(be[1]).to(be[0])
        self.vc = torch.zeros(nblocks, G, bs, DV).to(be[1]).to(be[0])
        self.tables = tables
        self.qk_f = rotary_inv_freq(n_rot, base).to(be[0]) if n_rot else None
        self.v_f = rotary_inv_freq(DV, base).to(be[0])

    def run(self, proj, portions, qw, kw, sink):
        """portions: per sequence (lo, hi) rows of proj[s] to feed now."""
        be, H, G, D, DV, bs = self.be, self.H, self.G, self.D, self.DV, self.bs
        a, b = H * D, H * D + G * D
        rows = torch.cat([proj[s][lo:hi] for s, (lo, hi) in enumerate(portions)])
        cu, pos, slots = [0], [], []
        for s, (lo, hi) in enumerate(portions):
            cu.append(cu[-1] + hi - lo)
            pos += list(range(lo, hi))
            slots += [self.tables[s][p // bs] * bs + p % bs for p in range(lo, hi)]
        dev = act(rows, be)
        qn = ops.qk_headnorm_rope_cache(
            dev[:, :a], dev[:, a:b], dev[:, b:], f32(qw, be), f32(kw, be),
            i64(pos, be), i32(slots, be), self.kc, self.vc, self.eps, H,
            self.qk_f, True, self.v_f,
        )
        out = ops.ctx_attention_f32(
            qn, self.kc, self.vc, i32(self.tables, be), i32(cu, be),
            i32([hi for _, hi in portions], be), self.scale,
            max(hi - lo for lo, hi in portions), H, out_dtype=be[1],
            sink=f32(sink, be), chunk=self.chunk, out_inv_freq=self.v_f,
        )
        return [out[cu[s] : cu[s + 1]] for s in range(len(portions))]


class TestChunkSinkAttention:
    @pytest.mark.parametrize(
        "H,G,D,DV,bs,n_rot,chunk",
        [(4, 2, 16, 8, 16, 8, 8), (6, 2, 64, 32, 16, 16, 48), (5, 5, 40, 72, 8, 40, 20),
         (16, 1, 8, 200, 32, 0, 50), (8, 4, 128, 128, 16, 64, 37),
         (3, 1, 24, 16, 16, 24, 0)],
    )
    def test_paged_varlen_prefill_and_decode(self, be, H, G, D, DV, bs, n_rot, chunk):
        """Two sequences with scattered pages: a portion onto existing
        context beside a fresh prompt, then one decode token each."""
        base = 50.0
        lens = [150, 29]
        qw, kw = rnd(D, seed=40) * 0.3 + 1.0, rnd(D, seed=41) * 0.3 + 1.0
        sink = rnd(H, seed=39)
        width = H * D + G * D + G * DV
        proj = [rnd(n, width, seed=42 + n, dtype=be[1]) for n in lens]
        a, b = H * D, H * D + G * D
        want = [
            oracle_attention(p[:, :a], p[:, a:b], p[:, b:], qw, kw, sink, 1e-5, 0.2,
                             H, G, D, DV, n_rot, base, chunk)
            for p in proj
        ]
        nblocks = 48
        perm = torch.randperm(nblocks - 1, generator=torch.Generator().manual_seed(1)) + 1
        per = -(-max(lens) // bs)
        tables = [perm[:per].tolist(), perm[per : 2 * per].tolist()]
        att = PagedAttention(be, H, G, D, DV, bs, n_rot, base, chunk, nblocks, tables)
        first = att.run(proj, [(0, 71), (0, 28)], qw, kw, sink)
        second = att.run(proj, [(71, 149), (28, 29)], qw, kw, sink)
        third = att.run(proj, [(149, 150), (29, 29)], qw, kw, sink)[0]
        close(torch.cat([first[0], second[0], third]), want[0], be)
        close(torch.cat([first[1], second[1]]), want[1], be)

    @pytest.mark.parametrize("chunk,bs", [(16, 16), (24, 16), (64, 8), (100, 32)])
    def test_needle_at_the_chunk_edge(self, be, chunk, bs):
        """One key carries a huge score for every query. Queries of the
        needle's own chunk (from the needle on) return its value; the first
        query of the next chunk must not see it. Checked with the queries
        in a prompt portion and decoded one at a time."""
        H, G, D, DV = 2, 1, 8, 8
        needle = 2 * chunk - 1                      # last position of chunk 1
        T = 2 * chunk + 3
        k = torch.zeros(T, D)
        k[:, 1] = 1.0
        k[needle] = torch.tensor([30.0] + [0.0] * (D - 1))
        q = torch.zeros(T, H * D)
        q[:, 0] = q[:, D] = 1.0
        v = rnd(T, DV, seed=50)
        proj = [torch.cat([q, k, v], dim=1).to(be[1]).float()]
        qw = kw = torch.ones(D)
        sink = torch.full((H,), -30.0)
        want = oracle_attention(q, k, proj[0][:, H * D + D :], qw, kw, sink, 1e-6,
                                4.0, H, G, D, DV, 0, 10.0, chunk)
        # sanity of the construction itself
        vn = O.rms_unit(proj[0][:, H * D + D :].double().view(T, 1, DV), 1e-6)
        assert (want[needle, :DV] - vn[needle, 0]).abs().max() < 1e-6
        assert (want[needle + 1, :DV] - vn[needle + 1, 0]).abs().max() < 1e-6
        nb = -(-T // bs)
        tables = [list(range(nb, 0, -1))]
        for split in (T, needle - 1):               # whole prompt / then decode
            att = PagedAttention(be, H, G, D, DV, bs, 0, 10.0, chunk, nb + 1, tables,
                                 eps=1e-6, scale=4.0)
            outs = [att.run(proj, [(0, split)], qw, kw, sink)[0]]
            for p in range(split, T):
                outs.append(att.run(proj, [(p, p + 1)], qw, kw, sink)[0])
            close(torch.cat(outs), want, be)

    def test_far_key_inside_a_long_chunk(self, be):
        """Decode against 1000 keys of one chunk where only key 3 matters."""
        H, G, D, DV, bs, T = 2, 1, 8, 8, 16, 1000
        k = torch.zeros(T, D)
        k[:, 1] = 1.0
        k[3] = torch.tensor([4.0] + [0.0] * (D - 1))
        q = torch.zeros(T, H * D)
        q[:, 0] = q[:, D] = 5.0
        v = rnd(T, DV, seed=51)
        proj = [torch.cat([q, k, v], dim=1).to(be[1]).float()]
        qw = kw = torch.ones(D)
        sink = torch.full((H,), -20.0)
        want = oracle_attention(q, k, proj[0][:, H * D + D :], qw, kw, sink, 1e-6,
                                1.0, H, G, D, DV, 0, 10.0, 2048)
        nb = -(-T // bs)
        att = PagedAttention(be, H, G, D, DV, bs, 0, 10.0, 2048, nb + 1,
                             [list(range(1, nb + 1))], eps=1e-6, scale=1.0)
        out = att.run(proj, [(0, T - 1)], qw, kw, sink)[0]
        last = att.run(proj, [(T - 1, T)], qw, kw, sink)[0]
        close(torch.cat([out, last])[4:], want[4:], be)

    def test_sink_takes_weight_but_gives_nothing(self, be):
        """With a sink far above every score the output goes to zero; with
        a sink far below it the sink changes nothing."""
        H, G, D, DV, bs, T = 2, 2, 8, 8, 16, 20
        proj = [rnd(T, H * D + G * D + G * DV, seed=52, dtype=be[1])]
        qw = kw = torch.ones(D)
        tables = [[2, 1]]
        outs = {}
        for name, s in (("high", 40.0), ("low", -40.0), ("mixed", None)):
            sink = torch.tensor([40.0, -40.0]) if s is None else torch.full((H,), s)
            att = PagedAttention(be, H, G, D, DV, bs, 4, 10.0, 8, 3, tables)
            outs[name] = att.run(proj, [(0, T)], qw, kw, sink)[0].float().cpu()
        assert outs["high"].abs().max() < 1e-6
        assert outs["low"].abs().max() > 0.1
        assert torch.equal(outs["mixed"][:, :DV], outs["high"][:, :DV])
        assert torch.equal(outs["mixed"][:, DV:], outs["low"][:, DV:])

    def test_value_rotation_cancels_for_a_single_key(self, be):
        """Position 0 of every chunk sees only itself: rotating its value by
        its position and turning the output back must give the unit-norm
        value times its softmax weight, whatever the position."""
        H, G, D, DV, bs, chunk, T = 1, 1, 8, 12, 8, 5, 23
        proj = [rnd(T, D + D + DV, seed=53, dtype=be[1])]
        qw = kw = torch.ones(D)
        sink = torch.full((H,), -50.0)
        att = PagedAttention(be, H, G, D, DV, bs, 8, 7.0, chunk, 4, [[3, 1, 2]])
        out = att.run(proj, [(0, T)], qw, kw, sink)[0]
        vn = O.rms_unit(proj[0][:, 2 * D :].double(), 1e-5)
        first = list(range(0, T, chunk))
        close(out[first], vn[first], be)


class TestLargerShapes:
    """Head sizes, group sizes and lengths of a real model's layers."""

    def test_long_prompts_with_wide_heads(self, be):
        H, G, D, DV, bs, n_rot, chunk = 16, 4, 128, 128, 16, 64, 1024
        base = 500000.0
        lens = [2100, 130]
        qw, kw = rnd(D, seed=60) * 0.3 + 1.0, rnd(D, seed=61) * 0.3 + 1.0
        sink = rnd(H, seed=62)
        width = H * D + G * D + G * DV
        proj = [rnd(n, width, seed=63 + n, dtype=be[1]) for n in lens]
        a, b = H * D, H * D + G * D
        want = [
            oracle_attention(p[:, :a], p[:, a:b], p[:, b:], qw, kw, sink, 1e-5,
                             D ** -0.5, H, G, D, DV, n_rot, base, chunk)
            for p in proj
        ]
        per = -(-max(lens) // bs)
        nblocks = 2 * per + 1
        perm = torch.randperm(nblocks - 1, generator=torch.Generator().manual_seed(3)) + 1
        tables = [perm[:per].tolist(), perm[per : 2 * per].tolist()]
        att = PagedAttention(be, H, G, D, DV, bs, n_rot, base, chunk, nblocks, tables,
                             scale=D ** -0.5)
        first = att.run(proj, [(0, 2048), (0, 100)], qw, kw, sink)
        outs0, outs1 = [first[0]], [first[1]]
        for p in range(2048, 2100):             # both decode, the second ends early
            hi1 = min(100 + p - 2047, 130)
            lo1 = min(100 + p - 2048, 130)
            o = att.run(proj, [(p, p + 1), (lo1, hi1)], qw, kw, sink)
            outs0.append(o[0])
            outs1.append(o[1])
        # angles are 32-bit: at position 2000 one ulp of the angle is 1e-4
        close(torch.cat(outs0), want[0], be, f32_tol=3e-4)
        close(torch.cat(outs1), want[1][:130], be, f32_tol=3e-4)
