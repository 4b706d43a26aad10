"""Each mechanism of the 32-bit-residual / recurrent-state family alone:
``kserve_amd.ops`` against the float64 oracle functions of hybrid_oracle.py.

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
import hybrid_oracle as O  # noqa: E402

from kserve_amd import ops  # noqa: E402

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
    """Tensor in the activation dtype on the device."""
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


def layout(lens, starts):
    """Flat-batch tensors for portions of ``lens`` tokens starting at
    absolute positions ``starts``."""
    cu, seq, pos = [0], [], []
    for s, (n, p0) in enumerate(zip(lens, starts)):
        cu.append(cu[-1] + n)
        seq += [s] * n
        pos += list(range(p0, p0 + n))
    return cu, seq, pos


class TestEmbedding:
    @pytest.mark.parametrize("width", [16, 50, 256])
    def test_scaled_embedding_with_sinusoid(self, be, width):
        table = rnd(33, width, seed=1, dtype=be[1])
        toks = [3, 0, 32, 7, 7, 19]
        pos = [0, 1, 2, 500, 1001, 4095]
        from kserve_amd.ops.torch_ref import sinusoid_inv_freq

        got = ops.embed_scale_sinpos(
            act(table, be), i64(toks, be), i64(pos, be),
            sinusoid_inv_freq(width).to(be[0]), 2.5,
        )
        want = torch.zeros(len(toks), width, dtype=F64)
        for r, (t, p) in enumerate(zip(toks, pos)):
            for i in range(width):
                ang = p * 10000.0 ** (-(2 * (i // 2)) / width)
                want[r, i] = table[t, i].double() * 2.5 + (
                    math.cos(ang) if i % 2 else math.sin(ang)
                )
        assert got.dtype == torch.float32
        # fp32 angles at position ~4000 carry ~2e-4 absolute error
        close(got, want, be, f32_tol=3e-4, bf16_tol=3e-4)


class TestNorms:
    @pytest.mark.parametrize("width", [24, 256, 1000])
    def test_add_then_offset_norm(self, be, width):
        x = rnd(5, width, seed=2, scale=3.0)
        d0 = rnd(5, width, seed=3, dtype=be[1])
        d1 = rnd(5, width, seed=4, dtype=be[1])
        w = rnd(width, seed=5, scale=0.2)
        res = f32(x, be).clone()
        out = ops.add_rms_norm_f32res(
            res, f32(w, be), 1e-5, 1.0, be[1], act(d0, be), 0.7, act(d1, be), 1.4
        )
        summed = x.double() + 0.7 * d0.double() + 1.4 * d1.double()
        close(res, summed, be, bf16_tol=1e-5)  # the stream itself stays fp32
        close(out, O.offset_norm(summed, w.double(), 1e-5), be)

    def test_norm_without_delta_and_plain_weight(self, be):
        x = rnd(3, 40, seed=6)
        w = rnd(40, seed=7) + 1.0
        res = f32(x, be).clone()
        out = ops.add_rms_norm_f32res(res, f32(w, be), 1e-3, 0.0, be[1])
        close(res, x, be, bf16_tol=1e-7)
        close(out, O.rms(x.double(), 1e-3) * w.double(), be)

    @pytest.mark.parametrize("inner,groups", [(48, 1), (48, 3), (320, 5)])
    def test_gated_group_norm(self, be, inner, groups):
        y = rnd(4, inner, seed=8, scale=2.0)
        wide = rnd(4, inner + 9, seed=9, dtype=be[1])  # z is a column slice
        z = wide[:, 5 : 5 + inner]
        w = rnd(inner, seed=10) + 1.0
        got = ops.gated_group_rms_norm(
            f32(y, be), act(wide, be)[:, 5 : 5 + inner], f32(w, be), 1e-5, groups, be[1]
        )
        v = y.double() * O.silu(z.double())
        want = O.rms(v.reshape(4, groups, -1), 1e-5).reshape(4, inner) * w.double()
        close(got, want, be)


class TestClampedGLU:
    def test_branches_and_limits(self, be):
        x = rnd(6, 2 * 50, seed=11, scale=3.0, dtype=be[1])
        got = ops.clamped_swiglu(act(x, be), 1.702, 1.5)
        g = x[:, :50].double().clamp(max=1.5)
        u = x[:, 50:].double().clamp(-1.5, 1.5)
        want = g / (1 + torch.exp(-1.702 * g)) * (u + 1)
        # both clamps and the unclamped negative gate branch are exercised
        assert (x[:, :50] > 1.5).any() and (x[:, :50] < -1.5).any()
        assert (x[:, 50:] > 1.5).any() and (x[:, 50:] < -1.5).any()
        close(got, want, be)


class TestCausalConv:
    @pytest.mark.parametrize("taps", [1, 2, 4, 7])
    def test_portions_match_whole_sequence(self, be, taps):
        C, T = 37, 23
        wide = rnd(T, C + 6, seed=12, dtype=be[1])
        u = wide[:, 4 : 4 + C]
        w = rnd(C, taps, seed=13, scale=0.5)
        b = rnd(C, seed=14, scale=0.1)
        want = O.silu(O.causal_conv(u.double(), w.double(), b.double()))
        hist = max(taps - 1, 1)
        # the slot's old content is junk: a start at position 0 must ignore it
        state = torch.full((3, hist, C), 77.0).to(be[1]).to(be[0])
        dev_in = act(wide, be)[:, 4 : 4 + C]
        outs, at = [], 0
        for n in (1, 2, 1, 5, 2, 12):
            cu, seq, pos = layout([n], [at])
            outs.append(
                ops.causal_conv_silu(
                    dev_in[at : at + n], f32(w, be), f32(b, be), state,
                    i64(pos, be), i32(seq, be), i32(cu, be), i32([2], be),
                )
            )
            at += n
        close(torch.cat(outs), want, be)

    def test_batch_of_unequal_sequences(self, be):
        C, taps = 20, 4
        w = rnd(C, taps, seed=15, scale=0.5)
        b = rnd(C, seed=16, scale=0.1)
        seqs = [rnd(n, C, seed=20 + n, dtype=be[1]) for n in (9, 3, 14)]
        state = torch.zeros(4, taps - 1, C).to(be[1]).to(be[0])
        slots = [3, 1, 2]
        # first portions of different sizes, then the rest, as one batch each
        cuts = [4, 1, 11]
        got = [[], [], []]
        for part in (0, 1):
            chunks = [s[:c] if part == 0 else s[c:] for s, c in zip(seqs, cuts)]
            starts = [0 if part == 0 else c for c in cuts]
            cu, seq, pos = layout([len(c) for c in chunks], starts)
            out = ops.causal_conv_silu(
                act(torch.cat(chunks), be), f32(w, be), f32(b, be), state,
                i64(pos, be), i32(seq, be), i32(cu, be), i32(slots, be),
            )
            for s in range(3):
                got[s].append(out[cu[s] : cu[s + 1]])
        for s in range(3):
            want = O.silu(O.causal_conv(seqs[s].double(), w.double(), b.double()))
            close(torch.cat(got[s]), want, be)


class TestScan:
    @pytest.mark.parametrize(
        "H,G,P,N",
        [(2, 1, 4, 8), (4, 2, 24, 17), (6, 3, 16, 48), (3, 3, 70, 100), (2, 1, 8, 130)],
    )
    def test_portions_match_whole_sequence(self, be, H, G, P, N):
        T = 19
        inner = H * P
        xbc = rnd(T, inner + 2 * G * N, seed=30, scale=0.7)
        wide = rnd(T, H + 3, seed=31, dtype=be[1])
        dt_raw = wide[:, 2 : 2 + H]
        dt_bias = rnd(H, seed=32) - 1.0
        a_log = rnd(H, seed=33, scale=0.5)
        d_skip = rnd(H, seed=34)
        dt = O.softplus(dt_raw.double() + dt_bias.double())
        want = O.ssd(
            xbc[:, :inner].double().reshape(T, H, P),
            xbc[:, inner : inner + G * N].double().reshape(T, G, N),
            xbc[:, inner + G * N :].double().reshape(T, G, N),
            dt, a_log.double(), d_skip.double(), G,
        ).reshape(T, inner)
        state = torch.full((3, H, P, N), 5.0, device=be[0])  # junk in the slot
        dev_dt = act(wide, be)[:, 2 : 2 + H]
        outs, at = [], 0
        for n in (2, 1, 1, 7, 8):
            cu, _, pos = layout([n], [at])
            outs.append(
                ops.ssd_scan(
                    f32(xbc[at : at + n], be), dev_dt[at : at + n], f32(dt_bias, be),
                    f32(a_log, be), f32(d_skip, be), state, i64(pos, be),
                    i32(cu, be), i32([1], be), G,
                )
            )
            at += n
        close(torch.cat(outs), want, be, f32_tol=5e-5, bf16_tol=5e-5)

    def test_large_step_sizes_are_not_clamped(self, be):
        """softplus of a large argument is the argument itself."""
        H, P, N, T = 1, 4, 8, 3
        xbc = rnd(T, H * P + 2 * N, seed=35)
        dt_raw = torch.full((T, H), 40.0)
        state = torch.zeros(2, H, P, N, device=be[0])
        cu, _, pos = layout([T], [0])
        got = ops.ssd_scan(
            f32(xbc, be), act(dt_raw, be), f32(torch.zeros(H), be),
            f32(torch.tensor([-6.0]), be), f32(torch.ones(H), be), state,
            i64(pos, be), i32(cu, be), i32([1], be), 1,
        )
        want = O.ssd(
            xbc[:, :P].double().reshape(T, H, P), xbc[:, P : P + N].double().reshape(T, 1, N),
            xbc[:, P + N :].double().reshape(T, 1, N), dt_raw.double(),
            torch.tensor([-6.0], dtype=F64), torch.ones(H, dtype=F64), 1,
        ).reshape(T, H * P)
        close(got, want, be, f32_tol=5e-5, bf16_tol=5e-5)


def oracle_attention(q, k, v, gate, qw, kw, eps, scale, coef, every, H, G, D, DV, start):
    """q/k/v rows of one sequence from position 0; returns rows >= start."""
    T = q.shape[0]
    qn = O.rms(q.double(), eps) * qw.double()
    kn = O.rms(k.double(), eps) * kw.double()
    out = torch.zeros(T, H * DV, dtype=F64)
    for t in range(start, T):
        temp = 1.0 + coef * math.log((t + 1) // every + 1) if every else 1.0
        for h in range(H):
            g = h // (H // G)
            sc = (kn[: t + 1, g * D : (g + 1) * D] @ (qn[t, h * D : (h + 1) * D] * temp)) * scale
            wgt = torch.softmax(sc, 0)
            o = wgt @ v[: t + 1, g * DV : (g + 1) * DV].double()
            out[t, h * DV : (h + 1) * DV] = o / (1 + math.exp(-gate[t, h].item()))
    return out[start:]


class TestAttention:
    @pytest.mark.parametrize(
        "H,G,D,DV,bs",
        [(4, 2, 16, 8, 16), (6, 1, 64, 64, 16), (5, 5, 40, 72, 8),
         (32, 1, 8, 200, 32), (8, 4, 128, 128, 16)],
    )
    def test_paged_varlen_prefill_and_decode(self, be, H, G, D, DV, bs):
        """Two sequences with scattered pages: a portion onto existing
        context beside a fresh prompt, then one decode token each."""
        eps, scale, coef, every = 1e-5, 0.2, 0.6, 7
        lens = [70, 29]
        qw, kw = rnd(H * D, seed=40) + 1.0, rnd(G * D, seed=41) + 1.0
        width = H * D + G * D + G * DV + H
        proj = [rnd(n, width, seed=42 + n, dtype=be[1]) for n in lens]
        a, b, c = H * D, H * D + G * D, H * D + G * D + G * DV
        want = [
            oracle_attention(p[:, :a], p[:, a:b], p[:, b:c], p[:, c:], qw, kw, eps,
                             scale, coef, every, H, G, D, DV, 0)
            for p in proj
        ]
        nblocks = 24
        kc = torch.zeros(nblocks, G, bs, D).to(be[1]).to(be[0])
        vc = torch.zeros(nblocks, G, bs, DV).to(be[1]).to(be[0])
        perm = torch.randperm(nblocks - 1, generator=torch.Generator().manual_seed(1)) + 1
        per = -(-max(lens) // bs)
        tables = [perm[:per].tolist(), perm[per : 2 * per].tolist()]
        bt = i32(tables, be)

        def run(portions):
            """portions: per sequence (lo, hi) rows to feed now."""
            rows = torch.cat([proj[s][lo:hi] for s, (lo, hi) in enumerate(portions)])
            cu, _, pos = layout([hi - lo for lo, hi in portions], [lo for lo, _ in portions])
            slots = [
                tables[s][p // bs] * bs + p % bs
                for s, (lo, hi) in enumerate(portions) for p in range(lo, hi)
            ]
            dev = act(rows, be)
            qn = ops.qk_norm_temp_cache(
                dev[:, :a], dev[:, a:b], dev[:, b:c], f32(qw, be), f32(kw, be),
                i64(pos, be), i32(slots, be), kc, vc, eps, coef, every, H,
            )
            out = ops.ctx_attention_f32(
                qn, kc, vc, bt, i32(cu, be), i32([hi for _, hi in portions], be),
                scale, max(hi - lo for lo, hi in portions), H, gate=dev[:, c:],
                out_dtype=be[1],
            )
            return [out[cu[s] : cu[s + 1]] for s in range(len(portions))]

        first = run([(0, 33), (0, 28)])
        second = run([(33, 69), (28, 29)])       # portion beside one decode token
        third = run([(69, 70), (29, 29)])[0]     # decode alone (second seq idle)
        close(torch.cat([first[0], second[0], third]), want[0], be)
        close(torch.cat([first[1], second[1]]), want[1], be)

    def test_far_key_across_many_tiles(self, be):
        """Decode against 1000 keys where only key 3 matters."""
        H, G, D, DV, bs, T = 2, 1, 8, 8, 16, 1000
        k = torch.zeros(T, D)
        k[:, 1] = 1.0
        k[3] = torch.tensor([4.0] + [0.0] * (D - 1))
        v = rnd(T, DV, seed=50)
        nb = -(-T // bs)
        kc = torch.zeros(nb + 1, G, bs, D)
        vc = torch.zeros(nb + 1, G, bs, DV)
        for p in range(T):
            kc[1 + p // bs, 0, p % bs] = k[p]
            vc[1 + p // bs, 0, p % bs] = v[p]
        q = torch.zeros(1, H * D)
        q[0, 0] = q[0, D] = 5.0
        out = ops.ctx_attention_f32(
            f32(q, be), act(kc, be), act(vc, be), i32([list(range(1, nb + 1))], be),
            i32([0, 1], be), i32([T], be), 1.0, 1, H, out_dtype=be[1],
        )
        sc = k.double() @ q[0, :D].double()
        want = torch.softmax(sc, 0) @ v.to(be[1]).double()
        close(out[0, :DV], want, be)
        close(out[0, DV:], want, be)
        assert (want - v.to(be[1])[3].double()).abs().max() < 1e-3
