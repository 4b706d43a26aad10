"""The hybrid (state-space + attention) decoder through the engine, against
the float64 oracle in hybrid_oracle.py.

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
import hybrid_oracle as O  # noqa: E402

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


def two_kinds_config(**kw):
    """A state-space layer, a parallel layer with a feed-forward, another
    state-space layer with different sizes and a feed-forward."""
    return O.make_config(
        layers=[
            O.mamba_layer(heads=4, vdim=8, state=16, groups=2, conv=4, norm_groups=2),
            O.parallel_layer(
                left=O.attn_cfg(heads=4, kv_heads=2, dim=16, vdim=8, scale=0.3,
                                coef=0.7, every=5),
                right=O.ssm_cfg(heads=2, vdim=24, state=20, groups=1, conv=3,
                                norm_groups=1),
                mlp=O.dense_mlp(ff=40, limit=0.9),
            ),
            O.mamba_layer(heads=6, vdim=4, state=40, groups=3, conv=2,
                          norm_groups=4, mlp=O.dense_mlp(ff=24, limit=2.5)),
        ],
        **kw,
    )


def make_engine(cfg, sd, backend, num_blocks=64, block_size=16, max_seqs=4,
                eager=False, multi_step=1, max_len=512, batched_tokens=None,
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
    dt = torch.bfloat16 if backend[1] == "bfloat16" else torch.float32
    return O.random_weights(cfg, seed=seed, dtype=dt)


def rel_err(got, want):
    """Centered RMS difference over the vocabulary, relative to the RMS of
    the expected logits."""
    got, want = got.double().cpu(), want.double()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    scale = (want - want.mean(-1, keepdim=True)).pow(2).mean().sqrt()
    return (d.pow(2).mean(-1).sqrt() / scale).max().item()


def tol(backend):
    # bf16: worst position of a few hundred, inputs and products rounded
    return 6e-2 if backend[1] == "bfloat16" else 2e-4


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
        cfg = two_kinds_config()
        sd = weights_for(cfg, backend)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(37, cfg["vocab"], 1)
        res = []
        want = O.forward(cfg, sd, toks, res)
        eng.model.debug_residuals = []
        got = run_schedule(eng, [toks], [[(0, len(toks))]])[0]
        streams = eng.model.debug_residuals
        eng.model.debug_residuals = None
        assert rel_err(got, want) < tol(backend)
        assert len(streams) == len(cfg["layers"])
        for mine, ref in zip(streams, res):
            scale = ref.abs().max().item()
            assert (mine.double().cpu() - ref).abs().max().item() < tol(backend) * 4 * scale

    def test_first_tokens(self, backend):
        """Prompts of 1, 2 and 3 tokens: shorter than every convolution, all
        history before position 0 is zero."""
        cfg = two_kinds_config()
        sd = weights_for(cfg, backend, seed=3)
        eng = make_engine(cfg, sd, backend)
        for n in (1, 2, 3):
            toks = random_prompt(n, cfg["vocab"], 10 + n)
            got = run_schedule(eng, [toks], [[(0, n)]])[0]
            assert rel_err(got, O.forward(cfg, sd, toks)) < tol(backend)

    def test_sizes_equal_to_one(self, backend):
        """Single heads, one group, one tap, no temperature."""
        left = O.attn_cfg(heads=1, kv_heads=1, dim=8, vdim=24, scale=0.5)
        del left["q_temp"]
        cfg = O.make_config(
            vocab=31, width=24, emb_scale=1.0,
            layers=[
                O.parallel_layer(
                    left=left,
                    right=O.ssm_cfg(heads=1, vdim=16, state=8, groups=1, conv=1,
                                    norm_groups=1),
                    left_scale=1.0, right_scale=1.0,
                ),
                O.mamba_layer(heads=2, vdim=8, state=17, groups=1, conv=5, norm_groups=1),
            ],
        )
        sd = weights_for(cfg, backend, seed=4)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(21, cfg["vocab"], 5)
        got = run_schedule(eng, [toks], [[(0, 21)]])[0]
        assert rel_err(got, O.forward(cfg, sd, toks)) < tol(backend)


class TestSchedules:
    def test_prefill_then_decode(self, backend):
        cfg = two_kinds_config()
        sd = weights_for(cfg, backend, seed=5)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(70, cfg["vocab"], 6)
        want = O.forward(cfg, sd, toks)
        sched = [[(0, 30)]] + [[(0, 1)] for _ in range(40)]
        got = run_schedule(eng, [toks], sched)[0]
        assert rel_err(got, want) < tol(backend)

    def test_decode_steps_without_readback(self, backend):
        """Decode steps whose logits nobody reads must still run on their own
        inputs: only every 7th step is read back (the runner's staging
        buffers are refilled right behind the previous step's copies)."""
        cfg = two_kinds_config()
        sd = weights_for(cfg, backend, seed=16)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(90, cfg["vocab"], 17)
        want = O.forward(cfg, sd, toks)
        rp = TraceReplayer(eng)
        rp.step([{"id": "a", "tokens": toks[:20], "want": []}], [])
        got, rows = [], []
        for p in range(20, 90):
            read = p % 7 == 0 or p == 89
            out = rp.step([{"id": "a", "tokens": [toks[p]], "want": [0] if read else []}],
                          ["a"] if p == 89 else [])
            assert (out is not None) == read
            if read:
                got.append(out.float().cpu())
                rows.append(p)
        assert rel_err(torch.cat(got), want[rows]) < tol(backend)

    def test_token_by_token_from_the_start(self, backend):
        cfg = two_kinds_config()
        sd = weights_for(cfg, backend, seed=6)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(20, cfg["vocab"], 7)
        got = run_schedule(eng, [toks], [[(0, 1)] for _ in toks])[0]
        assert rel_err(got, O.forward(cfg, sd, toks)) < tol(backend)

    @pytest.mark.parametrize("sizes", [[2] * 20, [3, 17, 2, 16, 1, 5, 2, 2, 31],
                                       [16, 16, 16, 1, 15, 2, 14]])
    def test_portions(self, backend, sizes):
        """Portions down to two tokens, cut inside pages and shorter than the
        convolutions' history."""
        cfg = two_kinds_config()
        sd = weights_for(cfg, backend, seed=7)
        eng = make_engine(cfg, sd, backend)
        toks = random_prompt(sum(sizes), cfg["vocab"], 8)
        got = run_schedule(eng, [toks], [[(0, n)] for n in sizes])[0]
        assert rel_err(got, O.forward(cfg, sd, toks)) < tol(backend)

    def test_mixed_batches_and_reuse(self, backend):
        """Unequal requests side by side — portions next to decode tokens,
        requests skipped for a step — in a pool too small for all of them at
        once, so pages and state slots are handed out again."""
        cfg = two_kinds_config()
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
            assert rel_err(got[i], O.forward(cfg, sd, toks)) < tol(backend), i
        bm = eng.scheduler.block_manager
        assert bm.num_free_blocks == 9
        assert eng.scheduler.state_slots.num_free == 3

    def test_alone_equals_batched(self, backend):
        cfg = two_kinds_config()
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
            assert rel_err(together[i], alone.double()) < tol(backend) / 4

    def test_long_decode(self, backend):
        cfg = O.make_config(
            vocab=50, width=32,
            layers=[
                O.parallel_layer(
                    left=O.attn_cfg(heads=2, kv_heads=1, dim=8, vdim=16, every=64),
                    right=O.ssm_cfg(heads=2, vdim=8, state=8, groups=1, conv=4),
                ),
            ],
        )
        sd = weights_for(cfg, backend, seed=10)
        eng = make_engine(cfg, sd, backend, num_blocks=32)
        toks = random_prompt(300, cfg["vocab"], 11)
        got = run_schedule(eng, [toks], [[(0, 4)]] + [[(0, 1)]] * 296)[0]
        assert rel_err(got, O.forward(cfg, sd, toks)) < tol(backend)


class TestFarKeys:
    """One attention layer whose weights make a single early key decide the
    output: a key lost at a page border or cut off by a tile shows at once."""

    def _needle_setup(self, backend, page_pos, total):
        left = O.attn_cfg(heads=2, kv_heads=1, dim=8, vdim=8, scale=4.0, coef=0.0,
                          every=1000)
        cfg = O.make_config(
            vocab=40, width=16, emb_scale=10.0,
            layers=[O.parallel_layer(
                left=left,
                right=O.ssm_cfg(heads=1, vdim=8, state=4, groups=1, conv=2, norm_groups=1),
                left_scale=1.0, right_scale=0.0)],
        )
        sd = weights_for(cfg, backend, seed=12)
        # Token 1 is the needle. Every other embedding is made orthogonal to
        # its direction d; key row 0 reads d, the query is a constant that
        # reads key entry 0: the needle's score stands ~20 above all others.
        d = sd["embed"][1] / sd["embed"][1].norm()
        for j in range(cfg["vocab"]):
            if j != 1:
                sd["embed"][j] -= (sd["embed"][j] @ d) * d
        p = "l0.mix.left."
        sd[p + "q"].zero_()
        sd[p + "q.b"].zero_()
        sd[p + "q.b"][0] = sd[p + "q.b"][8] = 1.0
        sd[p + "k"][0] = 3.0 * d
        sd[p + "k.b"].zero_()
        sd[p + "q.norm"].fill_(1.0)
        sd[p + "k.norm"].fill_(1.0)
        sd["l0.norm1"].zero_()
        dt = torch.bfloat16 if backend[1] == "bfloat16" else torch.float32
        sd = {k: v.to(dt).float() for k, v in sd.items()}
        toks = [2 + (i % 30) for i in range(total)]
        toks[page_pos] = 1
        return cfg, sd, toks

    @pytest.mark.parametrize("page_pos", [0, 15, 16, 63, 64, 65, 127, 128])
    def test_needle_in_prompt_and_decode(self, backend, page_pos):
        cfg, sd, toks = self._needle_setup(backend, page_pos, 200)
        want = O.forward(cfg, sd, toks)
        plain = list(toks)
        plain[page_pos] = 3
        # the needle matters: without it the last logits move visibly
        assert rel_err(O.forward(cfg, sd, plain)[-1:], want[-1:]) > 0.2
        eng = make_engine(cfg, sd, backend, num_blocks=32)
        got = run_schedule(eng, [toks], [[(0, 150)]] + [[(0, 1)]] * 50)[0]
        assert rel_err(got, want) < tol(backend)


class TestGeneration:
    def test_greedy_through_scheduler(self, backend):
        """LLMEngine.generate: the scheduler's own prefill/decode batching,
        sampling, preemption-free pool."""
        cfg = two_kinds_config()
        sd = weights_for(cfg, backend, seed=13)
        eng = make_engine(cfg, sd, backend, multi_step=4)
        prompts = [random_prompt(n, cfg["vocab"], 60 + n) for n in (5, 19, 11)]
        outs = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=12,
                                                     ignore_eos=True))
        assert len(outs) == 3
        for p, o in zip(prompts, outs.values()):
            assert len(o.output_token_ids) == 12
            if backend[1] == "bfloat16":
                continue  # near-ties may flip; the logits are checked above
            seq = list(p)
            for t in o.output_token_ids:
                logits = O.forward(cfg, sd, seq)[-1]
                top2 = logits.topk(2).values
                if (top2[0] - top2[1]).item() > 1e-3:
                    assert int(logits.argmax()) == t
                seq.append(t)

    def test_mixed_batches_in_the_scheduler(self, backend):
        """With a token budget that admits one prompt per step, running
        requests ride along with the next prompt's prefill; the tokens are
        the same as without riders."""
        cfg = two_kinds_config()
        sd = weights_for(cfg, backend, seed=18)
        prompts = [random_prompt(n, cfg["vocab"], 90 + n) for n in (20, 18, 21)]
        sp = SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True)
        plain = make_engine(cfg, sd, backend, batched_tokens=24).generate(prompts, sp)
        eng = make_engine(cfg, sd, backend, batched_tokens=24, mixed=True)
        seen = []
        inner = eng.runner.execute_prefill

        def spy(batch, bm, logit_rows=None):
            seen.append(sorted(batch.num_scheduled_tokens))
            return inner(batch, bm, logit_rows=logit_rows)

        eng.runner.execute_prefill = spy
        mixed = eng.generate(prompts, sp)
        assert any(b[0] == 1 and b[-1] > 1 for b in seen), seen
        if backend[1] == "float32":
            for a, b in zip(plain.values(), mixed.values()):
                assert a.output_token_ids == b.output_token_ids

    def test_chunked_admission_and_preemption(self, backend):
        """A pool that cannot hold all requests: the scheduler preempts, the
        state slot goes back with the pages and the request restarts from
        position 0 with the same result."""
        cfg = two_kinds_config()
        sd = weights_for(cfg, backend, seed=14)
        prompts = [random_prompt(n, cfg["vocab"], 80 + n) for n in (30, 28, 25)]
        sp = SamplingParams(temperature=0.0, max_tokens=20, ignore_eos=True)
        roomy = make_engine(cfg, sd, backend, num_blocks=64).generate(prompts, sp)
        tight = make_engine(cfg, sd, backend, num_blocks=8, max_seqs=3).generate(prompts, sp)
        if backend[1] == "float32":
            for a, b in zip(roomy.values(), tight.values()):
                assert a.output_token_ids == b.output_token_ids


class TestConfigAndRegistry:
    def test_config_json_roundtrip(self, tmp_path):
        from kserve_amd.models.registry import load_model_config, native_modules_for

        cfg = two_kinds_config()
        (tmp_path / "config.json").write_text(json.dumps(cfg))
        mc = load_model_config(str(tmp_path))
        assert isinstance(mc, HybridModelConfig)
        assert [l.kind for l in mc.layers] == ["mamba2", "parallel", "mamba2"]
        assert mc.layers[1].attention.q_temp_every == 5
        assert mc.layers[2].mlp.limit == 2.5 and mc.layers[0].mlp is None
        assert native_modules_for(str(tmp_path)) == ("kserve_amd_seq_C",)

    def test_server_cli_picks_the_engine(self, tmp_path):
        from kserve_amd.runtimes.huggingfaceserver import detect_backend

        (tmp_path / "config.json").write_text(json.dumps(two_kinds_config()))
        assert detect_backend(str(tmp_path)) == "engine"

    def test_unknown_layer_type_is_refused(self):
        cfg = two_kinds_config()
        cfg["layers"][0]["type"] = "something-else"
        with pytest.raises(ValueError):
            HybridModelConfig.from_dict(cfg)

    def test_llama_config_still_resolves(self, tmp_path):
        from kserve_amd.engine.config import ModelConfig
        from kserve_amd.models.registry import load_model_config

        (tmp_path / "config.json").write_text(json.dumps({
            "model_type": "llama", "vocab_size": 64, "hidden_size": 32,
            "intermediate_size": 64, "num_hidden_layers": 1,
            "num_attention_heads": 2,
        }))
        assert isinstance(load_model_config(str(tmp_path)), ModelConfig)

    def test_checkpoint_loading_from_safetensors(self, tmp_path):
        from safetensors.torch import save_file

        from kserve_amd.engine.weights import load_safetensors_weights

        cfg = two_kinds_config()
        sd = O.random_weights(cfg, seed=15, dtype=torch.bfloat16)
        save_file({k: v.to(torch.bfloat16) for k, v in sd.items()},
                  str(tmp_path / "model.safetensors"))
        mc = HybridModelConfig.from_dict(cfg)
        mc.dtype = "float32"
        model = build_model(mc, device="cpu")
        load_safetensors_weights(model, str(tmp_path))
        assert torch.equal(model.layers[1].ssm.a_log, sd["l1.mix.right.A_log"])
        a = model.layers[1].attn.proj_width
        assert torch.equal(model.layers[1].fused_proj[a:], sd["l1.mix.right.in"])


class TestStateSlots:
    def test_slot_lifecycle(self):
        from kserve_amd.engine.state_manager import StateSlotManager

        m = StateSlotManager(4)
        a, b, c = m.allocate("a"), m.allocate("b"), m.allocate("c")
        assert sorted((a, b, c)) == [1, 2, 3] and m.num_free == 0
        assert m.allocate("a") == a
        with pytest.raises(RuntimeError):
            m.allocate("d")
        m.free("b")
        assert m.allocate("d") == b
        m.free("zzz")  # unknown ids are ignored

    def test_scheduler_waits_for_a_slot(self):
        from kserve_amd.engine.request import Request
        from kserve_amd.engine.scheduler import Scheduler

        s = Scheduler(SchedulerConfig(max_num_seqs=8, max_num_batched_tokens=64,
                                      max_model_len=64),
                      CacheConfig(block_size=16), 32, num_state_slots=3)
        reqs = [Request(f"r{i}", [1, 2, 3], SamplingParams(max_tokens=4)) for i in range(3)]
        for r in reqs:
            s.add_request(r)
        batch = s.schedule()
        assert [r.request_id for r in batch.requests] == ["r0", "r1"]
        assert {r.state_slot for r in batch.requests} == {1, 2}
        for r in batch.requests:
            r.num_computed_tokens = 3
        s.finish_requests([reqs[0]])
        batch = s.schedule()
        assert batch.is_prefill and batch.requests[0].request_id == "r2"
        assert batch.requests[0].state_slot == 1
