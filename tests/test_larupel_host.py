"""The Larupel design on the CPU: its configuration and what is refused, the run order and tensors
of a model whose layers lend keys and values, the states of the recurrent mixers, and the engine's
host logic (step function, cache, slots, batches) with the plain torch versions of the kernels put
in their place, against the plain whole-sequence implementation."""
import copy

import pytest
import torch

import larupel_configs as lc
import plain_larupel
import reference_ops
import traces
from helpers import compare, make_runner, prompts_for, random_weights, replay
from lucciola_amd import models  # noqa: F401  (registers the architectures)
from lucciola_amd.cache.manager import CacheManager
from lucciola_amd.cache.specs import CacheLayout, FixedStates, PagedKV
from lucciola_amd.config.engine_config import EngineConfig
from lucciola_amd.config.larupel_config import AttentionConfig, DeltaConfig, GeneralDeltaConfig, LarupelConfig
from lucciola_amd.config.model_config import ConfigError
from lucciola_amd.config.registry import architecture_for
from lucciola_amd.engine.batch import StepEntry
from lucciola_amd.engine.llm_engine import LLMEngine
from lucciola_amd.engine.loading import _build
from lucciola_amd.models.causal_lm import declared_tensors
from lucciola_amd.models.larupel import larupel_model_spec
from lucciola_amd.sampling.sampler import SamplingParams
from lucciola_amd.weights.loader import DictSource, ParamDecl, WeightsError, load_declared


def weights_of(cfg, seed, std=lc.STD):
    return random_weights(dict(cfg, initializer_range=std), seed)


def test_configuration_is_read_layer_by_layer():
    cfg = LarupelConfig.from_dict(lc.L_B)
    assert (cfg.vocab, cfg.width, cfg.norm_eps) == (131, 50, 3e-6)
    assert [l.type for l in cfg.layers] == ["delta", "attention", "general_delta", "attention", "attention",
                                            "general_delta", "attention"]
    assert isinstance(cfg.layers[0].mixer, DeltaConfig) and cfg.layers[0].mixer.conv == 2
    assert isinstance(cfg.layers[2].mixer, GeneralDeltaConfig) and (cfg.layers[2].mixer.heads, cfg.layers[2].mixer.dim) == (5, 6)
    assert isinstance(cfg.layers[1].mixer, AttentionConfig)
    assert [getattr(l.mixer, "kv_from", None) for l in cfg.layers] == [None, None, None, None, 1, None, 3]
    assert (cfg.layers[1].mixer.dim, cfg.layers[1].mixer.vdim, cfg.layers[1].mixer.scale) == (10, 6, 0.31)
    assert cfg.layers[0].mlp is None and cfg.layers[2].mlp.kind == "dense"
    assert (cfg.layers[1].mlp.experts, cfg.layers[1].mlp.top, cfg.layers[1].mlp.ff, cfg.layers[1].mlp.shared.ff) == (5, 1, 30, 22)
    assert cfg.layers[4].mlp.shared is None
    assert architecture_for(lc.L_B).name == "Larupel"


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="convolution"), "not a mixer"),
    (lambda c: c["layers"][0]["mixer"].pop("conv"), "conv"),
    (lambda c: c["layers"][1]["mixer"].update(heads=4, kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=4), "earlier"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=2), "attention layer"),
    (lambda c: c["layers"][6]["mixer"].update(kv_from=4), "of its own"),
    (lambda c: c["layers"][4]["mixer"].update(kv_from=3), "keeps"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "exceeds"),
    (lambda c: c["layers"][2]["mlp"].update(kind="gated"), "neither"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
])
def test_configuration_refuses(change, message):
    cfg = copy.deepcopy(lc.L_B)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        LarupelConfig.from_dict(cfg)


def test_run_order_and_tensors():
    spec = larupel_model_spec(LarupelConfig.from_dict(lc.L_B))
    assert [e.layer for e in spec.run_order] == list(range(7))
    assert [e.cache_of for e in spec.run_order] == [None, None, None, None, 1, None, 3]
    assert [l.block for l in spec.layers] == ["sandwich_mixer", "sandwich_residual", "sandwich_residual", "sandwich_mixer",
                                              "sandwich_residual", "sandwich_residual", "sandwich_residual"]
    names = declared_tensors(spec)
    assert names["embed"].shape == (131, 50) and names["head"].shape == (131, 50)
    assert names["final.norm.b"].shape == (50,) and names["l0.norm1b.b"].shape == (50,)
    assert "l0.norm2" not in names and "l0.mlp.gate" not in names
    # the gated delta rule: 3 kv heads of 7, 3 heads of 9, two taps
    assert names["l0.mix.q"].shape == (21, 50) and names["l0.mix.q.conv"].shape == (21, 2)
    assert names["l0.mix.v"].shape == (27, 50) and names["l0.mix.v.conv"].shape == (27, 2)
    assert names["l0.mix.b"].shape == (3, 50) and names["l0.mix.A_log"].shape == (3,) and names["l0.mix.norm"].shape == (9,)
    # attention: values shorter than keys; the lent layer has queries and an output of its own only
    assert names["l1.mix.q"].shape == (30, 50) and names["l1.mix.k"].shape == (10, 50) and names["l1.mix.v"].shape == (6, 50)
    assert names["l1.mix.o"].shape == (50, 18) and names["l1.mix.temp"].shape == (3,) and names["l1.mix.k.norm"].shape == (10,)
    assert "l4.mix.k" not in names and "l4.mix.v" not in names and "l4.mix.k.norm" not in names
    assert names["l4.mix.q.norm"].shape == (10,) and names["l4.mix.temp"].shape == (3,)
    # the generalized delta rule: the decay's inner size is the checkpoint's
    assert names["l2.mix.w1"].shape == (-1, 50) and names["l2.mix.w2"].shape == (30, -1) and names["l2.mix.a.b"].shape == (30,)
    assert names["l2.mix.norm"].shape == (30,) and names["l2.mix.r"].shape == (30, 50)
    # experts, router with bias, shared expert and its gate
    assert names["l1.mlp.e4.gate"].shape == (30, 50) and names["l1.mlp.router.b"].shape == (5,)
    assert names["l1.mlp.shared.up"].shape == (22, 50) and names["l1.mlp.shared.sg"].shape == (1, 50)
    assert "l4.mlp.shared.sg" not in names and names["l2.mlp.down"].shape == (50, 70)


def test_a_size_that_the_checkpoint_decides():
    decl = {"w": ParamDecl((-1, 4)), "u": ParamDecl((3, -1))}
    got = load_declared(DictSource({"w": torch.zeros(7, 4), "u": torch.zeros(3, 2)}), decl, torch.device("cpu"))
    assert got["w"].shape == (7, 4) and got["u"].shape == (3, 2)
    with pytest.raises(WeightsError, match="wrong shape"):
        load_declared(DictSource({"w": torch.zeros(7, 5), "u": torch.zeros(3, 2)}), decl, torch.device("cpu"))
    assert ParamDecl((-1, 4), free_size=9).concrete_shape() == (9, 4)


def test_states_and_pages_of_a_model():
    """Recurrent layers take a slot's worth of float32 state and no pages; attention layers that
    keep equal heads share a block table; a layer that reads another's keys keeps nothing."""
    cfg = lc.L_B
    weights = weights_of(cfg, 1)
    arch = architecture_for(cfg)
    model = _build(arch.model_spec(arch.read_config(cfg)), DictSource(weights), "float32", "cpu")
    needs = model.site_needs()
    assert needs[4] is None and needs[6] is None
    assert needs[0] == FixedStates(((3, 9, 7), (1, 69))) and needs[2] == FixedStates(((5, 6, 6),))
    assert isinstance(needs[1], PagedKV) and needs[1].head_dim == 32 and needs[3].num_kv_heads == 2
    cache = CacheManager(needs, block_size=4, num_blocks=10, max_seqs=3)
    assert len(cache.groups) == 2 and cache.has_fixed_state
    assert cache.state_bytes() == 3 * 4 * (3 * 7 * 9 + 69 + 5 * 6 * 6 + 20 * 20)
    state, tail = needs[0].allocate(CacheLayout(10, 4, 4, 3), torch.float32, "cpu")
    assert state.shape == (3, 3, 9, 7) and tail.shape == (3, 1, 69)
    state.fill_(5.0)
    tail.fill_(5.0)
    needs[0].start((state, tail), 1)
    assert float(state[1].abs().sum()) == 0 and float(tail[1].abs().sum()) == 0 and float(state[0, 0, 0, 0]) == 5.0


@pytest.mark.parametrize("key", ["A", "B", "C"])
@pytest.mark.parametrize("family", ["whole", "tail", "chunked", "mixed"])
def test_step_function_matches_plain(monkeypatch, key, family):
    reference_ops.install(monkeypatch)
    cfg, page, seed = lc.ALL[key]
    weights = weights_of(cfg, seed)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, {"A": [1, 12, 45], "B": [2, 40, 21], "C": [30, 9]}[key], seed)
    steps = {"whole": traces.whole, "tail": traces.tail_decode, "chunked": traces.chunked,
             "mixed": traces.mixed}[family](prompts)
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, "float32", "cpu", max_seqs=3)
    got = replay(runner, steps)
    refs = {n: plain_larupel.forward(cfg, weights, ids) for n, ids in prompts.items()}
    compare(got, cfg, weights, prompts, 5e-5, refs)
    assert not runner.cache.requests
    for g in runner.cache.groups:
        assert g.pool.num_free() == blocks


def test_stream_after_every_layer(monkeypatch):
    reference_ops.install(monkeypatch)
    cfg, page, seed = lc.ALL["B"]
    weights = weights_of(cfg, seed)
    ids = prompts_for({"vocab_size": cfg["vocab"]}, [19], seed)["r0"]
    want = []
    plain_larupel.forward(cfg, weights, ids, streams=want)
    runner = make_runner(cfg, weights, page, 8, "float32", "cpu")
    seen = []
    for layer in runner.model.layers:
        block, inner = layer.block, layer.block.forward

        def spy(stream, site, inner=inner):
            inner(stream, site)
            seen.append((stream.h + stream.pending.value().to(torch.float32)).double().clone())
        block.forward = spy
    runner.step([StepEntry("r", ids, [len(ids) - 1])])
    assert len(seen) == len(want) == 7
    for got, ref in zip(seen, want):
        assert float((got - ref).abs().max()) < 2e-5 * float(ref.abs().max())


def test_a_slot_that_is_used_again_starts_from_zero(monkeypatch):
    """One slot: every request finds the state and the convolutions' inputs of the one before it
    in its slot, and must not see them."""
    reference_ops.install(monkeypatch)
    cfg, page, seed = lc.ALL["A"]
    weights = weights_of(cfg, seed)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [14, 9, 11], seed)
    refs = {n: plain_larupel.forward(cfg, weights, ids) for n, ids in prompts.items()}
    runner = make_runner(cfg, weights, page, 2, "float32", "cpu", max_seqs=1)
    got = replay(runner, traces.chunked(prompts, sizes=(3, 2, 5)))
    compare(got, cfg, weights, prompts, 5e-5, refs)


def test_a_step_that_fails_leaves_the_states_reachable(monkeypatch):
    """A batch that does not fit changes nothing: the requests go on as if it had not been tried."""
    from lucciola_amd.cache.page_pool import OutOfPages
    reference_ops.install(monkeypatch)
    cfg, page, seed = lc.ALL["A"]
    weights = weights_of(cfg, seed)
    ids = prompts_for({"vocab_size": cfg["vocab"]}, [30], seed)["r0"]
    ref = plain_larupel.forward(cfg, weights, ids)
    runner = make_runner(cfg, weights, page, 2, "float32", "cpu", max_seqs=2)
    runner.step([StepEntry("a", ids[:20], [])])
    with pytest.raises(OutOfPages):
        runner.step([StepEntry("a", ids[20:], [9]), StepEntry("b", ids, [0])])
    logits = runner.step([StepEntry("a", ids[20:], [9])])
    assert float((logits[0].double() - ref[29]).abs().max()) < 5e-5 * float(ref[29].abs().max())


def test_greedy_generation_through_the_scheduler(monkeypatch):
    reference_ops.install(monkeypatch)
    cfg, page, seed = lc.ALL["A"]
    weights = weights_of(cfg, seed, std=0.2)
    arch = architecture_for(cfg)
    config = arch.read_config(cfg)
    model = _build(arch.model_spec(config), DictSource(weights), "float32", "cpu")
    engine = LLMEngine(model, config, EngineConfig(dtype="float32", block_size=page, max_blocks=40, max_seqs=3,
                                                   max_tokens_per_step=9, device="cpu", run_ahead=False))
    prompts = list(prompts_for({"vocab_size": cfg["vocab"]}, [4, 13, 27], seed + 1).values())
    got = engine.generate(prompts, SamplingParams(max_new_tokens=5))
    assert got == [plain_larupel.greedy(cfg, weights, p, 5) for p in prompts]
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


def test_the_bench_configurations_are_models_of_the_design():
    """What ``bench.py --workload designs`` builds for this design reads as a configuration, with the
    sizes of the model beside it."""
    import importlib.util
    import os
    spec = importlib.util.spec_from_file_location("bench", os.path.join(os.path.dirname(os.path.dirname(
        os.path.abspath(__file__))), "bench.py"))
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    for name, (width, heads, ff) in bench.DESIGN_SIZES.items():
        for routed in (True, False):
            cfg = LarupelConfig.from_dict(bench.larupel_design_config(name, routed=routed))
            assert (cfg.width, cfg.vocab, len(cfg.layers)) == (width, bench.DESIGN_VOCAB, bench.DESIGN_LAYERS)
            assert [l.type for l in cfg.layers] == ["attention", "general_delta", "delta", "attention"]
            assert cfg.layers[3].mixer.kv_from == 0 and cfg.layers[0].mixer.heads == heads
            assert [l.mlp.kind for l in cfg.layers] == (["dense", "moe", "moe", "dense"] if routed else ["dense"] * 4)
            declared_tensors(larupel_model_spec(cfg))
