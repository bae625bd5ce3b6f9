"""The Pubodra design on the GPU: every kernel it brought against the plain torch version of the
same operation, and the engine against the plain whole-sequence implementation
(``plain_pubodra``) in the four families of traces, in float32 and in bfloat16."""
import pytest
import torch

import plain_pubodra
import pubodra_configs
import reference_ops
import traces
from helpers import compare, make_runner, prompts_for, random_weights, replay
from lucciola_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {"float32": 2e-5, "bfloat16": 4e-2}
LENGTHS = {"A": [5, 1, 47, 90, 130], "B": [2, 61, 33, 100], "C": [150, 9, 230, 70]}
_cache = {}


def case(key):
    if key not in _cache:
        cfg, page, seed = pubodra_configs.ALL[key]
        weights = random_weights(cfg, seed, std=pubodra_configs.STD)
        prompts = prompts_for({"vocab_size": cfg["vocab"]}, LENGTHS[key], seed)
        refs = {n: plain_pubodra.forward(cfg, weights, ids) for n, ids in prompts.items()}
        _cache[key] = (cfg, page, weights, prompts, refs)
    return _cache[key]


def close(got, want, dtype, what, terms=1):
    """``terms``: how many times longer the sums are than the few hundred terms the bounds are set for
    (float32 rounding grows with the length of a sum)."""
    tol = (3e-6 if dtype == torch.float32 else 1.2e-2) * max(1.0, terms) ** 0.5
    err = float((got.double() - want.double()).abs().max() / want.double().abs().max().clamp_min(1e-9))
    assert err < tol, f"{what}: relative error {err:.3e}"


# ------------------------------------------------------------------ kernels alone
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,rows", [(50, None), (192, None), (1030, [3, 0, 3])])
def test_dynamic_tanh(dtype, n, rows):
    g = torch.Generator().manual_seed(n)
    h = torch.randn(5, n, generator=g) * 3
    delta = torch.randn(5, n, generator=g).to(dtype)
    w, b = torch.randn(n, generator=g), torch.randn(n, generator=g)
    idx = torch.tensor(rows, dtype=torch.int32) if rows else None
    h_ref = h.clone()
    want = reference_ops.dynamic_tanh(h_ref, delta, w, b, 0.7, dtype, idx)
    h_dev = h.to(DEV)
    got = ops.dynamic_tanh(h_dev, delta.to(DEV), w.to(DEV), b.to(DEV), 0.7, dtype, idx.to(DEV) if rows else None)
    close(got.cpu(), want, dtype, "dynamic tanh")
    assert torch.equal(h_dev.cpu(), h_ref), "the stream after the addition"


def test_stream_add_and_activations():
    g = torch.Generator().manual_seed(1)
    h, delta, vec = torch.randn(7, 33, generator=g), torch.randn(7, 33, generator=g).bfloat16(), torch.randn(33, generator=g)
    want = h.clone()
    reference_ops.stream_add(want, delta, vec)
    got = h.to(DEV)
    ops.stream_add(got, delta.to(DEV), vec.to(DEV))
    assert torch.allclose(got.cpu(), want, atol=1e-6)
    for kind in ops.ACTIVATIONS:
        for dtype in (torch.float32, torch.bfloat16):
            x = (torch.randn(11, 37, generator=g) * 3).to(dtype)
            want = reference_ops.activation(x.clone(), kind)
            close(ops.activation(x.to(DEV), kind).cpu(), want, dtype, kind)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,G,N,K,pad_x,gap", [(1, 3, 21, 7, 5, 2), (16, 2, 64, 32, 5, 2), (77, 5, 18, 300, 5, 2),
                                                  (130, 1, 100, 9, 5, 2),
                                                  # whole 16-byte pieces: in bfloat16 the bfloat16 matrix instruction
                                                  (3, 4, 96, 32, 8, 8), (70, 3, 40, 136, 16, 0), (200, 2, 130, 512, 0, 64),
                                                  (1300, 16, 1100, 40, 0, 8)])     # many tiles: 128 x 128
def test_grouped_product_over_heads(dtype, rows, G, N, K, pad_x, gap):
    g = torch.Generator().manual_seed(rows * 7 + G)
    pad_o = 3
    x = torch.randn(rows, pad_x + G * (K + gap), generator=g).to(dtype)
    w = torch.randn(G, N, K, generator=g).bfloat16()
    gate = torch.randn(rows, G * N + 4, generator=g).to(dtype)
    for use_gate, act in ((False, None), (True, None), (False, "relu_squared")):
        out_ref = torch.zeros(rows, pad_o + G * N, dtype=dtype)
        out_dev = torch.zeros(rows, pad_o + G * N, dtype=dtype, device=DEV)
        gate_ref = ops.Strided(gate, 4, N) if use_gate else None
        gate_dev = ops.Strided(gate.to(DEV), 4, N) if use_gate else None
        reference_ops.grouped_gemm(ops.Strided(x, pad_x, K + gap), w, ops.Strided(out_ref, pad_o, N), rows, gate_ref, act)
        ops.grouped_gemm(ops.Strided(x.to(DEV), pad_x, K + gap), w.to(DEV), ops.Strided(out_dev, pad_o, N), rows, gate_dev, act)
        close(out_dev.cpu(), out_ref, dtype, f"grouped product gate={use_gate} act={act}")
        assert float(out_dev[:, :pad_o].abs().max()) == 0.0, "columns before the first group were written"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,E,top,H,I", [(1, 4, 4, 20, 12), (9, 5, 1, 33, 17), (70, 11, 3, 64, 40), (300, 3, 2, 48, 64),
                                         (700, 3, 2, 136, 200)])      # many rows an expert: tiles of 128
def test_routed_experts(dtype, T, E, top, H, I):
    g = torch.Generator().manual_seed(T + E)
    x = torch.randn(T, H, generator=g).to(dtype)
    logits = torch.randn(T, E, generator=g) * 2
    up, down = (torch.randn(E, I, H, generator=g) * 0.2).bfloat16(), (torch.randn(E, H, I, generator=g) * 0.2).bfloat16()
    r_ref = reference_ops.moe_route(logits, top, True, 1e-20)
    want = reference_ops.moe_combine(
        reference_ops.moe_experts(reference_ops.moe_experts(x, up, r_ref, dtype, "relu_squared", True), down, r_ref,
                                  torch.float32), r_ref, dtype)
    large = ops.moe_large_tiles(dtype, up.to(DEV), down.to(DEV))
    r = ops.moe_route(logits.to(DEV), top, True, 1e-20, large_tiles=large)
    assert r.tile == (128 if (large and T * top >= 192 * E) else 16 if T * top <= 16 * E else 64)
    assert torch.equal(r.ids.cpu(), r_ref.ids), "chosen experts"
    assert torch.allclose(r.weights.cpu(), r_ref.weights, atol=1e-6)
    starts = r.row_start.cpu().tolist()
    assert starts[0] == 0 and starts[-1] == T * top and starts == sorted(starts)
    hidden = ops.moe_experts(x.to(DEV), up.to(DEV), r, dtype, activation="relu_squared", gather=True)
    got = ops.moe_combine(ops.moe_experts(hidden, down.to(DEV), r, torch.float32), r, dtype)
    close(got.cpu(), want, dtype, "routed experts")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads,dim,rot,rank,rd,pairing,page,window",
                         [(3, 7, 10, 21, 6, "interleaved", 8, 17), (4, 16, 8, 32, 8, "interleaved", 4, 0),
                          (5, 0, 12, 40, 12, "half", 16, 70), (1, 5, 0, 9, 0, "interleaved", 2, 3),
                          (9, 8, 16, 300, 16, "interleaved", 16, 130), (2, 4, 4, 1100, 4, "interleaved", 16, 50)])
def test_latent_attention_kernels(dtype, heads, dim, rot, rank, rd, pairing, page, window):
    """Two requests of unequal length written to scattered pages in two portions each, then read."""
    g = torch.Generator().manual_seed(heads * 100 + rank)
    lengths = [150, 37]
    pages = sum(-(-n // page) for n in lengths) + 3
    width = heads * (dim + rot) + rank + rot + 3
    caches = [torch.zeros(pages, page, rank + rot, dtype=dtype), torch.zeros(pages, page, rank + rot, dtype=dtype, device=DEV)]
    table = torch.randn(200, rd, generator=g) if rd else None
    w = torch.rand(rank, generator=g) + 0.5
    order = torch.randperm(pages, generator=g).tolist()
    per = -(-max(lengths) // page)
    block_table = torch.full((2, per), -1, dtype=torch.int32)
    for r, n in enumerate(lengths):
        for b in range(-(-n // page)):
            block_table[r, b] = order.pop()
    done = [0, 0]
    for cut in (0.6, 1.0):
        tok_req, positions = [], []
        for r, n in enumerate(lengths):
            upto = int(n * cut)
            tok_req += [r] * (upto - done[r])
            positions += list(range(done[r], upto))
            done[r] = upto
        T = len(tok_req)
        tok_req, positions = torch.tensor(tok_req, dtype=torch.int32), torch.tensor(positions, dtype=torch.int32)
        slots = (block_table[tok_req.long(), (positions // page).long()] * page + positions % page).to(torch.int32)
        proj = torch.randn(T, width, generator=g).to(dtype)
        latent_q = torch.randn(T, heads, rank, generator=g).to(dtype)     # what the product per head would fill in
        outs = []
        for where, cache in zip(("cpu", DEV), caches):
            o = reference_ops if where == "cpu" else ops
            qa = torch.zeros(T, heads * (rank + rot), dtype=dtype, device=where)
            o.latent_prepare(proj.to(where), heads, dim, rot, rank, w.to(where), 1e-5, positions.to(where),
                             table.to(where) if rd else None, pairing, cache, slots.to(where), qa)
            qa.view(T, heads, rank + rot)[..., :rank] = latent_q.to(where)
            outs.append((qa.cpu(), o.latent_attention(qa, heads, rank, rot, tok_req.to(where), positions.to(where),
                                                      block_table.to(where), cache, page, 0.3, window).cpu()))
        close(outs[1][0], outs[0][0], dtype, "rotated queries")
        close(caches[1].cpu(), caches[0], dtype, "cache rows")
        caches[1].copy_(caches[0])        # the same rows on both sides for the attention itself
        close(outs[1][1], outs[0][1], dtype, "latent attention", terms=(rank + rot) / 300)


def test_rotary_table_stretched():
    """The part's table against the plain implementation's frequencies."""
    from lucciola_amd.parts.position import Rotary
    from lucciola_amd.parts.base import BuildContext
    scaling = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}
    part = Rotary(12, 5000.0, pairing="interleaved", scaling=scaling)
    part.bind({}, BuildContext(torch.float32, torch.device(DEV)))
    table = part.rotary_table(300).cpu().double()
    f, mag = plain_pubodra.rotary_frequencies(12, 5000.0, scaling)
    angle = torch.arange(table.shape[0], dtype=torch.float64)[:, None] * f[None, :]
    assert torch.allclose(table[:, :6], torch.cos(angle) * mag, atol=1e-6)
    assert torch.allclose(table[:, 6:], torch.sin(angle) * mag, atol=1e-6)


# ------------------------------------------------------------------ the engine
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["A", "B", "C"])
@pytest.mark.parametrize("family", ["whole", "tail", "chunked", "mixed"])
def test_replay_families(dtype, key, family):
    cfg, page, weights, prompts, refs = case(key)
    steps = {"whole": traces.whole, "tail": traces.tail_decode, "chunked": traces.chunked,
             "mixed": traces.mixed}[family](prompts)
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, dtype, DEV)
    got = replay(runner, steps)
    assert len(got) == sum(len(p) for p in prompts.values())
    worst = compare(got, cfg, weights, prompts, TOL[dtype], refs)
    print(f"{key} {family} {dtype}: worst relative error {worst:.3e}")
    assert not runner.cache.requests
    for g in runner.cache.groups:
        assert g.pool.num_free() == blocks


# ------------------------------------------------------------------ one mechanism a model
def _one_layer(mixer, mlp, **more):
    cfg = {"architecture": "Pubodra", "vocab": 97, "width": 40, "norm": {"eps": 2e-6},
           "layers": [{"type": "latent_attention", "mixer": mixer, "mlp": mlp}]}
    cfg.update(more)
    return cfg


MECHANISMS = {
    "mixer alone": _one_layer(pubodra_configs._mixer(3, 8, 6, 5, 12, 0.3, 11, base=200.0), None),
    "one head, nothing rotated": _one_layer({"heads": 1, "dim": 9, "rot_dim": 0, "vdim": 7, "kv_rank": 10, "scale": 0.4,
                                              "mask": {"size": 5}}, None),
    "everything rotated, no window": _one_layer(pubodra_configs._mixer(2, 0, 12, 6, 8, 0.3, None, base=50.0,
                                                                        scaling=pubodra_configs.YARN), None),
    "dense feed-forward": _one_layer(pubodra_configs._mixer(2, 4, 4, 4, 8, 0.5, 64), pubodra_configs._dense(33)),
    "every expert chosen": _one_layer(pubodra_configs._mixer(2, 4, 4, 4, 8, 0.5, 64), pubodra_configs._moe(12, 4, 4)),
    "one expert of many": _one_layer(pubodra_configs._mixer(2, 4, 4, 4, 8, 0.5, 64), pubodra_configs._moe(20, 70, 1)),
    "a stack run once": _one_layer(pubodra_configs._mixer(2, 4, 4, 4, 8, 0.5, 3), pubodra_configs._dense(16),
                                   loop={"start": 0, "stop": 1, "times": 1}),
    "one layer run four times": _one_layer(pubodra_configs._mixer(2, 4, 4, 4, 8, 0.5, 7), pubodra_configs._moe(16, 3, 2),
                                           loop={"start": 0, "stop": 1, "times": 4}),
}


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_each_mechanism(name, dtype):
    """Models of one layer that have one mechanism each, with sizes of 1, of 0 and equal to one
    another, fed whole, in portions and token by token."""
    cfg = MECHANISMS[name]
    weights = random_weights(cfg, 5, std=0.15 if dtype == "float32" else 0.06)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [23, 2, 58], 3)
    refs = {n: plain_pubodra.forward(cfg, weights, ids) for n, ids in prompts.items()}
    every_token = [([(n, [t], [0])], [n] if i == len(ids) - 1 else []) for n, ids in prompts.items()
                   for i, t in enumerate(ids)]
    for steps in (traces.whole(prompts), traces.chunked(prompts, sizes=(2, 9, 3, 2, 17)), every_token):
        runner = make_runner(cfg, weights, 4, 40, dtype, DEV)
        compare(replay(runner, steps), cfg, weights, prompts, TOL[dtype], refs)


# ------------------------------------------------------------------ edges of the window, far keys
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,page", [(33, 16), (64, 16), (17, 4), (0, 8)])
def test_one_key_carries_the_weight(dtype, window, page):
    """Among 300 cached rows one row's score stands out (its latent lies along the query); it is put
    far back, on both sides of every page border near the window's edge, just inside and just
    outside the window, and is read by a lone token and by the last row of a portion.  Where the
    query sees it, the result is that row's latent; where it does not, it is not."""
    heads, rank, rot, n = 2, 16, 4, 300
    g = torch.Generator().manual_seed(window + page)
    pages = -(-n // page) + 2
    order = torch.randperm(pages, generator=g).tolist()
    block_table = torch.tensor([order[:-(-n // page)]], dtype=torch.int32)
    base = (torch.randn(n, rank + rot, generator=g) * 0.1)
    marker = torch.zeros(rank + rot)
    marker[3] = 6.0
    p = n - 1
    edge = p - window + 1 if window else 0
    places = sorted({0, 1, edge - 1, edge, edge + 1, p - 1, p} | {b + d for b in range(edge - page, edge + page + 1, 1)
                                                                  if b % page == 0 for d in (-1, 0)})
    for place in [j for j in places if 0 <= j <= p]:
        rows = base.clone()
        rows[place] = marker
        cache = torch.zeros(pages, page, rank + rot, dtype=dtype)
        for j in range(n):
            cache[block_table[0, j // page], j % page] = rows[j].to(dtype)
        qa = torch.zeros(heads * (rank + rot))
        qa[3] = qa[rank + rot + 3] = 4.0
        seen = place >= edge
        for portion in (1, 7):
            T = portion
            positions = torch.arange(p - T + 1, p + 1, dtype=torch.int32)
            q = qa.to(dtype).repeat(T, 1)
            args = (heads, rank, rot, torch.zeros(T, dtype=torch.int32), positions, block_table)
            want = reference_ops.latent_attention(q, *args, cache, page, 1.0, window)
            got = ops.latent_attention(q.to(DEV), heads, rank, rot, args[3].to(DEV), positions.to(DEV),
                                       block_table.to(DEV), cache.to(DEV), page, 1.0, window).cpu()
            close(got, want, dtype, f"marker at {place}, window {window}, portion of {portion}")
            last = got[-1].float().view(heads, rank)
            assert (float(last[0, 3]) > 5.5) == seen, f"marker at {place} (edge {edge}): seen is {seen}"


# ------------------------------------------------------------------ the engine's other ways in
def engine_for(cfg, weights, page, blocks, dtype, **kw):
    from lucciola_amd.config.engine_config import EngineConfig
    from lucciola_amd.config.registry import architecture_for
    from lucciola_amd.engine.llm_engine import LLMEngine
    from lucciola_amd.engine.loading import _build
    from lucciola_amd.weights.loader import DictSource
    arch = architecture_for(cfg)
    config = arch.read_config(cfg)
    model = _build(arch.model_spec(config), DictSource(weights), dtype, DEV)
    return LLMEngine(model, config, EngineConfig(dtype=dtype, block_size=page, max_blocks=blocks, device=DEV, **kw))


@pytest.mark.parametrize("key", ["A", "B", "C"])
def test_greedy_generation_through_the_engine(key):
    from lucciola_amd.sampling.sampler import SamplingParams
    cfg, page, seed = pubodra_configs.ALL[key]
    weights = random_weights(cfg, seed, std=0.2)
    prompts = list(prompts_for({"vocab_size": cfg["vocab"]}, [5, 11, 37], seed + 30).values())
    engine = engine_for(cfg, weights, page, 64, "float32", max_tokens_per_step=16, max_seqs=4)
    got = engine.generate(prompts, SamplingParams(max_new_tokens=8))
    assert got == [plain_pubodra.greedy(cfg, weights, p, 8) for p in prompts]
    engine.runner.cache.check()
    assert not engine.runner.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("key", ["A", "C"])
def test_long_decoding_and_stale_pages(dtype, key):
    """A short prompt, then 260 tokens one by one (in bfloat16 through captured steps), past every
    window, in a cache whose pages hold the rows of other requests when they are taken."""
    cfg, page, seed = pubodra_configs.ALL[key]
    weights = random_weights(cfg, seed, std=pubodra_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [268, 270], seed + 7)
    refs = {n: plain_pubodra.forward(cfg, weights, ids) for n, ids in prompts.items()}
    steps = traces.tail_decode(prompts, tail=260)
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, dtype, DEV)
    for stored in runner.cache.storage.values():
        stored[0].normal_(0, 30.0)
    compare(replay(runner, steps), cfg, weights, prompts, TOL[dtype], refs)
    if dtype == "bfloat16":
        assert runner.graph_replays > 200


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(tmp_path, dtype):
    import json
    import os
    import subprocess
    import sys
    import numpy as np
    from lucciola_amd.weights.random_init import write_model_folder
    from lucciola_amd.weights.safetensors_io import SafetensorsFile
    cfg, page, seed = pubodra_configs.ALL["B"]
    folder = write_model_folder(str(tmp_path / "model"), dict(cfg, initializer_range=pubodra_configs.STD), seed)
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        weights = {n: f.get(n).clone() for n in f.names()}
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [70, 33, 50, 3, 61], seed)
    steps = traces.mixed(prompts, seed=3)
    lines, index, fed = [], {}, {}
    for i, (entries, end) in enumerate(steps):
        lines.append(json.dumps({"step": i, "end": end, "entries": [{"id": n, "tokens": t, "want": w} for n, t, w in entries]}))
        rows = []
        for n, t, w in entries:
            rows += [(n, fed.get(n, 0) + k) for k in w]
            fed[n] = fed.get(n, 0) + len(t)
        index[i] = rows
    out = tmp_path / "out"
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                           "--out", str(out), "--max-tokens", str(traces.max_live_tokens(steps, 64))],
                          input="\n".join(lines) + "\n", text=True, capture_output=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split() == [x for i in range(len(steps)) for x in ("done", str(i))]
    got = {}
    for i, rows in index.items():
        data = np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"])
        for r, key in enumerate(rows):
            got[key] = torch.from_numpy(data[r].astype("float64"))
    refs = {n: plain_pubodra.forward(cfg, weights, ids) for n, ids in prompts.items()}
    compare(got, cfg, weights, prompts, TOL[dtype], refs)


def test_float32_logits_do_not_depend_on_the_cut():
    """The same bits whole, in portions and token by token: every sum's order follows from the
    token alone."""
    cfg, page, seed = pubodra_configs.ALL["B"]
    weights = random_weights(cfg, seed, std=pubodra_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [75, 40], seed)
    runs = []
    for steps in (traces.whole(prompts), traces.chunked(prompts), traces.tail_decode(prompts, tail=30), traces.mixed(prompts)):
        runs.append(replay(make_runner(cfg, weights, page, 40, "float32", DEV), steps))
    for other in runs[1:]:
        for key, row in runs[0].items():
            assert torch.equal(row, other[key]), f"{key}: the bits differ between two cuts"


# ------------------------------------------------------------------ the matrix-core latent attention kernel
@pytest.mark.parametrize("heads,rank,rot,page,window", [(4, 32, 16, 16, 0), (3, 48, 8, 4, 37), (16, 64, 32, 16, 100),
                                                        (70, 16, 0, 8, 0), (9, 512, 64, 16, 130), (2, 208, 24, 32, 64)])
def test_latent_attention_on_the_matrix_cores(heads, rank, rot, page, window):
    """A step of portions (of 40, 2 and 17 tokens after histories of 150, 0 and 33) beside lone tokens
    (after 299 and 64), against the plain version and against the general kernel; then the same
    with the keys of every tile shared out over several workgroups."""
    from lucciola_amd.engine.batch import HostLayout, Plan
    g = torch.Generator().manual_seed(heads + rank)
    history, fresh = [150, 0, 299, 33, 64], [40, 2, 1, 17, 1]
    n_pages = sum(-(-(h + f) // page) for h, f in zip(history, fresh)) + 2
    order = torch.randperm(n_pages, generator=g).tolist()
    width = max(-(-(h + f) // page) for h, f in zip(history, fresh))
    block_table = torch.full((len(history), width), -1, dtype=torch.int32)
    cache = (torch.randn(n_pages, page, rank + rot, generator=g) * 0.5).bfloat16()
    for r, (h, f) in enumerate(zip(history, fresh)):
        for b in range(-(-(h + f) // page)):
            block_table[r, b] = order.pop()
    q_start = [0]
    for f in fresh:
        q_start.append(q_start[-1] + f)
    T = q_start[-1]
    tok_req = torch.tensor([r for r, f in enumerate(fresh) for _ in range(f)], dtype=torch.int32)
    positions = torch.tensor([history[r] + i for r, f in enumerate(fresh) for i in range(f)], dtype=torch.int32)
    qa = torch.randn(T, heads * (rank + rot), generator=g).bfloat16()
    arrays, info = ops.plan_latent_attention(HostLayout(len(fresh), T, q_start, history, page, False))
    plan = Plan({k: torch.from_numpy(v).to(DEV) for k, v in arrays.items()}, info)
    want = reference_ops.latent_attention(qa, heads, rank, rot, tok_req, positions, block_table, cache, page, 0.2, window)
    args = (qa.to(DEV), heads, rank, rot, tok_req.to(DEV), positions.to(DEV), block_table.to(DEV), cache.to(DEV), page,
            0.2, window)
    plain = ops.latent_attention(*args)
    close(plain.cpu(), want, torch.bfloat16, "general kernel")
    assert ops.library().lc_latent_bf16_supported(rank, rot)
    fast = ops.latent_attention(*args, plan=plan, max_ctx=300)
    close(fast.cpu(), want, torch.bfloat16, "matrix-core kernel")
    shared = ops.latent_attention(*args, plan=plan, max_ctx=1 << 20)       # a wide table: many shares, most of them empty
    close(shared.cpu(), want, torch.bfloat16, "matrix-core kernel with shares")


def test_matrix_core_path_is_the_one_that_serves():
    """A bfloat16 engine with sizes the kernel takes runs it (and the general kernel when switched off),
    with the same logits within rounding."""
    cfg, page, weights, prompts, refs = case("C")
    steps = traces.mixed(prompts)
    blocks = traces.max_live_tokens(steps, page) // page
    fast = replay(make_runner(cfg, weights, page, blocks, "bfloat16", DEV), steps)
    before = ops.latent_matrix_cores(False)
    try:
        slow = replay(make_runner(cfg, weights, page, blocks, "bfloat16", DEV), steps)
    finally:
        ops.latent_matrix_cores(before)
    compare(fast, cfg, weights, prompts, TOL["bfloat16"], refs)
    compare(slow, cfg, weights, prompts, TOL["bfloat16"], refs)
    assert any(not torch.equal(fast[k], slow[k]) for k in fast), "both runs took the same kernel"


def test_command_line(tmp_path):
    """A model folder made from a configuration and a seed, then greedy tokens through
    ``python -m lucciola_amd``: the architecture is found by config.json alone."""
    import json
    import os
    import subprocess
    import sys
    from lucciola_amd.weights.safetensors_io import SafetensorsFile
    cfg, page, seed = pubodra_configs.ALL["A"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    config_file = tmp_path / "config.json"
    config_file.write_text(json.dumps(dict(cfg, initializer_range=0.2)))
    folder = str(tmp_path / "model")
    run = [sys.executable, "-m", "lucciola_amd"]
    made = subprocess.run(run + ["--random-config", str(config_file), "--seed", "4", "--write-model", folder],
                          cwd=root, capture_output=True, text=True, timeout=300)
    assert made.returncode == 0, made.stderr[-2000:]
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as f:
        weights = {n: f.get(n).clone() for n in f.names()}
    prompts = [[3, 17, 150, 9], [88] * 30 + [5, 6]]
    proc = subprocess.run(run + ["--model", folder, "--dtype", "float32", "--max-new-tokens", "6", "--max-blocks", "64",
                                 "--block-size", str(page), "--max-tokens-per-step", "12"]
                          + [x for p in prompts for x in ("--prompt-ids", ",".join(map(str, p)))],
                          cwd=root, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = [[int(t) for t in line.split()] for line in proc.stdout.strip().splitlines()]
    assert got == [plain_pubodra.greedy(cfg, weights, p, 6) for p in prompts]


@pytest.mark.parametrize("ahead", [False, True])
def test_generation_survives_preemption(ahead):
    """With so few pages that running requests are preempted and recomputed (the windows give pages
    back, full attention in one layer of B does not), every request's tokens are the plain
    implementation's; also with the next step queued before this step's tokens are read."""
    from lucciola_amd.sampling.sampler import SamplingParams
    cfg, page, seed = pubodra_configs.ALL["B"]
    weights = random_weights(cfg, seed, std=0.2)
    prompts = list(prompts_for({"vocab_size": cfg["vocab"]}, [9, 14, 6, 11], seed + 40).values())
    tight = engine_for(cfg, weights, page, 9, "float32", max_tokens_per_step=12, max_seqs=4, run_ahead=ahead)
    got = tight.generate(prompts, SamplingParams(max_new_tokens=20))
    assert tight.scheduler.num_preemptions > 0
    for prompt, tokens in zip(prompts, got):
        assert tokens == plain_pubodra.greedy(cfg, weights, prompt, 20)
    tight.runner.cache.check()
    assert not tight.runner.cache.requests


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("seed", range(12))
def test_random_configurations(seed, dtype):
    """Configurations drawn at random, requests in mixed steps with so few pages that they are used
    again, against the plain implementation."""
    cfg, page = pubodra_configs.random_configuration(seed)
    weights = random_weights(cfg, 100 + seed, std=pubodra_configs.STD)
    prompts = prompts_for({"vocab_size": cfg["vocab"]}, [3, 120, 41, 77, 1, 150], seed)
    refs = {n: plain_pubodra.forward(cfg, weights, ids) for n, ids in prompts.items()}
    steps = traces.mixed(prompts, seed=seed)
    blocks = traces.max_live_tokens(steps, page) // page
    runner = make_runner(cfg, weights, page, blocks, dtype, DEV)
    compare(replay(runner, steps), cfg, weights, prompts, TOL[dtype], refs)
    assert not runner.cache.requests


@pytest.mark.parametrize("heads,rank,rot,page,window", [(16, 512, 64, 16, 0), (20, 64, 32, 16, 90), (3, 48, 8, 4, 37),
                                                        (32, 208, 24, 32, 0), (1, 16, 0, 8, 5), (70, 64, 16, 16, 0)])
def test_a_step_of_lone_tokens_on_the_matrix_cores(heads, rank, rot, page, window):
    """A step of lone tokens only (after 299, 0, 64, 31 and 700 cached tokens), where a workgroup
    serves up to 64 heads of one token, against the plain version; then with the keys shared out."""
    from lucciola_amd.engine.batch import HostLayout, Plan
    g = torch.Generator().manual_seed(heads * 3 + rank)
    history = [299, 0, 64, 31, 700]
    n_pages = sum(-(-(h + 1) // page) for h in history) + 2
    order = torch.randperm(n_pages, generator=g).tolist()
    width = max(-(-(h + 1) // page) for h in history)
    block_table = torch.full((len(history), width), -1, dtype=torch.int32)
    cache = (torch.randn(n_pages, page, rank + rot, generator=g) * 0.5).bfloat16()
    for r, h in enumerate(history):
        for b in range(-(-(h + 1) // page)):
            block_table[r, b] = order.pop()
    T = len(history)
    tok_req = torch.arange(T, dtype=torch.int32)
    positions = torch.tensor(history, dtype=torch.int32)
    qa = torch.randn(T, heads * (rank + rot), generator=g).bfloat16()
    arrays, info = ops.plan_latent_attention(HostLayout(T, T, list(range(T + 1)), history, page, True))
    plan = Plan({k: torch.from_numpy(v).to(DEV) for k, v in arrays.items()}, info)
    want = reference_ops.latent_attention(qa, heads, rank, rot, tok_req, positions, block_table, cache, page, 0.2, window)
    args = (qa.to(DEV), heads, rank, rot, tok_req.to(DEV), positions.to(DEV), block_table.to(DEV), cache.to(DEV), page,
            0.2, window)
    close(ops.latent_attention(*args, plan=plan, max_ctx=701).cpu(), want, torch.bfloat16, "lone tokens")
    close(ops.latent_attention(*args, plan=plan, max_ctx=1 << 20).cpu(), want, torch.bfloat16, "lone tokens, many shares")
