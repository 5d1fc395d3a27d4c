"""GPU tier: the layer-list engine (HybridEngine over libtinyllm_hybrid.so) against the plain float64 restatement in
tests/layer_list_oracle.py, on small made-up configurations with random (or crafted) weights.

float32 runs are held to a relative RMS error of 2e-4 per logits row (summation order only); bfloat16 runs to 4e-2
(matrices, matrix-product inputs and K/V pages rounded to 8 bits of mantissa, everything else in float32).
"""

import json
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import layer_list_oracle as O

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 2e-4, torch.bfloat16: 4e-2}


def make_model(config, weights, dtype=torch.float32):
    from tiny_llm_hip.layer_list import FAMILIES

    read_config, _ = FAMILIES[config["architecture"]]
    cfg = read_config(config)
    return SimpleNamespace(family=cfg.family, config=cfg, tensors={k: torch.from_numpy(np.asarray(v)) for k, v in weights.items()}, dtype=dtype)


def make_engine(config, weights, dtype=torch.float32, **pool):
    from tiny_llm_hip.models import engine_for

    kw = dict(page_size=16, num_pages=64, max_batch=4, max_prefill_rows=512)
    kw.update(pool)
    return engine_for(make_model(config, weights, dtype), dtype=dtype, **kw)


def rel_err(got, want):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    return float(np.max(np.sqrt(((got - want) ** 2).mean(-1)) / np.sqrt((want ** 2).mean(-1))))


def tokens_for(config, n, seed=0, avoid=()):
    rng = np.random.default_rng(seed)
    pool = [t for t in range(config["vocab"]) if t not in avoid]
    return [int(pool[i]) for i in rng.integers(0, len(pool), n)]


def whole(engine, tokens, slot=0):
    engine.begin(slot)
    try:
        n = engine.step([(slot, tokens, list(range(len(tokens))))])
        return engine.logits_host(n)
    finally:
        engine.release(slot)


def in_portions(engine, tokens, sizes, slot=0):
    """The sequence cut into portions of the given sizes (cycled); every row's logits."""
    engine.begin(slot)
    rows, at, i = [], 0, 0
    try:
        while at < len(tokens):
            part = tokens[at:at + sizes[i % len(sizes)]]
            rows.append(engine.logits_host(engine.step([(slot, part, list(range(len(part))))])))
            at += len(part)
            i += 1
    finally:
        engine.release(slot)
    return np.concatenate(rows, 0)


MIXED = O.fonapel_config([O.delta_layer(), O.attention_layer(), O.attention_layer(heads=2, kv_heads=2, dim=16, vdim=8, rot_dims=16, ff=0),
                          O.delta_layer(heads=2, kv_heads=2, dim=32, vdim=16, conv=4)], loop=(1, 3, 2))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layer", ["attention", "attention_ff", "delta", "delta_ff", "attention_full_rot", "attention_no_rot", "delta_wide_key",
                                   "delta_many_columns", "attention_very_wide_head", "attention_large_group"])
def test_each_mixer_alone(layer, dtype):
    spec = {"attention": O.attention_layer(ff=0), "attention_ff": O.attention_layer(ff=48), "delta": O.delta_layer(ff=0),
            "delta_ff": O.delta_layer(ff=40), "attention_full_rot": O.attention_layer(dim=16, rot_dims=16, ff=0),
            "attention_no_rot": O.attention_layer(rot_dims=0, ff=0),
            "attention_very_wide_head": O.attention_layer(heads=2, kv_heads=1, dim=264, vdim=260, rot_dims=64, ff=0),  # beyond the tile kernel: a wave per row
            "attention_large_group": O.attention_layer(heads=24, kv_heads=1, dim=16, vdim=8, rot_dims=4, ff=0),  # 24 query heads on one K/V head: two blocks of 16
            "delta_wide_key": O.delta_layer(heads=2, kv_heads=1, dim=136, vdim=20, ff=0),         # a wave per state column
            "delta_many_columns": O.delta_layer(heads=20, kv_heads=10, dim=72, vdim=128, ff=0)}[layer]  # 16 lanes per column, 8 rows each
    config = O.fonapel_config([spec])
    W = O.make_fonapel_weights(config, seed=1)
    toks = tokens_for(config, 37, seed=2)
    engine = make_engine(config, W, dtype)
    try:
        assert rel_err(whole(engine, toks), O.fonapel_forward(config, W, toks)) < TOL[dtype]
    finally:
        engine.close()


def test_row_attention_twin_of_the_tile_kernel(monkeypatch):
    """TL_HYBRID_ATTN_ROWS=1 runs every attention on the one-wave-per-row kernel; both forms must give the restatement's logits."""
    W = O.make_fonapel_weights(MIXED, seed=27)
    toks = tokens_for(MIXED, 90, seed=28)
    want = O.fonapel_forward(MIXED, W, toks)
    monkeypatch.setenv("TL_HYBRID_ATTN_ROWS", "1")
    engine = make_engine(MIXED, W)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[torch.float32]
        assert rel_err(in_portions(engine, toks, [50, 1, 7]), want) < TOL[torch.float32]
    finally:
        engine.close()


def test_stream_after_every_layer_run_and_loop_passes():
    W = O.make_fonapel_weights(MIXED, seed=3)
    toks = tokens_for(MIXED, 29, seed=4)
    streams = []
    want = O.fonapel_forward(MIXED, W, toks, streams)
    engine = make_engine(MIXED, W)
    try:
        assert engine.stats()["layer_runs"] == len(streams) == 6
        engine.set_trace(True)
        engine.begin(0)
        n = engine.step([(0, toks, list(range(len(toks))))])
        for run, ref in enumerate(streams):
            assert rel_err(engine.read_trace(run, len(toks)), ref) < 1e-5, f"layer run {run}"
        assert rel_err(engine.logits_host(n), want) < TOL[torch.float32]
        engine.release(0)
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prefill_against_token_by_token(dtype):
    W = O.make_fonapel_weights(MIXED, seed=5)
    toks = tokens_for(MIXED, 45, seed=6)
    want = O.fonapel_forward(MIXED, W, toks)
    engine = make_engine(MIXED, W, dtype)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[dtype]
        assert rel_err(in_portions(engine, toks, [1]), want) < TOL[dtype]
        assert rel_err(in_portions(engine, toks, [30, 1]), want) < TOL[dtype]  # a prompt, then decoding
    finally:
        engine.close()


@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [16], [15, 17, 1], [33, 2, 2, 40], [70, 13]])
def test_portions_of_several_sizes(sizes):
    W = O.make_fonapel_weights(MIXED, seed=7)
    toks = tokens_for(MIXED, 83, seed=8)
    engine = make_engine(MIXED, W)
    try:
        assert rel_err(in_portions(engine, toks, sizes), O.fonapel_forward(MIXED, W, toks)) < TOL[torch.float32]
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_unequal_requests_in_one_batch_against_each_alone(dtype):
    """Portions of some requests beside single tokens of others; every request's rows must equal its whole-sequence logits."""
    W = O.make_fonapel_weights(MIXED, seed=9)
    prompts = [tokens_for(MIXED, n, seed=10 + n) for n in (70, 9, 41, 25)]
    want = [O.fonapel_forward(MIXED, W, p) for p in prompts]
    cuts = [[20, 1, 1, 30, 1, 1, 1, 15], [2, 1, 1, 1, 1, 1, 1, 1], [1, 17, 3, 19, 1], [25]]
    engine = make_engine(MIXED, W, dtype)
    try:
        at = [0] * 4
        got = [[] for _ in prompts]
        for s in range(4):
            engine.begin(s)
        turn = 0
        while any(at[i] < len(prompts[i]) for i in range(4)):
            entries, who = [], []
            for i in range(4):
                if at[i] < len(prompts[i]) and turn < len(cuts[i]) + 64:
                    n = cuts[i][turn] if turn < len(cuts[i]) else 1
                    part = prompts[i][at[i]:at[i] + n]
                    if (turn + i) % 5 == 4 and len(entries) > 0:
                        continue  # a request may sit out a step
                    entries.append((i, part, list(range(len(part)))))
                    who.append((i, len(part)))
                    at[i] += len(part)
            turn += 1
            if not entries:
                continue
            rows = engine.logits_host(engine.step(entries))
            r = 0
            for i, n in who:
                got[i].append(rows[r:r + n])
                r += n
        for i in range(4):
            assert rel_err(np.concatenate(got[i], 0), want[i]) < TOL[dtype], f"request {i}"
    finally:
        engine.close()


def test_pages_and_slots_are_used_again():
    """A pool of 6 pages of 16 tokens and 2 slots serves 6 requests one after the other and in pairs."""
    W = O.make_fonapel_weights(MIXED, seed=11)
    engine = make_engine(MIXED, W, page_size=16, num_pages=6, max_batch=2, max_prefill_rows=96)
    try:
        prompts = [tokens_for(MIXED, n, seed=20 + n) for n in (40, 33, 48, 17, 31, 47)]
        want = [O.fonapel_forward(MIXED, W, p) for p in prompts]
        for k in range(0, 6, 2):
            a, b = prompts[k], prompts[k + 1]
            engine.begin(0)
            engine.begin(1)
            ra = [engine.logits_host(engine.step([(0, a[:10], list(range(10)))]))]
            both = engine.logits_host(engine.step([(0, a[10:], list(range(len(a) - 10))), (1, b, list(range(len(b))))]))
            ra.append(both[:len(a) - 10])
            assert rel_err(np.concatenate(ra, 0), want[k]) < TOL[torch.float32]
            assert rel_err(both[len(a) - 10:], want[k + 1]) < TOL[torch.float32]
            engine.release(0)
            engine.release(1)
        st = engine.stats()
        assert st["reused_page_allocations"] > 0 and st["reused_slot_begins"] == 4 and st["pages_in_use"] == 0
        engine.begin(0)
        engine.step([(0, tokens_for(MIXED, 96, seed=1), [])])  # all 6 pages
        engine.begin(1)
        with pytest.raises(RuntimeError, match="pool exhausted"):
            engine.step([(1, [1], [])])
        engine.release(0)
        engine.step([(1, [1], [])])  # a failed step leaves the engine usable
    finally:
        engine.close()


def _needle_model(scale=2.0):
    """One attention layer whose query token B looks for key token A: the score of (B, A) towers over every other, so a lost,
    shifted or doubled key changes the logits at B by much more than the tolerance."""
    config = O.fonapel_config([O.attention_layer(heads=2, kv_heads=1, dim=32, vdim=16, rot_dims=8, scale=scale, ff=0)], width=64, vocab=50)
    W = O.make_fonapel_weights(config, seed=12)
    A, B = 48, 49
    W["embed"][:, :2] = 0.0
    W["embed"][A] *= 0.05
    W["embed"][B] *= 0.05
    W["embed"][A, 0] = 8.0
    W["embed"][B, 1] = 8.0
    u = np.zeros(32, dtype=np.float32)
    u[8:] = np.where(np.arange(24) % 2 == 0, 1.0, -1.0)  # outside the rotated dimensions: the match does not depend on distance
    W["l0.mix.k"][:, 0] += 4.0 * u
    for h in range(2):
        W["l0.mix.q"][h * 32:(h + 1) * 32, 1] += 4.0 * u
    W["l0.mix.v"][:, 0] += 2.0
    for k in W:
        W[k] = torch.from_numpy(W[k]).to(torch.bfloat16).float().numpy()
    return config, W, A, B


@pytest.mark.parametrize("needle_at", [0, 3, 15, 16, 17, 31, 32, 250])
@pytest.mark.parametrize("query", ["prompt", "decoded"])
def test_far_keys_and_page_borders(needle_at, query):
    config, W, A, B = _needle_model()
    toks = tokens_for(config, 300, seed=13, avoid=(A, B))
    toks[needle_at] = A
    toks[-1] = B
    want = O.fonapel_forward(config, W, toks)[-1]
    other = list(toks)
    other[needle_at] = toks[needle_at - 1] if needle_at else toks[1]
    assert rel_err(O.fonapel_forward(config, W, other)[-1][None], want[None]) > 0.2  # the needle does decide the answer
    engine = make_engine(config, W, page_size=16, num_pages=24, max_batch=1)
    try:
        engine.begin(0)
        if query == "prompt":
            engine.step([(0, toks[:100], []), ])
            n = engine.step([(0, toks[100:], [len(toks) - 101])])
        else:
            engine.step([(0, toks[:-1], [])])
            n = engine.step([(0, toks[-1:], [0])])
        assert rel_err(engine.logits_host(n), want[None]) < TOL[torch.float32]
        engine.release(0)
    finally:
        engine.close()


@pytest.mark.parametrize("needle_at", [5, 63, 64, 127, 128, 255, 256, 511, 512, 640, 767, 768])
def test_decoding_over_a_split_key_range(needle_at):
    """From 256 keys on a single-token step splits a row's keys over workgroups (64 keys each, doubled beyond 64 splits) and merges the
    partial sums: the needle sits at the splits' borders; the query is decoded alone, then greedy decoding goes on through the captured step."""
    config, W, A, B = _needle_model()
    toks = tokens_for(config, 800, seed=23, avoid=(A, B))
    toks[needle_at] = A
    toks[-1] = B
    ref = O.fonapel_forward(config, W, toks)
    engine = make_engine(config, W, page_size=16, num_pages=64, max_batch=2, max_prefill_rows=1024)
    try:
        engine.begin(1)
        engine.step([(1, toks[:-1], [])])
        n = engine.step([(1, toks[-1:], [0])])
        assert rel_err(engine.logits_host(n), ref[-1][None]) < TOL[torch.float32]
        engine.release(1)
        engine.begin(0)
        engine.prefill(0, toks[:790])
        engine.set_token(0, toks[790])
        engine.decode_free_running(9, [0])       # feeds 790, then its own greedy ids
        engine.synchronize()
        assert engine.context_len(0) == 799
        engine.release(0)
    finally:
        engine.close()


@pytest.mark.parametrize("needle_at", [100, 4095, 4096, 4223])
def test_decoding_over_more_keys_than_64_tiles(needle_at):
    """Beyond 4,096 keys the splits take 128 keys each (two tiles per workgroup)."""
    config, W, A, B = _needle_model()
    toks = tokens_for(config, 4300, seed=26, avoid=(A, B))
    toks[needle_at] = A
    toks[-1] = B
    want = O.fonapel_forward(config, W, toks)[-1]
    engine = make_engine(config, W, page_size=64, num_pages=70, max_batch=1, max_prefill_rows=2048)
    try:
        engine.begin(0)
        engine.prefill(0, toks[:-1], want_logits=False)
        n = engine.step([(0, toks[-1:], [0])])
        assert rel_err(engine.logits_host(n), want[None]) < TOL[torch.float32]
        engine.release(0)
    finally:
        engine.close()


WIDE = O.fonapel_config([O.delta_layer(heads=4, kv_heads=2, dim=32, vdim=32, conv=4, ff=256), O.attention_layer(heads=4, kv_heads=2, dim=64, vdim=32, rot_dims=32, ff=256)],
                        width=128, vocab=200, loop=(0, 2, 2))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_large_chunks_take_the_wide_tile_products(dtype):
    """From 192 rows the bfloat16 products run on the 256-wide LDS-DMA tile GEMM with float32 epilogues; the same prompt in small
    portions (64-wide tiles, row kernel) must give the same logits."""
    W = O.make_fonapel_weights(WIDE, seed=24)
    toks = tokens_for(WIDE, 300, seed=25)
    want = O.fonapel_forward(WIDE, W, toks)
    engine = make_engine(WIDE, W, dtype, page_size=64, num_pages=8, max_batch=2)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[dtype]
        assert rel_err(in_portions(engine, toks, [250, 3, 40, 1]), want) < TOL[dtype]
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_first_tokens_where_the_sink_weighs_most(dtype):
    """At position 0 a weight is exp(s) / (1 + exp(s)): without the 1 in the denominator it would be exactly 1."""
    config = O.fonapel_config([O.attention_layer(scale=0.02, ff=0), O.delta_layer(ff=0)])
    W = O.make_fonapel_weights(config, seed=14)
    toks = tokens_for(config, 4, seed=15)
    want = O.fonapel_forward(config, W, toks)
    engine = make_engine(config, W, dtype)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[dtype]
        assert rel_err(in_portions(engine, toks, [1]), want) < TOL[dtype]
        assert rel_err(whole(engine, toks[:1]), want[:1]) < TOL[dtype]
    finally:
        engine.close()


ODD = O.fonapel_config([O.attention_layer(heads=3, kv_heads=1, dim=24, vdim=40, rot_dims=10, base=777.0, scale=0.3, ff=100),
                        O.delta_layer(heads=6, kv_heads=2, dim=20, vdim=12, conv=2, ff=0),
                        O.delta_layer(heads=1, kv_heads=1, dim=72, vdim=33, conv=1, ff=52),
                        O.attention_layer(heads=5, kv_heads=5, dim=10, vdim=6, rot_dims=10, ff=36)],
                       width=88, vocab=97, eps=1e-3, residual_mult=1.0)


@pytest.mark.parametrize("loop", [None, (0, 2, 2), (2, 4, 3), (1, 2, 1), (0, 4, 2)])
def test_other_sizes_and_loop_shapes(loop):
    """Sizes that are no multiples of 8, unequal head groups in both mixers, one tap, no feed-forward, loops at either end."""
    config = dict(ODD)
    if loop:
        config["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    W = O.make_fonapel_weights(config, seed=16)
    toks = tokens_for(config, 41, seed=17)
    want = O.fonapel_forward(config, W, toks)
    engine = make_engine(config, W)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[torch.float32]
        assert rel_err(in_portions(engine, toks, [5, 1, 2, 9]), want) < TOL[torch.float32]
    finally:
        engine.close()


def test_long_greedy_decoding_on_the_device_and_graph_replays():
    """160 greedy steps through the captured decode step; the ids are the float64 restatement's greedy choices, and replaying the
    graph gives what eager launches give."""
    W = O.make_fonapel_weights(MIXED, seed=18)
    prompt = tokens_for(MIXED, 21, seed=19)
    engine = make_engine(MIXED, W, page_size=16, num_pages=16, max_batch=2)
    try:
        ids = engine.generate(prompt, 161, slot=1)
        assert engine.stats()["graph_replays"] >= 160 and engine.stats()["graph_captures"] == 1
        full = prompt + ids
        ref = O.fonapel_forward(MIXED, W, full[:-1])
        for k, tok in enumerate(ids):
            row = ref[len(prompt) - 1 + k]
            assert row[tok] >= row.max() - 1e-3 * np.abs(row).max(), f"generated token {k}"
        engine.begin(0)
        engine.prefill(0, prompt)
        engine.decode(40, slots=[0], use_graph=False)
        assert engine.read_tokens(0, 41) == ids[:41]
        engine.release(0)
    finally:
        engine.close()


@pytest.mark.parametrize("mixed", [True, False])
def test_greedy_generation_through_the_scheduler(mixed):
    """engine.batch_generate_ids (continuous batching: chunked prefill in a staging slot, adoption into decode slots, retirement)
    over the layer-list engine: every request's ids are what the request alone generates."""
    from tiny_llm_hip.engine import batch_generate_ids

    W = O.make_fonapel_weights(MIXED, seed=20)
    prompts = [tokens_for(MIXED, n, seed=30 + n) for n in (5, 23, 40, 9, 31)]
    limits = [12, 7, 9, 15, 4]
    engine = make_engine(MIXED, W, page_size=16, num_pages=40, max_batch=4, max_prefill_rows=64)
    try:
        alone = [engine.generate(p, n, slot=0) for p, n in zip(prompts, limits)]
        done = dict(batch_generate_ids(engine, prompts, limits, batch_size=3, prefill_step=16, mixed_steps=mixed))
        assert sorted(done) == list(range(5))
        for i in range(5):
            assert done[i] == alone[i], f"request {i}"
        assert engine.stats()["pages_in_use"] == 0
    finally:
        engine.close()


def test_checkpoint_directory_through_loader_registry_and_command_line(tmp_path, capsys):
    from safetensors.torch import save_file

    config = O.fonapel_config([O.delta_layer(), O.attention_layer()], loop=(0, 2, 2))
    W = O.make_fonapel_weights(config, seed=21)
    (tmp_path / "config.json").write_text(json.dumps(config))
    save_file({k: torch.from_numpy(v).to(torch.bfloat16) for k, v in W.items()}, str(tmp_path / "model.safetensors"))
    from tiny_llm_hip import load
    from tiny_llm_hip.models import engine_for

    model, tokenizer = load(str(tmp_path))
    assert tokenizer is None and model.family == "Fonapel"
    prompt = tokens_for(config, 11, seed=22)
    engine = engine_for(model, dtype=torch.float32, page_size=16, num_pages=8, max_batch=1, max_prefill_rows=32)
    try:
        want = engine.generate(prompt, 6)
    finally:
        engine.close()
    import main as cli

    out = cli.main(["--model", str(tmp_path), "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--dtype", "float32"])
    assert [int(t) for t in out.split()] == want
    # the sampler path: temperature ~ 0 must reproduce the greedy ids
    out = cli.main(["--model", str(tmp_path), "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--dtype", "float32",
                    "--sampler-temp", "1e-4", "--sampler-top-k", "1"])
    assert [int(t) for t in out.split()] == want


def test_trace_replay_command_line(tmp_path):
    """bin/trace_run on a checkpoint directory: steps as JSON lines on stdin, one packed pass per step, logits files and "done" lines out.
    The first step is larger than the engine's row workspace (it is fed in portions); then two requests share steps, one ends and its
    slot and pages serve a third."""
    import subprocess
    import sys
    from pathlib import Path

    from safetensors.torch import save_file

    config, W, A, B = _needle_model()
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(config))
    save_file({k: torch.from_numpy(v).to(torch.bfloat16) for k, v in W.items()}, str(model_dir / "model.safetensors"))
    long = tokens_for(config, 4200, seed=29, avoid=(A, B))
    long[7], long[-1] = A, B
    short = tokens_for(config, 30, seed=30)
    third = tokens_for(config, 50, seed=31)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": long[:4150], "want": [0, 4149]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": long[4150:4199], "want": []}, {"id": "y", "tokens": short[:29], "want": [28]}], "end": []},
             {"step": 2, "entries": [{"id": "y", "tokens": short[29:], "want": [0]}, {"id": "x", "tokens": long[4199:], "want": [0]}], "end": ["x"]},
             {"step": 3, "entries": [], "end": []},
             {"step": 4, "entries": [{"id": "z", "tokens": third, "want": [49, 3]}, {"id": "y", "tokens": [5], "want": []}], "end": ["y", "z"]}]
    root = Path(__file__).resolve().parent.parent
    run = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", "float32", "--out", str(out_dir),
                          "--max-tokens", str(4224 + 64 + 64), "--slots", "2"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=110)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    ref_long, ref_short, ref_third = (O.fonapel_forward(config, W, t) for t in (long, short, third))
    got = {i: np.fromfile(out_dir / f"{i}.f32", dtype="<f4").reshape(-1, config["vocab"]) for i in (0, 1, 2, 4)}
    assert not (out_dir / "3.f32").exists()
    assert rel_err(got[0], ref_long[[0, 4149]]) < TOL[torch.float32]
    assert rel_err(got[1], ref_short[[28]]) < TOL[torch.float32]
    assert rel_err(got[2], np.stack([ref_short[29], ref_long[4199]])) < TOL[torch.float32]
    assert rel_err(got[4], ref_third[[49, 3]]) < TOL[torch.float32]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(1, 64, 128), (3, 50, 77), (8, 300, 256), (9, 64, 64), (70, 130, 96), (200, 97, 203), (64, 64, 8), (256, 512, 256),
                                   (300, 132, 128), (1000, 260, 192)])
@pytest.mark.parametrize("kernel", [0, 1, 2, 3])
def test_linear_kernels_against_torch(shape, dtype, kernel):
    import ctypes

    import tiny_llm_ext_hybrid as ext

    M, N, K = shape
    if kernel == 1 and M > 8:
        pytest.skip("the row kernel takes at most 8 rows")
    if kernel == 3 and (dtype != torch.bfloat16 or K % 64 or K < 128 or N % 4):
        pytest.skip("the 256-wide tile GEMM takes bfloat16, whole 64-wide K steps (two at least) and columns in fours")
    gen = torch.Generator().manual_seed(M * 1000 + N)
    a = torch.randn(M, K, generator=gen).to(dtype).cuda()
    w = torch.randn(N, K, generator=gen).to(dtype).cuda()
    out = torch.full((M, N), float("nan"), dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    ext.check(ext.lib().tl_hybrid_linear(ext.HY_BF16 if dtype == torch.bfloat16 else ext.HY_F32, a.data_ptr(), K, w.data_ptr(), out.data_ptr(), N, M, N, K,
                                         kernel, None))
    torch.cuda.synchronize()
    want = a.double().cpu() @ w.double().cpu().T
    assert rel_err(out.cpu().numpy(), want.numpy()) < 1e-5
