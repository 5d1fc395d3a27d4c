"""GPU tier: the Zefapel family on the layer-list engine against the plain float64 restatement in tests/layer_list_oracle.py, on
small made-up configurations with random (or crafted) weights: sequential blocks with Dynamic Tanh norms and layer scale; the
matrix-memory, gated-linear-attention and latent-attention mixers; dense and mixture-of-experts feed-forwards.

float32 runs are held to a relative RMS error of 2e-4 per logits row, bfloat16 runs to 4e-2 (layer_list_engine_helpers.TOL).
"""

import json

import numpy as np
import pytest
import torch

import layer_list_oracle as O
from layer_list_engine_helpers import TOL, in_portions, make_engine, rel_err, tokens_for, whole

pytestmark = pytest.mark.gpu

# every mixer and both feed-forward kinds; the last layer reads the third's latent cache
MIXED = O.zefapel_config([O.mlstm_layer(mlp=O.dense_ff()), O.gla_layer(mlp=O.moe_ff()), O.latent_layer(mlp=O.dense_ff(40)),
                          O.latent_layer(kv_from=2, mlp=O.moe_ff(experts=4, identity=2, top=3, groups=2, keep=1, shared=0))])

LAYERS = {
    "mlstm": O.mlstm_layer(),
    "mlstm_dense": O.mlstm_layer(mlp=O.dense_ff()),
    "mlstm_one_head_wide_key": O.mlstm_layer(heads=1, dim=136, vdim=20),            # a wave per state column
    "mlstm_many_columns": O.mlstm_layer(heads=20, dim=72, vdim=127),                  # 16 lanes per column; the normaliser's column starts a block
    "mlstm_32_lanes_per_column": O.mlstm_layer(heads=12, dim=40, vdim=100),               # 1,212 columns: between one wave and a DPP row per column
    "gla_32_lanes_per_column": O.gla_layer(heads=10, dim=72, vdim=128, a_rank=8),
    "gla_wide_key_many_columns": O.gla_layer(heads=10, dim=264, vdim=250, a_rank=8),      # 16 rows a lane at most: 32 lanes although the columns are many
    "gla": O.gla_layer(),
    "gla_moe": O.gla_layer(mlp=O.moe_ff()),
    "gla_narrow": O.gla_layer(heads=5, dim=10, vdim=7, tau=1.0, a_rank=3),
    "gla_wide_key": O.gla_layer(heads=2, dim=264, vdim=12, tau=20.0, a_rank=16),
    "latent": O.latent_layer(),
    "latent_plain_frequencies": O.latent_layer(scaling=None),
    "latent_frequency_ramp": O.latent_layer(rot_dim=16, scaling=(8.0, 32, 4.0, 0.5)),
    "latent_many_heads": O.latent_layer(heads=24, dim=8, vdim=8, rot_dim=4, q_rank=16, kv_rank=24),   # two blocks of 16 query heads on the one K/V head
    "latent_three_heads_odd_sizes": O.latent_layer(heads=3, dim=20, vdim=12, rot_dim=6, q_rank=9, kv_rank=26),
    "latent_mid_tile": O.latent_layer(heads=4, dim=24, vdim=16, rot_dim=16, q_rank=24, kv_rank=104),       # key rows of 120, values of 104: the 128 / 128 tile
    "latent_widest_tile": O.latent_layer(heads=2, dim=16, vdim=16, rot_dim=8, q_rank=16, kv_rank=216),    # key rows of 224, values of 216: the 256 / 256 tile
    "latent_wide_latent": O.latent_layer(heads=2, dim=16, vdim=16, rot_dim=8, q_rank=16, kv_rank=264),  # beyond the tile kernel: a wave per row
    "latent_moe": O.latent_layer(mlp=O.moe_ff(experts=9, identity=6, top=5, groups=5, keep=3)),
}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("layer", sorted(LAYERS))
def test_each_mechanism_alone(layer, dtype):
    config = O.zefapel_config([LAYERS[layer]])
    W = O.make_zefapel_weights(config, seed=1)
    toks = tokens_for(config, 37, seed=2)
    engine = make_engine(config, W, dtype)
    try:
        want = O.zefapel_forward(config, W, toks)
        assert rel_err(whole(engine, toks), want) < TOL[dtype]
        assert rel_err(in_portions(engine, toks, [9, 1, 2]), want) < TOL[dtype]
    finally:
        engine.close()


@pytest.mark.parametrize("mlp", ["identity_only_choice", "no_identity", "one_group", "all_taken", "negative_choices", "many_experts"])
def test_expert_choice(mlp):
    """The router's branches: identity experts, groups that shut experts out, choices that are all negative (an expert outside the
    kept groups counts as minus infinity, not as 0), every expert taken, more experts than a wave has lanes."""
    spec = {"identity_only_choice": O.moe_ff(experts=2, identity=4, top=3, groups=3, keep=2, shared=0),
            "no_identity": O.moe_ff(experts=6, identity=0, top=2, groups=2, keep=1, shared=16),
            "one_group": O.moe_ff(experts=3, identity=1, top=2, groups=1, keep=1, shared=0),
            "all_taken": O.moe_ff(experts=3, identity=3, top=6, groups=3, keep=3, shared=8),
            "negative_choices": O.moe_ff(experts=6, identity=3, top=3, groups=3, keep=2, shared=8),
            "many_experts": O.moe_ff(experts=70, identity=10, top=6, groups=8, keep=3, ff=8, shared=8)}[mlp]
    config = O.zefapel_config([O.gla_layer(mlp=spec)])
    W = O.make_zefapel_weights(config, seed=3)
    if mlp == "negative_choices":
        W["l0.mlp.correction"] = W["l0.mlp.correction"] - 2.0
    toks = tokens_for(config, 60, seed=4)
    engine = make_engine(config, W)
    try:
        assert rel_err(whole(engine, toks), O.zefapel_forward(config, W, toks)) < TOL[torch.float32]
    finally:
        engine.close()


def test_stream_after_every_layer():
    W = O.make_zefapel_weights(MIXED, seed=5)
    toks = tokens_for(MIXED, 29, seed=6)
    streams = []
    want = O.zefapel_forward(MIXED, W, toks, streams)
    engine = make_engine(MIXED, W)
    try:
        assert engine.stats()["layer_runs"] == len(streams) == 4
        engine.set_trace(True)
        engine.begin(0)
        n = engine.step([(0, toks, list(range(len(toks))))])
        for run, ref in enumerate(streams):
            assert rel_err(engine.read_trace(run, len(toks)), ref) < 1e-5, f"layer {run}"
        assert rel_err(engine.logits_host(n), want) < TOL[torch.float32]
        engine.release(0)
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_prefill_against_token_by_token(dtype):
    W = O.make_zefapel_weights(MIXED, seed=7)
    toks = tokens_for(MIXED, 45, seed=8)
    want = O.zefapel_forward(MIXED, W, toks)
    engine = make_engine(MIXED, W, dtype)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[dtype]
        assert rel_err(in_portions(engine, toks, [1]), want) < TOL[dtype]
        assert rel_err(in_portions(engine, toks, [30, 1]), want) < TOL[dtype]  # a prompt, then decoding
    finally:
        engine.close()


@pytest.mark.parametrize("sizes", [[2], [3, 2, 7], [16], [15, 17, 1], [33, 2, 2, 40], [70, 13], [64, 1, 63, 2]])
def test_portions_of_several_sizes(sizes):
    """Portions end inside pages (16 tokens), inside the recurrences' 32-token tiles and inside the gate scan's 64-token tiles."""
    W = O.make_zefapel_weights(MIXED, seed=9)
    toks = tokens_for(MIXED, 150, seed=10)
    engine = make_engine(MIXED, W)
    try:
        assert rel_err(in_portions(engine, toks, sizes), O.zefapel_forward(MIXED, W, toks)) < TOL[torch.float32]
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_unequal_requests_in_one_batch_against_each_alone(dtype):
    """Portions of some requests beside single tokens of others; every request's rows must equal its whole-sequence logits."""
    W = O.make_zefapel_weights(MIXED, seed=11)
    prompts = [tokens_for(MIXED, n, seed=10 + n) for n in (70, 9, 41, 25)]
    want = [O.zefapel_forward(MIXED, W, p) for p in prompts]
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
                if at[i] < len(prompts[i]):
                    n = cuts[i][turn] if turn < len(cuts[i]) else 1
                    if (turn + i) % 5 == 4 and entries:
                        continue  # a request may sit out a step
                    part = prompts[i][at[i]:at[i] + n]
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


def test_pages_and_state_slots_are_used_again():
    """6 pages of 16 tokens and 2 slots serve 6 requests in pairs: a slot's matrix states, normalisers and running maxima start at
    zero again, and pages that held another request's latents are overwritten before they are read."""
    W = O.make_zefapel_weights(MIXED, seed=12)
    engine = make_engine(MIXED, W, page_size=16, num_pages=6, max_batch=2, max_prefill_rows=96)
    try:
        prompts = [tokens_for(MIXED, n, seed=20 + n) for n in (40, 33, 48, 17, 31, 47)]
        want = [O.zefapel_forward(MIXED, W, p) for p in prompts]
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
    finally:
        engine.close()


def test_a_sequence_changes_slots():
    """move(): the recurrent states travel with the sequence, the latent pages stay where they are."""
    W = O.make_zefapel_weights(MIXED, seed=13)
    toks = tokens_for(MIXED, 50, seed=14)
    want = O.zefapel_forward(MIXED, W, toks)
    engine = make_engine(MIXED, W)
    try:
        engine.begin(2)
        a = engine.logits_host(engine.step([(2, toks[:23], list(range(23)))]))
        engine.move(2, 0)
        b = engine.logits_host(engine.step([(0, toks[23:], list(range(27)))]))
        assert rel_err(np.concatenate([a, b], 0), want) < TOL[torch.float32]
        engine.release(0)
    finally:
        engine.close()


def _latent_needle_model():
    """One latent-attention layer whose query token B looks for key token A through ONE unrotated dimension that only these two
    tokens excite (so the match does not depend on distance): the score of (B, A) towers over every other, and a lost, shifted
    or doubled key changes the logits at B by much more than the tolerance."""
    config = O.zefapel_config([O.latent_layer(heads=2, dim=16, vdim=16, rot_dim=8, q_rank=12, kv_rank=24, scale=0.5)], width=64, vocab=50)
    W = O.make_zefapel_weights(config, seed=15)
    A, B = 48, 49
    W["embed"][:, :2] = 0.0
    W["embed"][A] *= 0.05
    W["embed"][B] *= 0.05
    W["embed"][A, 0] = 8.0
    W["embed"][B, 1] = 8.0
    W["l0.norm1.b"][:2] = 0.0                     # the norm has no statistics: channels 0 and 1 stay 0 for every other token
    W["l0.norm1"][:2] = 1.0
    m = "l0.mix."
    W[m + "dkv"][0, :] = 0.0
    W[m + "dkv"][0, 0] = 6.0                      # latent channel 0 <- stream channel 0 (token A only)
    W[m + "dq"][0, :] = 0.0
    W[m + "dq"][0, 1] = 6.0                       # query latent channel 0 <- stream channel 1 (token B only)
    for h in range(2):
        W[m + "uk"][h * 16, :] = 0.0
        W[m + "uk"][h * 16 + 1:(h + 1) * 16, 0] = 0.0
        W[m + "uk"][h * 16, 0] = 4.0              # unrotated key dimension 0 of every head <- latent channel 0 alone
        W[m + "uq"][h * 24, :] = 0.0
        W[m + "uq"][h * 24 + 1:(h + 1) * 24, 0] = 0.0
        W[m + "uq"][h * 24, 0] = 4.0
    W[m + "uv"][:, 0] += 1.0
    for k in W:
        W[k] = torch.from_numpy(np.asarray(W[k], dtype=np.float32)).to(torch.bfloat16).float().numpy()
    return config, W, A, B


def _needle_prompt(config, A, B, n, needle_at, seed):
    toks = tokens_for(config, n, seed=seed, avoid=(A, B))
    toks[needle_at] = A
    toks[-1] = B
    return toks


@pytest.mark.parametrize("needle_at", [0, 3, 15, 16, 17, 31, 32, 250])
@pytest.mark.parametrize("query", ["prompt", "decoded"])
def test_far_keys_and_page_borders(needle_at, query):
    config, W, A, B = _latent_needle_model()
    toks = _needle_prompt(config, A, B, 300, needle_at, 16)
    want = O.zefapel_forward(config, W, toks)[-1]
    other = list(toks)
    other[needle_at] = toks[needle_at - 1] if needle_at else toks[1]
    assert rel_err(O.zefapel_forward(config, W, other)[-1][None], want[None]) > 0.2  # the needle does decide the answer
    engine = make_engine(config, W, page_size=16, num_pages=24, max_batch=1)
    try:
        engine.begin(0)
        if query == "prompt":
            engine.step([(0, toks[:100], [])])
            n = engine.step([(0, toks[100:], [len(toks) - 101])])
        else:
            engine.step([(0, toks[:-1], [])])
            n = engine.step([(0, toks[-1:], [0])])
        assert rel_err(engine.logits_host(n), want[None]) < TOL[torch.float32]
        engine.release(0)
    finally:
        engine.close()


@pytest.mark.parametrize("needle_at", [5, 63, 64, 255, 256, 511, 512, 767, 768])
def test_decoding_over_a_split_key_range(needle_at):
    """From 256 keys on a single-token step splits a row's keys over workgroups and merges the partial sums (here sums of latents,
    projected to values afterwards): the needle sits at the splits' borders."""
    config, W, A, B = _latent_needle_model()
    toks = _needle_prompt(config, A, B, 800, needle_at, 17)
    ref = O.zefapel_forward(config, W, toks)
    engine = make_engine(config, W, page_size=16, num_pages=64, max_batch=2, max_prefill_rows=1024)
    try:
        engine.begin(1)
        engine.step([(1, toks[:-1], [])])
        n = engine.step([(1, toks[-1:], [0])])
        assert rel_err(engine.logits_host(n), ref[-1][None]) < TOL[torch.float32]
        engine.release(1)
    finally:
        engine.close()


def test_a_layer_reads_another_layers_latent_cache():
    """kv_from: the reading layer has its own key / value projections and queries; a needle written by the owning layer is found
    through the reader's projections too, in a prompt cut at the needle and decoded."""
    config, W, A, B = _latent_needle_model()
    config["layers"].append(O.latent_layer(heads=2, dim=16, vdim=16, rot_dim=8, q_rank=12, kv_rank=24, scale=0.5, kv_from=0, mlp=O.dense_ff(32)))
    W2 = O.make_zefapel_weights(config, seed=18)
    W2.update({k: v for k, v in W.items() if not k.startswith("l1.")})
    toks = _needle_prompt(config, A, B, 120, 31, 19)
    want = O.zefapel_forward(config, W2, toks)
    engine = make_engine(config, W2, page_size=16, num_pages=16, max_batch=1)
    try:
        assert engine.stats()["kv_bytes"] == 16 * 16 * 32 * 4  # one pool of [c | rotated part] rows for both layers
        assert rel_err(in_portions(engine, toks, [31, 1, 1, 50, 1]), want) < TOL[torch.float32]
    finally:
        engine.close()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_first_tokens(dtype):
    """The gates' running maximum starts at 0, not at minus infinity: with a very negative input gate the first tokens' read-outs are
    floored by exp(-m) = 1 rather than by the gate itself."""
    config = O.zefapel_config([O.mlstm_layer(), O.gla_layer(), O.latent_layer()])
    W = O.make_zefapel_weights(config, seed=20)
    W["l0.mix.i.b"] = W["l0.mix.i.b"] - 6.0
    toks = tokens_for(config, 4, seed=21)
    want = O.zefapel_forward(config, W, toks)
    engine = make_engine(config, W, dtype)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[dtype]
        assert rel_err(in_portions(engine, toks, [1]), want) < TOL[dtype]
        assert rel_err(whole(engine, toks[:1]), want[:1]) < TOL[dtype]
    finally:
        engine.close()


def test_gates_far_from_zero_over_a_long_sequence():
    """Forget gates near 1 and large input gates: the running maximum climbs and the state's scale e^-m falls far below 1; a chunk
    border must hand the maximum on exactly."""
    config = O.zefapel_config([O.mlstm_layer(heads=2, dim=16, vdim=8, gate_cap=14.0)])
    W = O.make_zefapel_weights(config, seed=22)
    W["l0.mix.i.b"] = W["l0.mix.i.b"] + 9.0
    W["l0.mix.f.b"] = W["l0.mix.f.b"] + 6.0
    toks = tokens_for(config, 400, seed=23)
    want = O.zefapel_forward(config, W, toks)
    engine = make_engine(config, W)
    try:
        assert rel_err(in_portions(engine, toks, [64, 65, 1, 127]), want) < TOL[torch.float32]
    finally:
        engine.close()


ODD = O.zefapel_config([O.latent_layer(heads=3, dim=24, vdim=40, rot_dim=10, q_rank=7, kv_rank=18, base=777.0, scale=0.3, mlp=O.dense_ff(100)),
                        O.gla_layer(heads=6, dim=20, vdim=12, tau=3.0, a_rank=5),
                        O.latent_layer(heads=5, dim=10, vdim=6, rot_dim=10, q_rank=7, kv_rank=18, base=777.0, scale=0.3, kv_from=0, mlp=O.moe_ff(experts=7, identity=2, top=4, groups=3, keep=2, ff=12, shared=20)),
                        O.mlstm_layer(heads=1, dim=72, vdim=33, mlp=O.dense_ff(52)),
                        O.latent_layer(heads=1, dim=8, vdim=8, rot_dim=10, q_rank=4, kv_rank=18, base=777.0, scale=1.0, kv_from=0)],
                       width=88, vocab=97, eps=1e-3, embed_scale=1.25)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_other_sizes(dtype):
    """Sizes that are no multiples of 8, one head, heads * vdim != width, no feed-forward, two readers of one latent cache (with head
    counts and widths of their own), a latent layer first, a recurrence last but one."""
    W = O.make_zefapel_weights(ODD, seed=24)
    toks = tokens_for(ODD, 41, seed=25)
    want = O.zefapel_forward(ODD, W, toks)
    engine = make_engine(ODD, W, dtype)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[dtype]
        assert rel_err(in_portions(engine, toks, [5, 1, 2, 9]), want) < TOL[dtype]
    finally:
        engine.close()


WIDE = O.zefapel_config([O.mlstm_layer(heads=2, dim=32, vdim=64, mlp=O.dense_ff(256)),
                         O.latent_layer(heads=4, dim=32, vdim=32, rot_dim=16, q_rank=64, kv_rank=64, mlp=O.moe_ff(experts=4, identity=2, top=2, groups=3, keep=2, ff=64, shared=64)),
                         O.gla_layer(heads=2, dim=32, vdim=64, a_rank=16, mlp=O.dense_ff(128))], width=128, vocab=200)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_large_chunks_take_the_wide_tile_products(dtype):
    """From 192 rows the bfloat16 products run on the 256-wide tile GEMM (the layer scale rides its float32 epilogue); the same prompt
    in small portions (64-wide tiles, row kernel) must give the same logits."""
    W = O.make_zefapel_weights(WIDE, seed=26)
    toks = tokens_for(WIDE, 300, seed=27)
    want = O.zefapel_forward(WIDE, W, toks)
    engine = make_engine(WIDE, W, dtype, page_size=64, num_pages=8, max_batch=2)
    try:
        assert rel_err(whole(engine, toks), want) < TOL[dtype]
        assert rel_err(in_portions(engine, toks, [250, 3, 40, 1]), want) < TOL[dtype]
    finally:
        engine.close()


def test_long_greedy_decoding_on_the_device_and_graph_replays():
    """160 greedy steps through the captured decode step; the ids are the float64 restatement's greedy choices, and replaying the
    graph gives what eager launches give."""
    W = O.make_zefapel_weights(MIXED, seed=28)
    prompt = tokens_for(MIXED, 21, seed=29)
    engine = make_engine(MIXED, W, page_size=16, num_pages=16, max_batch=2)
    try:
        ids = engine.generate(prompt, 161, slot=1)
        assert engine.stats()["graph_replays"] >= 160 and engine.stats()["graph_captures"] == 1
        full = prompt + ids
        ref = O.zefapel_forward(MIXED, W, full[:-1])
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
    """engine.batch_generate_ids (continuous batching: chunked prefill in a staging slot, adoption into decode slots, retirement):
    every request's ids are what the request alone generates."""
    from tiny_llm_hip.engine import batch_generate_ids

    W = O.make_zefapel_weights(MIXED, seed=30)
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


def _save(tmp_path, config, W):
    from safetensors.torch import save_file

    tmp_path.mkdir(exist_ok=True)
    (tmp_path / "config.json").write_text(json.dumps(config))
    save_file({k: torch.from_numpy(np.asarray(v, dtype=np.float32)).to(torch.bfloat16) for k, v in W.items()}, str(tmp_path / "model.safetensors"))


def test_checkpoint_directory_through_loader_registry_and_command_line(tmp_path):
    W = O.make_zefapel_weights(MIXED, seed=31)
    _save(tmp_path, MIXED, W)
    from tiny_llm_hip import load
    from tiny_llm_hip.models import engine_for

    model, tokenizer = load(str(tmp_path))
    assert tokenizer is None and model.family == "Zefapel"
    assert model.config.layers[1].a_rank == 6  # read from the tensor
    prompt = tokens_for(MIXED, 11, seed=32)
    engine = engine_for(model, dtype=torch.float32, page_size=16, num_pages=8, max_batch=1, max_prefill_rows=32)
    try:
        want = engine.generate(prompt, 6)
    finally:
        engine.close()
    import main as cli

    out = cli.main(["--model", str(tmp_path), "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--dtype", "float32"])
    assert [int(t) for t in out.split()] == want
    out = cli.main(["--model", str(tmp_path), "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "6", "--dtype", "float32",
                    "--sampler-temp", "1e-4", "--sampler-top-k", "1"])
    assert [int(t) for t in out.split()] == want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_replay_command_line(tmp_path, dtype):
    """bin/trace_run on a checkpoint directory: two requests share steps, one ends, and its slot and pages serve a third."""
    import subprocess
    import sys
    from pathlib import Path

    W = O.make_zefapel_weights(MIXED, seed=33)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    _save(model_dir, MIXED, W)
    long, short, third = (tokens_for(MIXED, n, seed=34 + n) for n in (150, 30, 50))
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": long[:100], "want": [0, 99]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": long[100:149], "want": []}, {"id": "y", "tokens": short[:29], "want": [28]}], "end": []},
             {"step": 2, "entries": [{"id": "y", "tokens": short[29:], "want": [0]}, {"id": "x", "tokens": long[149:], "want": [0]}], "end": ["x"]},
             {"step": 3, "entries": [], "end": []},
             {"step": 4, "entries": [{"id": "z", "tokens": third, "want": [49, 3]}, {"id": "y", "tokens": [5], "want": []}], "end": ["y", "z"]}]
    root = Path(__file__).resolve().parent.parent
    run = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", str(model_dir), "--dtype", dtype, "--out", str(out_dir),
                          "--max-tokens", str(192 + 64), "--slots", "2"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                         capture_output=True, text=True, timeout=110)
    assert run.returncode == 0, run.stderr[-2000:]
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    ref_long, ref_short, ref_third = (O.zefapel_forward(MIXED, W, t) for t in (long, short, third))
    got = {i: np.fromfile(out_dir / f"{i}.f32", dtype="<f4").reshape(-1, MIXED["vocab"]) for i in (0, 1, 2, 4)}
    tol = TOL[torch.float32 if dtype == "float32" else torch.bfloat16]
    assert rel_err(got[0], ref_long[[0, 99]]) < tol
    assert rel_err(got[1], ref_short[[28]]) < tol
    assert rel_err(got[2], np.stack([ref_short[29], ref_long[149]])) < tol
    assert rel_err(got[4], ref_third[[49, 3]]) < tol
