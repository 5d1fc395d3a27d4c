"""CPU tier: host logic of the Zefapel family on the layer-list engine -- config reader, tensor table, weight packing, loader
checks -- and the float64 restatement's own consistency (each recurrence against its unrolled sum, latent attention against its
absorbed form, the router against a brute-force choice)."""

import itertools
import json
import math

import numpy as np
import pytest
import torch

import layer_list_oracle as O

CONFIG = O.zefapel_config([O.mlstm_layer(heads=3, dim=24, vdim=40, gate_cap=9.0, mlp=O.dense_ff(100)),
                           O.gla_layer(heads=6, dim=20, vdim=12, tau=3.0, a_rank=5, mlp=O.moe_ff(experts=7, identity=2, top=4, groups=3, keep=2, ff=12, shared=20)),
                           O.latent_layer(heads=5, dim=10, vdim=6, rot_dim=14, q_rank=7, kv_rank=18, base=777.0, scale=0.3, scaling=(3.0, 100, 20.0, 2.0)),
                           O.latent_layer(heads=2, dim=8, vdim=16, rot_dim=14, q_rank=4, kv_rank=18, base=777.0, scale=0.9, scaling=(3.0, 100, 20.0, 2.0), kv_from=2)],
                          width=88, vocab=97, eps=1e-3, embed_scale=1.25)


def test_config_reader_takes_every_size_and_constant_from_the_file():
    from tiny_llm_hip.layer_list import zefapel_config

    cfg = zefapel_config(CONFIG)
    m, g, a, b = cfg.layers
    assert (cfg.family, cfg.width, cfg.vocab, cfg.norm_eps, cfg.embed_scale, cfg.norm_kind, cfg.block, cfg.layer_scale, cfg.loop) == \
        ("Zefapel", 88, 97, 1e-3, 1.25, "dyt", "sequential", True, None)
    assert (m.kind, m.rec_kind, m.heads, m.dim, m.vdim, m.gate_cap, m.ff, m.ff_kind, m.ff_act) == ("linrec", "expgate", 3, 24, 40, 9.0, 100, "gated", "silu")
    assert (g.kind, g.rec_kind, g.heads, g.dim, g.vdim, g.tau, g.a_rank) == ("linrec", "channel", 6, 20, 12, 3.0, -1)  # the rank comes with the tensors
    assert (g.ff_kind, g.ff_act, g.experts, g.identity, g.top, g.groups, g.keep, g.expert_ff, g.shared_ff, g.ff) == ("moe", "relu2", 7, 2, 4, 3, 2, 12, 20, 20 + 7 * 12)
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dim, a.rot_dims, a.q_rank, a.kv_rank, a.rot_base, a.scale, a.kv_from, a.ff) == \
        ("latent", 5, 1, 10, 6, 14, 14, 7, 18, 777.0, 0.3, -1, 0)
    assert a.rot_scaling == (3.0, 100.0, 20.0, 2.0) and (b.kv_from, b.heads, b.vdim, b.scale) == (2, 2, 16, 0.9)
    bad = json.loads(json.dumps(CONFIG))
    bad["layers"][3]["mixer"]["kv_from"] = 3
    with pytest.raises(ValueError, match="earlier layer"):
        zefapel_config(bad)
    bad = json.loads(json.dumps(CONFIG))
    bad["layers"][1]["mlp"]["router"]["groups"]["count"] = 4
    with pytest.raises(ValueError, match="equal groups"):
        zefapel_config(bad)
    with pytest.raises(ValueError, match="unknown mixer type"):
        zefapel_config(dict(CONFIG, layers=[dict(CONFIG["layers"][0], type="window")]))
    with pytest.raises(ValueError, match="lacks"):
        zefapel_config({k: v for k, v in CONFIG.items() if k != "embedding"})


def test_packed_matrices_are_the_named_projections_side_by_side():
    from tiny_llm_hip.layer_list import pack_layer_list, zefapel_config

    W = O.make_zefapel_weights(CONFIG, seed=1)
    cfg = zefapel_config(CONFIG)
    cfg.layers[1].a_rank = 5
    T = {k: torch.from_numpy(np.asarray(v)) for k, v in W.items()}
    packed = pack_layer_list(cfg, T, torch.float32, "cpu")
    h = torch.randn(3, 88)
    m, g, a, b = packed["layers"]
    cat = lambda p, names: torch.cat([h @ T[p + n].T for n in names], 1)
    same = lambda x, y: x.shape == y.shape and torch.allclose(x, y, atol=1e-5)  # (products of differently shaped matrices: summation order)
    assert same(h @ m["w_in"].T, cat("l0.mix.", ("q", "k", "v", "g", "i", "f")))
    assert same(h @ m["w_in2"].T, cat("l0.mlp.", ("gate", "up"))) and torch.equal(m["w_out2"], T["l0.mlp.down"]) and torch.equal(m["w_out"], T["l0.mix.o"])
    assert same(h @ g["w_in"].T, cat("l1.mix.", ("q", "k", "v", "g", "a1")))
    moe_in = cat("l1.mlp.", ["shared.up"] + [f"e{e}.up" for e in range(7)] + ["router", "shared.sg"])  # 20 + 84 + 9 + 1 = 114 -> 120 rows
    assert g["w_in2"].shape[0] == 120 and same((h @ g["w_in2"].T)[:, :114], moe_in) and not g["w_in2"][114:].any()
    assert torch.equal(g["w_out2"], torch.cat([T["l1.mlp.shared.down"]] + [T[f"l1.mlp.e{e}.down"] for e in range(7)], 1))
    assert same(h @ a["w_in"].T, cat("l2.mix.", ("dq", "dkv", "g"))) and same(h @ b["w_in"].T, cat("l3.mix.", ("dq", "g")))
    assert "w_in2" not in a and "ls2" not in a and "ls1" in a and "dkv_norm" not in b
    # per head: the key projection transposed, the value projection as stored
    assert a["uk_t"].shape == (5, 18, 10) and torch.equal(a["uk_t"][3].T, T["l2.mix.uk"][30:40]) and torch.equal(b["uv"][1], T["l3.mix.uv"][16:32])
    assert m["norm_alpha"] == float(W["l0.norm1.alpha"]) and torch.equal(m["norm2_bias"], T["l0.norm2.b"]) and packed["final_norm_alpha"] == float(W["final.norm.alpha"])


def test_loader_checks_names_and_shapes(tmp_path):
    from safetensors.torch import save_file

    from tiny_llm_hip.layer_list import FAMILIES
    from tiny_llm_hip.loader import load, load_weights

    W = {k: torch.from_numpy(np.asarray(v, dtype=np.float32)).to(torch.bfloat16) for k, v in O.make_zefapel_weights(CONFIG, seed=2).items()}
    (tmp_path / "config.json").write_text(json.dumps(CONFIG))
    save_file(W, str(tmp_path / "model.safetensors"))
    model, tokenizer = load(str(tmp_path), device="cpu")
    assert tokenizer is None and model.family == "Zefapel" and set(model.tensors) == set(W) and model.config.layers[1].a_rank == 5
    assert set(FAMILIES["Zefapel"][1](model.config)) == set(W)  # the table names exactly the checkpoint's tensors
    bad = dict(W)
    bad["l2.mix.uk"] = bad["l2.mix.uk"][:, :17].contiguous()
    save_file(bad, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="l2.mix.uk: expected shape"):
        load_weights(tmp_path)
    del bad["l2.mix.uk"]
    save_file(bad, str(tmp_path / "model.safetensors"))
    with pytest.raises(KeyError, match="l2.mix.uk"):
        load_weights(tmp_path)


def test_restatement_is_causal():
    W = O.make_zefapel_weights(CONFIG, seed=3)
    rng = np.random.default_rng(4)
    toks = [int(t) for t in rng.integers(0, 97, 30)]
    full = O.zefapel_forward(CONFIG, W, toks)
    other = toks[:20] + [int(t) for t in rng.integers(0, 97, 10)]
    assert np.allclose(O.zefapel_forward(CONFIG, W, other)[:20], full[:20], atol=1e-9)
    assert np.allclose(O.zefapel_forward(CONFIG, W, toks[:11]), full[:11], atol=1e-9)


def test_matrix_memory_matches_its_unrolled_sum():
    """Without the running maximum: S_t = sum_j exp(i_j + sum_{l=j+1..t} f_l) k_j v_j^T, the same sum for n, and the floor
    exp(-m_t) in the denominator becomes 1 once everything is multiplied through by exp(m_t)."""
    rng = np.random.default_rng(5)
    L, H, D, V = 9, 2, 4, 3
    q, k, v = rng.normal(size=(L, H, D)), rng.normal(size=(L, H, D)), rng.normal(size=(L, H, V))
    li, lf = rng.normal(size=(L, H)) * 2, -np.abs(rng.normal(size=(L, H)))
    got = O.matrix_memory(q, k, v, li, lf)
    for h in range(H):
        for t in range(L):
            w = np.array([math.exp(li[j, h] + lf[j + 1:t + 1, h].sum()) for j in range(t + 1)])
            num = (w[:, None] * v[:t + 1, h] * (k[:t + 1, h] @ q[t, h])[:, None]).sum(0)
            den = abs((w * (k[:t + 1, h] @ q[t, h])).sum())
            m = 0.0
            for j in range(t + 1):
                m = max(lf[j, h] + m, li[j, h])
            assert np.allclose(got[t, h], num * math.exp(-m) / (max(den * math.exp(-m), math.exp(-m)) + 1e-6), rtol=1e-9, atol=1e-12)


def test_gated_linear_attention_matches_its_unrolled_sum():
    rng = np.random.default_rng(6)
    L, H, D, V = 8, 2, 3, 4
    q, k, v = rng.normal(size=(L, H, D)), rng.normal(size=(L, H, D)), rng.normal(size=(L, H, V))
    a = rng.uniform(0.5, 1.0, size=(L, H, D))
    got = O.gated_linear_attention(q, k, v, a)
    for h in range(H):
        for t in range(L):
            want = sum(((q[t, h] * k[j, h] * np.prod(a[j + 1:t + 1, h], axis=0)).sum()) * v[j, h] for j in range(t + 1))
            assert np.allclose(got[t, h], want, atol=1e-12)


def test_latent_attention_equals_its_absorbed_form():
    """Scores through per-head keys W_uk c equal scores of W_uk^T q against the latent itself, and values W_uv c summed with the
    weights equal W_uv applied to the weighted sum of latents: what lets a cache hold only [c | rotated part]."""
    rng = np.random.default_rng(7)
    L, H, D, R, C, V = 7, 3, 4, 2, 5, 6
    q, c, kr = rng.normal(size=(L, H, D + R)), rng.normal(size=(L, C)), rng.normal(size=(L, R))
    uk, uv = rng.normal(size=(H, D, C)), rng.normal(size=(H, V, C))
    k = np.concatenate([np.einsum("hdc,lc->lhd", uk, c), np.broadcast_to(kr[:, None], (L, H, R))], -1)
    naive = O.causal_softmax_attention(q, k, np.einsum("hvc,lc->lhv", uv, c), 0.4)
    qa = np.concatenate([np.einsum("hdc,lhd->lhc", uk, q[..., :D]), q[..., D:]], -1)
    ka = np.broadcast_to(np.concatenate([c, kr], -1)[:, None], (L, H, C + R))
    lat = O.causal_softmax_attention(qa, ka, np.broadcast_to(c[:, None], (L, H, C)), 0.4)
    assert np.allclose(np.einsum("hvc,lhc->lhv", uv, lat), naive, atol=1e-12)


def test_scaled_frequencies():
    f, mult = O.scaled_frequencies(8, 10000.0, None)
    assert mult == 1.0 and np.allclose(f, [1.0, 0.1, 0.01, 0.001])
    # dims 8, base 1e4, original 2 pi 100: where(turns) = 4 log10(100 / turns) / 4 ... fast 100 -> 0, slow 1 -> 2: ramp 0, 1/2, 1, 1
    f, mult = O.scaled_frequencies(8, 10000.0, {"factor": 4.0, "original": 2 * math.pi * 100, "fast": 100.0, "slow": 1.0})
    assert np.allclose(f, [1.0, 0.1 * (0.5 / 4 + 0.5), 0.01 / 4, 0.001 / 4]) and math.isclose(mult, 0.1 * math.log(4.0) + 1.0)


def test_router_against_a_brute_force_choice():
    rng = np.random.default_rng(8)
    for _ in range(50):
        E, groups, keep, top = 15, 5, 2, 4
        z, corr = rng.normal(size=E) * 2, rng.normal(size=E) * 0.3 - (1.0 if _ % 2 else 0.0)
        s = np.exp(z) / np.exp(z).sum()
        choice = s + corr
        gmax = [choice[3 * g:3 * g + 3].max() for g in range(groups)]
        best_groups = max(itertools.combinations(range(groups), keep), key=lambda gs: sorted((gmax[g] for g in gs), reverse=True))
        allowed = [j for j in range(E) if j // 3 in best_groups]
        best = max(itertools.combinations(allowed, top), key=lambda js: sorted((choice[j] for j in js), reverse=True))
        got = O.route(z, corr, top, groups, keep)
        assert sorted(got) == sorted(best) and all(math.isclose(got[j], s[j]) for j in got)
