"""CPU tier: host logic around the layer-list engine -- the config reader and weight packing of the Fonapel family, the
checkpoint loader's checks, the float64 restatement's own consistency, and the scheduler's mixed steps on a stand-in engine."""

import json

import numpy as np
import pytest
import torch

import layer_list_oracle as O


def test_config_reader_takes_every_size_from_the_file():
    from tiny_llm_hip.layer_list import fonapel_config

    config = O.fonapel_config([O.attention_layer(heads=6, kv_heads=2, dim=24, vdim=40, rot_dims=10, base=777.0, scale=0.3, ff=100),
                               O.delta_layer(heads=6, kv_heads=3, dim=20, vdim=12, conv=5, ff=0)], width=88, vocab=97, loop=(1, 2, 4),
                              eps=1e-3, residual_mult=0.7)
    cfg = fonapel_config(config)
    a, d = cfg.layers
    assert (cfg.width, cfg.vocab, cfg.norm_eps, cfg.residual_mult, cfg.loop, cfg.layer_runs) == (88, 97, 1e-3, 0.7, (1, 2, 4), 5)
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.rot_dims, a.rot_base, a.scale, a.ff) == ("attention", 6, 2, 24, 40, 10, 777.0, 0.3, 100)
    assert a.sink and a.gated and a.qk_unit_rms
    assert (d.kind, d.heads, d.kv_heads, d.dim, d.vdim, d.conv_taps, d.ff) == ("delta", 6, 3, 20, 12, 5, 0)
    with pytest.raises(ValueError, match="unknown mixer type"):
        fonapel_config(dict(config, layers=[dict(config["layers"][0], type="window")]))
    with pytest.raises(ValueError, match="loop"):
        fonapel_config(dict(config, loop={"start": 1, "stop": 3, "times": 2}))
    with pytest.raises(ValueError, match="lacks"):
        fonapel_config({k: v for k, v in config.items() if k != "width"})


def test_packed_matrices_are_the_named_projections_side_by_side():
    from tiny_llm_hip.layer_list import fonapel_config, pack_layer_list

    config = O.fonapel_config([O.delta_layer(), O.attention_layer()], loop=(0, 2, 2))
    W = O.make_fonapel_weights(config, seed=1)
    packed = pack_layer_list(fonapel_config(config), {k: torch.from_numpy(v) for k, v in W.items()}, torch.float32, "cpu")
    h = torch.randn(3, config["width"])
    d, a = packed["layers"]
    want = torch.cat([h @ torch.from_numpy(W[f"l0.mix.{n}"]).T for n in ("q", "k", "v", "g", "a", "b")] + [h @ torch.from_numpy(W["l0.mlp.up"]).T], 1)
    assert torch.equal(h @ d["w_in"].T, want)
    want = torch.cat([h @ torch.from_numpy(W[f"l1.mix.{n}"]).T for n in ("q", "k", "v", "g")] + [h @ torch.from_numpy(W["l1.mlp.up"]).T], 1)
    assert torch.equal(h @ a["w_in"].T, want)
    o, act = torch.randn(3, W["l1.mix.o"].shape[1]), torch.randn(3, W["l1.mlp.down"].shape[1])
    both = torch.cat([o, act], 1) @ a["w_out"].T
    assert torch.allclose(both, o @ torch.from_numpy(W["l1.mix.o"]).T + act @ torch.from_numpy(W["l1.mlp.down"]).T, atol=1e-5)
    assert d["conv"].shape == (2 * 2 * 16 + 4 * 24, 3) and packed["loop_in"].shape == (64, 128) and packed["loop_step"].shape == (2, 64)


def test_loader_checks_names_and_shapes(tmp_path):
    from safetensors.torch import save_file

    from tiny_llm_hip.loader import load, load_weights

    config = O.fonapel_config([O.attention_layer(), O.delta_layer()])
    W = {k: torch.from_numpy(v).to(torch.bfloat16) for k, v in O.make_fonapel_weights(config, seed=2).items()}
    (tmp_path / "config.json").write_text(json.dumps(config))
    save_file(W, str(tmp_path / "model.safetensors"))
    model, tokenizer = load(str(tmp_path), device="cpu")
    assert tokenizer is None and model.family == "Fonapel" and model.dtype == torch.bfloat16 and set(model.tensors) == set(W)
    assert load_weights(tmp_path, dtype=torch.float32).dtype == torch.float32
    bad = dict(W)
    bad["l1.mix.q.conv"] = bad["l1.mix.q.conv"][:, :2].contiguous()
    save_file(bad, str(tmp_path / "model.safetensors"))
    with pytest.raises(ValueError, match="l1.mix.q.conv: expected shape"):
        load_weights(tmp_path)
    del bad["l1.mix.q.conv"]
    save_file(bad, str(tmp_path / "model.safetensors"))
    with pytest.raises(KeyError, match="l1.mix.q.conv"):
        load_weights(tmp_path)


def test_restatement_is_causal_and_its_recurrence_matches_the_unrolled_sum():
    config = O.fonapel_config([O.delta_layer(), O.attention_layer()], loop=(0, 2, 2))
    W = O.make_fonapel_weights(config, seed=3)
    toks = [3, 17, 99, 4, 4, 56, 23, 8, 71]
    full = O.fonapel_forward(config, W, toks)
    assert np.allclose(O.fonapel_forward(config, W, toks[:5]), full[:5], atol=1e-12)
    # with decay 1 and beta 1 on orthonormal keys the delta rule stores each value under its key
    k = np.eye(4)[:, None, :]
    v = np.arange(12.0).reshape(4, 1, 3)
    out = O.gated_delta_rule(k, k, v, np.ones((4, 1)), np.ones((4, 1)))
    assert np.allclose(out, v)
    # one position: weight exp(s) / (1 + exp(s))
    o = O.sink_attention(np.ones((1, 1, 2)), np.ones((1, 1, 2)), np.full((1, 1, 1), 5.0), 0.5)
    assert np.isclose(o[0, 0, 0], 5.0 * np.e / (1 + np.e))


class _StandInEngine:
    """The request-level surface of the engines with a toy rule in place of a model: the next id of a slot is a hash of every
    id the slot has seen, so a token fed to the wrong slot, twice or not at all changes the output."""

    supports_mixed_steps = True
    vocab = 1009

    def __init__(self, max_batch):
        self.max_batch, self.hist, self.pending, self.mixed_calls = max_batch, {}, {}, 0

    def _next(self, slot):
        h = 7
        for t in self.hist[slot]:
            h = (h * 31 + t + 1) % self.vocab
        return h

    def begin(self, slot):
        assert slot not in self.hist
        self.hist[slot] = []

    def release(self, slot):
        del self.hist[slot]
        self.pending.pop(slot, None)

    def move(self, src, dst):
        assert dst not in self.hist
        self.hist[dst] = self.hist.pop(src)
        self.pending[dst] = self.pending.pop(src)

    def prefill(self, slot, tokens, chunk=None, want_logits=True):
        self.hist[slot] += list(tokens)
        if want_logits:
            self.pending[slot] = self._next(slot)

    def read_tokens(self, slot, count):
        assert count == 1
        return [self.pending[slot]]

    def decode(self, steps, batch=None):
        assert steps == 1
        for s in range(batch):
            if s in self.hist:
                self.hist[s].append(self.pending[s])
                self.pending[s] = self._next(s)

    def read_pending(self, count):
        return [self.pending.get(s, 0) for s in range(count)]

    def step(self, entries):
        self.mixed_calls += 1
        self._rows = []
        for slot, toks, want in entries:
            for i, t in enumerate(toks):
                self.hist[slot].append(t)
                if i in want:
                    self.pending[slot] = self._next(slot)
                    self._rows.append(self.pending[slot])
        return len(self._rows)

    def argmax(self, rows):
        return self._rows[:rows]


@pytest.mark.parametrize("mixed", [True, False])
def test_scheduler_mixed_steps_feed_every_slot_its_own_tokens(mixed, built_libs):
    from tiny_llm_hip.engine import batch_generate_ids

    prompts = [[5, 6, 7], list(range(40)), [9] * 17, [1, 2], list(range(100, 133))]
    limits = [9, 5, 12, 7, 3]

    def alone(p, n):
        e = _StandInEngine(1)
        e.begin(0)
        e.prefill(0, p)
        out = [e.pending[0]]
        for _ in range(n - 1):
            e.decode(1, batch=1)
            out.append(e.pending[0])
        return out

    engine = _StandInEngine(4)
    done = dict(batch_generate_ids(engine, prompts, limits, batch_size=3, prefill_step=8, mixed_steps=mixed))
    assert {i: done[i] for i in range(5)} == {i: alone(p, n) for i, (p, n) in enumerate(zip(prompts, limits))}
    assert (engine.mixed_calls > 0) == mixed and not engine.hist
