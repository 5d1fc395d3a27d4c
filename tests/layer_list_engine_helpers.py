"""Shared helpers of the layer-list engine's GPU tests: build an engine from a config dict and named arrays, run a sequence whole
or in portions, compare rows of logits."""

from types import SimpleNamespace

import numpy as np
import torch

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
