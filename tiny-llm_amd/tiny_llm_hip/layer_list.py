"""Layer-list model descriptions: decoder-only models given as a list of layers, each a token mixer of some kind plus an
optional feed-forward, served by the layer-list engine (``hybrid_engine.HybridEngine``, include/tinyllm_hybrid.h).

A *family* turns a checkpoint's ``config.json`` into a ``LayerListConfig`` and names its tensors; ``FAMILIES`` is the
registry ``loader.load_weights`` and ``models.engine_for`` consult (key: config.json's ``architecture``).  The engine itself
knows mixer kinds and their options, not families.

Fonapel (the one family so far) -- per layer, with h = norm(x) and one norm for both branches:

    x <- x + m * (mixer(h) + ff(h))            norm: x / sqrt(mean x^2 + eps) * (1 + w)
    ff(h) = W_down gelu_erf(W_up h)

    mixer "attention": grouped-query attention; rotary positions on the first rot.dims dimensions (adjacent pairs, angle
        p * base^(-2i/dims)); then q and k divided by their RMS over the head; scores q.k * scale, causal;
        weights exp(s_j) / (1 + sum_j exp(s_j)); heads * sigmoid(W_g h); W_o.
    mixer "delta": gated delta rule.  q, k (kv_heads x dim), v (heads x vdim) each pass a causal depthwise convolution
        of `conv` taps and SiLU; q, k -> unit vectors (x / sqrt(sum x^2 + 1e-6)), q * dim^-1/2;
        beta = sigmoid(W_b h); g = exp(-exp(A_log) * softplus(W_a h + dt_bias)); per head
        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;
        o / rms(o) * norm * silu(W_g h); W_o.

    loop {start, stop, times}: layers start..stop-1 run `times` times with the same weights and separate caches; each pass
        is entered through x <- W_in [x ; x0] + step[t] (x0 = the embedding output).
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Callable

import torch

__all__ = ["LayerSpec", "LayerListConfig", "FAMILIES", "fonapel_config", "pack_layer_list"]


@dataclass
class LayerSpec:
    kind: str                       # "attention" | "delta"
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    ff: int = 0                     # 0: no feed-forward
    ff_act: str = "gelu_erf"
    # attention
    rot_dims: int = 0
    rot_base: float = 10000.0
    scale: float = 1.0
    qk_unit_rms: bool = False
    sink: bool = False
    gated: bool = False
    # delta
    conv_taps: int = 0
    unit_eps: float = 1e-6


@dataclass
class LayerListConfig:
    family: str
    width: int
    vocab: int
    norm_eps: float
    residual_mult: float
    layers: list[LayerSpec]
    norm_offset: float = 1.0        # norm weights stored around zero are applied as (1 + w)
    loop: tuple[int, int, int] | None = None  # (start, stop, times)
    prefix: Callable[[int], str] = field(default=lambda i: f"l{i}.")

    @property
    def layer_runs(self) -> int:
        if not self.loop:
            return len(self.layers)
        start, stop, times = self.loop
        return len(self.layers) + (stop - start) * (times - 1)


def fonapel_config(config: dict) -> LayerListConfig:
    """config.json of a Fonapel checkpoint -> LayerListConfig.  Every size comes from the file."""
    for key in ("layers", "norm", "residual_mult", "vocab", "width"):
        if key not in config:
            raise ValueError(f"config.json lacks {key!r}")
    layers = []
    for i, entry in enumerate(config["layers"]):
        kind, mc, mlp = entry.get("type"), entry.get("mixer") or {}, entry.get("mlp")
        ff = 0
        if mlp is not None:
            if mlp.get("kind", "dense") != "dense":
                raise ValueError(f"layer {i}: unsupported mlp.kind={mlp.get('kind')!r} (dense only)")
            ff = int(mlp["ff"])
        common = dict(heads=int(mc["heads"]), kv_heads=int(mc["kv_heads"]), dim=int(mc["dim"]), vdim=int(mc["vdim"]), ff=ff)
        if kind == "attention":
            rot = mc.get("rot") or {}
            layers.append(LayerSpec(kind="attention", rot_dims=int(rot.get("dims", 0)), rot_base=float(rot.get("base", 10000.0)),
                                    scale=float(mc["scale"]), qk_unit_rms=True, sink=True, gated=True, **common))
        elif kind == "delta":
            layers.append(LayerSpec(kind="delta", conv_taps=int(mc["conv"]), unit_eps=1e-6, **common))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
    loop = None
    lp = config.get("loop")
    if lp:
        loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        if not (0 <= loop[0] < loop[1] <= len(layers)) or loop[2] < 1:
            raise ValueError(f"loop {lp!r} does not fit {len(layers)} layers")
    return LayerListConfig(family="Fonapel", width=int(config["width"]), vocab=int(config["vocab"]),
                           norm_eps=float(config["norm"]["eps"]), residual_mult=float(config["residual_mult"]),
                           layers=layers, norm_offset=1.0, loop=loop)


def _fonapel_tensor_shapes(cfg: LayerListConfig) -> dict[str, tuple[int, ...]]:
    """Every tensor a Fonapel checkpoint must hold, with its shape (the loader checks the file against this)."""
    W = cfg.width
    want: dict[str, tuple[int, ...]] = {"embed": (cfg.vocab, W), "final.norm": (W,), "head": (cfg.vocab, W)}
    if cfg.loop:
        want["loop.in"] = (W, 2 * W)
        want["loop.step"] = (cfg.loop[2], W)
    for i, L in enumerate(cfg.layers):
        p = cfg.prefix(i)
        want[p + "norm1"] = (W,)
        hv = L.heads * L.vdim
        if L.kind == "attention":
            want.update({p + "mix.q": (L.heads * L.dim, W), p + "mix.k": (L.kv_heads * L.dim, W), p + "mix.v": (L.kv_heads * L.vdim, W),
                         p + "mix.g": (hv, W), p + "mix.o": (W, hv)})
        else:
            qk = L.kv_heads * L.dim
            want.update({p + "mix.q": (qk, W), p + "mix.k": (qk, W), p + "mix.v": (hv, W), p + "mix.g": (hv, W), p + "mix.o": (W, hv),
                         p + "mix.q.conv": (qk, L.conv_taps), p + "mix.k.conv": (qk, L.conv_taps), p + "mix.v.conv": (hv, L.conv_taps),
                         p + "mix.a": (L.heads, W), p + "mix.b": (L.heads, W), p + "mix.A_log": (L.heads,), p + "mix.dt_bias": (L.heads,),
                         p + "mix.norm": (L.vdim,)})
        if L.ff:
            want.update({p + "mlp.up": (L.ff, W), p + "mlp.down": (W, L.ff)})
    return want


# architecture name (config.json) -> (config reader, tensor table)
FAMILIES: dict[str, tuple[Callable[[dict], LayerListConfig], Callable[[LayerListConfig], dict]]] = {
    "Fonapel": (fonapel_config, _fonapel_tensor_shapes),
}


def pack_layer_list(cfg: LayerListConfig, tensors: dict[str, torch.Tensor], dtype: torch.dtype, device: Any) -> dict:
    """The engine's weight layout from a family's named tensors: per layer one input matrix (every projection that reads
    the normed input, rows concatenated: q | k | v | gate | [a | b] | up) and one output matrix ([W_o | W_down] side by
    side); vectors in float32.  Matrices are cast to ``dtype`` (bfloat16 as stored, or float32)."""
    def mat(name):
        return tensors[name].to(device=device, dtype=dtype)

    def vec(name):
        return tensors[name].to(device=device, dtype=torch.float32).contiguous()

    packed = {"embed": mat("embed").contiguous(), "head": mat("head").contiguous(), "final_norm": vec("final.norm"), "layers": []}
    if cfg.loop:
        packed["loop_in"] = mat("loop.in").contiguous()
        packed["loop_step"] = vec("loop.step")
    for i, L in enumerate(cfg.layers):
        p = cfg.prefix(i)
        rows = [mat(p + "mix.q"), mat(p + "mix.k"), mat(p + "mix.v")]
        if L.kind == "delta" or L.gated:
            rows.append(mat(p + "mix.g"))
        entry: dict[str, Any] = {"norm": vec(p + "norm1")}
        if L.kind == "delta":
            rows += [mat(p + "mix.a"), mat(p + "mix.b")]
            entry["conv"] = torch.cat([vec(p + "mix.q.conv"), vec(p + "mix.k.conv"), vec(p + "mix.v.conv")], 0).contiguous()
            entry["a_log"], entry["dt_bias"], entry["out_norm"] = vec(p + "mix.A_log"), vec(p + "mix.dt_bias"), vec(p + "mix.norm")
        out = [mat(p + "mix.o")]
        if L.ff:
            rows.append(mat(p + "mlp.up"))
            out.append(mat(p + "mlp.down"))
        entry["w_in"] = torch.cat(rows, 0).contiguous()
        entry["w_out"] = torch.cat(out, 1).contiguous()
        packed["layers"].append(entry)
    return packed
