"""Small Milenex configurations and model folders for the tests.

The folders are written here with draws of the tests' own (not by the framework's random-weights mode): matrices
N(0, 1/in) so that activations stay of order one through every layer, norm weights spread visibly around zero, shifts
spread over (0, 1), convolutions whose earlier taps count, sinks of order one, distance penalties that matter within a
window, mixing matrices near the identity with visible off-diagonal terms, routers whose scores are spread out and
corrections that change the choice, and limits that the experts' branches reach.
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, Optional

import torch


def attention(heads, kv_heads, dim, vdim, window=None, conv=None, dims=None, base=10000.0, scale=None, mlp=None):
    mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else 1.5 * dim ** -0.5)
    if window is not None:
        mixer["mask"] = dict(size=window)
    if conv is not None:
        mixer["conv"] = conv
    if dims is not None:
        mixer["rot"] = dict(base=base, dims=dims)
    return dict(type="attention", mixer=mixer, mlp=mlp)


def attention_2(heads, kv_heads, dim, vdim, window=None, scale=None, mlp=None):
    mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else 1.5 * dim ** -0.5)
    if window is not None:
        mixer["mask"] = dict(size=window)
    return dict(type="attention_2", mixer=mixer, mlp=mlp)


def dense(ff):
    return dict(kind="dense", ff=ff)


def moe(experts, top, ff, limit, groups=None, shared=None):
    router = dict(experts=experts, top=top)
    if groups is not None:
        router["groups"] = dict(count=groups[0], keep=groups[1])
    out = dict(kind="moe", expert=dict(ff=ff, limit=limit), router=router)
    if shared is not None:
        out["shared"] = dict(ff=shared[0], limit=shared[1])
    return out


# Configurations that differ in every size and constant: one key/value head for all query heads, one for each, and
# groups; head sizes that are no multiple of four, beyond 64 and beyond a wave; more mixing heads than a workgroup has
# waves; rotation of a whole head, of a part, of none; convolutions of one to five taps or none; windows from 6 to 70
# tokens (inside one 64-key tile, across two) and none; layers without a feed-forward, dense ones, experts with one group
# and several, one chosen expert and all of the kept groups', with and without a shared expert; no loop, a loop over the
# first layers, over the middle, over the last, of one to three passes.
CONFIGS: Dict[str, dict] = {
    "A": dict(architecture="Milenex", vocab=96, width=48, norm=dict(eps=1e-5), loop=dict(start=0, stop=2, times=2), layers=[
        attention(4, 2, 12, 20, window=9, conv=3, dims=8, base=500.0, scale=0.5, mlp=dense(80)),
        attention_2(3, 3, 10, 6, window=11, scale=0.6, mlp=moe(6, 2, 24, 1.0, groups=(3, 2), shared=(16, 0.7))),
        attention_2(6, 2, 8, 12, window=20, mlp=None),
        attention(2, 1, 16, 8, window=33, conv=2, dims=16, base=50.0, mlp=moe(4, 1, 20, 0.8))]),
    "B": dict(architecture="Milenex", vocab=131, width=64, norm=dict(eps=1e-6), layers=[
        attention_2(6, 1, 24, 130, window=50, mlp=dense(96)),
        attention(2, 2, 40, 24, window=70, conv=5, dims=24, mlp=None),
        attention(3, 1, 72, 200, window=17, conv=1, dims=72, base=1000.0, scale=0.2, mlp=dense(40))]),
    "C": dict(architecture="Milenex", vocab=77, width=42, norm=dict(eps=1e-3), loop=dict(start=1, stop=2, times=3), layers=[
        attention(5, 1, 7, 5, window=6, conv=4, dims=6, base=30.0, scale=0.7, mlp=moe(5, 5, 12, 0.5, shared=(9, 2.0))),
        attention_2(12, 4, 6, 9, window=70, mlp=moe(8, 3, 10, 1.5, groups=(4, 2))),
        attention_2(2, 2, 5, 3, mlp=dense(30))]),                                    # no window: every key
    "D": dict(architecture="Milenex", vocab=64, width=32, norm=dict(eps=1e-5), loop=dict(start=1, stop=3, times=2), layers=[
        attention(2, 2, 8, 8, mlp=dense(48)),                                      # no window, no convolution, no rotation
        attention(4, 4, 4, 3, window=64, conv=2, dims=2, base=7.0, scale=1.1, mlp=None),
        attention_2(18, 6, 8, 12, window=65, scale=0.5, mlp=moe(3, 2, 16, 1.0, groups=(1, 1), shared=(8, 1.0)))]),
    # ones and equals: a window of one key (the row's own) and of two, one tap, one head, one expert a group with every group
    # kept, one expert in all, a loop over every layer, a rotation of one pair
    "E": dict(architecture="Milenex", vocab=50, width=24, norm=dict(eps=1e-6), loop=dict(start=0, stop=4, times=2), layers=[
        attention_2(1, 1, 4, 4, window=1, scale=1.0, mlp=moe(4, 1, 8, 2.0, groups=(4, 4))),
        attention(1, 1, 2, 1, window=2, conv=1, dims=2, base=2.0, scale=1.0, mlp=moe(1, 1, 8, 1.0, shared=(8, 1.0))),
        attention_2(4, 4, 4, 4, window=128, mlp=dense(8)),
        attention(3, 3, 6, 2, window=1, conv=2, dims=4, mlp=moe(6, 2, 8, 1.0, groups=(6, 2)))]),
}
SEEDS = {"A": 13, "B": 24, "C": 35, "D": 46, "E": 57}


def every_expert(config: dict) -> dict:
    """The configuration with routers that have nothing to choose: one group, every expert used, each still weighed by its
    score.  For runs in reduced precision: where a choice is a close call (a few rows in a hundred, with any weights), a
    rounding turns it, and the rows after it are then another model's."""
    import copy
    out = copy.deepcopy(config)
    for layer in out["layers"]:
        mlp = layer.get("mlp")
        if mlp is not None and mlp["kind"] == "moe":
            mlp["router"]["top"] = mlp["router"]["experts"]
            mlp["router"].pop("groups", None)
    return out


def tensors_for(config: dict, seed: int, query_factor: float = 1.0) -> Dict[str, torch.Tensor]:
    gen = torch.Generator().manual_seed(seed)

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=gen) * std + mean

    def uniform(*shape, lo=0.0, hi=1.0):
        return torch.rand(*shape, generator=gen) * (hi - lo) + lo

    def matrix(out, inn, factor=1.0):
        return normal(out, inn, std=factor / math.sqrt(inn))
    W = config["width"]
    t = {"embed": normal(config["vocab"], W), "head": matrix(config["vocab"], W), "final.norm": normal(W, std=0.2)}

    def unit(prefix, ff):
        t[prefix + "gate"], t[prefix + "up"], t[prefix + "down"] = matrix(ff, W, 1.5), matrix(ff, W, 1.5), matrix(W, ff)
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        t[p + "norm1"], t[p + "shift"] = normal(W, std=0.2), uniform(W, lo=0.05, hi=0.95)
        H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = matrix(H * d, W, query_factor), matrix(G * d, W), matrix(G * e, W)
        t[p + "mix.o"], t[p + "mix.sink"] = matrix(W, H * e), normal(H, mean=0.5)
        if layer["type"] == "attention":
            taps = m.get("conv")
            if taps:
                for name, channels in (("q", H * d), ("k", G * d), ("v", G * e)):
                    w = normal(channels, taps, std=0.5)
                    w[:, -1] += 1.0
                    t[p + f"mix.{name}.conv"] = w
        else:
            t[p + "mix.r1"], t[p + "mix.r2"] = uniform(H, lo=0.2, hi=1.0), uniform(H, lo=0.1, hi=2.0)
            t[p + "mix.talk"] = torch.eye(H) * 0.8 + normal(H, H, std=0.25)
            t[p + "mix.g"] = matrix(H, W, 1.5)
        mlp = layer["mlp"]
        if mlp is None:
            continue
        t[p + "norm2"] = normal(W, std=0.2)
        if mlp["kind"] == "dense":
            t[p + "mlp.up"], t[p + "mlp.down"] = matrix(mlp["ff"], W, 1.5), matrix(W, mlp["ff"])
            continue
        E = mlp["router"]["experts"]
        t[p + "mlp.router"], t[p + "mlp.correction"] = matrix(E, W, 2.0), normal(E, std=0.15)
        for j in range(E):
            unit(p + f"mlp.e{j}.", mlp["expert"]["ff"])
        if mlp.get("shared") is not None:
            unit(p + "mlp.shared.", mlp["shared"]["ff"])
            t[p + "mlp.shared.sg"] = matrix(1, W, 1.5)
    return t


def write_folder(root, name: str, dtype: str, config: Optional[dict] = None, seed: Optional[int] = None, tag: str = "", **draw) -> str:
    """config.json and model.safetensors of configuration ``name`` (or of ``config``) under ``root``."""
    from safetensors.torch import save_file
    config = config or CONFIGS[name]
    out = os.path.join(str(root), f"milenex_{name}_{dtype}{tag}")
    if not os.path.exists(os.path.join(out, "model.safetensors")):
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "config.json"), "w", encoding="utf-8") as fh:
            json.dump(config, fh)
        store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
        tensors = tensors_for(config, SEEDS.get(name, 1) if seed is None else seed, **draw)
        save_file({k: v.to(store).contiguous() for k, v in tensors.items()}, os.path.join(out, "model.safetensors"))
    return out
