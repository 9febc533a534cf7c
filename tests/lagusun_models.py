"""Small Lagusun configurations and model folders for the tests.

The folders are written here with draws of the tests' own (not by the framework's random-weights mode): matrices
N(0, 1/in) so that activations stay of order one through every layer, norm weights and the sublayers' channel scales
spread visibly around one, biases of a size that counts, head biases of the sigmoid weights below zero (a window's keys
add up, they are not normalised), a map back into the loop that keeps the stream's size, pass vectors of order 0.3,
routers whose scores are spread out and corrections that change the choice.
"""
from __future__ import annotations

import copy
import json
import math
import os
from typing import Dict, Optional

import torch


def attention(heads, kv_heads, dim, block=None, dims=None, base=10000.0, scale=None, mlp=None):
    mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=scale if scale is not None else 1.5 * dim ** -0.5)
    if block is not None:
        mixer["mask"] = dict(size=block)
    if dims is not None:
        mixer["rot"] = dict(base=base, dims=dims)
    return dict(type="attention", mixer=mixer, mlp=mlp)


def attention_2(heads, kv_heads, dim, vdim, window=None, dims=None, base=10000.0, scaling=None, softcap=None, scale=None, mlp=None):
    mixer = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale if scale is not None else 4.0 * dim ** -0.5)
    if window is not None:
        mixer["mask"] = dict(size=window)
    if dims is not None:
        mixer["rot"] = dict(base=base, dims=dims)
        if scaling is not None:
            mixer["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    if softcap is not None:
        mixer["softcap"] = softcap
    return dict(type="attention_2", mixer=mixer, mlp=mlp)


def moe(experts, top, ff, scale=None, shared=None):
    router = dict(experts=experts, top=top)
    if scale is not None:
        router["scale"] = scale
    return dict(kind="moe", expert=dict(ff=ff), router=router, shared=dict(ff=shared) if shared else None)


# Configurations that differ in every size and constant: one key/value head for all query heads, one for each, and
# groups; head sizes that are no multiple of four, beyond 64 and beyond a wave; values of another size than the keys;
# rotation of a whole head, of a part, of one pair, of none, with frequencies scaled in all three of their ranges and
# not at all; blocks and windows of 1 to 100 positions (inside one 64-key tile, across two, no multiple of a page) and
# none; score caps that bend the scores and none; norms in one to four groups; layers without a feed-forward, one to
# eight experts of which one to all are chosen, with and without a shared expert, with and without a factor on the
# weights; no loop, a loop from the first layer, over the middle, over the last layers, over all, of one to three
# passes; an embedding factor of one (absent) and others.
CONFIGS: Dict[str, dict] = {
    "A": dict(architecture="Lagusun", vocab=96, width=48, norm=dict(eps=1e-5, groups=3), embedding=dict(scale=2.5),
              loop=dict(start=1, stop=3, times=2), layers=[
        attention(4, 2, 12, block=9, dims=8, base=500.0, scale=0.5, mlp=moe(6, 2, 24, scale=1.5, shared=16)),
        attention_2(3, 3, 10, 6, window=11, dims=10, base=100.0, scaling=(4.0, 1.0, 3.0, 40), softcap=3.0, mlp=moe(4, 1, 20)),
        attention_2(6, 2, 8, 12, window=20, dims=4, base=30.0, softcap=30.0, scale=0.6, mlp=None),
        attention(2, 1, 16, block=33, dims=16, base=50.0, mlp=moe(5, 5, 12, scale=0.5, shared=9))]),
    "B": dict(architecture="Lagusun", vocab=131, width=64, norm=dict(eps=1e-6, groups=1), layers=[
        attention_2(6, 1, 24, 130, window=50, dims=12, base=1000.0, scaling=(6.0, 1.0, 3.0, 64), mlp=moe(3, 2, 40, shared=24)),
        attention(2, 2, 40, block=70, dims=24, mlp=None),
        attention(3, 1, 72, block=17, dims=72, base=1000.0, scale=0.2, mlp=moe(8, 3, 16, scale=2.5))]),
    "C": dict(architecture="Lagusun", vocab=77, width=42, norm=dict(eps=1e-3, groups=2), embedding=dict(scale=0.7),
              loop=dict(start=0, stop=1, times=3), layers=[
        attention(5, 1, 7, block=6, dims=6, base=30.0, scale=0.7, mlp=moe(5, 2, 12, shared=9)),
        attention_2(12, 4, 6, 9, window=70, dims=6, base=20.0, scaling=(2.0, 0.5, 2.0, 16), softcap=1.5, mlp=moe(8, 3, 10, scale=3.0)),
        attention_2(2, 2, 5, 3, mlp=moe(2, 1, 30))]),                                # no window, no rotation, no cap
    "D": dict(architecture="Lagusun", vocab=64, width=32, norm=dict(eps=1e-5, groups=4), embedding=dict(scale=4.0),
              loop=dict(start=1, stop=3, times=2), layers=[
        attention(2, 2, 8, mlp=moe(3, 2, 16)),                                       # no block: every key; no rotation
        attention(4, 4, 4, block=64, dims=2, base=7.0, scale=1.1, mlp=None),
        attention_2(18, 6, 8, 12, window=65, dims=8, base=300.0, scaling=(16.0, 2.0, 8.0, 100), scale=0.5, mlp=moe(3, 3, 16, shared=8))]),
    # ones and equals: a block and a window of one key (the row's own) and of two, one head, one expert in all, a loop
    # over every layer, a loop of one pass, a rotation of one pair, one group
    "E": dict(architecture="Lagusun", vocab=50, width=24, norm=dict(eps=1e-6, groups=1), embedding=dict(scale=1.0),
              loop=dict(start=0, stop=4, times=2), layers=[
        attention_2(1, 1, 4, 4, window=1, dims=2, base=2.0, scale=1.0, mlp=moe(4, 1, 8)),
        attention(1, 1, 2, block=2, dims=2, base=2.0, scale=1.0, mlp=moe(1, 1, 8, shared=8)),
        attention_2(4, 4, 4, 4, window=100, softcap=0.5, mlp=moe(2, 2, 8, scale=1.0)),
        attention(3, 3, 6, block=1, dims=4, mlp=moe(6, 2, 8))]),
    "F": dict(architecture="Lagusun", vocab=40, width=20, norm=dict(eps=1e-4, groups=5), loop=dict(start=1, stop=2, times=1), layers=[
        attention_2(2, 1, 6, 10, window=2, dims=6, base=9.0, mlp=moe(3, 1, 6, shared=4)),
        attention(2, 1, 10, block=100, dims=10, base=9.0, mlp=moe(4, 2, 6))]),
    # widths at which the products take their matrix-core forms: multiples of 64 throughout, a prompt of a few hundred rows
    "G": dict(architecture="Lagusun", vocab=300, width=192, norm=dict(eps=1e-5, groups=2), embedding=dict(scale=8.0),
              loop=dict(start=0, stop=2, times=2), layers=[
        attention(6, 3, 32, block=48, dims=16, base=5000.0, mlp=moe(4, 2, 128, scale=1.5, shared=64)),
        attention_2(4, 2, 48, 64, window=40, dims=32, base=5000.0, scaling=(4.0, 1.0, 2.0, 128), softcap=20.0, mlp=moe(8, 2, 64, shared=128)),
        attention_2(8, 8, 16, 16, window=130, dims=16, softcap=10.0, mlp=moe(4, 3, 64))]),
}
SEEDS = {"A": 13, "B": 24, "C": 35, "D": 46, "E": 57, "F": 68, "G": 79}


def every_expert(config: dict) -> dict:
    """The configuration with routers that have nothing to choose: every expert used, each still weighed by its score.
    For runs in reduced precision: where a choice is a close call (a few rows in a hundred, with any weights), a rounding
    turns it, and the rows after it are then another model's."""
    out = copy.deepcopy(config)
    for layer in out["layers"]:
        if layer.get("mlp") is not None:
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return out


def passes(config: dict) -> int:
    loop = config.get("loop")
    return loop["times"] if loop and loop["start"] < loop["stop"] else 0


def tensors_for(config: dict, seed: int, query_factor: float = 1.0) -> Dict[str, torch.Tensor]:
    gen = torch.Generator().manual_seed(seed)

    def normal(*shape, std=1.0, mean=0.0):
        return torch.randn(*shape, generator=gen) * std + mean

    def matrix(out, inn, factor=1.0):
        return normal(out, inn, std=factor / math.sqrt(inn))
    W = config["width"]
    t = {"embed": normal(config["vocab"], W, std=1.0 / float(config.get("embedding", {}).get("scale", 1.0))),
         "head": matrix(config["vocab"], W), "final.norm": normal(W, std=0.2, mean=1.0)}
    if passes(config):
        t["loop.in"] = torch.cat([torch.eye(W) * 0.7 + matrix(W, W, 0.5), matrix(W, W, 0.7)], dim=1)
        t["loop.step"] = normal(passes(config), W, std=0.3)
    for i, layer in enumerate(config["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        t[p + "norm1"], t[p + "ls1"] = normal(W, std=0.2, mean=1.0), normal(W, std=0.3, mean=1.0)
        H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.o"] = matrix(H * d, W, query_factor), matrix(G * d, W), matrix(W, H * e)
        if layer["type"] == "attention":
            t[p + "mix.q.norm"], t[p + "mix.k.norm"] = normal(H * d, std=0.3, mean=1.0), normal(G * d, std=0.3, mean=1.0)
        else:
            t[p + "mix.v"] = matrix(G * e, W)
            t[p + "mix.q.b"], t[p + "mix.k.b"], t[p + "mix.v.b"] = normal(H * d, std=0.3), normal(G * d, std=0.3), normal(G * e, std=0.3)
            t[p + "mix.pb"] = normal(H, std=0.7, mean=-2.0)
        mlp = layer["mlp"]
        if mlp is None:
            continue
        t[p + "norm2"], t[p + "ls2"] = normal(W, std=0.2, mean=1.0), normal(W, std=0.3, mean=1.0)
        E = mlp["router"]["experts"]
        t[p + "mlp.router"], t[p + "mlp.correction"] = matrix(E, W, 2.0), normal(E, std=0.15)
        units = [(f"e{j}.", mlp["expert"]["ff"]) for j in range(E)] + ([("shared.", mlp["shared"]["ff"])] if mlp.get("shared") else [])
        for name, ff in units:
            t[p + "mlp." + name + "up"], t[p + "mlp." + name + "down"] = matrix(ff, W, 1.5), matrix(W, ff)
    return t


def write_folder(root, name: str, dtype: str, config: Optional[dict] = None, seed: Optional[int] = None, tag: str = "", **draw) -> str:
    """config.json and model.safetensors of configuration ``name`` (or of ``config``) under ``root``."""
    from safetensors.torch import save_file
    config = config or CONFIGS[name]
    out = os.path.join(str(root), f"lagusun_{name}_{dtype}{tag}")
    if not os.path.exists(os.path.join(out, "model.safetensors")):
        os.makedirs(out, exist_ok=True)
        with open(os.path.join(out, "config.json"), "w", encoding="utf-8") as fh:
            json.dump(config, fh)
        store = torch.bfloat16 if dtype == "bfloat16" else torch.float32
        tensors = tensors_for(config, SEEDS.get(name, 1) if seed is None else seed, **draw)
        save_file({k: v.to(store).contiguous() for k, v in tensors.items()}, os.path.join(out, "model.safetensors"))
    return out
