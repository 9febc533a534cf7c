"""A plain, slow implementation of the Lagusun decoder for the tests.

Whole sequences, no cache, no state carried between calls, one function for each mechanism, written from the
design's equations and sharing no code with the engine: it reads config.json with ``json`` and the weights with
the ``safetensors`` package.  Arithmetic is float64 by default.

The design, in this file's notation (a linear weight is stored [out, in] and applied as W x; t counts a
sequence's tokens from 0):

  embedding  x0 = E[token] * c                                 (c: ``embedding.scale``)
  layer      x += a1 * mixer(N1(x));  x += a2 * ff(N2(x))     (a1, a2: a vector each, element by element; a layer may
                                                                have no ff)
  N(v)       v cut into n equal runs of neighbouring channels; a run r becomes r / sqrt(mean(r^2) + eps); then all times g
  loop       layers a..b-1 run n times in a row with the same weights (each pass with a cache of its own); right before
             the first layer of pass t (t = 0 too)  x = W_in [x; x0] + s_t
  rotation   of a head's first ``dims`` elements, in two halves: (lo_i, hi_i) = (element i, element i + dims/2) turns by the
             angle t = p w_i at position p, w_i = base^(-2i/dims): lo' = lo cos t - hi sin t, hi' = hi cos t + lo sin t;
             with ``scaling`` the slow w_i are divided by a factor, the fast ones kept, those between blended
  mixers     ``attention``    q = Wq h, k = Wk h, values = k straight out of its product; q and k each normed across all
                              heads together (one mean square a token, a weight a channel), then rotated; a row sees the keys of its
                              own block of ``mask.size`` positions up to itself; softmax with one more term, exp(0),
                              in the denominator
             ``attention_2``  q, k, v with biases; q and k rotated, then each head divided by its root mean square;
                              each value head divided by its root mean square; scores capped by c tanh(s / c); a row
                              sees itself and the ``mask.size`` - 1 keys before it; a key in sight counts with
                              sigmoid(score + b_head), whatever the other keys score
  ff         sigmoid router over all experts, chosen by score + correction, the chosen scores divided by their sum and
             multiplied by a constant; an expert is W_down gelu(W_up v) with the exact gelu; one more expert of that form
             stands outside the router and counts fully for every token
  output     logits = W_head N(x)
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Optional, Sequence

import torch


# --- mechanisms -----------------------------------------------------------------

def unit_rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    """v / sqrt(mean(v^2) + eps) over the last axis."""
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def grouped_norm(v: torch.Tensor, g: torch.Tensor, eps: float, groups: int) -> torch.Tensor:
    """v [..., W] as ``groups`` runs of W / groups channels, every run through unit_rms by itself; then all channels times g."""
    parts = v.reshape(*v.shape[:-1], groups, v.shape[-1] // groups)
    return unit_rms(parts, eps).reshape(v.shape) * g


def scaled_frequencies(dims: int, base: float, scaling: Optional[dict]) -> torch.Tensor:
    """w_i = base^(-2i/dims) for i < dims/2.  With ``scaling`` (factor F, low, high, original L) a pair is judged by
    r = L w / (2 pi), the turns it makes over L positions: r > high leaves w, r < low gives w / F, and from low to high
    w (s + (1 - s) / F) with s = (r - low) / (high - low)."""
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling is not None:
            factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength > original / low:
                f = f / factor
            elif wavelength >= original / high:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


def half_rotation(v: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """v [T, heads, d]: among the first 2 len(freqs) elements of a head, element i is paired with element i + len(freqs)."""
    half = len(freqs)
    if half == 0:
        return v.clone()
    ang = positions.to(torch.float64)[:, None] * freqs[None, :]
    c, s = torch.cos(ang).to(v.dtype)[:, None, :], torch.sin(ang).to(v.dtype)[:, None, :]
    a, b = v[..., :half], v[..., half:2 * half]
    out = v.clone()
    out[..., :half] = a * c - b * s
    out[..., half:2 * half] = b * c + a * s
    return out


def block_mask(n: int, size: int) -> torch.Tensor:
    """[n, n] bool: row i sees column j <= i of the same block of ``size`` positions counted from 0."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def window_mask(n: int, size: int) -> torch.Tensor:
    """[n, n] bool: row i sees column j with 0 <= i - j < size."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & (i - j < size)


def softmax_plus_one(scores: torch.Tensor, mask: torch.Tensor) -> torch.Tensor:
    """p_j = exp(s_j) / (1 + sum over the visible j of exp(s_j)); scores [..., T, T]."""
    s = scores.masked_fill(~mask, -math.inf)
    top = torch.clamp(s.max(dim=-1, keepdim=True).values, min=0.0)
    e = torch.exp(s - top)
    return e / (torch.exp(-top) + e.sum(dim=-1, keepdim=True))


def capped(scores: torch.Tensor, cap: float) -> torch.Tensor:
    return cap * torch.tanh(scores / cap)


def sigmoid_weights(scores: torch.Tensor, mask: torch.Tensor, head_bias: torch.Tensor) -> torch.Tensor:
    """scores [heads, T, T]: sigmoid(score + b_head) where visible, zero elsewhere; nothing is normalised."""
    return torch.sigmoid(scores + head_bias[:, None, None]) * mask


def per_head(weights: torch.Tensor, values: torch.Tensor, heads: int, kv_heads: int) -> torch.Tensor:
    """weights [heads, T, T], values [T, kv_heads, e] -> [T, heads * e]; query head a reads head a // (heads / kv_heads)."""
    share = heads // kv_heads
    out = [weights[a] @ values[:, a // share, :] for a in range(heads)]
    return torch.cat(out, dim=-1)


def scores_of(q: torch.Tensor, k: torch.Tensor, heads: int, kv_heads: int, scale: float) -> torch.Tensor:
    """q [T, heads, d], k [T, kv_heads, d] -> [heads, T, T]."""
    share = heads // kv_heads
    return torch.stack([q[:, a, :] @ k[:, a // share, :].T for a in range(heads)]) * scale


def exact_gelu(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def route(z: torch.Tensor, correction: torch.Tensor, top: int, factor: float):
    """z [T, E] router logits -> (chosen [T, top], weights [T, top], margin [T]): s = sigmoid(z); the ``top`` largest
    s + correction are chosen; their s, divided by their sum, times ``factor``.  margin: how far the last chosen
    choice score lies above the best one left out (inf if none is left out)."""
    s = torch.sigmoid(z)
    choice = s + correction
    order = torch.argsort(choice, dim=-1, descending=True, stable=True)
    chosen = order[:, :top]
    picked = torch.gather(s, 1, chosen)
    weights = picked / (picked.sum(dim=-1, keepdim=True) + 1e-20) * factor
    ranked = torch.gather(choice, 1, order)
    margin = ranked[:, top - 1] - ranked[:, top] if top < z.shape[1] else torch.full((z.shape[0],), math.inf, dtype=z.dtype)
    return chosen, weights, margin


# --- the model ---------------------------------------------------------------------

class PlainLagusun:
    def __init__(self, folder: str, dtype: torch.dtype = torch.float64):
        from safetensors.torch import load_file
        with open(os.path.join(folder, "config.json"), encoding="utf-8") as fh:
            self.cfg = json.load(fh)
        self.dtype = dtype
        self.w: Dict[str, torch.Tensor] = {k: (v if v.dtype == torch.int32 else v.to(dtype))
                                           for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
        self.eps = float(self.cfg["norm"]["eps"])
        self.groups = int(self.cfg["norm"].get("groups", 1))
        self.margins: List[torch.Tensor] = []

    # ---- order of layer runs ----
    def runs(self):
        """(layer, pass or None) for every layer run; a pass number marks the first layer of a pass."""
        n, loop = len(self.cfg["layers"]), self.cfg.get("loop")
        if not loop or loop["start"] == loop["stop"]:
            return [(i, None) for i in range(n)]
        out = [(i, None) for i in range(loop["start"])]
        for t in range(loop["times"]):
            out += [(i, t if i == loop["start"] else None) for i in range(loop["start"], loop["stop"])]
        return out + [(i, None) for i in range(loop["stop"], n)]

    def norm(self, v, name):
        return grouped_norm(v, self.w[name], self.eps, self.groups)

    # ---- mixers ----
    def attention(self, p: str, m: dict, h: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        w, T = self.w, h.shape[0]
        H, G, d = m["heads"], m["kv_heads"], m["dim"]
        q, k = h @ w[p + "q"].T, h @ w[p + "k"].T
        v = k.reshape(T, G, d)                                       # the values: k straight out of its product
        q = unit_rms(q, self.eps) * w[p + "q.norm"]                  # one mean square over all heads of the token
        k = unit_rms(k, self.eps) * w[p + "k.norm"]
        rot = m.get("rot")
        freqs = scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling")) if rot else torch.zeros(0, dtype=torch.float64)
        q = half_rotation(q.reshape(T, H, d), positions, freqs)
        k = half_rotation(k.reshape(T, G, d), positions, freqs)
        s = scores_of(q, k, H, G, m["scale"])
        mask = block_mask(T, m["mask"]["size"]) if m.get("mask") else window_mask(T, T)
        return per_head(softmax_plus_one(s, mask), v, H, G) @ w[p + "o"].T

    def attention_2(self, p: str, m: dict, h: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        w, T = self.w, h.shape[0]
        H, G, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        q = (h @ w[p + "q"].T + w[p + "q.b"]).reshape(T, H, d)
        k = (h @ w[p + "k"].T + w[p + "k.b"]).reshape(T, G, d)
        v = (h @ w[p + "v"].T + w[p + "v.b"]).reshape(T, G, e)
        rot = m.get("rot")
        freqs = scaled_frequencies(rot["dims"], rot["base"], rot.get("scaling")) if rot else torch.zeros(0, dtype=torch.float64)
        q = unit_rms(half_rotation(q, positions, freqs), self.eps)
        k = unit_rms(half_rotation(k, positions, freqs), self.eps)
        v = unit_rms(v, self.eps)
        s = scores_of(q, k, H, G, m["scale"])
        if m.get("softcap"):
            s = capped(s, m["softcap"])
        mask = window_mask(T, m["mask"]["size"]) if m.get("mask") else window_mask(T, T)
        return per_head(sigmoid_weights(s, mask, w[p + "pb"]), v, H, G) @ w[p + "o"].T

    # ---- feed-forward ----
    def unit(self, p: str, h: torch.Tensor) -> torch.Tensor:
        return exact_gelu(h @ self.w[p + "up"].T) @ self.w[p + "down"].T

    def experts(self, p: str, mlp: dict, h: torch.Tensor) -> torch.Tensor:
        r = mlp["router"]
        z = h.to(torch.float64) @ self.w[p + "router"].to(torch.float64).T
        chosen, weights, margin = route(z, self.w[p + "correction"].to(torch.float64), r["top"], float(r.get("scale", 1.0)))
        self.margins.append(margin)
        out = torch.zeros_like(h)
        for e in range(r["experts"]):
            rows, slot = torch.nonzero(chosen == e, as_tuple=True)
            if len(rows):
                out[rows] += weights[rows, slot, None].to(h.dtype) * self.unit(p + f"e{e}.", h[rows])
        if mlp.get("shared"):
            out = out + self.unit(p + "shared.", h)
        return out

    # ---- whole sequences ----
    def forward(self, ids: Sequence[int], return_layers: bool = False):
        """float logits [T, vocab] of one sequence from its first token (and, if asked, the stream after every layer run)."""
        w, cfg = self.w, self.cfg
        self.margins = []
        ids = torch.as_tensor(list(ids), dtype=torch.long)
        positions = torch.arange(len(ids))
        x0 = w["embed"][ids] * float(cfg.get("embedding", {}).get("scale", 1.0))
        x, after = x0.clone(), []
        for i, turn in self.runs():
            layer, p = cfg["layers"][i], f"l{i}."
            if turn is not None:
                x = torch.cat([x, x0], dim=-1) @ w["loop.in"].T + w["loop.step"][turn]
            h = self.norm(x, p + "norm1")
            mixer = self.attention if layer["type"] == "attention" else self.attention_2
            x = x + mixer(p + "mix.", layer["mixer"], h, positions) * w[p + "ls1"]
            if layer.get("mlp") is not None:
                x = x + self.experts(p + "mlp.", layer["mlp"], self.norm(x, p + "norm2")) * w[p + "ls2"]
            after.append(x.clone())
        logits = (self.norm(x, "final.norm") @ w["head"].T).to(torch.float32)
        return (logits, after) if return_layers else logits

    def closest_call(self) -> Optional[torch.Tensor]:
        """[T]: the smallest routing margin of every token over all routers of the last forward (None without routers)."""
        return torch.stack(self.margins).min(dim=0).values if self.margins else None
