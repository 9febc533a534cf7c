"""A plain, slow implementation of the Milenex decoder for the tests.

Whole sequences, no cache, no state carried between calls, one function for each mechanism, written from the
design's equations and sharing no code with the engine: it reads config.json with ``json`` and the weights with
the ``safetensors`` package.  Arithmetic is float64 by default.

The design, in this file's notation (a linear weight is stored [out, in] and applied as W x; t counts a
sequence's tokens from 0):

  layer      x += mixer(shift(N1(x)));  x += ff(N2(x))       (a layer may have no ff)
  N(v)       v / sqrt(mean(v^2) + eps) * (1 + g)
  shift(h)   h_t + (h_(t-1) - h_t) * m, element by element, h_(-1) = 0; the h on the right are the unshifted ones
  loop       layers a..b-1 run n times in a row with the same weights (each pass with a state of its own); before
             every pass but the first the embedding's output is added to x
  mixers     ``attention``    q, k, v, each through a short causal convolution over time, q and k rotated by
                              position (neighbouring pairs) and divided by their root mean square per head;
                              softmax over a window of the last keys with a sink in the denominator
             ``attention_2``  no rotation: a distance penalty on the scores; windowed softmax with a sink; the
                              heads' weights mixed by a matrix; a gate per head on the output
  ff         ``dense``        W_down gelu(W_up v), the exact gelu
             ``moe``          softmax router over all experts, chosen by score + correction among the best groups,
                              weighted by the plain scores; a shared expert with a gate per token
  expert     W_down (g sigmoid(1.702 g) (u + 1)) with g = min(W_gate v, L), u = clamp(W_up v, -L, L)
  output     logits = W_head N(x)
"""
from __future__ import annotations

import json
import math
import os
from typing import Dict, List, Sequence

import torch


# --- mechanisms -----------------------------------------------------------------

def unit_rms(v: torch.Tensor, eps: float) -> torch.Tensor:
    """v / sqrt(mean(v^2) + eps) over the last axis."""
    return v / torch.sqrt((v * v).mean(dim=-1, keepdim=True) + eps)


def zero_centred_norm(v: torch.Tensor, g: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(v, eps) * (1.0 + g)


def token_shift(h: torch.Tensor, m: torch.Tensor) -> torch.Tensor:
    """h [T, W] of one sequence from its first token: h_t + (h_(t-1) - h_t) m."""
    before = torch.cat([torch.zeros_like(h[:1]), h[:-1]], dim=0)
    return h + (before - h) * m


def short_convolution(u: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """u [T, C] of one sequence from its first token, w [C, taps]: y_t = sum_j w[:, j] u_(t - taps + 1 + j)."""
    taps = w.shape[1]
    y = torch.zeros_like(u)
    for j in range(taps):
        back = taps - 1 - j
        if back < u.shape[0]:
            y[back:] += u[:u.shape[0] - back] * w[:, j]
    return y


def neighbour_rotation(v: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """v [T, heads, d]: among the first ``dims`` elements of a head, element 2i is paired with element 2i + 1; the pair
    (a, b) at position p becomes (a cos - b sin, b cos + a sin) of the angle p * base^(-2i/dims)."""
    if dims == 0:
        return v.clone()
    i = torch.arange(dims // 2, dtype=torch.float64)
    ang = positions.to(torch.float64)[:, None] * base ** (-2.0 * i / dims)[None, :]
    c, s = torch.cos(ang).to(v.dtype)[:, None, :], torch.sin(ang).to(v.dtype)[:, None, :]
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out = v.clone()
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def window_weights(q: torch.Tensor, k: torch.Tensor, scale: float, window: int, sink: float, r1: float = 0.0,
                   r2: float = 0.0) -> torch.Tensor:
    """One head: q, k [T, d] -> weights [T, T].  score(i, j) = q_i . k_j * scale - r1 ln(1 + r2 (i - j)) for
    0 <= i - j < window; weight = exp(score) / (sum over the visible j of exp(score) + exp(sink))."""
    T = q.shape[0]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    dist = (i - j).to(q.dtype)
    s = (q @ k.T) * scale
    if r1 != 0.0 or r2 != 0.0:
        s = s - r1 * torch.log1p(r2 * dist.clamp(min=0))
    seen = (i - j >= 0) & (i - j < window)
    s = s.masked_fill(~seen, float("-inf"))
    top = torch.maximum(s.max(dim=-1, keepdim=True).values, torch.full((T, 1), sink, dtype=q.dtype))
    e = torch.exp(s - top)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink - top))


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def clamped_glu(gate: torch.Tensor, up: torch.Tensor, limit: float) -> torch.Tensor:
    g = torch.clamp(gate, max=limit)
    u = torch.clamp(up, min=-limit, max=limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def route(z: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int):
    """z [T, E] router logits -> (chosen experts [T, top], their weights [T, top]).  s = softmax(z); the choice goes by
    s + correction; a group of E / groups neighbouring experts counts by its largest choice score, only the ``keep``
    best groups' experts can be chosen; the weights are s of the chosen, as they are."""
    T, E = z.shape
    s = torch.softmax(z, dim=-1)
    choice = s + correction
    per = E // groups
    best = choice.view(T, groups, per).max(dim=-1).values
    kept = torch.topk(best, keep, dim=-1).indices
    allowed = torch.zeros(T, groups, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    choice = choice.masked_fill(~allowed.repeat_interleave(per, dim=1), float("-inf"))
    chosen = torch.topk(choice, top, dim=-1).indices
    return chosen, torch.gather(s, 1, chosen)


def route_margin(z: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int) -> torch.Tensor:
    """[T]: how far every row's choice is from another one -- the smaller of the gap between the last kept group's score
    and the best group's left out, and the gap between the last chosen expert's choice score and the best one's left out
    among the kept groups (infinite where nothing is left out).  A test in reduced precision knows by it which rows'
    choice a rounding could turn."""
    T, E = z.shape
    choice = torch.softmax(z, dim=-1) + correction
    per = E // groups
    best = choice.view(T, groups, per).max(dim=-1).values.sort(dim=-1, descending=True).values
    inf = torch.full((T,), float("inf"), dtype=z.dtype)
    group_gap = best[:, keep - 1] - best[:, keep] if keep < groups else inf
    kept = torch.topk(choice.view(T, groups, per).max(dim=-1).values, keep, dim=-1).indices
    allowed = torch.zeros(T, groups, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    ranked = choice.masked_fill(~allowed.repeat_interleave(per, dim=1), float("-inf")).sort(dim=-1, descending=True).values
    expert_gap = ranked[:, top - 1] - ranked[:, top] if top < keep * per else inf
    return torch.minimum(group_gap, expert_gap)


# --- the model --------------------------------------------------------------------

class PlainMilenex:
    def __init__(self, folder: str, dtype: torch.dtype = torch.float64):
        from safetensors import safe_open
        with open(os.path.join(folder, "config.json")) as fh:
            self.cfg = json.load(fh)
        self.w: Dict[str, torch.Tensor] = {}
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
            for name in f.keys():
                self.w[name] = f.get_tensor(name).to(dtype)
        self.dtype = dtype
        self.eps = float(self.cfg["norm"]["eps"])
        self.margins: List[torch.Tensor] = []      # of the last forward: every routed feed-forward run's route_margin

    def closest_call(self) -> torch.Tensor:
        """[T] of the last forward: per token the smallest routing margin of any layer run (infinite without routers)."""
        return torch.stack(self.margins).min(dim=0).values if self.margins else None

    def lin(self, name: str, x: torch.Tensor) -> torch.Tensor:
        return x @ self.w[name].T

    @staticmethod
    def window(m: dict, T: int) -> int:
        """The mixer's window; without one every earlier token is seen."""
        return int(m["mask"]["size"]) if m.get("mask") is not None else T

    def attention(self, p: str, m: dict, h: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        T, H, G, d, e = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        q, k, v = self.lin(p + "q", h), self.lin(p + "k", h), self.lin(p + "v", h)
        if m.get("conv"):
            q, k, v = (short_convolution(u, self.w[p + n + ".conv"]) for u, n in ((q, "q"), (k, "k"), (v, "v")))
        q, k, v = q.view(T, H, d), k.view(T, G, d), v.view(T, G, e)
        rot = m.get("rot")
        if rot is not None:
            q = neighbour_rotation(q, positions, int(rot["dims"]), float(rot["base"]))
            k = neighbour_rotation(k, positions, int(rot["dims"]), float(rot["base"]))
        q, k = unit_rms(q, self.eps), unit_rms(k, self.eps)
        o = torch.zeros(T, H, e, dtype=h.dtype)
        for a in range(H):
            g = a // (H // G)
            o[:, a] = window_weights(q[:, a], k[:, g], float(m["scale"]), self.window(m, T), float(self.w[p + "sink"][a])) @ v[:, g]
        return self.lin(p + "o", o.reshape(T, H * e))

    def attention_2(self, p: str, m: dict, h: torch.Tensor) -> torch.Tensor:
        T, H, G, d, e = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        q, k, v = self.lin(p + "q", h).view(T, H, d), self.lin(p + "k", h).view(T, G, d), self.lin(p + "v", h).view(T, G, e)
        w = torch.stack([window_weights(q[:, a], k[:, a // (H // G)], float(m["scale"]), self.window(m, T),
                                        float(self.w[p + "sink"][a]), float(self.w[p + "r1"][a]), float(self.w[p + "r2"][a]))
                         for a in range(H)])
        mixed = torch.einsum("hg,gij->hij", self.w[p + "talk"], w)
        gate = torch.sigmoid(self.lin(p + "g", h))
        o = torch.zeros(T, H, e, dtype=h.dtype)
        for a in range(H):
            o[:, a] = (mixed[a] @ v[:, a // (H // G)]) * gate[:, a:a + 1]
        return self.lin(p + "o", o.reshape(T, H * e))

    def expert(self, p: str, limit: float, h: torch.Tensor) -> torch.Tensor:
        return self.lin(p + "down", clamped_glu(self.lin(p + "gate", h), self.lin(p + "up", h), limit))

    def feed_forward(self, p: str, m: dict, h: torch.Tensor) -> torch.Tensor:
        if m["kind"] == "dense":
            return self.lin(p + "down", gelu_erf(self.lin(p + "up", h)))
        r = m["router"]
        groups = r.get("groups") or dict(count=1, keep=1)
        z = self.lin(p + "router", h)
        chosen, weights = route(z, self.w[p + "correction"], int(r["top"]), int(groups["count"]), int(groups["keep"]))
        self.margins.append(route_margin(z, self.w[p + "correction"], int(r["top"]), int(groups["count"]), int(groups["keep"])))
        out = torch.zeros_like(h)
        for t in range(h.shape[0]):
            for e, wt in zip(chosen[t].tolist(), weights[t]):
                out[t] += wt * self.expert(f"{p}e{e}.", float(m["expert"]["limit"]), h[t:t + 1])[0]
        if m.get("shared") is not None:
            out = out + self.expert(p + "shared.", float(m["shared"]["limit"]), h) * torch.sigmoid(self.lin(p + "shared.sg", h))
        return out

    def layer(self, n: int, x: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
        layer, p = self.cfg["layers"][n], f"l{n}."
        h = token_shift(zero_centred_norm(x, self.w[p + "norm1"], self.eps), self.w[p + "shift"])
        if layer["type"] == "attention":
            x = x + self.attention(p + "mix.", layer["mixer"], h, positions)
        elif layer["type"] == "attention_2":
            x = x + self.attention_2(p + "mix.", layer["mixer"], h)
        else:
            raise ValueError(f"layer {n}: unknown type {layer['type']!r}")
        if layer.get("mlp") is not None:
            x = x + self.feed_forward(p + "mlp.", layer["mlp"], zero_centred_norm(x, self.w[p + "norm2"], self.eps))
        return x

    def order(self) -> List[tuple]:
        """(layer, whether the embedding's output is added before it) for every layer run."""
        n, loop = len(self.cfg["layers"]), self.cfg.get("loop")
        if not loop:
            return [(i, False) for i in range(n)]
        a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
        runs = [(i, False) for i in range(a)]
        for turn in range(times):
            runs += [(i, turn > 0 and i == a) for i in range(a, b)]
        return runs + [(i, False) for i in range(b, n)]

    def forward(self, tokens: Sequence[int], return_layers: bool = False):
        """float logits [T, vocab] of a whole sequence from position 0 (and the residual stream after every layer run)."""
        ids = torch.as_tensor(list(tokens), dtype=torch.long)
        positions = torch.arange(len(ids))
        emb = self.w["embed"][ids]
        x = emb.clone()
        self.margins = []
        after: List[torch.Tensor] = []
        for n, add in self.order():
            if add:
                x = x + emb
            x = self.layer(n, x, positions)
            after.append(x)
        logits = self.lin("head", zero_centred_norm(x, self.w["final.norm"], self.eps))
        return (logits, after) if return_layers else logits
