"""A plain, slow implementation of the Tegolix decoder, one function per mechanism, written from the
design's equations with torch on the CPU (64-bit by default). It shares no code with the engine: it
reads config.json and model.safetensors itself. The tests compare the engine with it.

Notation. rms(x) = x / sqrt(mean(x^2) + eps); n(x) = rms(x) (1 + w) is the layers' norm, whose weight is
stored around zero. A layer computes
    x <- x + s1 * n1b(mixer(n1 x)),   x <- x + s2 * n2b(ff(n2 x)),   x <- x + rms(P (gelu(G x) * e_i(token))) * c
with s1, s2 learned vectors, and e_i(token) layer i's slice of a second, narrow token table. The mixer is
gated linear attention ("gla"), or a pair of mixers side by side that read the same input ("parallel"):
on the left grouped-query attention inside a sliding window with capped scores, a norm on every query and
key head, rotated values and a gate per head; on the right an RWKV-style recurrence with token shift, a
data-dependent decay and a bonus for the current token. The feed-forward is a relu-gated unit or a
mixture of silu-gated experts with identity experts and a shared expert behind a gate of its own.
"""

from __future__ import annotations

import json
import math
import os

import torch
from safetensors import safe_open


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by its root mean square over the last dimension, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """The layers' norm: its weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rotary_frequencies(dims: int, base: float, scaling: dict | None) -> tuple[torch.Tensor, float]:
    """(f_i for i < dims/2, the factor on cos and sin). Without scaling f_i = base^(-2i/dims) and the
    factor is 1. With scaling (factor s, original length L, fast, slow): d(t) = dims ln(L / (2 pi t)) /
    (2 ln base), lo = max(floor d(fast), 0), hi = min(ceil d(slow), dims - 1), r_i = clamp((i - lo) /
    max(hi - lo, 0.001), 0, 1); f_i <- f_i / s * r_i + f_i (1 - r_i); the factor is 0.1 ln s + 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / max(dims, 1))
    if not scaling:
        return f, 1.0
    s, length = float(scaling["factor"]), float(scaling["original"])

    def d(t: float) -> float:
        return dims * math.log(length / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(d(float(scaling["fast"]))), 0)
    hi = min(math.ceil(d(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / s * ramp + f * (1.0 - ramp), 0.1 * math.log(s) + 1.0


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor, amplitude: float = 1.0,
                  back: bool = False) -> torch.Tensor:
    """x [n, heads, D]: the first 2 len(freqs) dimensions of a head turn by positions * f_i (by minus that
    with `back`), dimension i paired with i + len(freqs); the rest pass."""
    half = freqs.shape[0]
    if half == 0:
        return x
    angle = positions.to(torch.float64)[:, None] * freqs[None, :]
    if back:
        angle = -angle
    cos = (torch.cos(angle) * amplitude).to(x.dtype)[:, None, :]
    sin = (torch.sin(angle) * amplitude).to(x.dtype)[:, None, :]
    out = x.clone()
    u, v = x[..., :half], x[..., half:2 * half]
    out[..., :half] = u * cos - v * sin
    out[..., half:2 * half] = v * cos + u * sin
    return out


def window_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_positions: torch.Tensor, scale: float,
                     softcap: float, window: int) -> torch.Tensor:
    """q [n, H, D] at `q_positions` over keys k [m, G, D] and values v [m, G, V] at positions 0..m-1: query i sees
    key j where 0 <= i - j (< window, if there is one); score = q.k scale, capped as cap tanh(score / cap) if there
    is a cap; an ordinary softmax over what is seen."""
    n, H, _ = q.shape
    G = k.shape[1]
    i, j = q_positions[:, None], torch.arange(k.shape[0])[None, :]
    see = j <= i
    if window:
        see = see & ((i - j) < window)
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        s = s.masked_fill(~see, float("-inf"))
        out[:, h] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def left_attention(h: torch.Tensor, positions: torch.Tensor, W: dict, m: dict, eps: float, past: dict) -> torch.Tensor:
    """The attention half of the "parallel" mixer for the rows h at `positions`; `past` holds the keys and the
    (rotated) values so far."""
    H, G, D, V = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    n = h.shape[0]
    q = unit_rms((h @ W["q"].T).reshape(n, H, D), eps) * W["q.norm"]         # head by head, one weight for all heads
    k = unit_rms((h @ W["k"].T).reshape(n, G, D), eps) * W["k.norm"]
    v = (h @ W["v"].T).reshape(n, G, V)
    rot = m.get("rot") or {}
    if rot.get("dims"):
        freqs, amp = rotary_frequencies(int(rot["dims"]), float(rot["base"]), rot.get("scaling"))
        q, k = rotate_halves(q, positions, freqs, amp), rotate_halves(k, positions, freqs, amp)
    value_freqs = rotary_frequencies(V, float(rot["base"]), None)[0] if rot else torch.zeros(0, dtype=torch.float64)
    v = rotate_halves(v, positions, value_freqs)                             # the value of position j turns by j, all of it
    past["k"] = torch.cat([past["k"], k]) if "k" in past else k
    past["v"] = torch.cat([past["v"], v]) if "v" in past else v
    window = int((m.get("mask") or {}).get("size", 0))
    o = window_attention(q, past["k"], past["v"], positions, float(m["scale"]), float(m.get("softcap") or 0.0), window)
    o = rotate_halves(o, positions, value_freqs, back=True)                  # and the sum at position i turns back by i
    o = o * torch.sigmoid(h @ W["g"].T)[:, :, None]                          # one gate per head
    return o.reshape(n, H * V) @ W["o"].T


def right_recurrence(h: torch.Tensor, W: dict, m: dict, eps: float, state: dict) -> torch.Tensor:
    """The recurrent half of the "parallel" mixer, token by token. state: S [H, D, D] and the previous token's h,
    zeros at the start. Each of r, k, v, g, w reads h + (h' - h) mu of its own; the decay is
    w = exp(-exp(W2 tanh(W1 x_w) + w0)); o = (S + diag(u) k v^T)^T r, then S <- diag(w) S + k v^T."""
    H, D = int(m["heads"]), int(m["dim"])
    if "S" not in state:
        state["S"] = torch.zeros(H, D, D, dtype=h.dtype)
        state["prev"] = torch.zeros(h.shape[1], dtype=h.dtype)
    rows = []
    for t in range(h.shape[0]):
        x, prev = h[t], state["prev"]
        mix = {s: x + (prev - x) * W[f"mu.{s}"] for s in ("r", "k", "v", "g", "w")}
        r = (W["r"] @ mix["r"]).reshape(H, D)
        k = (W["k"] @ mix["k"]).reshape(H, D)
        v = (W["v"] @ mix["v"]).reshape(H, D)
        gate = torch.nn.functional.silu(W["g"] @ mix["g"])
        w = torch.exp(-torch.exp(W["w2"] @ torch.tanh(W["w1"] @ mix["w"]) + W["w0"])).reshape(H, D)
        kv = k[:, :, None] * v[:, None, :]
        o = torch.einsum("hkv,hk->hv", state["S"] + W["u"][:, :, None] * kv, r)
        state["S"] = w[:, :, None] * state["S"] + kv
        state["prev"] = x
        rows.append(((unit_rms(o, eps).reshape(H * D) * W["norm"]) * gate) @ W["o"].T)
    return torch.stack(rows)


def gated_linear_attention(h: torch.Tensor, W: dict, m: dict, eps: float, state: dict) -> torch.Tensor:
    """The "gla" mixer, token by token. state: S [H, D, V], zeros at the start. alpha = sigmoid(A2 A1 h + b)^(1/tau)
    per head and key channel; S <- diag(alpha) S + k v^T; o = S^T (q D^(-1/2)); each head's o through rms and a weight
    over V, the heads side by side times silu(W_g h), then W_o."""
    H, D, V, tau = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["tau"])
    if "S" not in state:
        state["S"] = torch.zeros(H, D, V, dtype=h.dtype)
    rows = []
    for t in range(h.shape[0]):
        x = h[t]
        q = (W["q"] @ x).reshape(H, D) * D ** -0.5
        k = (W["k"] @ x).reshape(H, D)
        v = (W["v"] @ x).reshape(H, V)
        alpha = torch.exp(torch.nn.functional.logsigmoid(W["a2"] @ (W["a1"] @ x) + W["a2.b"]) / tau).reshape(H, D)
        state["S"] = alpha[:, :, None] * state["S"] + k[:, :, None] * v[:, None, :]
        o = torch.einsum("hkv,hk->hv", state["S"], q)
        o = (unit_rms(o, eps) * W["norm"]).reshape(H * V)
        rows.append((o * torch.nn.functional.silu(W["g"] @ x)) @ W["o"].T)
    return torch.stack(rows)


def gated_unit(h: torch.Tensor, W: dict, act) -> torch.Tensor:
    return (act(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


def chosen_experts(logits: torch.Tensor, correction: torch.Tensor, top: int) -> tuple[torch.Tensor, torch.Tensor]:
    """(indices [n, top], weights [n, top]): s = softmax over every router output; the `top` largest s + correction
    are chosen; their weights are their s, as they are."""
    s = torch.softmax(logits, dim=-1)
    idx = torch.topk(s + correction, top, dim=-1).indices
    return idx, torch.gather(s, 1, idx)


def choice_margin(logits: torch.Tensor, correction: torch.Tensor, top: int) -> torch.Tensor:
    """[n]: how far the last chosen expert's choice score lies above the best one left out (infinite where all are
    chosen): a rounding of the scores by less than that chooses the same experts."""
    ranked = torch.sort(torch.softmax(logits, dim=-1) + correction, dim=-1, descending=True).values
    if top >= ranked.shape[-1]:
        return torch.full(ranked.shape[:-1], float("inf"), dtype=ranked.dtype)
    return ranked[..., top - 1] - ranked[..., top]


def expert_mixture(h: torch.Tensor, W: dict, mlp: dict, margins: list | None = None) -> torch.Tensor:
    """The router's last `identity` outputs stand for experts that hand their input through. `margins`, if given,
    collects every token's `choice_margin`."""
    router = mlp["router"]
    real = int(router["experts"])
    silu = torch.nn.functional.silu
    idx, weights = chosen_experts(h @ W["router"].T, W["correction"], int(router["top"]))
    if margins is not None:
        margins.append(choice_margin(h @ W["router"].T, W["correction"], int(router["top"])))
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for w, e in zip(weights[t], idx[t]):
            e = int(e)
            if e >= real:
                out[t] += w * h[t]
            else:
                out[t] += w * gated_unit(h[t:t + 1], {n: W[f"e{e}.{n}"] for n in ("gate", "up", "down")}, silu)[0]
    if mlp.get("shared"):
        shared = gated_unit(h, {n: W[f"shared.{n}"] for n in ("gate", "up", "down")}, silu)
        out = out + shared * torch.sigmoid(h @ W["shared.sg"].T)
    return out


class PlainTegolix:
    """The whole decoder over one request, fed in any portions; keeps that request's caches and states."""

    def __init__(self, config: dict, weights: dict[str, torch.Tensor], dtype: torch.dtype = torch.float64) -> None:
        self.c, self.dtype = config, dtype
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
        self.memory: list[dict] = [dict() for _ in config["layers"]]
        self.fed = 0
        self.after_layers: list[torch.Tensor] = []      # the residual stream after every layer, of the last call
        self.margins: torch.Tensor | None = None        # per token of the last call: the routers' smallest `choice_margin`

    @classmethod
    def from_folder(cls, folder: str, dtype: torch.dtype = torch.float64) -> "PlainTegolix":
        with open(os.path.join(folder, "config.json")) as f:
            config = json.load(f)
        weights = {}
        with safe_open(os.path.join(folder, "model.safetensors"), "pt", "cpu") as f:
            for name in f.keys():
                weights[name] = f.get_tensor(name)
        return cls(config, weights, dtype)

    def _sub(self, prefix: str) -> dict:
        return {k[len(prefix):]: v for k, v in self.w.items() if k.startswith(prefix)}

    def forward(self, tokens: list[int]) -> torch.Tensor:
        """Feeds the request's next tokens; returns logits [len(tokens), vocab]."""
        c, eps = self.c, float(self.c["norm"]["eps"])
        positions = torch.arange(self.fed, self.fed + len(tokens))
        self.fed += len(tokens)
        ids = torch.tensor(tokens)
        x = self.w["embed"][ids]
        side = int((c.get("token_side") or {}).get("dim", 0))
        self.after_layers = []
        margins: list[torch.Tensor] = []
        for i, layer in enumerate(c["layers"]):
            p = f"l{i}."
            h = layer_norm(x, self.w[p + "norm1"], eps)
            W, m, mem = self._sub(p + "mix."), layer["mixer"], self.memory[i]
            if layer["type"] == "gla":
                y = gated_linear_attention(h, W, m, eps, mem)
            elif layer["type"] == "parallel":
                left = left_attention(h, positions, self._sub(p + "mix.left."), m["left"], eps, mem.setdefault("left", {}))
                right = right_recurrence(h, self._sub(p + "mix.right."), m["right"], eps, mem.setdefault("right", {}))
                y = float(m["left_scale"]) * left + float(m["right_scale"]) * right
            else:
                raise ValueError(layer["type"])
            x = x + layer_norm(y, self.w[p + "norm1b"], eps) * self.w[p + "ls1"]
            mlp = layer.get("mlp")
            if mlp is not None:
                h = layer_norm(x, self.w[p + "norm2"], eps)
                F = self._sub(p + "mlp.")
                y = gated_unit(h, F, torch.relu) if mlp["kind"] == "dense" else expert_mixture(h, F, mlp, margins)
                x = x + layer_norm(y, self.w[p + "norm2b"], eps) * self.w[p + "ls2"]
            if side:
                e = self.w["side.embed"][ids][:, i * side:(i + 1) * side]
                y = (gelu_tanh(x @ self.w[p + "side.gate"].T) * e) @ self.w[p + "side.proj"].T
                x = x + unit_rms(y, eps) * self.w[p + "side.norm"]
            self.after_layers.append(x.clone())
        self.margins = torch.stack(margins).min(0).values if margins else torch.full((len(tokens),), float("inf"), dtype=x.dtype)
        return layer_norm(x, self.w["final.norm"], eps) @ self.w["head"].T

    def reset(self) -> None:
        """Forgets the request: the next tokens are a new request's first."""
        self.memory = [dict() for _ in self.c["layers"]]
        self.fed = 0

    def logits(self, tokens: list[int]) -> torch.Tensor:
        """[len(tokens), vocab] for a request of its own, fed whole."""
        self.reset()
        return self.forward(tokens)

    def streams(self, tokens: list[int]) -> list[torch.Tensor]:
        """The residual stream after every layer, for a request of its own, fed whole."""
        self.logits(tokens)
        return self.after_layers

    def greedy(self, tokens: list[int], n: int) -> list[int]:
        self.reset()
        row, out = self.forward(tokens)[-1], []
        for _ in range(n):
            out.append(int(row.argmax()))
            row = self.forward(out[-1:])[-1]
        return out
