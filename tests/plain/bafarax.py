"""A plain, slow implementation of the Bafarax decoder, one function per mechanism, written from
the design's equations with torch on the CPU (64-bit by default). It shares no code with the
engine: it reads config.json and model.safetensors itself. The tests compare the engine with it.

Notation. rms(x) = x / sqrt(mean(x^2) + eps). A layer computes x <- x + mixer(n1 x), then
x <- x + ff(n2 x) with n(x) = rms(x) (1 + w). The mixer is one of three: grouped-query attention
inside chunks of positions with a learned sink per head ("attention"), attention through a
low-rank latent with a shared rotated key part, a sliding window and an output gate
("latent_attention"), or the matrix memory of an mLSTM with a stabilised exponential input gate
("mlstm"). The feed-forward is a silu-gated unit or a mixture of small experts with a squared relu.
A layer may run with the weights of an earlier one, keeping a cache or state of its own.
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


def rotary_frequencies(dims: int, base: float, scaling: dict | None) -> tuple[torch.Tensor, float]:
    """(f_i for i < dims/2, the factor on cos and sin). Without scaling f_i = base^(-2i/dims) and the
    factor is 1. With scaling (factor s, original length L, fast, slow): d(t) = dims ln(L / (2 pi t)) /
    (2 ln base), lo = max(floor d(fast), 0), hi = min(ceil d(slow), dims - 1), r_i = clamp((i - lo) /
    max(hi - lo, 0.001), 0, 1); f_i <- f_i / s * r_i + f_i (1 - r_i); the factor is 0.1 ln s + 1."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = torch.tensor(float(base), dtype=torch.float64) ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    s, length = float(scaling["factor"]), float(scaling["original"])

    def d(t: float) -> float:
        return dims * math.log(length / (2.0 * math.pi * t)) / (2.0 * math.log(base))

    lo = max(math.floor(d(float(scaling["fast"]))), 0)
    hi = min(math.ceil(d(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / s * ramp + f * (1.0 - ramp), 0.1 * math.log(s) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, freqs: torch.Tensor, amplitude: float, interleaved: bool) -> torch.Tensor:
    """x [n, ..., D]: the first 2 len(freqs) dimensions of the last axis turn by positions * f_i, pair i
    being dimensions (2i, 2i + 1) if `interleaved`, else (i, i + len(freqs)); the rest pass."""
    half = freqs.shape[0]
    if half == 0:
        return x
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    angle = (positions.to(torch.float64)[:, None] * freqs[None, :])
    cos = (torch.cos(angle) * amplitude).to(x.dtype).reshape(shape)
    sin = (torch.sin(angle) * amplitude).to(x.dtype).reshape(shape)
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:2 * half:2], x[..., 1:2 * half:2]
        out[..., 0:2 * half:2] = u * cos - v * sin
        out[..., 1:2 * half:2] = v * cos + u * sin
    else:
        u, v = x[..., :half], x[..., half:2 * half]
        out[..., :half] = u * cos - v * sin
        out[..., half:2 * half] = v * cos + u * sin
    return out


def visibility(q_positions: torch.Tensor, keys: int, kind: str, size: int) -> torch.Tensor:
    """[n, keys] booleans: whether the query at position i sees key position j. Causal, and then by the
    mask's kind: "window": i - j < size; "chunk": floor(i / size) = floor(j / size); "full": all before."""
    i, j = q_positions[:, None], torch.arange(keys)[None, :]
    see = j <= i
    if kind == "window":
        see &= (i - j) < size
    elif kind == "chunk":
        see &= torch.div(i, size, rounding_mode="floor") == torch.div(j, size, rounding_mode="floor")
    return see


def masked_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, q_positions: torch.Tensor, scale: float,
                     kind: str, size: int, sinks: torch.Tensor | None) -> torch.Tensor:
    """q [n, H, D] at `q_positions` over keys k [m, G, D] and values v [m, G, V] at positions 0..m-1.
    weight_j = exp(s_j) / (sum over visible j' of exp(s_j') [+ exp(sink_h)]), s_j = q.k_j scale."""
    n, H, _ = q.shape
    G = k.shape[1]
    see = visibility(q_positions, k.shape[0], kind, size)
    out = torch.zeros(n, H, v.shape[2], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~see, float("-inf"))
        top = s.max(dim=-1, keepdim=True).values
        if sinks is not None:
            top = torch.maximum(top, sinks[h])
        e = torch.exp(s - top)
        total = e.sum(-1, keepdim=True) + (torch.exp(sinks[h] - top) if sinks is not None else 0.0)
        out[:, h] = (e / total) @ v[:, g]
    return out


def mask_of(mixer: dict, default: str) -> tuple[str, int]:
    mask = mixer.get("mask")
    return (default, int(mask["size"])) if mask else ("full", 0)


def chunk_attention(h: torch.Tensor, positions: torch.Tensor, W: dict, m: dict, eps: float, past: dict) -> torch.Tensor:
    """The "attention" mixer for the rows h at `positions`; `past` holds the keys and values so far."""
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    n = h.shape[0]
    q = unit_rms(h @ W["q"].T, eps) * W["q.norm"]           # over the whole projection, before the heads are cut
    k = unit_rms(h @ W["k"].T, eps) * W["k.norm"]
    v = h @ W["v"].T
    rot = m.get("rot") or {}
    freqs, amp = rotary_frequencies(int(rot.get("dims", 0)), float(rot.get("base", 1.0)), rot.get("scaling")) \
        if rot.get("dims") else (torch.zeros(0, dtype=torch.float64), 1.0)
    q = rotate(q.reshape(n, H, D), positions, freqs, amp, interleaved=False)
    k = rotate(k.reshape(n, G, D), positions, freqs, amp, interleaved=False)
    past["k"] = torch.cat([past["k"], k]) if "k" in past else k
    past["v"] = torch.cat([past["v"], v.reshape(n, G, V)]) if "v" in past else v.reshape(n, G, V)
    kind, size = mask_of(m, "chunk")
    o = masked_attention(q, past["k"], past["v"], positions, float(m["scale"]), kind, size, W["sink"])
    return o.reshape(n, H * V) @ W["o"].T


def latent_attention(h: torch.Tensor, positions: torch.Tensor, W: dict, m: dict, eps: float, past: dict) -> torch.Tensor:
    """The "latent_attention" mixer; `past` holds the latents and the shared rotated key parts so far."""
    H, D, R, V, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    n = h.shape[0]
    cq = unit_rms(h @ W["dq"].T, eps) * W["dq.norm"]
    q = (cq @ W["uq"].T).reshape(n, H, D + R)
    down = h @ W["dkv"].T
    c = unit_rms(down[:, :C], eps) * W["dkv.norm"]
    rot = m["rot"]
    freqs, amp = rotary_frequencies(R, float(rot["base"]), rot.get("scaling"))
    kr = rotate(down[:, C:C + R], positions, freqs, amp, interleaved=True)
    qr = rotate(q[..., D:], positions, freqs, amp, interleaved=True)
    past["c"] = torch.cat([past["c"], c]) if "c" in past else c
    past["kr"] = torch.cat([past["kr"], kr]) if "kr" in past else kr
    keys = torch.cat([(past["c"] @ W["uk"].T).reshape(-1, H, D), past["kr"][:, None, :].expand(-1, H, -1)], dim=-1)
    values = (past["c"] @ W["uv"].T).reshape(-1, H, V)
    kind, size = mask_of(m, "window")
    o = masked_attention(torch.cat([q[..., :D], qr], dim=-1), keys, values, positions, float(m["scale"]), kind, size, None)
    return (o.reshape(n, H * V) * torch.sigmoid(h @ W["g"].T)) @ W["o"].T


def mlstm(h: torch.Tensor, W: dict, m: dict, eps: float, state: dict) -> torch.Tensor:
    """The "mlstm" mixer, token by token. state: S [H, D, V], n [H, D], m [H], zeros at the start.
    m_t = max(f + m', i); S = exp(f + m' - m_t) S' + exp(i - m_t) k v^T; n likewise with k;
    o = S^T q / (max(|n.q|, exp(-m_t)) + 1e-6); then rms per head, a weight, a sigmoid gate, W_o."""
    H, D, V, cap = m["heads"], m["dim"], m["vdim"], float(m["gate_cap"])
    if "S" not in state:
        state["S"] = torch.zeros(H, D, V, dtype=h.dtype)
        state["n"] = torch.zeros(H, D, dtype=h.dtype)
        state["m"] = torch.zeros(H, dtype=h.dtype)
    rows = []
    for t in range(h.shape[0]):
        x = h[t]
        q = (W["q"] @ x).reshape(H, D) * D ** -0.5
        k = (W["k"] @ x).reshape(H, D)
        v = (W["v"] @ x).reshape(H, V)
        i = cap * torch.tanh((W["i"] @ x + W["i.b"]) / cap)
        f = torch.nn.functional.logsigmoid(cap * torch.tanh((W["f"] @ x + W["f.b"]) / cap))
        m_new = torch.maximum(f + state["m"], i)
        keep, take = torch.exp(f + state["m"] - m_new), torch.exp(i - m_new)
        state["S"] = keep[:, None, None] * state["S"] + take[:, None, None] * k[:, :, None] * v[:, None, :]
        state["n"] = keep[:, None] * state["n"] + take[:, None] * k
        state["m"] = m_new
        num = torch.einsum("hdv,hd->hv", state["S"], q)
        den = torch.maximum((state["n"] * q).sum(-1).abs(), torch.exp(-m_new)) + 1e-6
        o = unit_rms(num / den[:, None], eps).reshape(H * V) * W["norm"]
        rows.append((o * torch.sigmoid(W["g"] @ x)) @ W["o"].T)
    return torch.stack(rows)


def gated_unit(h: torch.Tensor, W: dict) -> torch.Tensor:
    return (torch.nn.functional.silu(h @ W["gate"].T) * (h @ W["up"].T)) @ W["down"].T


def chosen_experts(logits: torch.Tensor, top: int) -> tuple[torch.Tensor, torch.Tensor]:
    """(indices [n, top] of the largest logits, their weights: the softmax over those logits alone)."""
    best, idx = torch.topk(logits, top, dim=-1)
    return idx, torch.softmax(best, dim=-1)


def expert_mixture(h: torch.Tensor, W: dict, mlp: dict) -> torch.Tensor:
    idx, weights = chosen_experts(h @ W["router"].T, int(mlp["router"]["top"]))
    out = torch.zeros(h.shape[0], W["e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        for w, e in zip(weights[t], idx[t]):
            e = int(e)
            out[t] += w * (torch.relu(W[f"e{e}.up"] @ h[t]) ** 2) @ W[f"e{e}.down"].T
    return out


class PlainBafarax:
    """The whole decoder over one request, fed in any portions; keeps that request's caches and states."""

    def __init__(self, config: dict, weights: dict[str, torch.Tensor], dtype: torch.dtype = torch.float64) -> None:
        self.c, self.dtype = config, dtype
        self.w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
        self.memory: list[dict] = [dict() for _ in config["layers"]]
        self.fed = 0
        self.after_layers: list[torch.Tensor] = []      # the residual stream after every layer, of the last call

    @classmethod
    def from_folder(cls, folder: str, dtype: torch.dtype = torch.float64) -> "PlainBafarax":
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
        x = self.w["embed"][torch.tensor(tokens)] * float((c.get("embedding") or {}).get("scale", 1.0))
        self.after_layers = []
        for i, layer in enumerate(c["layers"]):
            src = layer.get("weights_of", i)
            h = layer_norm(x, self.w[f"l{src}.norm1"], eps)
            W, m, kind = self._sub(f"l{src}.mix."), layer["mixer"], layer["type"]
            if kind == "attention":
                x = x + chunk_attention(h, positions, W, m, eps, self.memory[i])
            elif kind == "latent_attention":
                x = x + latent_attention(h, positions, W, m, eps, self.memory[i])
            elif kind == "mlstm":
                x = x + mlstm(h, W, m, eps, self.memory[i])
            else:
                raise ValueError(kind)
            mlp = layer.get("mlp")
            if mlp is not None:
                h = layer_norm(x, self.w[f"l{src}.norm2"], eps)
                F = self._sub(f"l{src}.mlp.")
                x = x + (gated_unit(h, F) if mlp["kind"] == "dense" else expert_mixture(h, F, mlp))
            self.after_layers.append(x.clone())
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
