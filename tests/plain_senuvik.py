"""A plain, slow implementation of the Senuvik decoder, one function per mechanism, in float64 and token by token.

It shares no code with the package: tests compare the engine with it.  A model is a raw configuration (the
``config.json`` dictionary) and a dictionary of tensors by checkpoint name.  ``Model.start()`` gives a ``Sequence``
that is fed tokens one at a time (or in runs) and keeps what the design carries from token to token: keys and
values of the attention layers, the state-space memory and the convolution's last inputs, the time-mixing memory
and the previous token's input.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


# ---------------------------------------------------------------------------------------------------- mechanisms
def rms_norm(x: torch.Tensor, weight, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) * weight over the last axis (``weight=None``: no weight)."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0.0)


def plain_frequencies(dims: int, base: float) -> torch.Tensor:
    return torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)  # (angles stay float64)


def linear_frequencies(dims: int, base: float, factor: float) -> tuple[torch.Tensor, float]:
    return plain_frequencies(dims, base) / factor, 1.0


def yarn_frequencies(dims: int, base: float, factor: float, original: float, fast: float,
                     slow: float) -> tuple[torch.Tensor, float]:
    """Frequencies stretched where a pair turns slowly over the original length, and the factor on cos and sin."""
    f = plain_frequencies(dims, base)
    at = lambda t: dims * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(base))
    lo = max(math.floor(at(fast)), 0)
    hi = min(math.ceil(at(slow)), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(dims // 2)], dtype=F)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(head: torch.Tensor, position: int, frequencies: torch.Tensor, gain: float, dims: int,
           neighbours: bool) -> torch.Tensor:
    """Turn the first ``dims`` numbers of a head: pairs (2i, 2i + 1) or (i, i + dims / 2)."""
    out = head.clone()
    for i in range(dims // 2):
        a, b = (2 * i, 2 * i + 1) if neighbours else (i, i + dims // 2)
        angle = position * float(frequencies[i])
        c, s = math.cos(angle) * gain, math.sin(angle) * gain
        u, v = head[a], head[b]
        out[a] = u * c - v * s
        out[b] = v * c + u * s
    return out


def window_sees(i: int, j: int, size, keep_first: int) -> bool:
    """Whether the token at i sees the key at j: behind it, and within the window or among the kept first tokens."""
    if j > i:
        return False
    return size is None or i - j < size or j < keep_first


def softmax_attention_token(q: torch.Tensor, keys: torch.Tensor, values: torch.Tensor, seen: list, scale: float,
                            softcap=None, sink=None) -> torch.Tensor:
    """One head's output for one token: q [dim], keys [n, dim], values [n, vdim], seen: indices of the visible keys."""
    scores = (keys[seen] @ q) * scale
    if softcap is not None:
        scores = softcap * torch.tanh(scores / softcap)
    top = scores.max() if sink is None else torch.maximum(scores.max(), sink)
    weights = torch.exp(scores - top)
    denominator = weights.sum() + (torch.exp(sink - top) if sink is not None else 0.0)
    return (weights / denominator) @ values[seen]


def router_choice(logits: torch.Tensor, top: int) -> tuple[list, torch.Tensor]:
    """The ``top`` largest logits (lowest index first among equals) and the softmax over them alone."""
    order = sorted(range(logits.shape[0]), key=lambda e: (-float(logits[e]), e))[:top]
    chosen = logits[order]
    weights = torch.exp(chosen - chosen.max())
    return order, weights / weights.sum()


def gated_unit(x: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, act) -> torch.Tensor:
    return down @ (act(gate @ x) * (up @ x))


def state_space_token(memory: torch.Tensor, x: torch.Tensor, b: torch.Tensor, c: torch.Tensor, dt: torch.Tensor,
                      a_log: torch.Tensor, d: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """One head: memory [N, vdim], x [vdim], b, c [N], dt, a_log, d scalars.  Returns (new memory, y)."""
    memory = torch.exp(-torch.exp(a_log) * dt) * memory + dt * torch.outer(b, x)
    return memory, memory.t() @ c + d * x


def time_mix_token(memory: torch.Tensor, r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, w: torch.Tensor,
                   u: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """One head: memory [dim, dim] (key channel, value channel); the bonus u counts for the current token only."""
    out = (memory + torch.outer(u * k, v)).t() @ r
    return w[:, None] * memory + torch.outer(k, v), out


# ---------------------------------------------------------------------------------------------------- the model
class Model:
    def __init__(self, config: dict, tensors: dict, dtype: torch.dtype = F) -> None:
        self.config = config
        self.dtype = dtype  # float64 is the yardstick; bfloat16 shows what rounding everything to 16 bits costs
        self.t = {name: value.to(dtype) for name, value in tensors.items()}
        self.eps = float(config["norm"]["eps"])
        self.width = int(config["width"])
        self.layers = config["layers"]

    def start(self) -> "Sequence":
        return Sequence(self)

    def logits(self, tokens) -> torch.Tensor:
        """Logits [len(tokens), vocab] of one sequence from its start."""
        return self.start().feed(tokens)


class Sequence:
    def __init__(self, model: Model) -> None:
        self.m = model
        self.position = 0
        self.kv: dict[int, tuple[list, list]] = {}      # layer -> (keys [G, dim] per token, values [G, vdim] per token)
        self.state: dict[tuple, torch.Tensor] = {}      # (layer, what) -> tensor
        self.stream_after: list[list[torch.Tensor]] = []  # per token, the stream after every layer

    def feed(self, tokens) -> torch.Tensor:
        return torch.stack([self.token(int(t)) for t in tokens])

    # -- one token through the whole model
    def token(self, token: int) -> torch.Tensor:
        m, t = self.m, self.m.t
        x = t["embed"][token].clone()
        after = []
        for index, layer in enumerate(m.layers):
            p = f"l{index}."
            mixed = self.mixer(index, layer, rms_norm(x, t[p + "norm1"], m.eps))
            x = x + rms_norm(mixed, t[p + "norm1b"], m.eps) * t[p + "ls1"]
            if layer.get("mlp") is not None:
                fed = self.feed_forward(p + "mlp.", layer["mlp"], rms_norm(x, t[p + "norm2"], m.eps))
                x = x + rms_norm(fed, t[p + "norm2b"], m.eps) * t[p + "ls2"]
            after.append(x.clone())
        self.stream_after.append(after)
        self.position += 1
        return t["head"] @ rms_norm(x, t["final.norm"], m.eps)

    def mixer(self, index: int, layer: dict, h: torch.Tensor) -> torch.Tensor:
        kind, sizes, p = layer["type"], layer["mixer"], f"l{index}.mix."
        if kind == "attention":
            return self.attention(index, sizes, p, h)
        if kind == "mamba2":
            return self.mamba2(index, sizes, p, h)
        if kind == "parallel":
            left = self.left(index, sizes["left"], p + "left.", h)
            right = self.right(index, sizes["right"], p + "right.", h)
            return float(sizes["left_scale"]) * left + float(sizes["right_scale"]) * right
        raise ValueError(kind)

    # -- softmax attention with a window, kept first tokens and a sink
    def attention(self, index: int, c: dict, p: str, h: torch.Tensor) -> torch.Tensor:
        m, t = self.m, self.m.t
        H, G, dim, vdim = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        rot = c["rot"]
        scaling = rot.get("scaling") or {}
        frequencies, gain = linear_frequencies(rot["dims"], rot["base"], float(scaling.get("factor", 1.0)))
        q = rms_norm(t[p + "q"] @ h + t[p + "q.b"], t[p + "q.norm"], m.eps).reshape(H, dim)
        q = torch.stack([rotate(q[i], self.position, frequencies, gain, rot["dims"], True) for i in range(H)])
        source = c.get("kv_from")
        if source is None:
            k = rms_norm(t[p + "k"] @ h + t[p + "k.b"], t[p + "k.norm"], m.eps).reshape(G, dim)
            k = torch.stack([rotate(k[i], self.position, frequencies, gain, rot["dims"], True) for i in range(G)])
            v = (t[p + "v"] @ h + t[p + "v.b"]).reshape(G, vdim)
            keys, values = self.kv.setdefault(index, ([], []))
            keys.append(k)
            values.append(v)
        else:
            keys, values = self.kv[source]
        mask = c.get("mask") or {}
        seen = [j for j in range(self.position + 1)
                if window_sees(self.position, j, mask.get("size"), int(mask.get("keep_first", 0)))]
        all_k, all_v = torch.stack(keys), torch.stack(values)
        out = [softmax_attention_token(q[i], all_k[:, i // (H // G)], all_v[:, i // (H // G)], seen, float(c["scale"]),
                                       sink=t[p + "sink"][i]) for i in range(H)]
        return t[p + "o"] @ torch.cat(out)

    # -- the left branch of a parallel layer: causal attention, rotation by halves, capped scores, a gate per head
    def left(self, index: int, c: dict, p: str, h: torch.Tensor) -> torch.Tensor:
        t = self.m.t
        H, G, dim, vdim = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
        rot = c["rot"]
        s = rot.get("scaling")
        if s is not None:
            frequencies, gain = yarn_frequencies(rot["dims"], rot["base"], s["factor"], s["original"], s["fast"], s["slow"])
        else:
            frequencies, gain = plain_frequencies(rot["dims"], rot["base"]), 1.0
        q = (t[p + "q"] @ h).reshape(H, dim)
        k = (t[p + "k"] @ h).reshape(G, dim)
        q = torch.stack([rotate(q[i], self.position, frequencies, gain, rot["dims"], False) for i in range(H)])
        k = torch.stack([rotate(k[i], self.position, frequencies, gain, rot["dims"], False) for i in range(G)])
        v = (t[p + "v"] @ h).reshape(G, vdim)
        keys, values = self.kv.setdefault(index, ([], []))
        keys.append(k)
        values.append(v)
        all_k, all_v = torch.stack(keys), torch.stack(values)
        seen = list(range(self.position + 1))
        gate = torch.sigmoid(t[p + "g"] @ h)
        out = [softmax_attention_token(q[i], all_k[:, i // (H // G)], all_v[:, i // (H // G)], seen, float(c["scale"]),
                                       softcap=c.get("softcap")) * gate[i] for i in range(H)]
        return t[p + "o"] @ torch.cat(out)

    # -- the right branch: time mixing with a decay per channel that depends on the token
    def right(self, index: int, c: dict, p: str, h: torch.Tensor) -> torch.Tensor:
        m, t = self.m, self.m.t
        heads, dim = c["heads"], c["dim"]
        before = self.state.get((index, "previous"), torch.zeros_like(h))
        mix = {s: h + (before - h) * t[p + "mu." + s] for s in "rkvgw"}
        r = (t[p + "r"] @ mix["r"]).reshape(heads, dim)
        k = (t[p + "k"] @ mix["k"]).reshape(heads, dim)
        v = (t[p + "v"] @ mix["v"]).reshape(heads, dim)
        gate = silu(t[p + "g"] @ mix["g"])
        w = torch.exp(-torch.exp(t[p + "w2"] @ torch.tanh(t[p + "w1"] @ mix["w"]) + t[p + "w0"])).reshape(heads, dim)
        memory = self.state.get((index, "memory"), torch.zeros((heads, dim, dim), dtype=m.dtype))
        outs, new = [], []
        for i in range(heads):
            s, o = time_mix_token(memory[i], r[i], k[i], v[i], w[i], t[p + "u"][i])
            new.append(s)
            outs.append(rms_norm(o, None, m.eps))
        self.state[(index, "memory")] = torch.stack(new)
        self.state[(index, "previous")] = h.clone()
        return t[p + "o"] @ (torch.cat(outs) * t[p + "norm"] * gate)

    # -- the state-space mixer
    def mamba2(self, index: int, c: dict, p: str, h: torch.Tensor) -> torch.Tensor:
        m, t = self.m, self.m.t
        heads, vdim, N, G, taps = c["heads"], c["vdim"], c["state"], c["groups"], c["conv"]
        inner = heads * vdim
        proj = t[p + "in"] @ h
        z, xbc, dt = proj[:inner], proj[inner: 2 * inner + 2 * G * N], proj[2 * inner + 2 * G * N:]
        past = self.state.get((index, "past"), torch.zeros((taps - 1, xbc.shape[0]), dtype=m.dtype))
        inputs = torch.cat([past, xbc[None]], dim=0)                         # the last `taps` inputs, oldest first
        xbc = silu((inputs * t[p + "conv"].t()).sum(0) + t[p + "conv.b"])
        self.state[(index, "past")] = inputs[1:]
        x = xbc[:inner].reshape(heads, vdim)
        b = xbc[inner: inner + G * N].reshape(G, N)
        cc = xbc[inner + G * N:].reshape(G, N)
        dt = softplus(dt + t[p + "dt_bias"])
        memory = self.state.get((index, "memory"), torch.zeros((heads, N, vdim), dtype=m.dtype))
        ys, new = [], []
        for i in range(heads):
            g = i // (heads // G)
            s, y = state_space_token(memory[i], x[i], b[g], cc[g], dt[i], t[p + "A_log"][i], t[p + "D"][i])
            new.append(s)
            ys.append(y)
        self.state[(index, "memory")] = torch.stack(new)
        y = torch.cat(ys) * silu(z)
        parts = int(c.get("norm_groups", 1))
        y = rms_norm(y.reshape(parts, inner // parts), None, m.eps).reshape(inner) * t[p + "norm"]
        return t[p + "o"] @ y

    # -- feed-forwards
    def feed_forward(self, p: str, c: dict, h: torch.Tensor) -> torch.Tensor:
        t = self.m.t
        if c["kind"] == "dense":
            return gated_unit(h, t[p + "gate"], t[p + "up"], t[p + "down"], gelu_tanh)
        chosen, weights = router_choice(t[p + "router"] @ h, int(c["router"]["top"]))
        out = torch.zeros_like(h)
        for e, weight in zip(chosen, weights):
            out = out + weight * gated_unit(h, t[f"{p}e{e}.gate"], t[f"{p}e{e}.up"], t[f"{p}e{e}.down"], silu)
        if c.get("shared") is not None:
            shared = gated_unit(h, t[p + "shared.gate"], t[p + "shared.up"], t[p + "shared.down"], silu)
            out = out + torch.sigmoid(t[p + "shared.sg"] @ h)[0] * shared
        return out


def forward(config: dict, tensors: dict, tokens, dtype: torch.dtype = F) -> torch.Tensor:
    """Logits [len(tokens), vocab] of one sequence from its start."""
    return Model(config, tensors, dtype).logits(tokens)
