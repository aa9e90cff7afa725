"""A plain, slow Nokipel: one function per mechanism, written from the design's equations with torch tensor
arithmetic only.  It shares no code with the package; the tests compare the engine with it.

A model is ``(raw, weights)``: ``raw`` the dictionary a ``config.json`` of this design holds, ``weights`` a
name -> tensor dictionary.  Everything runs in ``dtype`` (float64 by default, the yardstick).  ``forward`` runs a
whole sequence and can hand back the stream after every layer run; ``Stepper`` keeps a sequence's keys, values and
memories from call to call and is fed any number of tokens at a time.

The design in this file's notation (t a token at position p counted from 0, h a sublayer's input):

    x_0 = E[token] * c_embed
    a layer:  x <- x + mix(N(x; w1)),  x <- x + ff(N(x; w2))
    N(y; w):  y cut into n equal consecutive parts, each divided by sqrt(mean(part^2) + eps), the whole times w
    run order: layers 0 .. start-1 once; layers start .. stop-1 `times` times over (each pass with keys, values and
               memories of its own; before every pass but the first x <- x + x_0); layers stop .. once
    logits = H N(x; w_final)

    'attention', query head a of H on key head floor(a / (H / G)):
      q = W_q h + b_q, k = W_k h + b_k, v = W_v h + b_v
      q, k: the first R numbers of each head turn in neighbouring pairs: (y_2i, y_2i+1) at position p becomes
            (y_2i cos - y_2i+1 sin, y_2i+1 cos + y_2i sin) of the angle p * base^(-2i / R)
      s_ij = (q_i . k_j) * scale for j <= i with floor(i / C) = floor(j / C), nothing else is seen (C counted from 0)
      o_i = softmax_j(s_ij) v_j;  out = W_o concat(o)

    'lightning', head a:
      q = silu(W_q h), k = silu(W_k h), v = silu(W_v h)
      S_t = d_a S_(t-1) + k_t v_t^T  (S before the first token is 0),  o_t = S_t^T q_t
      out = W_o (concat(o) / sqrt(mean(concat(o)^2) + eps) * w_norm * sigmoid(W_g h))

    dense feed-forward: g = min(W_gate h, L), u = clamp(W_up h, -L, L);  W_down (g sigmoid(1.702 g) (u + 1))

    routed feed-forward with E experts and I identity experts behind them (E + I router outputs):
      z = W_r h,  s = softmax(z),  c = s + correction
      the E + I outputs in `count` equal groups of neighbours; a group's score is its largest c; outside the `keep`
      best groups c counts as -inf; the `top` largest c are chosen
      w_e = s_e / (sum of the chosen s + 1e-20) * c_route
      out = sum_chosen w_e * expert_e(h)  [+ sigmoid(W_sg h) * shared(h)]
      expert_e(h) = W_down silu(W_gate h) * (W_up h)  for e < E,   h itself for e >= E
"""

from __future__ import annotations

import math

import torch


def grouped_norm(x, w, groups: int, eps: float):
    """Each of `groups` equal consecutive parts over its own root mean square (eps inside the root), times w."""
    parts = x.reshape(*x.shape[:-1], groups, x.shape[-1] // groups)
    parts = parts / torch.sqrt((parts * parts).mean(dim=-1, keepdim=True) + eps)
    return parts.reshape(x.shape) * w


def silu(z):
    return z * torch.sigmoid(z)


def turn_pairs(y, positions, dims: int, base: float):
    """y [T, heads, dim]: neighbouring pairs of the first `dims` numbers of each head turned by the position."""
    if not dims:
        return y
    i = torch.arange(dims // 2, dtype=y.dtype)
    freq = float(base) ** (-2.0 * i / dims)
    angle = positions.to(y.dtype)[:, None] * freq[None, :]                  # [T, dims / 2]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    even, odd = y[..., 0:dims:2], y[..., 1:dims:2]
    out = y.clone()
    out[..., 0:dims:2] = even * cos - odd * sin
    out[..., 1:dims:2] = odd * cos + even * sin
    return out


def chunk_sees(i: int, j: int, size) -> bool:
    """Whether the query at position i sees the key at position j."""
    if j > i:
        return False
    return size is None or i // size == j // size


def softmax_attention_token(q, keys, values, i: int, key_positions, size, scale: float):
    """One query head's output at position i: q [dim], keys [n, dim], values [n, vdim]."""
    seen = [n for n, j in enumerate(key_positions) if chunk_sees(i, j, size)]
    scores = torch.stack([(q * keys[n]).sum() * scale for n in seen])
    weights = torch.softmax(scores, dim=0)
    return (weights[:, None] * values[seen]).sum(dim=0)


def lightning_token(S, q, k, v, decay):
    """One head, one token: the memory after the token and what the token reads from it."""
    S = decay * S + k[:, None] * v[None, :]
    return S, S.t() @ q


def dense_feed_forward(h, w_gate, w_up, w_down, limit: float):
    g = torch.clamp(h @ w_gate.t(), max=limit)
    u = torch.clamp(h @ w_up.t(), min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ w_down.t()


def gated_expert(h, w_gate, w_up, w_down):
    return (silu(h @ w_gate.t()) * (h @ w_up.t())) @ w_down.t()


def router_choice(z, correction, top: int, count: int, keep: int, scale: float):
    """z [n] router outputs of one token -> (chosen indices, their weights)."""
    s = torch.softmax(z, dim=0)
    c = s + correction
    n = z.shape[0]
    per = n // count
    group_score = torch.stack([c[g * per:(g + 1) * per].max() for g in range(count)])
    kept = sorted(range(count), key=lambda g: (-float(group_score[g]), g))[:keep]
    allowed = torch.full_like(c, -math.inf)
    for g in kept:
        allowed[g * per:(g + 1) * per] = c[g * per:(g + 1) * per]
    chosen = sorted(range(n), key=lambda e: (-float(allowed[e]), e))[:top]
    picked = s[chosen]
    return chosen, picked / (picked.sum() + 1e-20) * scale


class Model:
    def __init__(self, raw: dict, weights: dict, dtype=torch.float64):
        self.raw = raw
        self.dtype = dtype
        self.w = {name: t.to(dtype) for name, t in weights.items()}
        self.eps = float(raw["norm"]["eps"])
        self.groups = int(raw["norm"].get("groups", 1))
        loop = raw.get("loop") or {}
        n = len(raw["layers"])
        start, stop, times = int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1))
        # (layer, pass, whether the embedding's rows are added before it)
        self.runs = [(i, 0, False) for i in range(0, start)]
        for p in range(times if stop > start else 0):
            self.runs += [(i, p, p > 0 and i == start) for i in range(start, stop)]
        self.runs += [(i, 0, False) for i in range(max(stop, start), n)]

    def norm(self, x, name):
        return grouped_norm(x, self.w[name], self.groups, self.eps)

    # ---- mixers: h [T, width] the tokens of one call at `positions`; `kept` the sequence's record for this run
    def attention(self, prefix, sizes, h, positions, kept):
        H, G, D, V = int(sizes["heads"]), int(sizes.get("kv_heads", sizes["heads"])), int(sizes["dim"]), int(sizes["vdim"])
        w = self.w
        T = h.shape[0]
        q = (h @ w[prefix + "q"].t() + w[prefix + "q.b"]).reshape(T, H, D)
        k = (h @ w[prefix + "k"].t() + w[prefix + "k.b"]).reshape(T, G, D)
        v = (h @ w[prefix + "v"].t() + w[prefix + "v.b"]).reshape(T, G, V)
        rot = sizes.get("rot")
        if rot:
            q = turn_pairs(q, positions, int(rot["dims"]), float(rot["base"]))
            k = turn_pairs(k, positions, int(rot["dims"]), float(rot["base"]))
        kept.setdefault("k", []).extend(k)
        kept.setdefault("v", []).extend(v)
        kept.setdefault("p", []).extend(int(p) for p in positions)
        keys, values = torch.stack(kept["k"]), torch.stack(kept["v"])
        size = int(sizes["mask"]["size"]) if sizes.get("mask") else None
        out = torch.zeros((T, H, V), dtype=self.dtype)
        for t in range(T):
            for a in range(H):
                g = a // (H // G)
                out[t, a] = softmax_attention_token(q[t, a], keys[:, g], values[:, g], int(positions[t]), kept["p"],
                                                    size, float(sizes["scale"]))
        return out.reshape(T, H * V) @ w[prefix + "o"].t()

    def lightning(self, prefix, sizes, h, positions, kept):
        H, D, V = int(sizes["heads"]), int(sizes["dim"]), int(sizes["vdim"])
        w = self.w
        T = h.shape[0]
        q = silu(h @ w[prefix + "q"].t()).reshape(T, H, D)
        k = silu(h @ w[prefix + "k"].t()).reshape(T, H, D)
        v = silu(h @ w[prefix + "v"].t()).reshape(T, H, V)
        S = kept.setdefault("S", torch.zeros((H, D, V), dtype=self.dtype))
        out = torch.zeros((T, H, V), dtype=self.dtype)
        for t in range(T):
            for a in range(H):
                S[a], out[t, a] = lightning_token(S[a], q[t, a], k[t, a], v[t, a], float(sizes["decay"][a]))
        flat = out.reshape(T, H * V)
        flat = flat / torch.sqrt((flat * flat).mean(dim=-1, keepdim=True) + self.eps) * w[prefix + "norm"]
        return (flat * torch.sigmoid(h @ w[prefix + "g"].t())) @ w[prefix + "o"].t()

    # ---- feed-forwards
    def feed_forward(self, prefix, mlp, h):
        w = self.w
        if mlp["kind"] == "dense":
            return dense_feed_forward(h, w[prefix + "gate"], w[prefix + "up"], w[prefix + "down"], float(mlp["limit"]))
        router = mlp["router"]
        experts, identity = int(router["experts"]), int(router.get("identity", 0))
        groups = router.get("groups") or {"count": 1, "keep": 1}
        correction = w.get(prefix + "correction")
        out = torch.zeros_like(h)
        for t in range(h.shape[0]):
            z = w[prefix + "router"] @ h[t]
            chosen, weights = router_choice(z, correction if correction is not None else torch.zeros_like(z),
                                            int(router["top"]), int(groups["count"]), int(groups["keep"]),
                                            float(router.get("scale", 1.0)))
            for e, weight in zip(chosen, weights):
                if e >= experts:
                    out[t] += weight * h[t]
                else:
                    out[t] += weight * gated_expert(h[t], w[f"{prefix}e{e}.gate"], w[f"{prefix}e{e}.up"], w[f"{prefix}e{e}.down"])
        if mlp.get("shared"):
            shared = gated_expert(h, w[prefix + "shared.gate"], w[prefix + "shared.up"], w[prefix + "shared.down"])
            out = out + torch.sigmoid(h @ w[prefix + "shared.sg"].t()) * shared
        return out

    def run_tokens(self, tokens, positions, record, taps=None):
        """The stream of `tokens` at `positions` through all layer runs; `record[run]` is the sequence's memory."""
        scale = float((self.raw.get("embedding") or {}).get("scale", 1.0))
        x0 = self.w["embed"][torch.as_tensor(tokens)] * scale
        x = x0.clone()
        positions = torch.as_tensor(positions)
        for run, (index, _pass, adds) in enumerate(self.runs):
            layer = self.raw["layers"][index]
            prefix = f"l{index}."
            if adds:
                x = x + x0
            mixer = self.attention if layer["type"] == "attention" else self.lightning
            x = x + mixer(prefix + "mix.", layer["mixer"], self.norm(x, prefix + "norm1"), positions, record.setdefault(run, {}))
            if layer.get("mlp"):
                x = x + self.feed_forward(prefix + "mlp.", layer["mlp"], self.norm(x, prefix + "norm2"))
            if taps is not None:
                taps.append(x.clone())
        return x

    def logits(self, x):
        return self.norm(x, "final.norm") @ self.w["head"].t()


def forward(raw, weights, tokens, dtype=torch.float64, taps=None):
    """Logits [T, vocab] of a whole sequence."""
    model = Model(raw, weights, dtype)
    return model.logits(model.run_tokens(list(tokens), list(range(len(tokens))), {}, taps))


class Stepper:
    """One sequence fed in pieces: what it has seen stays between calls."""

    def __init__(self, raw, weights, dtype=torch.float64):
        self.model = Model(raw, weights, dtype)
        self.record: dict = {}
        self.fed = 0

    def feed(self, tokens):
        positions = list(range(self.fed, self.fed + len(tokens)))
        self.fed += len(tokens)
        return self.model.logits(self.model.run_tokens(list(tokens), positions, self.record))
