"""Mixers with a state of fixed size per request (``FixedState`` cache units) instead of a growing cache.

``Retention``: linear attention with a fixed decay per head and neither softmax nor denominator.  With
``q, k`` (heads x dim) turned by the position and ``k`` scaled by ``dim^-1/2`` after the turn, ``v`` (heads x vdim):
``S_t = decay_h S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t``; each head's ``o_t`` is divided by its root mean square
(no weight), the heads are concatenated, multiplied by ``silu(W_g x)`` and projected.  The state ``S`` [heads, dim,
vdim] is float32.

``LightningAttention``: the same memory and read-out with activated queries, keys and values, no rotation, one
norm with a weight over all heads' read-outs together and a ``sigmoid`` gate.

``GatedLinearRecurrence``: two branches of ``width`` channels, ``y = gelu_tanh(W_y x + b_y)`` and
``u = conv(W_x x + b_x)`` (a causal convolution over each channel's last ``taps`` inputs); per block of channels
``r = sigmoid(A_b u_b + a_b)``, ``i = sigmoid(B_b u_b + b_b)``; ``a = exp(-8 r softplus(lambda))``,
``S_t = a S_(t-1) + sqrt(1 - a^2) i u_t``; the output is ``W_o (S_t y_t)``.  Its state is ``S`` [width] and the
convolution's last ``taps - 1`` inputs, both float32.

``StateSpace``: a state-space layer with one decay per head and token (the duality form): one product makes
``z | x | B | C | dt``; ``x, B, C`` pass a causal convolution and ``silu``; ``dt = softplus(dt + bias)``; per head
``S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T`` and ``y_t = S_t^T C_t + D x_t``; ``y silu(z)`` is normed in
groups, weighted and projected.  Its state is ``S`` [heads, state, vdim] and the convolution's last inputs.

``TimeMixing``: a memory with a decay per key channel that the token itself sets.  Every projection reads its own
mix of the token's input and the one before it; ``o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t``, then
``S_t = diag(w_t) S_(t-1) + k_t v_t^T`` with ``w = exp(-exp(W_2 tanh(W_1 mix) + w_0))``; each head's ``o`` is divided by
its root mean square, weighted, gated by ``silu`` and projected.  Its state is ``S`` [heads, dim, dim] and the input
of the token before.

These two run the same walk (``ops.memory_walk``).  All of them read their sequences' slots and lengths from the step's device tensors (``csrc/recurrent.hip``), run a step's
tokens in order from the state the earlier steps left and write it back, so a prompt may be cut anywhere.
"""

from __future__ import annotations

from typing import Optional

import torch

from ..cache.manager import FixedState
from ..config.specs import PartSpec
from ..kernels import ops
from ..weights.tensors import TensorSpec
from .base import Part, build_part, register_part
from .latent_attention import positions_bound
from .linear import linear


class Retention(Part):
    graph_safe = True  # (a captured step's rotation tables reach the bound the step was captured for)

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, decay: tuple, eps: float,
                 position: PartSpec) -> None:
        if min(hidden_size, num_heads, head_dim, value_dim) < 1:
            raise ValueError("sizes must be positive")
        decay = tuple(float(d) for d in decay)
        if len(decay) != num_heads:
            raise ValueError(f"one decay per head: {len(decay)} for {num_heads} heads")
        if not eps > 0:
            raise ValueError("eps must be positive")
        ops.plan_retention(head_dim, value_dim)  # (refuses heads the kernel has no room for)
        self.hidden_size = hidden_size
        self.num_heads = num_heads
        self.head_dim = head_dim
        self.value_dim = value_dim
        self.decay_values = decay
        self.eps = float(eps)
        self.position = build_part("position", position)

    def cache_need(self) -> FixedState:
        return FixedState((self.num_heads, self.head_dim, self.value_dim))

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, d, v, hidden = self.num_heads, self.head_dim, self.value_dim, self.hidden_size
        return {
            prefix + "q": TensorSpec((h * d, hidden)),
            prefix + "k": TensorSpec((h * d, hidden)),
            prefix + "v": TensorSpec((h * v, hidden)),
            prefix + "g": TensorSpec((h * v, hidden)),
            prefix + "o": TensorSpec((hidden, h * v)),
        }

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        self.w_in = torch.cat([tensors[prefix + n] for n in ("q", "k", "v", "g")], dim=0).contiguous()
        self.w_o = tensors[prefix + "o"].contiguous()
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=device)

    def forward(self, x: torch.Tensor, batch, view, writes: bool = True) -> torch.Tensor:
        if not writes:
            raise ValueError("a recurrent mixer moves its state on whenever it runs")
        h, d, v = self.num_heads, self.head_dim, self.value_dim
        rot = self.position.rotary_dim if self.position.rotates else 0
        if rot and batch.max_context > self.position.max_position:
            raise ValueError(f"position {batch.max_context - 1} is beyond the rotary table of {self.position.max_position}")
        bound = positions_bound(batch)
        cos, sin = self.position.tables(x.device, bound) if rot else (None, None)
        proj = linear(x, self.w_in)
        out = ops.retention(proj, (0, h * d, 2 * h * d, 2 * h * d + h * v), cos, sin, rot, self.decay, view.state,
                            batch.seq_slot, batch.positions, batch.q_start_loc, batch.sequences, h, d, v, self.eps,
                            d ** -0.5, bound - 1)
        return linear(out, self.w_o)


class LightningAttention(Part):
    """Linear attention with a fixed decay per head and activated inputs: ``q = act(W_q x)``, ``k = act(W_k x)``
    (heads x dim), ``v = act(W_v x)`` (heads x vdim), per head ``S_t = decay_h S_(t-1) + k_t v_t^T`` and
    ``o_t = S_t^T q_t`` (no rotation, no other scale).  The heads' read-outs, concatenated, are divided by their
    common root mean square and multiplied by the weight ``norm`` (one number per column), then by ``sigmoid(W_g x)``,
    and projected.  The memory ``S`` [heads, dim, vdim] is float32, starts at zero and is carried in the request's
    state slot; activations after the projection, decays, the walk and the norm are float32.  ``activation``,
    ``norm_span`` (how many heads share a root mean square: all of them by default) and ``gate`` are parameters of
    the kernels that ``Retention`` runs too."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, value_dim: int, decay: tuple, eps: float,
                 activation: Optional[str] = "silu", gate: str = "sigmoid", norm_span: Optional[int] = None,
                 norm_weight: bool = True) -> None:
        for name, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("head_dim", head_dim),
                            ("value_dim", value_dim)):
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer, got {value!r}")
        decay = tuple(float(d) for d in decay)
        if len(decay) != num_heads:
            raise ValueError(f"one decay per head: {len(decay)} for {num_heads} heads")
        if not eps > 0:
            raise ValueError("eps must be positive")
        if activation not in ops.RETENTION_ACTIVATIONS or gate not in ops.RETENTION_GATES:
            raise ValueError(f"activation {activation!r} or gate {gate!r} is none the kernels have")
        ops.plan_retention(head_dim, value_dim)  # (refuses heads the kernel has no room for)
        self.hidden_size, self.num_heads, self.head_dim, self.value_dim = hidden_size, num_heads, head_dim, value_dim
        self.decay_values, self.eps = decay, float(eps)
        self.activation, self.gate = activation, gate
        self.norm_span = num_heads if norm_span is None else int(norm_span)
        if self.norm_span < 1 or num_heads % self.norm_span:
            raise ValueError(f"runs of {self.norm_span} heads do not divide {num_heads} heads")
        self.has_norm_weight = bool(norm_weight)

    def cache_need(self) -> FixedState:
        return FixedState((self.num_heads, self.head_dim, self.value_dim))

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, d, v, hidden = self.num_heads, self.head_dim, self.value_dim, self.hidden_size
        out = {
            prefix + "q": TensorSpec((h * d, hidden)),
            prefix + "k": TensorSpec((h * d, hidden)),
            prefix + "v": TensorSpec((h * v, hidden)),
            prefix + "g": TensorSpec((h * v, hidden)),
            prefix + "o": TensorSpec((hidden, h * v)),
        }
        if self.has_norm_weight:
            out[prefix + "norm"] = TensorSpec((h * v,), init="norm", keeps_float32=True)
        return out

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        self.w_in = torch.cat([tensors[prefix + n] for n in ("q", "k", "v", "g")], dim=0).contiguous()
        self.w_o = tensors[prefix + "o"].contiguous()
        self.decay = torch.tensor(self.decay_values, dtype=torch.float32, device=device)
        self.norm_weight = tensors[prefix + "norm"].float().contiguous() if self.has_norm_weight else None

    def warm_up(self, rows: int) -> None:
        blank = lambda width: torch.zeros((rows, width), dtype=self.w_in.dtype, device=self.w_in.device)
        linear(blank(self.hidden_size), self.w_in)
        linear(blank(self.num_heads * self.value_dim), self.w_o)

    def forward(self, x: torch.Tensor, batch, view, writes: bool = True) -> torch.Tensor:
        if not writes:
            raise ValueError("a recurrent mixer moves its state on whenever it runs")
        h, d, v = self.num_heads, self.head_dim, self.value_dim
        proj = linear(x, self.w_in)
        out = ops.retention(proj, (0, h * d, 2 * h * d, 2 * h * d + h * v), None, None, 0, self.decay, view.state,
                            batch.seq_slot, batch.positions, batch.q_start_loc, batch.sequences, h, d, v, self.eps,
                            1.0, 0, activation=self.activation, norm_span=self.norm_span,
                            norm_weight=self.norm_weight, gate=self.gate)
        return linear(out, self.w_o)


SCAN_SEGMENT_TOKENS = 64  # portions from which the recurrence's tokens are cut into stretches


class GatedLinearRecurrence(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, width: int, blocks: int, taps: int) -> None:
        if min(hidden_size, width, blocks, taps) < 1 or width % blocks:
            raise ValueError(f"{width} channels in {blocks} equal blocks, {taps} taps: sizes must be positive and divide")
        if taps > ops.MAX_CONV_TAPS:
            raise ValueError(f"the convolution takes up to {ops.MAX_CONV_TAPS} taps, not {taps}")
        self.hidden_size = hidden_size
        self.width = width
        self.blocks = blocks
        self.taps = taps

    def cache_need(self) -> tuple:
        return (FixedState((self.width,)), FixedState((max(self.taps - 1, 1), self.width)))

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        w, b, hidden = self.width, self.blocks, self.hidden_size
        per = w // b
        return {
            prefix + "y": TensorSpec((w, hidden)), prefix + "y.b": TensorSpec((w,)),
            prefix + "x": TensorSpec((w, hidden)), prefix + "x.b": TensorSpec((w,)),
            prefix + "conv": TensorSpec((w, self.taps)), prefix + "conv.b": TensorSpec((w,)),
            prefix + "ra": TensorSpec((b, per, per)), prefix + "ra.b": TensorSpec((b, per)),
            prefix + "ri": TensorSpec((b, per, per)), prefix + "ri.b": TensorSpec((b, per)),
            prefix + "lam": TensorSpec((w,)),
            prefix + "o": TensorSpec((hidden, w)),
        }

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        self.w_in = torch.cat([tensors[prefix + "y"], tensors[prefix + "x"]], dim=0).contiguous()
        self.b_in = torch.cat([tensors[prefix + "y.b"], tensors[prefix + "x.b"]], dim=0).contiguous()
        self.conv_w = tensors[prefix + "conv"].contiguous()
        self.conv_b = tensors[prefix + "conv.b"].contiguous()
        # per block the weights of its r gate over those of its i gate: one block-diagonal product makes both
        self.w_gates = torch.cat([tensors[prefix + "ra"], tensors[prefix + "ri"]], dim=1).contiguous()
        self.b_gates = torch.cat([tensors[prefix + "ra.b"], tensors[prefix + "ri.b"]], dim=1).contiguous()
        self.rate = (-8.0 * torch.nn.functional.softplus(tensors[prefix + "lam"].float())).contiguous()
        self.w_o = tensors[prefix + "o"].contiguous()

    def forward(self, x: torch.Tensor, batch, view, writes: bool = True) -> torch.Tensor:
        if not writes:
            raise ValueError("a recurrent mixer moves its state on whenever it runs")
        state, past = view[0].state, view[1].state
        w = self.width
        proj = linear(x, self.w_in, self.b_in)
        y_pre, x_in = proj[:, :w], proj[:, w:]
        u = ops.causal_conv(x_in, self.conv_w, self.conv_b, past, batch.seq_of_token, batch.seq_slot, batch.q_start_loc)
        gates = ops.block_linear(u, self.w_gates, self.b_gates, out_dtype=torch.float32)
        # long portions run as stretches side by side (the portion lengths are the host's, and a captured step's own)
        segments = 16 if batch.max_q_len >= SCAN_SEGMENT_TOKENS else 1
        out = ops.gated_recurrence(y_pre, x_in, u, gates, w // self.blocks, self.rate, state, past, batch.seq_slot,
                                   batch.q_start_loc, batch.sequences, self.taps, segments)
        return linear(out, self.w_o)


class StateSpace(Part):
    """``W_in x`` is laid out ``[z: inner | x: inner | B: groups * state | C: groups * state | dt: heads]`` with
    ``inner = heads * vdim``; head h uses the B and C of group ``h // (heads / groups)``.  Tensors: ``in``, ``conv``
    [inner + 2 groups state, taps] with ``conv.b`` (the last tap is the token's own input), ``dt_bias``, ``A_log``,
    ``D`` [heads], ``norm`` [inner], ``o``.  The gate ``silu(z)`` comes before the norm, which runs over
    ``norm_groups`` equal parts of the row.  Products and the convolution with its activation run in the engine's
    type; step sizes, decays, the memory, the read-out and the norm are float32."""

    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, value_dim: int, state: int, groups: int, taps: int,
                 norm_groups: int, eps: float) -> None:
        for name, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("value_dim", value_dim),
                            ("state", state), ("groups", groups), ("taps", taps), ("norm_groups", norm_groups)):
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer, got {value!r}")
        if num_heads % groups or (num_heads * value_dim) % norm_groups:
            raise ValueError(f"{num_heads} heads of {value_dim} in {groups} groups, normed in {norm_groups} parts: no equal parts")
        if taps > ops.MAX_CONV_TAPS or not eps > 0:
            raise ValueError(f"up to {ops.MAX_CONV_TAPS} taps and a positive eps, got {taps}, {eps}")
        ops.plan_memory_walk(state, value_dim, False)  # (refuses memories the walk has no room for)
        self.hidden_size, self.num_heads, self.value_dim, self.state = hidden_size, num_heads, value_dim, state
        self.groups, self.taps, self.norm_groups, self.eps = groups, taps, norm_groups, float(eps)
        self.inner = num_heads * value_dim
        self.conv_width = self.inner + 2 * groups * state

    def cache_need(self) -> tuple:
        return (FixedState((self.num_heads, self.state, self.value_dim)),
                FixedState((max(self.taps - 1, 1), self.conv_width)))

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        small = dict(keeps_float32=True)
        return {
            prefix + "in": TensorSpec((2 * self.inner + 2 * self.groups * self.state + self.num_heads, self.hidden_size)),
            prefix + "conv": TensorSpec((self.conv_width, self.taps)),
            prefix + "conv.b": TensorSpec((self.conv_width,)),
            prefix + "dt_bias": TensorSpec((self.num_heads,), **small),
            prefix + "A_log": TensorSpec((self.num_heads,), **small),
            prefix + "D": TensorSpec((self.num_heads,), init="norm", **small),
            prefix + "norm": TensorSpec((self.inner,), init="norm", **small),
            prefix + "o": TensorSpec((self.hidden_size, self.inner)),
        }

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        w_in = tensors[prefix + "in"]
        if w_in.shape[0] % 8:  # (the rows of the product's result stay 16-byte aligned)
            w_in = torch.cat([w_in, w_in.new_zeros((8 - w_in.shape[0] % 8, self.hidden_size))], dim=0)
        self.w_in = w_in.contiguous()
        self.conv_w = tensors[prefix + "conv"].contiguous()
        self.conv_b = tensors[prefix + "conv.b"].contiguous()
        self.dt_bias = tensors[prefix + "dt_bias"].float().contiguous()
        self.a_log = tensors[prefix + "A_log"].float().contiguous()
        self.skip = tensors[prefix + "D"].float().contiguous()
        self.norm_weight = tensors[prefix + "norm"].float().contiguous()
        self.w_o = tensors[prefix + "o"].contiguous()

    def warm_up(self, rows: int) -> None:
        blank = lambda width: torch.zeros((rows, width), dtype=self.w_in.dtype, device=self.w_in.device)
        linear(blank(self.hidden_size), self.w_in)
        linear(blank(self.inner), self.w_o)

    def forward(self, x: torch.Tensor, batch, view, writes: bool = True) -> torch.Tensor:
        if not writes:
            raise ValueError("a recurrent mixer moves its state on whenever it runs")
        memory, past = view[0].state, view[1].state
        inner, bc = self.inner, self.groups * self.state
        proj = linear(x, self.w_in)
        z, taken, raw_dt = proj[:, :inner], proj[:, inner: inner + self.conv_width], proj[:, 2 * inner + 2 * bc:2 * inner + 2 * bc + self.num_heads]
        mixed = ops.causal_conv(taken, self.conv_w, self.conv_b, past, batch.seq_of_token, batch.seq_slot,
                                batch.q_start_loc, activation="silu", out_dtype=torch.float32)
        ops.conv_keep(taken, past, batch.seq_slot, batch.q_start_loc, batch.sequences, self.taps)
        steps, decay, log_decay = ops.space_steps(raw_dt, self.dt_bias, self.a_log)
        # (prompts' portions walk in blocks on the matrix cores, single tokens and short portions token by token:
        # which of the two follows from the step's shape, which a captured step repeats)
        y = ops.memory_walk(decay, mixed[:, inner: inner + bc], mixed[:, inner + bc:], mixed[:, :inner], memory,
                            batch.seq_slot, batch.q_start_loc, batch.sequences, self.num_heads, self.state,
                            self.value_dim, heads_per_group=self.num_heads // self.groups, value_scale=steps,
                            skip=self.skip, log_decay=log_decay)
        out = ops.gated_group_norm(y, z, self.norm_weight, self.norm_groups, self.eps, x.dtype, gate_first=True)
        return linear(out, self.w_o)


class TimeMixing(Part):
    """Tensors: ``mu.r``, ``mu.k``, ``mu.v``, ``mu.g``, ``mu.w`` [hidden] (how much of the token before each mix takes),
    ``r``, ``k``, ``v``, ``g`` [heads * dim, hidden], ``w1`` [rank, hidden] and ``w2`` [heads * dim, rank] (the rank is
    the checkpoint's), ``w0`` [heads * dim], ``u`` [heads, dim], ``norm`` [heads * dim], ``o``.  Mixes and products run
    in the engine's type; the products' results that enter the memory, decays, the memory, the read-out and its norm
    are float32."""

    graph_safe = True
    MIXES = ("r", "k", "v", "g", "w")

    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, eps: float, decay_rank: Optional[int] = None) -> None:
        for name, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("head_dim", head_dim)):
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer, got {value!r}")
        if not eps > 0:
            raise ValueError("eps must be positive")
        ops.plan_memory_walk(head_dim, head_dim, True)  # (refuses memories the walk has no room for)
        self.hidden_size, self.num_heads, self.head_dim, self.eps = hidden_size, num_heads, head_dim, float(eps)
        self.decay_rank = decay_rank  # None: whatever the checkpoint holds
        self.channels = num_heads * head_dim

    def cache_need(self) -> tuple:
        return (FixedState((self.num_heads, self.head_dim, self.head_dim)), FixedState((self.hidden_size,)))

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        c, hidden = self.channels, self.hidden_size
        small = dict(keeps_float32=True)
        drawn_rank = self.decay_rank or max(8, min(64, hidden // 16 // 8 * 8 or 8))
        out = {prefix + "mu." + name: TensorSpec((hidden,), **small) for name in self.MIXES}
        out.update({prefix + name: TensorSpec((c, hidden)) for name in ("r", "k", "v", "g")})
        out[prefix + "w1"] = TensorSpec((self.decay_rank, hidden), drawn=(drawn_rank, hidden))
        out[prefix + "w2"] = TensorSpec((c, self.decay_rank), drawn=(c, drawn_rank))
        out[prefix + "w0"] = TensorSpec((c,), **small)
        out[prefix + "u"] = TensorSpec((self.num_heads, self.head_dim), **small)
        out[prefix + "norm"] = TensorSpec((c,), init="norm", **small)
        out[prefix + "o"] = TensorSpec((hidden, c))
        return out

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        self.mu = torch.stack([tensors[prefix + "mu." + name].float() for name in self.MIXES]).contiguous()
        self.w_r, self.w_k, self.w_v, self.w_g = (tensors[prefix + name].contiguous() for name in ("r", "k", "v", "g"))
        self.w_1 = tensors[prefix + "w1"].contiguous()
        w_2 = tensors[prefix + "w2"]
        if self.w_1.shape[0] != w_2.shape[1]:
            raise ValueError(f"{prefix}w1 {tuple(self.w_1.shape)} and {prefix}w2 {tuple(w_2.shape)} disagree on the rank")
        self.w_2t = w_2.t().contiguous()  # [rank, channels]: the decay kernel's threads read neighbouring channels
        self.w_0 = tensors[prefix + "w0"].float().contiguous()
        self.bonus = tensors[prefix + "u"].float().contiguous()
        self.norm_weight = tensors[prefix + "norm"].float().contiguous()
        self.w_o = tensors[prefix + "o"].contiguous()

    def warm_up(self, rows: int) -> None:
        blank = lambda width: torch.zeros((rows, width), dtype=self.w_o.dtype, device=self.w_o.device)
        for weight in (self.w_r, self.w_k, self.w_v, self.w_g):
            linear(blank(self.hidden_size), weight)
        linear(blank(self.channels), self.w_o)

    def forward(self, x: torch.Tensor, batch, view, writes: bool = True) -> torch.Tensor:
        if not writes:
            raise ValueError("a recurrent mixer moves its state on whenever it runs")
        memory, before = view[0].state, view[1].state
        mixes = ops.shift_mix(x, before, self.mu, batch.seq_of_token, batch.seq_slot, batch.q_start_loc)
        f32 = torch.float32
        r = linear(mixes[0], self.w_r, out_dtype=f32)
        k = linear(mixes[1], self.w_k, out_dtype=f32)
        v = linear(mixes[2], self.w_v, out_dtype=f32)
        gate = linear(mixes[3], self.w_g)
        low = linear(mixes[4], self.w_1, out_dtype=f32)
        decay = ops.time_decay(low, self.w_2t, self.w_0, x, before, batch.seq_of_token, batch.seq_slot, batch.q_start_loc)
        y = ops.memory_walk(decay, k, r, v, memory, batch.seq_slot, batch.q_start_loc, batch.sequences, self.num_heads,
                            self.head_dim, self.head_dim, bonus=self.bonus, read_first=True)
        out = ops.gated_group_norm(y, gate, self.norm_weight, self.num_heads, self.eps, x.dtype, gate_first=False)
        return linear(out, self.w_o)


register_part("mixer", "retention", Retention)
register_part("mixer", "state_space", StateSpace)
register_part("mixer", "time_mixing", TimeMixing)
register_part("mixer", "lightning_attention", LightningAttention)
register_part("mixer", "gated_linear_recurrence", GatedLinearRecurrence)
