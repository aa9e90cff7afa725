"""Grouped-query softmax attention over a window of the paged cache, without rotation, whose scores are shaped by
the position in other ways.  Every step is a parameter of the part and may be left out:

* a per-head RMS norm of queries and keys (``qk_norm``: ``"weight"`` with one weight vector for all query heads
  and one for all key heads, ``"unit"`` without weights, ``None``), or (``"whole"``) one RMS norm over all query
  heads of a token together and one over all its key heads, with a weight for every number of the projection;
* a factor on the queries that grows with the logarithm of the position (``q_temperature = (coef, every)``:
  ``1 + coef * ln(floor((p + 1) / every) + 1)``);
* ``score = q . k * scale``, then a smooth cap (``softcap``: ``c * tanh(score / c)``), then a bias on the distance
  itself (``slope_base = b``: head h of H loses ``2^(-b (h + 1) / H) * (i - j)``);
* a window (``window``: the token itself and the ``window - 1`` before it; with ``keep_first`` the first that many
  tokens of the sequence stay visible from behind the window too, at their own positions), or chunks (``chunk``: the token sees the
  keys of its own chunk of that many positions up to itself; chunks are counted from position 0 of the sequence);
* biases on the projections of queries, keys and values (``qkv_bias``);
* a rotation of the first numbers of every query and key head by the position (``position``: a position part such
  as ``rotary_pairs``, applied after the heads' norm);
* a sink (``sink``: one learned number per head whose exponential stands in the softmax's denominator, and
  nowhere else);
* a gate on every head's output (``head_gate``: ``sigmoid(W_g x)_h``, read from the layer's own input);
* key and value heads of different sizes;
* no keys and values of its own (``own_kv=False``): the layer has no tensors for them and reads the cache unit that
  another layer of the same head sizes writes, with its own queries, mask and everything else.

One product makes queries, keys, values and gate logits; one kernel norms and scales the heads, lays the queries
out and writes the cache (``ops.heads_prepare``); the attention kernel shapes the scores, and applies sink and
gate in its epilogue: bfloat16 with head sizes up to 128 on the matrix cores (``ops.scored_attention_mfma``, the
heads zero-padded to 64 or 128 numbers: no score and no output changes), anything else, and float32, in the
generic form.  Norm statistics, the logarithm, scores, softmax, value sums and the gate are float32.
"""

from __future__ import annotations

import warnings
from typing import Optional

import torch

from ..cache.manager import PagedKV
from ..config.specs import PartSpec
from ..kernels import ops
from ..weights.tensors import TensorSpec
from .base import Part, build_part, register_part
from .latent_attention import positions_bound
from .linear import linear

_SAID_GENERIC: set = set()
PROMPT_ROW_TILES = 2  # tiles of 16 (token, head) rows that a workgroup of the matrix-core form takes of a prompt's portion


def _round8(n: int) -> int:
    return -(-n // 8) * 8


class ScoredAttention(Part):
    graph_safe = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, value_dim: int,
                 scale: float, eps: float, window: Optional[int] = None, qk_norm: Optional[str] = None,
                 q_temperature: Optional[tuple] = None, softcap: Optional[float] = None,
                 slope_base: Optional[float] = None, sink: bool = False, head_gate: bool = False,
                 chunk: Optional[int] = None, qkv_bias: bool = False, position: Optional[PartSpec] = None,
                 keep_first: int = 0, own_kv: bool = True) -> None:
        for name, value in (("hidden_size", hidden_size), ("num_heads", num_heads), ("num_kv_heads", num_kv_heads),
                            ("head_dim", head_dim), ("value_dim", value_dim)):
            if isinstance(value, bool) or not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer, got {value!r}")
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads are no multiple of {num_kv_heads} key heads")
        if max(head_dim, value_dim) > 256:
            raise ValueError(f"heads of up to 256 numbers, got {head_dim} and {value_dim}")
        if window is not None and window < 1:
            raise ValueError("window must be positive")
        if chunk is not None and (isinstance(chunk, bool) or not isinstance(chunk, int) or chunk < 1 or window is not None):
            raise ValueError(f"chunks hold a positive number of tokens and stand in a window's place, got {chunk!r}")
        if isinstance(keep_first, bool) or not isinstance(keep_first, int) or keep_first < 0:
            raise ValueError(f"keep_first is a count of tokens, got {keep_first!r}")
        if window is None:
            keep_first = 0  # (every key is seen anyway)
        if qk_norm not in ops.NORM_MODES:
            raise ValueError(f"qk_norm must be one of {list(ops.NORM_MODES)}, got {qk_norm!r}")
        if not eps > 0:
            raise ValueError("eps must be positive")
        if softcap is not None and not softcap > 0:
            raise ValueError("softcap must be positive")
        if q_temperature is not None:
            coef, every = q_temperature
            if isinstance(every, bool) or int(every) != every or every < 1:
                raise ValueError(f"the temperature's period must be a positive integer, got {every!r}")
            q_temperature = (float(coef), int(every))
        self.hidden_size, self.num_heads, self.num_kv_heads = hidden_size, num_heads, num_kv_heads
        self.head_dim, self.value_dim = head_dim, value_dim
        self.scale, self.eps, self.window = float(scale), float(eps), window
        self.qk_norm, self.q_temperature, self.softcap = qk_norm, q_temperature, softcap
        self.slope_base, self.sink, self.head_gate = slope_base, bool(sink), bool(head_gate)
        self.chunk, self.qkv_bias = chunk, bool(qkv_bias)
        self.keep_first, self.own_kv = keep_first, bool(own_kv)
        self.position = build_part("position", position) if position is not None else None
        if self.position is not None and self.position.rotates and self.position.rotary_dim > head_dim:
            raise ValueError(f"{self.position.rotary_dim} turning numbers in heads of {head_dim}")
        # the head sizes the kernels and the cache see: those of the matrix-core form where it has them
        sizes = tuple(next((s for s in (64, 128) if s >= n), None) for n in (head_dim, value_dim))
        self.mfma_dims = sizes if sizes in ops.SCORED_MFMA_DIMS else None
        self.kernel_dim, self.kernel_vdim = self.mfma_dims or (_round8(head_dim), _round8(value_dim))

    def cache_need(self) -> PagedKV:
        # (a chunk's keys all lie inside a window of the chunk's length: pages behind it go back to the pool)
        return PagedKV(self.num_kv_heads, self.kernel_dim, self.window if self.chunk is None else self.chunk,
                       value_dim=self.kernel_vdim if self.kernel_vdim != self.kernel_dim else None,
                       keep_first=self.keep_first)

    def expected_tensors(self, prefix: str) -> dict[str, TensorSpec]:
        h, g, d, v, width = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim, self.hidden_size
        out = {prefix + "q": TensorSpec((h * d, width))}
        if self.own_kv:
            out[prefix + "k"] = TensorSpec((g * d, width))
            out[prefix + "v"] = TensorSpec((g * v, width))
        out[prefix + "o"] = TensorSpec((width, h * v))
        if self.qkv_bias:
            out[prefix + "q.b"] = TensorSpec((h * d,))
            if self.own_kv:
                out[prefix + "k.b"] = TensorSpec((g * d,))
                out[prefix + "v.b"] = TensorSpec((g * v,))
        if self.qk_norm in ("weight", "whole"):
            whole = self.qk_norm == "whole"
            out[prefix + "q.norm"] = TensorSpec((h * d if whole else d,), init="norm", keeps_float32=True)
            if self.own_kv:
                out[prefix + "k.norm"] = TensorSpec((g * d if whole else d,), init="norm", keeps_float32=True)
        if self.sink:
            out[prefix + "sink"] = TensorSpec((h,), keeps_float32=True)
        if self.head_gate:
            out[prefix + "g"] = TensorSpec((h, width))
        return out

    def bind(self, tensors, prefix, dtype, device) -> None:
        super().bind(tensors, prefix, dtype, device)
        h, g, d, v = self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim
        blocks = [tensors[prefix + "q"]]
        if self.own_kv:
            blocks += [tensors[prefix + "k"], tensors[prefix + "v"]]
        self.offsets = (0, h * d, h * d + g * d) if self.own_kv else (0, 0, 0)
        self.gate_offset = None
        if self.head_gate:
            # gate logits ride in the same product, on columns that start at a multiple of 8 (and the row is
            # padded to one), so that the rows of the result stay 16-byte aligned
            pad = lambda rows: blocks[0].new_zeros((rows, self.hidden_size))
            used = h * d + (g * d + g * v if self.own_kv else 0)
            if used % 8:
                blocks.append(pad(8 - used % 8))
            self.gate_offset = _round8(used)
            blocks.append(tensors[prefix + "g"])
            if h % 8:
                blocks.append(pad(8 - h % 8))
        self.w_in = torch.cat(blocks, dim=0).contiguous()
        self.b_in = None
        if self.qkv_bias:
            names = ("q.b", "k.b", "v.b") if self.own_kv else ("q.b",)
            bias = torch.cat([tensors[prefix + name] for name in names], dim=0)
            self.b_in = torch.cat([bias, bias.new_zeros(self.w_in.shape[0] - bias.shape[0])]).contiguous()
        self.q_weight = self.k_weight = None
        if self.qk_norm in ("weight", "whole"):
            self.q_weight = tensors[prefix + "q.norm"].float().contiguous()
            if self.own_kv:
                self.k_weight = tensors[prefix + "k.norm"].float().contiguous()
        self.sinks = tensors[prefix + "sink"].float().contiguous() if self.sink else None
        self.slopes = None
        if self.slope_base is not None:
            self.slopes = torch.tensor([2.0 ** (-self.slope_base * (i + 1) / h) for i in range(h)],
                                       dtype=torch.float32, device=device)
        w_o = tensors[prefix + "o"]
        if self.kernel_vdim != v:  # the attention's rows hold padded heads: zero columns under the padding
            wide = w_o.new_zeros((self.hidden_size, h, self.kernel_vdim))
            wide[:, :, :v] = w_o.reshape(self.hidden_size, h, v)
            w_o = wide.reshape(self.hidden_size, h * self.kernel_vdim)
        self.w_o = w_o.contiguous()

    def warm_up(self, rows: int) -> None:
        blank = lambda width: torch.zeros((rows, width), dtype=self.w_in.dtype, device=self.w_in.device)
        linear(blank(self.hidden_size), self.w_in, self.b_in)
        linear(blank(self.num_heads * self.kernel_vdim), self.w_o)

    def forward(self, x: torch.Tensor, batch, view, writes: bool = True) -> torch.Tensor:
        if writes and not self.own_kv:
            raise ValueError("a layer without keys and values of its own reads the cache unit that another layer writes")
        proj = linear(x, self.w_in, self.b_in)
        rotary = None
        if self.position is not None and self.position.rotates:
            if batch.max_context > self.position.max_position:
                raise ValueError(f"position {batch.max_context - 1} is beyond the rotary table of {self.position.max_position}")
            cos, sin = self.position.tables(x.device, positions_bound(batch))
            rotary = (cos, sin, self.position.rotary_dim, getattr(self.position, "pairing", "halves") == "neighbours")
        q = ops.heads_prepare(proj, self.offsets, self.num_heads, self.num_kv_heads, self.head_dim, self.value_dim,
                              self.kernel_dim, self.kernel_vdim, self.qk_norm, self.q_weight, self.k_weight, self.eps,
                              self.q_temperature, batch.positions, batch.seq_of_token, batch.seq_slot,
                              view.block_table, view.k_pool, view.v_pool, batch.tokens, write_kv=writes, rotary=rotary)
        gate = proj[:, self.gate_offset:] if self.head_gate else None
        context = self.attend(q, gate, batch, view)
        return linear(context, self.w_o)

    def attend(self, q: torch.Tensor, gate, batch, view) -> torch.Tensor:
        shape = dict(window=self.window, scale=self.scale, softcap=self.softcap, slopes=self.slopes,
                     sinks=self.sinks, gate=gate, chunk=self.chunk, keep_first=self.keep_first)
        h, g = self.num_heads, self.num_kv_heads
        group = h // g
        page_size = view.page_size
        if q.dtype == torch.bfloat16 and self.mfma_dims and group <= 64 and page_size >= 4 and not page_size & (page_size - 1):
            # rows of a tile: a token's heads of one key head, and as many tokens as fill the tile
            least = 1 if group <= 16 else 2 if group <= 32 else 4
            # the most keys a token sees in this step (a captured step: in any of its replays)
            bound = batch.static_plan.max_keys if batch.static_plan is not None else batch.max_context
            reach = self.window if self.chunk is None else self.chunk  # the most keys a token sees, if bounded
            if reach is not None and self.keep_first:
                reach += -(-self.keep_first // 32) * 32 + 32  # (the kept first keys are walked in whole blocks of 32)
            bound = bound if reach is None else min(bound, reach)

            def shares(tiles: int, span: int) -> dict:
                """Few tiles over many keys: the keys in shares of at least 128, about two workgroups a compute unit."""
                reach = bound + span + 32                        # a tile's range starts at a multiple of 32
                wanted = min(2 * ops.compute_units() // max(tiles * g, 1), reach // 128)
                if wanted < 2:
                    return {}
                per = -(-(-(-reach // wanted)) // 128) * 128
                return dict(n_splits=-(-reach // per), keys_per_split=per)

            if batch.static_plan is not None and batch.static_plan.decode_rows in (None, batch.sequences):
                # a captured step of single tokens: tile i is sequence i, nothing comes from the host
                return ops.scored_attention_mfma(q, view.k_pool, view.v_pool, view.block_table, None, None,
                                                 batch.sequences, batch.seq_slot, batch.seq_start, batch.seq_q_len,
                                                 batch.q_start_loc, batch.tokens, h, g, self.kernel_dim,
                                                 self.kernel_vdim, 1, least, **shape, **shares(batch.sequences, 1))
            row_tiles = max(least, PROMPT_ROW_TILES if batch.max_q_len * group > 16 else 1)
            while row_tiles > least and -(-batch.tokens * group // (16 * row_tiles)) * g < ops.compute_units():
                row_tiles //= 2  # (fewer rows a tile where the tiles would not fill the compute units)
            per_tile = (16 * row_tiles) // group
            tile_seq, tile_q0, n_tiles = batch.tiles(per_tile, decode=None)
            return ops.scored_attention_mfma(q, view.k_pool, view.v_pool, view.block_table, tile_seq, tile_q0, n_tiles,
                                             batch.seq_slot, batch.seq_start, batch.seq_q_len, batch.q_start_loc,
                                             batch.tokens, h, g, self.kernel_dim, self.kernel_vdim, per_tile,
                                             row_tiles, **shape, **shares(n_tiles, per_tile))
        if q.dtype == torch.bfloat16 and (self.kernel_dim, self.kernel_vdim, group, page_size) not in _SAID_GENERIC:
            _SAID_GENERIC.add((self.kernel_dim, self.kernel_vdim, group, page_size))
            warnings.warn(f"bfloat16 attention with heads of {self.head_dim} and {self.value_dim} numbers, {group} query "
                          f"heads per key head and pages of {page_size} takes the generic kernel (the matrix-core form "
                          f"takes heads of up to 128 numbers, up to 64 heads per key head and pages of a power of two >= 4)",
                          RuntimeWarning, stacklevel=2)
        return ops.scored_attention_generic(q, view.k_pool, view.v_pool, view.block_table, batch.positions,
                                            batch.seq_of_token, batch.seq_slot, batch.tokens, h, g, self.kernel_dim,
                                            self.kernel_vdim, **shape)


register_part("mixer", "scored_attention", ScoredAttention)
