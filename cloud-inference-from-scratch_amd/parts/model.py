"""The decoder, generic over its parts: embedding, the layers in the order the
:class:`~cie_amd.config.specs.ModelSpec` lists, final norm, row selection and
the float32 output head (reference: ``Qwen2CausalLM.forward``,
src/cloud_engine/model.py:194-228).
"""

from __future__ import annotations

from typing import Any

import torch

from ..config.specs import ModelSpec
from ..kernels import ops
from ..weights.loader import torch_dtype
from ..weights.tensors import TensorSpec
from .base import BLOCKS, build_part
from .block import normalise
from .linear import StreamRows, linear


def _blocks(spec: ModelSpec) -> list[Any]:
    blocks = []
    for layer in spec.layers:
        if layer.block not in BLOCKS:
            raise KeyError(f"unknown block kind {layer.block!r}; known: {sorted(BLOCKS)}")
        blocks.append(BLOCKS[layer.block](layer))
    return blocks


def _expected(spec: ModelSpec, blocks: list[Any], final_norm: Any) -> dict[str, TensorSpec]:
    out: dict[str, TensorSpec] = {spec.embedding_name: TensorSpec((spec.vocab_size, spec.hidden_size))}
    out.update(final_norm.expected_tensors(spec.final_norm_name + "."))
    if not spec.tie_word_embeddings:
        out[spec.head_name] = TensorSpec((spec.vocab_size, spec.hidden_size))
    for index, block in enumerate(blocks):
        out.update(block.expected_tensors(spec.layer_prefix.format(index=index)))
    return out


def expected_tensors(spec: ModelSpec) -> dict[str, TensorSpec]:
    """Name -> what is expected of every checkpoint tensor of ``spec``, in a fixed order."""
    return _expected(spec, _blocks(spec), build_part("norm", spec.final_norm))


class DecoderModel:
    def __init__(self, spec: ModelSpec) -> None:
        self.spec = spec
        self.blocks = _blocks(spec)
        self.final_norm = build_part("norm", spec.final_norm)
        self.embedding: torch.Tensor | None = None
        self.head: torch.Tensor | None = None
        # blocks that read what every earlier layer left (``keeps_history``) are handed a float32 tensor
        # [calls + 1, tokens, hidden] of the step: row 0 the embedding's rows, row i + 1 what call i left
        self.keeps_history = any(getattr(block, "keeps_history", False) for block in self.blocks)
        # a run order that lets the embedding's rows join the stream again keeps a copy of them for the step
        self.keeps_embedding = any(call.adds_embedding for call in spec.order)
        if self.keeps_embedding and self.keeps_history:
            raise ValueError("a run order adds the embedding's rows again to layers that average over the depth: not built")
        calls = [self.blocks[call.layer] for call in spec.order]
        if len(set(map(id, calls))) == len(calls):  # (a layer that runs twice has no single successor)
            for block, follower in zip(calls, calls[1:] + [None]):
                link = getattr(block, "link_next", None)
                if link is not None:
                    link(follower)

    def expected_tensors(self) -> dict[str, TensorSpec]:
        return _expected(self.spec, self.blocks, self.final_norm)

    def cache_needs(self) -> list[Any]:
        """The need of every cache unit: that of the layer which writes it."""
        needs: list[Any] = [None] * self.spec.cache_units
        seen: set[int] = set()
        for call in self.spec.order:
            need = self.blocks[call.layer].cache_need()
            if call.writes and call.cache not in seen:
                needs[call.cache] = need
                seen.add(call.cache)
        for call in self.spec.order:
            if call.writes:
                continue
            need = self.blocks[call.layer].cache_need()
            if need == needs[call.cache]:
                continue
            # a reader with a mask of its own: the unit keeps what either of them still sees
            join = getattr(needs[call.cache], "joined", None)
            try:
                if join is None or type(need) is not type(needs[call.cache]):
                    raise ValueError("not a paged cache on both sides")
                needs[call.cache] = join(need)
            except ValueError as error:
                raise ValueError(
                    f"layer {call.layer} reads cache unit {call.cache} whose shape it does not share ({error})"
                ) from error
        return needs

    @property
    def graph_safe(self) -> bool:
        """Whether a decode step of this model may be captured in a graph."""
        return all(getattr(block, "graph_safe", False) for block in self.blocks) and self.final_norm.graph_safe

    def load(self, source: Any, dtype: str, device: str | torch.device) -> "DecoderModel":
        """Bind weights from a source (``SafetensorsSource`` or ``RandomSource``)."""
        device = torch.device(device)
        self.dtype = torch_dtype(dtype)
        self.device = device
        expected = self.expected_tensors()
        tied_optional = (
            {self.spec.head_name: self.spec.embedding_name, "model." + self.spec.head_name: self.spec.embedding_name}
            if self.spec.tie_word_embeddings else {}
        )
        # (a source that can hand out tensors one by one is asked to: the model then needs its own size of
        # device memory and one layer's tensors, not twice its size)
        take = getattr(source, "open", None) or source.load
        tensors = take(expected, dtype, device, tied_optional=tied_optional)
        self.embedding = tensors[self.spec.embedding_name].contiguous()
        self.head = self.embedding if self.spec.tie_word_embeddings else tensors[self.spec.head_name].contiguous()
        self.final_norm.bind(tensors, self.spec.final_norm_name + ".", self.dtype, device)
        for index, block in enumerate(self.blocks):
            block.bind(tensors, self.spec.layer_prefix.format(index=index), self.dtype, device)
        return self

    def warm_up(self, row_counts) -> None:
        """Run every part's products once on blank rows of the given counts, so that what a product
        does at the first call of a shape (the library's products time their candidates) happens
        before the first request.  Layers of one specification share their shapes: one of each runs."""
        if self.dtype != torch.bfloat16 or self.device.type != "cuda":
            return
        seen = set()
        for block in self.blocks:
            key = repr(block.spec)
            if key in seen:
                continue
            seen.add(key)
            warm = getattr(block, "warm_up", None)
            if warm is not None:
                for rows in row_counts:
                    warm(rows)

    def forward(self, batch, cache) -> torch.Tensor:
        """Run the step's tokens; float32 logits ``[len(logit_rows), vocab]``."""
        history = None
        if self.keeps_history:
            history = torch.empty((len(self.spec.order) + 1, batch.token_ids.shape[0], self.embedding.shape[1]),
                                  dtype=torch.float32, device=self.embedding.device)
        first = self.blocks[self.spec.order[0].layer] if self.spec.order else None
        rows = None
        if getattr(first, "reads_stream", False) and self.embedding.dtype != torch.float32:
            # a first layer whose products read the stream itself: the embedding kernel also leaves it in their type
            rows = torch.empty((batch.token_ids.shape[0], self.embedding.shape[1]), dtype=self.embedding.dtype,
                               device=self.embedding.device)
        residual = ops.embed(self.embedding, batch.token_ids, feed=batch.token_feed, pool=batch.token_pool,
                             out=history[0] if history is not None else None, scale=self.spec.embedding_scale,
                             rows=rows)
        pending = StreamRows(rows) if rows is not None else None
        embedded = residual.clone() if self.keeps_embedding else None
        for call in self.spec.order:
            block = self.blocks[call.layer]
            extra = {"history": history} if getattr(block, "keeps_history", False) else {}
            if call.adds_embedding:
                extra["plus"] = embedded
            residual, pending = block.forward(residual, pending, batch, cache.view(call.cache), call.writes, **extra)
        if batch.logit_rows.shape[0] == 0:  # a step of prompt portions that end before their prompts do
            return torch.empty((0, self.head.shape[0]), dtype=torch.float32, device=residual.device)
        selected = normalise(self.final_norm, residual, pending, self.dtype, rows=batch.logit_rows)
        logits = linear(selected, self.head, None, out_dtype=torch.float32)
        if self.spec.logit_softcap is not None:
            ops.soft_cap_(logits, self.spec.logit_softcap)
        return logits
