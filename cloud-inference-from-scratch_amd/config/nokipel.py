"""Configuration of the Nokipel decoder, read from its ``config.json``.

The file lists the layers one by one: ``layers[i] = {"type", "mixer", "mlp"}``.  ``type`` is ``attention`` (grouped-query
softmax attention with biases on queries, keys and values, a rotation of the first ``rot.dims`` numbers of every query
and key head in pairs of neighbours, and chunks of ``mask.size`` positions outside of which a token sees nothing) or
``lightning`` (linear attention with one ``decay`` per head, activated queries, keys and values, one norm over all
heads' read-outs and a sigmoid gate).  ``mlp`` is ``{"kind": "dense", "ff", "limit"}`` (a gated unit with bounded
inputs), ``{"kind": "moe", "router": {experts, top, identity, scale, groups: {count, keep}}, "expert": {ff},
"shared": {ff}}`` (softmax scores over ``experts + identity`` router outputs, a correction for the choice, groups,
weights normalised over the chosen and scaled; the last ``identity`` outputs hand the token's row on; a shared expert
behind a sigmoid gate) or ``null``.  ``loop = {start, stop, times}`` lets layers ``start .. stop - 1`` run ``times``
times over with the same weights, each pass on cache units of its own, and the embedding's rows join the stream again
in front of every pass but the first.  Beside these: ``vocab``, ``width``, ``norm.eps``, ``norm.groups`` (every norm
of the stream takes its statistics over that many equal parts of the row), ``embedding.scale``.  Every size and every
constant that the file gives is read from it; what the design itself fixes (the dense unit's 1.702 and + 1, the
experts' plain silu, which mixer has which steps) is handed to the parts as parameters here.

Layers are ``pre_norm`` blocks; tensors are named ``embed``, ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.norm2``,
``l<i>.mlp.*``, ``final.norm`` and ``head``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any

from .givizen import _need, _positive, _positive_int
from .specs import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec

MIXER_TYPES = ("attention", "lightning")
DENSE_ALPHA = 1.702    # the dense unit: g * sigmoid(1.702 g) * (u + 1)
DENSE_OFFSET = 1.0
EXPERT_ALPHA = 1.0     # an expert's unit: silu(g) * u
EXPERT_OFFSET = 0.0


def _count(table: dict, key: str, where: str, default: int | None = None) -> int:
    value = table.get(key, default)
    if isinstance(value, bool) or not isinstance(value, int) or value < 0:
        raise ConfigError(f"{where}: {key} must be a count, got {value!r}")
    return value


@dataclass(frozen=True)
class NokipelConfig:
    raw: dict = field(compare=False)

    architecture = "Nokipel"

    @classmethod
    def from_hf_config(cls, raw: dict[str, Any]) -> "NokipelConfig":
        _need(raw, ("layers", "norm", "vocab", "width"), "config")
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config: layers must be a list with at least one layer")
        _need(raw["norm"], ("eps",), "config.norm")
        _positive(raw["norm"], "eps", "config.norm")
        for key in ("vocab", "width"):
            _positive_int(raw, key, "config")
        if raw.get("embedding") is not None:
            _need(raw["embedding"], ("scale",), "config.embedding")
        config = cls(copy.deepcopy(raw))
        spec = config.model_spec()
        from ..parts.model import expected_tensors  # (the parts are built once here: what one refuses is a ConfigError)

        try:
            expected_tensors(spec)
        except (KeyError, TypeError, ValueError) as error:
            if isinstance(error, ConfigError):
                raise
            raise ConfigError(f"config: {error}") from error
        return config

    def to_hf_config(self) -> dict[str, Any]:
        out = copy.deepcopy(self.raw)
        out["architecture"] = self.architecture
        return out

    @property
    def hidden_size(self) -> int:
        return int(self.raw["width"])

    @property
    def vocab_size(self) -> int:
        return int(self.raw["vocab"])

    @property
    def eps(self) -> float:
        return float(self.raw["norm"]["eps"])

    @property
    def norm_groups(self) -> int:
        groups = self.raw["norm"].get("groups", 1)
        if isinstance(groups, bool) or not isinstance(groups, int) or groups < 1 or self.hidden_size % groups:
            raise ConfigError(f"config.norm: groups must be a positive integer that divides the width, got {groups!r}")
        return groups

    def loop(self) -> tuple[int, int, int]:
        """(start, stop, times): layers start .. stop - 1 run ``times`` times in a row.  No loop: (0, 0, 1)."""
        loop = self.raw.get("loop")
        if loop is None:
            return 0, 0, 1
        _need(loop, ("start", "stop", "times"), "config.loop")
        start, stop = _count(loop, "start", "config.loop"), _count(loop, "stop", "config.loop")
        times = _positive_int(loop, "times", "config.loop")
        if not start <= stop <= len(self.raw["layers"]):
            raise ConfigError(f"config.loop: layers {start} .. {stop} do not lie among {len(self.raw['layers'])} layers")
        return start, stop, times

    def _mixer(self, kind: str, sizes: Any, where: str) -> PartSpec:
        if kind not in MIXER_TYPES:
            raise ConfigError(f"{where}: unknown layer type {kind!r}; known: {MIXER_TYPES}")
        if kind == "lightning":
            _need(sizes, ("heads", "dim", "vdim", "decay"), where)
            decay = sizes["decay"]
            if not isinstance(decay, list) or not all(isinstance(d, (int, float)) and not isinstance(d, bool) for d in decay):
                raise ConfigError(f"{where}: decay must be a list of numbers, one per head")
            return PartSpec.of(
                "lightning_attention", hidden_size=self.hidden_size, num_heads=_positive_int(sizes, "heads", where),
                head_dim=_positive_int(sizes, "dim", where), value_dim=_positive_int(sizes, "vdim", where),
                decay=tuple(float(d) for d in decay), eps=self.eps, activation="silu", gate="sigmoid",
                norm_span=None, norm_weight=True)
        _need(sizes, ("heads", "dim", "vdim", "scale"), where)
        heads = _positive_int(sizes, "heads", where)
        dim = _positive_int(sizes, "dim", where)
        chunk = None
        if sizes.get("mask") is not None:
            _need(sizes["mask"], ("size",), where + ".mask")
            chunk = _positive_int(sizes["mask"], "size", where + ".mask")
        position = None
        if sizes.get("rot") is not None:
            _need(sizes["rot"], ("dims", "base"), where + ".rot")
            position = PartSpec.of("rotary_pairs", head_dim=dim, theta=_positive(sizes["rot"], "base", where + ".rot"),
                                   max_position=None, rotary_dim=_positive_int(sizes["rot"], "dims", where + ".rot"))
        return PartSpec.of(
            "scored_attention", hidden_size=self.hidden_size, num_heads=heads,
            num_kv_heads=_positive_int(sizes, "kv_heads", where) if "kv_heads" in sizes else heads, head_dim=dim,
            value_dim=_positive_int(sizes, "vdim", where), scale=float(sizes["scale"]), eps=self.eps, chunk=chunk,
            qkv_bias=True, position=position)

    def _feed_forward(self, mlp: Any, where: str) -> PartSpec:
        if mlp is None:
            return PartSpec.of("none", hidden_size=self.hidden_size)
        _need(mlp, ("kind",), where)
        if mlp["kind"] == "dense":
            _need(mlp, ("ff", "limit"), where)
            return PartSpec.of("clamped_gated_mlp", hidden_size=self.hidden_size,
                               intermediate_size=_positive_int(mlp, "ff", where), limit=_positive(mlp, "limit", where),
                               alpha=DENSE_ALPHA, offset=DENSE_OFFSET)
        if mlp["kind"] != "moe":
            raise ConfigError(f"{where}: unknown kind {mlp['kind']!r}; known: ('dense', 'moe')")
        _need(mlp, ("router", "expert"), where)
        router = mlp["router"]
        _need(router, ("experts", "top"), where + ".router")
        _need(mlp["expert"], ("ff",), where + ".expert")
        groups = None
        if router.get("groups") is not None:
            _need(router["groups"], ("count", "keep"), where + ".router.groups")
            groups = (_positive_int(router["groups"], "count", where + ".router.groups"),
                      _positive_int(router["groups"], "keep", where + ".router.groups"))
        shared = mlp.get("shared")
        if shared is not None:
            _need(shared, ("ff",), where + ".shared")
        return PartSpec.of(
            "routed_experts", hidden_size=self.hidden_size,
            experts=_positive_int(router, "experts", where + ".router"), top=_positive_int(router, "top", where + ".router"),
            expert_ff=_positive_int(mlp["expert"], "ff", where + ".expert"), expert_limit=None,
            shared_ff=_positive_int(shared, "ff", where + ".shared") if shared is not None else None, shared_limit=None,
            alpha=EXPERT_ALPHA, offset=EXPERT_OFFSET, scoring="softmax", correction=True, groups=groups,
            identity=_count(router, "identity", where + ".router", 0), normalize=True,
            route_scale=float(router.get("scale", 1.0)), weight_on="output", shared_gate=shared is not None)

    def model_spec(self) -> ModelSpec:
        norm = PartSpec.of("rms_norm_groups", size=self.hidden_size, eps=self.eps, groups=self.norm_groups)
        layers = []
        for index, layer in enumerate(self.raw["layers"]):
            where = f"layers[{index}]"
            _need(layer, ("type", "mixer"), where)
            try:
                layers.append(LayerSpec(
                    mixer=self._mixer(layer["type"], layer["mixer"], where + ".mixer"),
                    feed_forward=self._feed_forward(layer.get("mlp"), where + ".mlp"),
                    norm1=norm, norm2=norm, block="pre_norm",
                    names=(("norm1", "norm1"), ("mixer", "mix"), ("norm2", "norm2"), ("feed_forward", "mlp")),
                ))
            except (TypeError, ValueError) as error:
                if isinstance(error, ConfigError):
                    raise
                raise ConfigError(f"{where}: {error}") from error
        start, stop, times = self.loop()
        # the run order: every run of a layer has a cache unit of its own
        runs = [(i, False) for i in range(start)]
        for turn in range(times if stop > start else 0):
            runs += [(i, turn > 0 and i == start) for i in range(start, stop)]
        runs += [(i, False) for i in range(max(start, stop), len(layers))]
        order = tuple(LayerCall(layer=i, cache=unit, writes=True, adds_embedding=adds)
                      for unit, (i, adds) in enumerate(runs))
        embedding = self.raw.get("embedding") or {}
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
            layers=tuple(layers), order=order, final_norm=norm, tie_word_embeddings=False, max_position=1 << 30,
            eos_token_id=self.raw.get("eos_token_id"), embedding_name="embed", final_norm_name="final.norm",
            head_name="head", layer_prefix="l{index}.", embedding_scale=float(embedding.get("scale", 1.0)),
        )
