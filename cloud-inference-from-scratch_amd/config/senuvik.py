"""Configuration of the Senuvik decoder, read from its ``config.json``.

The file lists the layers one by one: ``layers[i] = {"type", "mixer", "mlp"}``.  Every layer has a norm in front of
each sublayer and one on its output, and a learned scale per channel on what joins the stream
(``x += ls1 * norm1b(mixer(norm1(x)))``, ``x += ls2 * norm2b(mlp(norm2(x)))``: a ``sandwich_norm`` block).  ``type`` is

* ``attention``: grouped-query softmax attention with biases on queries, keys and values, one RMS norm over the whole
  query projection and one over the whole key projection, a rotation of the first ``rot.dims`` numbers of every head in
  pairs of neighbours with every frequency divided by ``rot.scaling.factor``, a window of ``mask.size`` tokens beside
  which the first ``mask.keep_first`` tokens stay visible, and a learned sink per head in the softmax's denominator.
  With ``kv_from: j`` the layer has no keys and values of its own and reads what layer j cached;
* ``mamba2``: a state-space layer (``heads``, ``vdim``, ``state``, ``groups``, ``conv`` taps, ``norm_groups``);
* ``parallel``: ``left_scale * left + right_scale * right`` of causal attention (rotation by halves with stretched
  frequencies, capped scores, a sigmoid gate per head) and time mixing (``heads``, ``dim``; a decay per key channel).

``mlp`` is ``{"kind": "dense", "ff"}`` (a gated unit with the tanh form of gelu), ``{"kind": "moe", "router": {experts,
top}, "expert": {ff}, "shared": {ff}}`` (the ``top`` largest router logits, weights the softmax over the chosen logits
alone, experts with silu, the weight on the expert's output; a shared expert behind a sigmoid gate of one logit per
token) or ``null``.  Beside the layers: ``vocab``, ``width``, ``norm.eps``.  Every size and constant that the file gives
is read from it; what the design fixes (which mixer has which steps, the activations, 0.1 ln(factor) + 1) is handed to
the parts as parameters here.

Tensors are named ``embed``, ``l<i>.norm1``, ``l<i>.norm1b``, ``l<i>.ls1``, ``l<i>.mix.*``, ``l<i>.norm2``,
``l<i>.norm2b``, ``l<i>.ls2``, ``l<i>.mlp.*``, ``final.norm`` and ``head``.
"""

from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any

from .givizen import _need, _positive, _positive_int
from .nokipel import _count
from .specs import ConfigError, LayerCall, LayerSpec, ModelSpec, PartSpec

MIXER_TYPES = ("attention", "mamba2", "parallel")
GELU_ALPHA = 2.0 * (2.0 / 3.141592653589793) ** 0.5   # 0.5 g (1 + tanh(sqrt(2 / pi) (g + c g^3))) = g sigmoid(alpha (g + c g^3))
GELU_CUBIC = 0.044715
NAMES = (("norm1", "norm1"), ("mixer", "mix"), ("norm1_out", "norm1b"), ("scale1", "ls1"),
         ("norm2", "norm2"), ("feed_forward", "mlp"), ("norm2_out", "norm2b"), ("scale2", "ls2"))


def _rotation(rot: Any, dim: int, kind: str, where: str) -> PartSpec | None:
    """The rotation of a mixer: ``rot = {dims, base, scaling}``; ``scaling = {factor}`` divides the frequencies,
    ``{factor, original, fast, slow}`` stretches the slow ones."""
    if rot is None:
        return None
    _need(rot, ("dims", "base"), where)
    dims = _positive_int(rot, "dims", where)
    if dims % 2 or dims > dim:
        raise ConfigError(f"{where}: dims must be even and at most the head size {dim}, got {dims}")
    scaling = None
    table = rot.get("scaling")
    if table is not None:
        _need(table, ("factor",), where + ".scaling")
        if any(key in table for key in ("original", "fast", "slow")):
            _need(table, ("original", "fast", "slow"), where + ".scaling")
            scaling = tuple(_positive(table, key, where + ".scaling") for key in ("factor", "original", "fast", "slow"))
        else:
            scaling = (_positive(table, "factor", where + ".scaling"),)
    return PartSpec.of(kind, head_dim=dim, theta=_positive(rot, "base", where), max_position=None, rotary_dim=dims,
                       scaling=scaling)


@dataclass(frozen=True)
class SenuvikConfig:
    raw: dict = field(compare=False)

    architecture = "Senuvik"

    @classmethod
    def from_hf_config(cls, raw: dict[str, Any]) -> "SenuvikConfig":
        _need(raw, ("layers", "norm", "vocab", "width"), "config")
        if not isinstance(raw["layers"], list) or not raw["layers"]:
            raise ConfigError("config: layers must be a list with at least one layer")
        _need(raw["norm"], ("eps",), "config.norm")
        _positive(raw["norm"], "eps", "config.norm")
        for key in ("vocab", "width"):
            _positive_int(raw, key, "config")
        config = cls(copy.deepcopy(raw))
        spec = config.model_spec()
        from ..parts.model import DecoderModel  # (the parts are built once here: what one refuses is a ConfigError)

        try:
            model = DecoderModel(spec)
            model.expected_tensors()
            model.cache_needs()
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

    # -- mixers
    def _attention(self, sizes: Any, where: str) -> PartSpec:
        _need(sizes, ("heads", "dim", "vdim", "scale"), where)
        heads, dim = _positive_int(sizes, "heads", where), _positive_int(sizes, "dim", where)
        window, keep = None, 0
        if sizes.get("mask") is not None:
            _need(sizes["mask"], ("size",), where + ".mask")
            window = _positive_int(sizes["mask"], "size", where + ".mask")
            keep = _count(sizes["mask"], "keep_first", where + ".mask", 0)
        return PartSpec.of(
            "scored_attention", hidden_size=self.hidden_size, num_heads=heads,
            num_kv_heads=_positive_int(sizes, "kv_heads", where) if "kv_heads" in sizes else heads, head_dim=dim,
            value_dim=_positive_int(sizes, "vdim", where), scale=float(sizes["scale"]), eps=self.eps, window=window,
            keep_first=keep, qk_norm="whole", qkv_bias=True, sink=True, own_kv=sizes.get("kv_from") is None,
            position=_rotation(sizes.get("rot"), dim, "rotary_pairs", where + ".rot"))

    def _left(self, sizes: Any, where: str) -> PartSpec:
        _need(sizes, ("heads", "dim", "vdim", "scale"), where)
        heads, dim = _positive_int(sizes, "heads", where), _positive_int(sizes, "dim", where)
        return PartSpec.of(
            "scored_attention", hidden_size=self.hidden_size, num_heads=heads,
            num_kv_heads=_positive_int(sizes, "kv_heads", where) if "kv_heads" in sizes else heads, head_dim=dim,
            value_dim=_positive_int(sizes, "vdim", where), scale=float(sizes["scale"]), eps=self.eps,
            softcap=_positive(sizes, "softcap", where) if sizes.get("softcap") is not None else None, head_gate=True,
            position=_rotation(sizes.get("rot"), dim, "rotary_half", where + ".rot"))

    def _right(self, sizes: Any, where: str) -> PartSpec:
        _need(sizes, ("heads", "dim"), where)
        return PartSpec.of("time_mixing", hidden_size=self.hidden_size, num_heads=_positive_int(sizes, "heads", where),
                           head_dim=_positive_int(sizes, "dim", where), eps=self.eps)

    def _mixer(self, kind: str, sizes: Any, where: str) -> PartSpec:
        if kind not in MIXER_TYPES:
            raise ConfigError(f"{where}: unknown layer type {kind!r}; known: {MIXER_TYPES}")
        if not isinstance(sizes, dict):
            raise ConfigError(f"{where}: must be a table")
        if kind == "attention":
            return self._attention(sizes, where)
        if kind == "mamba2":
            _need(sizes, ("heads", "vdim", "state", "groups", "conv"), where)
            return PartSpec.of(
                "state_space", hidden_size=self.hidden_size, num_heads=_positive_int(sizes, "heads", where),
                value_dim=_positive_int(sizes, "vdim", where), state=_positive_int(sizes, "state", where),
                groups=_positive_int(sizes, "groups", where), taps=_positive_int(sizes, "conv", where),
                norm_groups=_positive_int(sizes, "norm_groups", where) if "norm_groups" in sizes else 1, eps=self.eps)
        _need(sizes, ("left", "right"), where)
        return PartSpec.of("parallel_mixers", left=self._left(sizes["left"], where + ".left"),
                           right=self._right(sizes["right"], where + ".right"),
                           left_scale=float(sizes.get("left_scale", 1.0)), right_scale=float(sizes.get("right_scale", 1.0)))

    # -- feed-forwards
    def _feed_forward(self, mlp: Any, where: str) -> PartSpec:
        if mlp is None:
            return PartSpec.of("none", hidden_size=self.hidden_size)
        _need(mlp, ("kind",), where)
        if mlp["kind"] == "dense":
            _need(mlp, ("ff",), where)
            return PartSpec.of("clamped_gated_mlp", hidden_size=self.hidden_size,
                               intermediate_size=_positive_int(mlp, "ff", where), limit=None, alpha=GELU_ALPHA,
                               offset=0.0, cubic=GELU_CUBIC)
        if mlp["kind"] != "moe":
            raise ConfigError(f"{where}: unknown kind {mlp['kind']!r}; known: ('dense', 'moe')")
        _need(mlp, ("router", "expert"), where)
        _need(mlp["router"], ("experts", "top"), where + ".router")
        _need(mlp["expert"], ("ff",), where + ".expert")
        shared = mlp.get("shared")
        if shared is not None:
            _need(shared, ("ff",), where + ".shared")
        return PartSpec.of(
            "routed_experts", hidden_size=self.hidden_size,
            experts=_positive_int(mlp["router"], "experts", where + ".router"),
            top=_positive_int(mlp["router"], "top", where + ".router"),
            expert_ff=_positive_int(mlp["expert"], "ff", where + ".expert"), expert_limit=None,
            shared_ff=_positive_int(shared, "ff", where + ".shared") if shared is not None else None, shared_limit=None,
            alpha=1.0, offset=0.0, scoring="softmax", normalize=True, weight_on="output",
            shared_gate=shared is not None)

    def model_spec(self) -> ModelSpec:
        norm = PartSpec.of("rms_norm_groups", size=self.hidden_size, eps=self.eps, groups=1)
        layers, sources = [], []
        for index, layer in enumerate(self.raw["layers"]):
            where = f"layers[{index}]"
            _need(layer, ("type", "mixer"), where)
            try:
                layers.append(LayerSpec(
                    mixer=self._mixer(layer["type"], layer["mixer"], where + ".mixer"),
                    feed_forward=self._feed_forward(layer.get("mlp"), where + ".mlp"),
                    norm1=norm, norm2=norm, norm1_out=norm, norm2_out=norm, block="sandwich_norm", names=NAMES,
                ))
            except (TypeError, ValueError) as error:
                if isinstance(error, ConfigError):
                    raise
                raise ConfigError(f"{where}: {error}") from error
            source = layer["mixer"].get("kv_from") if layer["type"] == "attention" else None
            if source is not None:
                if isinstance(source, bool) or not isinstance(source, int) or not 0 <= source < index:
                    raise ConfigError(f"{where}.mixer: kv_from must name an earlier layer, got {source!r}")
                other = self.raw["layers"][source]
                if other.get("type") != "attention" or other["mixer"].get("kv_from") is not None:
                    raise ConfigError(f"{where}.mixer: kv_from names layer {source}, which has no keys and values of its own")
            sources.append(source)
        # the run order: a layer without keys and values of its own reads the cache unit of the layer it names
        unit_of: dict[int, int] = {}
        order = []
        for index, source in enumerate(sources):
            if source is None:
                unit_of[index] = len(unit_of)
                order.append(LayerCall(layer=index, cache=unit_of[index], writes=True))
            else:
                order.append(LayerCall(layer=index, cache=unit_of[source], writes=False))
        return ModelSpec(
            architecture=self.architecture, vocab_size=self.vocab_size, hidden_size=self.hidden_size,
            layers=tuple(layers), order=tuple(order), final_norm=norm, tie_word_embeddings=False, max_position=1 << 30,
            eos_token_id=self.raw.get("eos_token_id"), embedding_name="embed", final_norm_name="final.norm",
            head_name="head", layer_prefix="l{index}.",
        )
