"""CPU: what pins the plain Senuvik implementation (tests/plain_senuvik.py), and the configuration's reading, the
cache manager's kept first pages and the loader's free sizes, which need no GPU."""

from __future__ import annotations

import copy
import math

import pytest
import torch

import plain_senuvik as ps
import senuvik_util as su

F = torch.float64


def test_norm_is_the_root_mean_square_with_eps_inside_the_root():
    x = torch.randn(5, 12, dtype=F)
    w = torch.rand(12, dtype=F) + 0.5
    want = torch.stack([row / math.sqrt(float((row ** 2).sum()) / 12 + 1e-3) * w for row in x])
    assert torch.allclose(ps.rms_norm(x, w, 1e-3), want, rtol=1e-13, atol=0)


def test_gelu_tanh_is_the_gated_unit_with_a_cubic_inside_the_sigmoid():
    from cie_amd.config.senuvik import GELU_ALPHA, GELU_CUBIC

    g = torch.linspace(-6, 6, 241, dtype=F)
    assert torch.allclose(ps.gelu_tanh(g), g * torch.sigmoid(GELU_ALPHA * (g + GELU_CUBIC * g ** 3)), rtol=1e-12, atol=1e-15)
    assert torch.allclose(ps.gelu_tanh(g), torch.nn.functional.gelu(g, approximate="tanh"), rtol=1e-12, atol=1e-15)


def test_rotation_in_pairs_is_a_complex_multiplication_and_differs_from_the_halves():
    head = torch.randn(12, dtype=F)
    f = ps.plain_frequencies(8, 100.0)
    turned = ps.rotate(head, 7, f, 1.0, 8, neighbours=True)
    z = torch.view_as_complex(head[:8].reshape(4, 2).contiguous()) * torch.polar(torch.ones(4, dtype=F), 7 * f)
    assert torch.allclose(turned[:8], torch.view_as_real(z).reshape(8), rtol=1e-13, atol=1e-15)
    assert torch.equal(turned[8:], head[8:])
    halves = ps.rotate(head, 7, f, 1.0, 8, neighbours=False)
    z = torch.complex(head[:4], head[4:8]) * torch.polar(torch.ones(4, dtype=F), 7 * f)
    assert torch.allclose(halves[:4], z.real, rtol=1e-13, atol=1e-15) and torch.allclose(halves[4:8], z.imag, rtol=1e-13, atol=1e-15)
    assert not torch.allclose(turned, halves)
    assert torch.equal(ps.rotate(head, 0, f, 1.0, 8, True), head)


def test_scaled_frequencies_against_the_package_tables():
    """Two implementations of the same formulas, the package's tables and the plain ones, agree; the factor alone
    divides, the four constants stretch only the slow pairs."""
    from cie_amd.parts.position import RotaryHalf, RotaryPairs

    f, gain = ps.linear_frequencies(8, 100.0, 4.0)
    got, g = RotaryPairs(16, 100.0, None, rotary_dim=8, scaling=(4.0,)).inv_freq()
    assert g == 1.0 == gain and torch.allclose(got.double(), f, rtol=1e-6)
    f, gain = ps.yarn_frequencies(8, 1000.0, **su.YARN)
    got, g = RotaryHalf(16, 1000.0, None, rotary_dim=8, scaling=(4.0, 64, 16.0, 1.0)).inv_freq()
    assert abs(g - gain) < 1e-12 and abs(gain - (0.1 * math.log(4.0) + 1.0)) < 1e-12
    assert torch.allclose(got.double(), f, rtol=1e-6)
    plain = ps.plain_frequencies(8, 1000.0)
    assert torch.allclose(f[0], plain[0]) and torch.allclose(f[-1], plain[-1] / 4.0)  # fast pairs stay, slow ones stretch
    cos, sin = RotaryHalf(16, 1000.0, None, rotary_dim=8, scaling=(4.0, 64, 16.0, 1.0)).tables("cpu", 10)
    assert torch.allclose(cos[3].double(), torch.cos(3 * f) * gain, atol=1e-6) and torch.allclose(sin[3].double(), torch.sin(3 * f) * gain, atol=1e-6)


def test_window_kept_first_tokens_and_sink_against_library_attention():
    n, dim, size, keep = 30, 8, 5, 3
    q, k, v = torch.randn(n, dim, dtype=F), torch.randn(n, dim, dtype=F), torch.randn(n, 6, dtype=F)
    sink = torch.tensor(0.7, dtype=F)
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    mask = (j <= i) & ((i - j < size) | (j < keep))
    for a in range(n):
        for b in range(n):
            assert ps.window_sees(a, b, size, keep) == bool(mask[a, b])
    assert ps.window_sees(20, 2, size, keep) and not ps.window_sees(20, 3, size, keep)
    assert ps.window_sees(20, 16, size, keep) and not ps.window_sees(20, 15, size, keep)
    scores = (q @ k.t()) * 0.5
    scores = torch.cat([scores.masked_fill(~mask, -math.inf), sink.expand(n, 1)], dim=1)   # the sink as one more column ...
    want = torch.softmax(scores, dim=1)[:, :n] @ v                                         # ... that has no value
    for a in range(n):
        seen = [b for b in range(n) if mask[a, b]]
        got = ps.softmax_attention_token(q[a], k, v, seen, 0.5, sink=sink)
        assert torch.allclose(got, want[a], rtol=1e-12, atol=1e-14)
    capped = ps.softmax_attention_token(q[9], k, v, list(range(10)), 0.5, softcap=2.0)
    s = 2.0 * torch.tanh(((k[:10] @ q[9]) * 0.5) / 2.0)
    assert torch.allclose(capped, torch.softmax(s, 0) @ v[:10], rtol=1e-12, atol=1e-14)


def test_state_space_memory_against_its_closed_form():
    n, N, P = 9, 5, 4
    x, b, c = torch.randn(n, P, dtype=F), torch.randn(n, N, dtype=F), torch.randn(n, N, dtype=F)
    dt = torch.rand(n, dtype=F) + 0.1
    a_log, d = torch.tensor(0.3, dtype=F), torch.tensor(1.5, dtype=F)
    memory = torch.zeros(N, P, dtype=F)
    for t in range(n):
        memory, y = ps.state_space_token(memory, x[t], b[t], c[t], dt[t], a_log, d)
        want = d * x[t]
        for s in range(t + 1):
            fade = math.exp(-math.exp(0.3) * float(dt[s + 1: t + 1].sum()))
            want = want + fade * float(dt[s]) * float(c[t] @ b[s]) * x[s]
        assert torch.allclose(y, want, rtol=1e-11, atol=1e-13)


def test_time_mixing_memory_against_its_closed_form():
    n, D = 8, 5
    r, k, v = torch.randn(n, D, dtype=F), torch.randn(n, D, dtype=F), torch.randn(n, D, dtype=F)
    w, u = torch.rand(n, D, dtype=F), torch.randn(D, dtype=F)
    memory = torch.zeros(D, D, dtype=F)
    for t in range(n):
        memory, out = ps.time_mix_token(memory, r[t], k[t], v[t], w[t], u)
        want = float((r[t] * u * k[t]).sum()) * v[t]                       # the bonus, for the token itself only
        for s in range(t):
            fade = torch.prod(w[s + 1: t], dim=0) if t > s + 1 else torch.ones(D, dtype=F)  # the decays of the tokens between
            want = want + float((r[t] * fade * k[s]).sum()) * v[s]
        assert torch.allclose(out, want, rtol=1e-11, atol=1e-13)


def test_router_takes_the_largest_logits_and_weighs_them_among_themselves():
    logits = torch.tensor([0.1, 2.0, -1.0, 2.0, 0.5], dtype=F)
    chosen, weights = ps.router_choice(logits, 3)
    assert chosen == [1, 3, 4]                                              # lowest index first among equals
    e = torch.exp(torch.tensor([2.0, 2.0, 0.5], dtype=F))
    assert torch.allclose(weights, e / e.sum(), rtol=1e-13)
    chosen, weights = ps.router_choice(logits, 1)
    assert chosen == [1] and float(weights[0]) == 1.0


def test_a_layer_composed_by_hand():
    """The sandwich of norms, the scale per channel, experts with a gated shared expert."""
    raw = su.single({"type": "mamba2", "mixer": {"heads": 2, "vdim": 4, "state": 3, "groups": 1, "conv": 2, "norm_groups": 1},
                     "mlp": {"kind": "moe", "router": {"experts": 4, "top": 2}, "expert": {"ff": 6}, "shared": {"ff": 5}}}, width=16)
    w = {k: v.double() for k, v in su.make_weights(raw, seed=1).items()}
    seq = ps.Model(raw, w).start()
    logits = seq.token(3)
    x = w["embed"][3]
    mixed = ps.Model(raw, w).start().mamba2(0, raw["layers"][0]["mixer"], "l0.mix.", ps.rms_norm(x, w["l0.norm1"], 1e-6))
    x = x + ps.rms_norm(mixed, w["l0.norm1b"], 1e-6) * w["l0.ls1"]
    h = ps.rms_norm(x, w["l0.norm2"], 1e-6)
    z = w["l0.mlp.router"] @ h
    top = torch.topk(z, 2).indices.tolist()
    p = torch.softmax(z[top], 0)
    unit = lambda pre: w[pre + "down"] @ (torch.nn.functional.silu(w[pre + "gate"] @ h) * (w[pre + "up"] @ h))
    fed = sum(p[i] * unit(f"l0.mlp.e{e}.") for i, e in enumerate(top))
    fed = fed + torch.sigmoid(w["l0.mlp.shared.sg"] @ h)[0] * unit("l0.mlp.shared.")
    x = x + ps.rms_norm(fed, w["l0.norm2b"], 1e-6) * w["l0.ls2"]
    assert torch.allclose(seq.stream_after[0][0], x, rtol=1e-11, atol=1e-13)
    assert torch.allclose(logits, w["head"] @ ps.rms_norm(x, w["final.norm"], 1e-6), rtol=1e-11, atol=1e-13)


def test_a_layer_that_reads_another_layers_keys_sees_them_under_its_own_mask():
    raw = copy.deepcopy(su.SMALL_A)
    w = su.make_weights(raw, seed=2)
    tokens = list(range(40))
    base = ps.forward(raw, w, tokens)
    wider = copy.deepcopy(raw)
    wider["layers"][3]["mixer"]["mask"] = {"size": 40, "keep_first": 0}
    assert not torch.allclose(ps.forward(wider, w, tokens)[25:], base[25:])    # its own window matters ...
    assert torch.allclose(ps.forward(wider, w, tokens)[:20], base[:20])        # ... from where it is full
    assert "l3.mix.k" not in w and "l3.mix.v" not in w and "l3.mix.k.norm" not in w and "l3.mix.q.norm" in w


# ---------------------------------------------------------------------------------------------------- configuration
def test_the_configuration_hands_on_every_size_and_constant():
    from cie_amd.cache.manager import FixedState, PagedKV
    from cie_amd.config import config_from_dict
    from cie_amd.parts.model import DecoderModel

    config = config_from_dict(copy.deepcopy(su.SMALL_A))
    spec = config.model_spec()
    assert (spec.vocab_size, spec.hidden_size, len(spec.layers)) == (96, 64, 5)
    assert [layer.block for layer in spec.layers] == ["sandwich_norm"] * 5
    first = spec.layers[0].mixer.as_dict()
    assert (first["num_heads"], first["num_kv_heads"], first["head_dim"], first["value_dim"]) == (4, 2, 16, 24)
    assert (first["window"], first["keep_first"], first["scale"], first["qk_norm"], first["sink"], first["own_kv"]) == (9, 3, 0.3, "whole", True, True)
    assert first["position"].kind == "rotary_pairs" and first["position"].as_dict()["scaling"] == (2.0,)
    space = spec.layers[1].mixer.as_dict()
    assert (space["num_heads"], space["value_dim"], space["state"], space["groups"], space["taps"], space["norm_groups"]) == (4, 8, 12, 2, 4, 2)
    pair = spec.layers[2].mixer.as_dict()
    assert (pair["left_scale"], pair["right_scale"]) == (0.7, 0.4)
    left = pair["left"].as_dict()
    assert left["softcap"] == 5.0 and left["head_gate"] and left["position"].kind == "rotary_half"
    assert left["position"].as_dict()["scaling"] == (4.0, 64.0, 16.0, 1.0)
    assert pair["right"].as_dict()["head_dim"] == 12 and pair["right"].as_dict()["num_heads"] == 2
    reader = spec.layers[3].mixer.as_dict()
    assert not reader["own_kv"] and reader["window"] == 20
    # the run order: the reader reads unit 0 and writes nothing; the unit keeps what either layer still sees
    assert [(c.layer, c.cache, c.writes) for c in spec.order] == [(0, 0, True), (1, 1, True), (2, 2, True), (3, 0, False), (4, 3, True)]
    needs = DecoderModel(spec).cache_needs()
    # (the heads are padded up to the sizes the attention kernels take)
    assert (needs[0].kv_heads, needs[0].window, needs[0].keep_first) == (2, 20, 3) and needs[0].head_dim >= 16
    assert needs[1] == (FixedState((4, 12, 8)), FixedState((3, 24 + 32 + 2 * 2 * 12 - 24)))
    assert isinstance(needs[2][0], PagedKV) and (needs[2][0].kv_heads, needs[2][0].window) == (1, None)
    assert needs[2][1:] == (FixedState((2, 12, 12)), FixedState((64,)))
    dense = spec.layers[0].feed_forward.as_dict()
    assert dense["intermediate_size"] == 80 and abs(dense["alpha"] - 2 * math.sqrt(2 / math.pi)) < 1e-15 and dense["cubic"] == 0.044715
    moe = spec.layers[1].feed_forward.as_dict()
    assert (moe["experts"], moe["top"], moe["expert_ff"], moe["shared_ff"], moe["scoring"], moe["normalize"], moe["weight_on"],
            moe["shared_gate"]) == (6, 2, 24, 16, "softmax", True, "output", True)
    assert spec.layers[2].feed_forward.kind == "none"
    assert config.to_hf_config()["architecture"] == "Senuvik"


@pytest.mark.parametrize("change, message", [
    (lambda r: r["layers"][0].update(type="attention_9"), "unknown layer type"),
    (lambda r: r["layers"][3]["mixer"].update(kv_from=3), "earlier layer"),
    (lambda r: r["layers"][3]["mixer"].update(kv_from=1), "no keys and values"),
    (lambda r: r["layers"][3]["mixer"].update(heads=3, kv_heads=1), "heads differ"),
    (lambda r: r["layers"][0]["mixer"]["rot"].update(dims=7), "even"),
    (lambda r: r["layers"][1]["mixer"].update(groups=3), "equal parts"),
    (lambda r: r["layers"][1]["mixer"].pop("state"), "missing"),
    (lambda r: r["layers"][1]["mlp"]["router"].update(top=7), "router outputs"),
    (lambda r: r["layers"][0]["mlp"].update(kind="sparse"), "unknown kind"),
    (lambda r: r["layers"][2]["mixer"].pop("right"), "missing"),
    (lambda r: r.pop("width"), "missing"),
])
def test_the_configuration_refuses_what_does_not_fit(change, message):
    from cie_amd.config import ConfigError, config_from_dict

    raw = copy.deepcopy(su.SMALL_A)
    change(raw)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(raw)


def test_a_size_that_only_the_checkpoint_knows(tmp_path):
    """The rank of the decay's two small products is read off the tensors; the two must agree."""
    from cie_amd.config import config_from_dict
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights import write_tensors
    from cie_amd.weights.loader import SafetensorsSource, WeightError

    raw = su.single(copy.deepcopy(su.SMALL_A["layers"][2]), width=64)
    expected = expected_tensors(config_from_dict(raw).model_spec())
    assert expected["l0.mix.right.w1"].shape == (None, 64) and expected["l0.mix.right.w2"].shape == (24, None)
    for rank in (3, 16):
        weights = su.make_weights(raw, seed=1, rank=rank)
        folder = write_tensors(tmp_path / f"rank{rank}", raw, {k: v.to(torch.bfloat16) for k, v in weights.items()})
        tensors = SafetensorsSource(folder).load(expected, "float32", "cpu")
        assert tensors["l0.mix.right.w1"].shape == (rank, 64) and tensors["l0.mix.right.w2"].shape == (24, rank)
    weights["l0.mix.right.w1"] = weights["l0.mix.right.w1"][:, :60]
    folder = write_tensors(tmp_path / "narrow", raw, {k: v.to(torch.bfloat16) for k, v in weights.items()})
    with pytest.raises(WeightError, match="l0.mix.right.w1"):
        SafetensorsSource(folder).load(expected, "float32", "cpu")


def test_random_weights_mode_draws_every_tensor():
    from cie_amd.config import config_from_dict
    from cie_amd.parts.model import expected_tensors
    from cie_amd.weights.loader import RandomSource

    for raw in su.SMALL.values():
        expected = expected_tensors(config_from_dict(copy.deepcopy(raw)).model_spec())
        tensors = RandomSource(3).load(expected, "float32", "cpu")
        assert set(tensors) == {name for name, spec in expected.items() if not spec.optional}
        assert all(spec.fits(tuple(tensors[name].shape)) for name, spec in expected.items() if name in tensors)


# ---------------------------------------------------------------------------------------------------- cache manager
def test_pages_of_the_kept_first_tokens_stay_when_the_window_passes_them():
    from cie_amd.cache.manager import CacheManager, PagedKV

    manager = CacheManager([PagedKV(1, 8, window=6, keep_first=5)], page_size=4, kv_tokens=64, max_running=2,
                           max_model_len=64, prefill_chunk=16)
    manager.admit("a")
    manager.ensure_capacity_batch({"a": 30})
    manager.commit_lengths({"a": 30})
    table = manager.block_table(0, "a")
    # the next token sits at 30 and sees keys 25 .. 30 and 0 .. 4: pages 0 and 1 hold kept tokens, page 6 on the window
    assert [page >= 0 for page in table] == [True, True, False, False, False, False, True, True]
    manager.assert_invariants()
    assert manager.tokens_missing("a", 34) == 4 and manager.tokens_missing("a", 31) == 0
    manager.ensure_capacity_batch({"a": 41})
    manager.commit_lengths({"a": 41})
    table = manager.block_table(0, "a")
    assert [i for i, page in enumerate(table) if page >= 0] == [0, 1, 9, 10]
    manager.release("a")
    assert manager.stats().pages_used == 0
    # without kept tokens the first pages go too; a window that nothing has passed frees nothing
    manager = CacheManager([PagedKV(1, 8, window=6)], page_size=4, kv_tokens=64, max_running=2, max_model_len=64, prefill_chunk=16)
    manager.admit("b")
    manager.ensure_capacity_batch({"b": 30})
    manager.commit_lengths({"b": 30})
    assert [i for i, page in enumerate(manager.block_table(0, "b")) if page >= 0] == [6, 7]


def test_a_unit_read_under_two_masks_keeps_what_either_sees():
    from cie_amd.cache.manager import PagedKV

    a = PagedKV(2, 16, window=9, value_dim=24, keep_first=3)
    assert a.joined(PagedKV(2, 16, window=20, value_dim=24)) == PagedKV(2, 16, window=20, value_dim=24, keep_first=3)
    assert a.joined(PagedKV(2, 16, window=None, value_dim=24)) == PagedKV(2, 16, window=None, value_dim=24)
    assert a.joined(PagedKV(2, 16, window=4, value_dim=24, keep_first=8)).keep_first == 8
    with pytest.raises(ValueError):
        a.joined(PagedKV(1, 16, window=9, value_dim=24))
