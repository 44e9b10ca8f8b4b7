"""Kisadra without a GPU: the configuration reader and its refusals, the run order, the tensors
a model expects, and the plain implementation's mechanisms against direct formulas."""

from __future__ import annotations

import json
import math

import pytest
import torch

import kisadra_tiny as kt
from plain import kisadra_plain as plain
from turboserve_amd.config.kisadra_config import KisadraConfig
from turboserve_amd.config.model_config import UnsupportedModelError
from turboserve_amd.config.registry import parse_model_config
from turboserve_amd.weights.random_init import describe_model


def test_the_reader_takes_every_size_from_the_file():
    config = parse_model_config(kt.CONFIG_A)
    assert isinstance(config, KisadraConfig)
    assert (config.vocab_size, config.hidden_size, config.norm_eps) == (211, 64, 1e-5)
    assert [layer.type for layer in config.layers] == ["gla", "attention", "latent_attention"]
    state, chunks, latent = (layer.mixer for layer in config.layers)
    assert (state.heads, state.dim, state.vdim, state.tau, state.rank) == (2, 16, 24, 4.0, 8)
    assert (chunks.heads, chunks.kv_heads, chunks.dim, chunks.vdim, chunks.chunk, chunks.scale) == (4, 2, 16, 8, 20, 0.3)
    assert (latent.heads, latent.dim, latent.rot_dim, latent.vdim, latent.kv_rank, latent.rot_base, latent.rot_dims) == (3, 16, 8, 12, 24, 1000.0, 8)
    routed = config.layers[1].mlp
    assert (routed.experts, routed.identity, routed.top, routed.ff, routed.limit) == (6, 1, 2, 40, 1.5)
    assert config.layers[2].mlp is None and config.layers[0].mlp.ff == 96
    assert parse_model_config(kt.without_ranks(kt.CONFIG_A)).layers[0].mixer.rank is None


def test_the_run_order_of_a_loop():
    config = parse_model_config(kt.CONFIG_A)
    assert config.run_order() == [(0, False), (1, True), (2, False), (1, True), (2, False), (1, True), (2, False)]
    assert plain.run_order(kt.CONFIG_A) == config.run_order()
    empty = dict(kt.CONFIG_A, loop={"start": 2, "stop": 2, "times": 5})
    assert parse_model_config(empty).run_order() == [(0, False), (1, False), (2, False)]
    assert parse_model_config({k: v for k, v in kt.CONFIG_A.items() if k != "loop"}).run_order() == [(0, False), (1, False), (2, False)]


@pytest.mark.parametrize("damage,message", [
    (lambda c: c["layers"][0].update(type="conv"), "type"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=3), "rot.dims"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=8), "top"),
    (lambda c: c["layers"][1]["mlp"].update(kind="other"), "kind"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["layers"][0]["mixer"].update(tau=0), "tau"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), "size"),
])
def test_the_reader_refuses(damage, message):
    config = json.loads(json.dumps(kt.CONFIG_A))
    damage(config)
    with pytest.raises(UnsupportedModelError, match=message):
        parse_model_config(config)


def test_the_tensors_a_model_expects():
    _, model = describe_model(kt.CONFIG_A)
    specs = {name: spec.shape for name, spec in model.tensor_specs().items()}
    assert specs["embed"] == (211, 64) and specs["head"] == (211, 64) and specs["final.norm"] == (64,)
    assert specs["loop.in"] == (64, 128)
    assert specs["l0.norm1"] == (64,) and "l0.norm2" not in specs
    assert (specs["l0.mix.q"], specs["l0.mix.v"], specs["l0.mix.g"], specs["l0.mix.o"]) == ((32, 64), (48, 64), (48, 64), (64, 48))
    assert (specs["l0.mix.a1"], specs["l0.mix.a2"], specs["l0.mix.a2.b"], specs["l0.mix.norm"]) == ((8, 64), (32, 8), (32,), (24,))
    assert (specs["l1.mix.q"], specs["l1.mix.k"], specs["l1.mix.v"], specs["l1.mix.o"]) == ((64, 64), (32, 64), (16, 64), (64, 32))
    assert (specs["l1.mix.q.norm"], specs["l1.mix.k.norm"]) == ((64,), (32,))
    assert (specs["l1.mlp.router"], specs["l1.mlp.correction"]) == ((7, 64), (7,))
    assert "l1.mlp.e5.down" in specs and "l1.mlp.e6.gate" not in specs
    assert (specs["l2.mix.q"], specs["l2.mix.dkv"], specs["l2.mix.dkv.norm"]) == ((72, 64), (32, 64), (24,))
    assert (specs["l2.mix.uk"], specs["l2.mix.uv"], specs["l2.mix.o"]) == ((48, 24), (36, 24), (64, 36))
    assert not any(name.startswith("l2.mlp") for name in specs)
    # A file that does not name the decay input's width leaves it to the tensors.
    _, unnamed = describe_model(kt.without_ranks(kt.CONFIG_A))
    assert unnamed.tensor_specs()["l0.mix.a1"].shape == (-1, 64)
    # Each layer run has a cache of its own: pages for the attentions, a state for the other.
    needs = model.cache_needs()
    assert len(needs) == 7 and type(needs[0]).__name__ == "FixedState" and needs[0].shape == (2, 16, 24)
    assert (needs[2].num_kv_heads, needs[2].head_dim, needs[2].value_width) == (1, 32, 0)


def test_a_loop_over_nothing_leaves_its_matrix_unread():
    config = dict(kt.CONFIG_A, loop={"start": 1, "stop": 1, "times": 2})
    _, model = describe_model(config)
    assert "loop.in" not in model.tensor_specs() and "loop.in" in model.ignorable_names()


# -- the plain implementation against direct formulas -----------------------------------------------


def test_plain_gelu_and_slopes():
    z = torch.linspace(-6, 6, 25, dtype=torch.float64)
    want = torch.tensor([0.5 * v * (1 + math.tanh(math.sqrt(2 / math.pi) * (v + 0.044715 * v ** 3))) for v in z.tolist()])
    torch.testing.assert_close(plain.gelu_tanh(z), want.double())
    assert plain.distance_slopes(4) == [2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8]


def test_plain_state_walk_is_the_sum_it_stands_for():
    """``o_t = sum_{j <= t} (prod_{j < l <= t} a_l) (k_j . q_t) v_j`` per channel, written out."""
    g = torch.Generator().manual_seed(0)
    sizes = {"heads": 1, "dim": 3, "vdim": 2, "tau": 2.0}
    width, count = 5, 6
    tensors = {f"p.{n}": torch.randn(s, generator=g, dtype=torch.float64) for n, s in {
        "q": (3, width), "k": (3, width), "v": (2, width), "g": (2, width), "o": (width, 2), "a1": (2, width), "a2": (3, 2), "a2.b": (3,)}.items()}
    tensors["p.norm"] = torch.ones(2, dtype=torch.float64)
    tensors["p.o"] = torch.eye(2, dtype=torch.float64)[:, :2].repeat(3, 1)[:width]
    h = torch.randn(count, width, generator=g, dtype=torch.float64)
    got = plain.gated_linear_attention(h, tensors, "p", sizes, 1e-6)
    q, k, v = h @ tensors["p.q"].T / 3 ** 0.5, h @ tensors["p.k"].T, h @ tensors["p.v"].T
    a = torch.sigmoid(h @ tensors["p.a1"].T @ tensors["p.a2"].T + tensors["p.a2.b"]) ** 0.5
    gate = h @ tensors["p.g"].T
    for t in range(count):
        o = torch.zeros(2, dtype=torch.float64)
        for j in range(t + 1):
            kept = torch.ones(3, dtype=torch.float64)
            for l in range(j + 1, t + 1):
                kept = kept * a[l]
            o += (kept * k[j] * q[t]).sum() * v[j]
        o = o / torch.sqrt((o * o).mean() + 1e-6)
        torch.testing.assert_close(got[t], (o * gate[t] * torch.sigmoid(gate[t])) @ tensors["p.o"].T)


def test_plain_chunks_and_the_sink():
    """With one head, zero queries and values of one, a token's output is w / (1 + w), w the sum of
    exp(-m distance) over the positions of its chunk up to itself (m = 2^-8 for one head): the mask,
    the distance slope and the extra one in the denominator alone."""
    width = 4
    tensors = {"p.q": torch.zeros(2, width), "p.k": torch.zeros(2, width), "p.v": torch.zeros(1, width), "p.o": torch.ones(1, 1),
               "p.q.norm": torch.ones(2), "p.k.norm": torch.ones(2)}
    tensors["p.v"][0, 0] = 1.0
    h = torch.zeros(11, width)
    h[:, 0] = 1.0
    sizes = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 1, "scale": 1.0, "mask": {"size": 4}}
    got = plain.chunked_sink_attention(h, tensors, "p", sizes, 1e-6)[:, 0]
    mass = [sum(math.exp(-(2.0 ** -8) * d) for d in range(i % 4 + 1)) for i in range(11)]
    want = torch.tensor([w / (1.0 + w) for w in mass])
    torch.testing.assert_close(got, want)


def test_plain_routing_by_brute_force():
    g = torch.Generator().manual_seed(4)
    h, router, correction = torch.randn(20, 6, generator=g), torch.randn(9, 6, generator=g), 0.3 * torch.randn(9, generator=g)
    taken, weights = plain.routing(h, router, correction, 3)
    s = torch.softmax(h @ router.T, dim=-1)
    assert torch.equal(taken, torch.topk(s + correction, 3, dim=-1).indices)
    torch.testing.assert_close(weights, torch.gather(s, 1, taken))


def test_plain_rotation_turns_pairs_in_halves():
    x = torch.arange(1.0, 7.0).view(1, 6).repeat(2, 1)
    out = plain.turn_pairs(x, [0, 3], 4, 100.0)
    torch.testing.assert_close(out[0], x[0])
    for i in range(2):
        angle = 3 * 100.0 ** (-2.0 * i / 4)
        u, v = x[1, i], x[1, i + 2]
        assert math.isclose(float(out[1, i]), float(u * math.cos(angle) - v * math.sin(angle)), rel_tol=1e-6)
        assert math.isclose(float(out[1, i + 2]), float(v * math.cos(angle) + u * math.sin(angle)), rel_tol=1e-6)
    torch.testing.assert_close(out[1, 4:], x[1, 4:])
