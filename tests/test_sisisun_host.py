"""Sisisun on the host: the configuration reader, the plan and its tensor names, and the plain
implementation's own rules (routing, run order) against brute force."""

from __future__ import annotations

import copy
import itertools

import pytest
import torch

import sisisun_tiny as st
from plain import sisisun_plain as plain
from turboserve_amd.config.model_config import UnsupportedModelError
from turboserve_amd.config.registry import architecture_of, parse_model_config
from turboserve_amd.weights.random_init import describe_model


def test_the_configuration_is_read_layer_by_layer():
    config = parse_model_config(st.CONFIG_P)
    assert config.vocab_size == 211 and config.hidden_size == 64 and config.norm_eps == 1e-5
    assert [l.mixer.vdim for l in config.layers] == [16, 40, 16, 24]
    assert config.layers[2].mlp is None and config.layers[0].mlp.limit == 1.5
    routed = config.layers[1].mlp
    assert (routed.experts, routed.top, routed.groups, routed.keep, routed.shared_ff) == (8, 2, 4, 2, 64)
    assert config.layers[3].mlp.shared_ff == 0
    assert architecture_of(st.CONFIG_P).name == "Sisisun"


def test_the_run_order_repeats_the_slice_and_marks_where_a_pass_begins():
    config = parse_model_config(st.CONFIG_P)
    assert config.run_order() == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None)]
    assert config.run_order() == plain.run_order(st.CONFIG_P)
    assert parse_model_config(st.CONFIG_Q).run_order() == [(0, 0), (1, None)] == plain.run_order(st.CONFIG_Q)
    _, model = describe_model(st.CONFIG_P)
    entering = [None if call.enter is None else (call.enter.params["index"], call.enter.params["add_origin"])
                for call in model.plan.schedule]
    assert entering == [None, (0, False), None, (1, True), None, (2, True), None, None]
    assert len(model.cache_needs()) == 8  # a cache per layer run


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="recurrent"), "not implemented"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "not implemented"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "more than the kept groups hold"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3), "groups"),
    (lambda c: c["loop"].update(stop=9), "does not lie inside"),
    (lambda c: c.update(width="64"), "must be an int"),
    (lambda c: c["norm"].update(eps=0), "positive"),
])
def test_what_the_design_does_not_have_is_refused(change, message):
    config = copy.deepcopy(st.CONFIG_P)
    change(config)
    with pytest.raises(UnsupportedModelError, match=message):
        parse_model_config(config)


def test_tensor_names_and_shapes_follow_the_layers():
    _, model = describe_model(st.CONFIG_P)
    specs = {name: spec.shape for name, spec in model.tensor_specs().items()}
    assert specs["embed"] == (211, 64) and specs["head"] == (211, 64) and specs["final.norm"] == (64,)
    assert specs["loop.step"] == (3, 64)
    assert specs["l0.mix.q"] == (128, 64) and specs["l0.mix.k"] == (64, 64) and specs["l0.mix.v"] == (32, 64)
    assert specs["l0.mix.o"] == (64, 64) and specs["l0.mix.q.norm"] == (32,) == specs["l0.mix.k.norm"]
    assert specs["l1.mix.v"] == (80, 64) and specs["l1.mix.o"] == (64, 80)
    assert specs["l1.mlp.router"] == (8, 64) and specs["l1.mlp.e7.down"] == (64, 48) and specs["l1.mlp.shared.sg"] == (1, 64)
    assert "l2.norm2" not in specs and not any(name.startswith("l2.mlp") for name in specs)
    assert "l3.mlp.shared.gate" not in specs and specs["l3.mlp.e5.up"] == (40, 64)
    needs = model.cache_needs()
    assert (needs[0].num_kv_heads, needs[0].head_dim, needs[0].value_width) == (2, 32, 16)
    assert needs[1] == needs[3] == needs[5] and needs[1].value_width == 40


def test_the_routing_rule_against_brute_force():
    generator = torch.Generator().manual_seed(5)
    for experts, top, groups, keep in [(8, 2, 4, 2), (6, 1, 1, 1), (5, 3, 5, 3), (12, 3, 3, 2), (16, 4, 2, 1)]:
        size = experts // groups
        for _ in range(25):
            scores = torch.rand(experts, generator=generator).tolist()
            marks = [sum(sorted(scores[g * size:(g + 1) * size])[-2:]) for g in range(groups)]
            best = max(itertools.combinations(range(groups), keep), key=lambda kept: sum(marks[g] for g in kept))
            eligible = [e for e in range(experts) if e // size in best]
            want = sorted(sorted(eligible, key=lambda e: -scores[e])[:top])
            assert sorted(plain.route(scores, top, groups, keep)) == want


def test_the_plain_gated_units():
    x = torch.tensor([[3.0, -4.0, 0.5]])
    eye = torch.eye(3)
    tensors = {"p.gate": eye, "p.up": eye, "p.down": eye}
    g = torch.tensor([2.0, -4.0, 0.5])
    u = torch.tensor([2.0, -2.0, 0.5])
    assert torch.allclose(plain.clamped_glu(x, tensors, "p", 2.0)[0], g * torch.sigmoid(1.702 * g) * (u + 1))
    assert torch.allclose(plain.silu_glu(x, tensors, "p")[0], x[0] * torch.sigmoid(x[0]) * x[0])


def test_the_position_vectors():
    rows = plain.sinusoid_rows([0, 3], 6)
    assert torch.allclose(rows[0], torch.tensor([0.0, 1.0, 0.0, 1.0, 0.0, 1.0]))
    rate = 10000.0 ** (-2.0 / 6)
    assert torch.allclose(rows[1, 2:4], torch.tensor([torch.sin(torch.tensor(3 * rate)), torch.cos(torch.tensor(3 * rate))]))
    from turboserve_amd.parts.ends import sinusoid_table
    assert torch.allclose(sinusoid_table(40, 7, 10000.0), plain.sinusoid_rows(range(40), 7), atol=1e-6)


def test_a_random_model_folder_is_written_and_read_back(tmp_path):
    from turboserve_amd.config.model_config import read_config_json
    from turboserve_amd.weights.random_init import write_random_model

    folder = write_random_model(st.CONFIG_Q, tmp_path / "model", seed=3, dtype=torch.bfloat16, std=0.05)
    assert parse_model_config(read_config_json(folder)) == parse_model_config(st.CONFIG_Q)
    config, tensors = st.read_model_dir(folder)
    _, model = describe_model(config)
    assert set(tensors) == set(model.tensor_specs())
    assert float(tensors["l0.norm1"].abs().max()) == 0.0 and float(tensors["l0.mix.q.norm"].min()) == 1.0
    logits = plain.forward(config, tensors, [5, 1, 96, 40])
    assert logits.shape == (4, 97) and bool(torch.isfinite(logits).all())


def test_a_loop_over_no_layers_reads_no_offsets(tmp_path):
    config = copy.deepcopy(st.CONFIG_Q)
    config["loop"] = {"start": 1, "stop": 1, "times": 2}
    _, model = describe_model(config)
    assert "loop.step" not in model.tensor_specs() and "loop.step" in model.ignorable_names()
    assert plain.run_order(config) == [(0, None), (1, None)]
    _, looped = describe_model(st.CONFIG_Q)
    assert "loop.step" in looped.tensor_specs() and "loop.step" not in looped.ignorable_names()
