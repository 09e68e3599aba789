"""The Melizen configuration: its reader, the run order it makes of a loop, and the tensors it expects."""
import copy

import pytest

import gpullama3_java_amd as g
from gpullama3_java_amd.config import ConfigError
from gpullama3_java_amd.parts.model import expected_tensors
from melizen_models import CONFIGS, LOOPED, LOOP_AT_END, STRAIGHT
import plain_melizen as P


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_expected_tensors_are_the_design_s(name):
    cfg = g.config_from_dict(CONFIGS[name])
    want = P.tensor_shapes(CONFIGS[name])
    got = {k: tuple(v.shape) for k, v in expected_tensors(cfg.model_spec()).items()}
    assert got == want


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_round_trip(name):
    cfg = g.config_from_dict(CONFIGS[name])
    assert g.config_from_dict(cfg.to_dict()) == cfg
    assert cfg.max_position_embeddings == CONFIGS[name]["max_positions"]
    short = cfg.with_context_length(100)
    assert short.max_position_embeddings == 100
    # the table of positions keeps its stored size whatever the run's context
    assert short.model_spec().max_positions == CONFIGS[name]["max_positions"]


def test_run_order_of_a_loop():
    spec = g.config_from_dict(LOOPED).model_spec()
    assert [r.layer for r in spec.run_order] == [0, 1, 0, 1, 0, 1, 2, 3]
    assert [(r.before.row, r.before.embedding) if r.before else None for r in spec.run_order] == [
        (0, False), None, (1, True), None, (2, True), None, None, None]
    spec = g.config_from_dict(LOOP_AT_END).model_spec()
    assert [r.layer for r in spec.run_order] == [0, 1, 2, 1, 2]
    assert [r.before.row if r.before else None for r in spec.run_order] == [None, 0, None, 1, None]
    spec = g.config_from_dict(STRAIGHT).model_spec()
    assert [r.layer for r in spec.run_order] == [0, 1, 2, 3] and all(r.before is None for r in spec.run_order)
    assert [(l, t) for l, t in P.run_order(LOOPED)] == [(0, 0), (1, None), (0, 1), (1, None), (0, 2), (1, None), (2, None), (3, None)]


def test_what_the_description_carries():
    spec = g.config_from_dict(LOOPED).model_spec()
    delta, attn = spec.layers[0], spec.layers[1]
    assert delta.kind == attn.kind == "parallel" and delta.ffn_norm is None
    assert delta.mixer_norm.weight_offset == 1.0 and spec.final_norm.weight_offset == 1.0
    assert (delta.mixer.kind, delta.mixer.n_heads, delta.mixer.n_kv_heads, delta.mixer.key_dim, delta.mixer.value_dim,
            delta.mixer.conv_taps) == ("gated_delta", 4, 2, 32, 48, 3)
    assert (attn.mixer.n_heads, attn.mixer.n_kv_heads, attn.mixer.head_dim, attn.mixer.v_head_dim, attn.mixer.window,
            attn.mixer.scale, attn.mixer.sink, attn.mixer.position) == (6, 2, 32, 48, 40, 0.2, 0.0, None)
    assert attn.mixer.distance_bias.slopes(4) == [2.0 ** -2, 2.0 ** -4, 2.0 ** -6, 2.0 ** -8]
    assert (attn.ffn.activation, attn.ffn.limit, attn.ffn.up_shift, attn.ffn.intermediate) == ("quick_gelu", 3.0, 1.0, 128)
    assert spec.layers[2].ffn is None and spec.position_table_name == "pos" and spec.head_name == "head"
    assert g.config_from_dict(STRAIGHT).model_spec().layers[0].mixer.window is None


@pytest.mark.parametrize("change, key", [
    (lambda d: d.pop("width"), "width"),
    (lambda d: d["layers"][0].update(type="conv"), "type"),
    (lambda d: d["layers"][1]["mixer"].update(kv_heads=4), "kv_heads"),
    (lambda d: d["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda d: d["layers"][0]["mixer"].pop("conv"), "conv"),
    (lambda d: d["layers"][0]["mlp"].update(kind="routed"), "mlp"),
    (lambda d: d["loop"].update(stop=9), "loop"),
    (lambda d: d.update(norm=None), "norm"),
])
def test_errors_name_the_key(change, key):
    d = copy.deepcopy(LOOPED)
    change(d)
    with pytest.raises(ConfigError, match=key):
        g.config_from_dict(d)


def test_registered_by_the_folder_s_own_key():
    assert "Melizen" in g.registered_architectures()
    with pytest.raises(ConfigError, match="unknown architecture"):
        g.config_from_dict({**LOOPED, "architecture": "Nobody"})
