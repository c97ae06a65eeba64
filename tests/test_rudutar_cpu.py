"""Rudutar on the CPU: configuration and weights, every mechanism's plain torch reference against the plain
implementation's function, and the framework's host logic (model, parts, cache and state manager, step function,
scheduler) with the kernels replaced by those references."""
import copy

import pytest
import torch

import rudutar_cases as cases
import rudutar_mechanisms as mech
import torch_ops
from simply_amd.cache.manager import CacheError, CacheManager
from simply_amd.config import ConfigError, RudutarConfig, config_from_dict
from simply_amd.models import DecoderModel
from simply_amd.parts.base import CompositeNeed, PagedKVNeed, StateNeed

CPU = "cpu"


# ------------------------------------------------------------------ configuration, registry, cache needs
def test_config_round_trip_and_spec():
    cfg = config_from_dict(cases.MIXED)
    assert isinstance(cfg, RudutarConfig) and config_from_dict(cfg.to_dict()) == cfg
    spec = cfg.model_spec()
    assert all(l.mixer.kind == "gated_attention" and l.block.kind == "pre_norm" for l in spec.layers)
    assert [e.cache_from for e in spec.schedule] == [None, 0, None, 0, None, None]
    assert [None if l.feed_forward is None else l.feed_forward.kind for l in spec.layers] == \
        ["dense", "routed_experts", "routed_experts", None, "dense", "routed_experts"]
    assert spec.embedding.kind == "normed_embedding" and spec.head.params["soft_cap"] is None
    first, reader, second = (spec.layers[i].mixer.params for i in (0, 1, 2))
    # the layer whose pages others read keeps them for the longest of their windows
    assert (first["window"], first["cache_window"], reader["window"], reader["cache_window"]) == (7, 11, 11, 11)
    assert first["qk_norm"] == "head" and first["zero_sink"] and first["slope_exponent"] == 8.0 and first["conv_taps"] == 3
    assert reader["own_keys_values"] is False and reader["conv_taps"] == 2
    assert second["qk_norm"] == "row" and second["values"] == "keys" and second["output_gate"] == "head" and second["bias"]
    assert second["position_encoding"].kind == "partial_rope" and second["position_encoding"].params["dims"] == 6
    moe = spec.layers[1].feed_forward.params
    assert (moe["num_experts"], moe["top"], moe["num_groups"], moe["keep_groups"], moe["gated"], moe["router"]) == \
        (6, 2, 3, 2, False, "sigmoid")
    model = DecoderModel(spec)
    names = model.expected_tensors()
    assert names["l0.mix.q.conv"].shape == (60, 3) and names["l0.mix.v.conv"].shape == (28, 3)
    assert names["l2.mix.g"].shape == (4, 48) and names["l2.mix.q.norm"].shape == (48,) and names["l2.mix.k.b"].shape == (24,)
    assert names["l1.mlp.correction"].shape == (6,) and names["l1.mlp.shared.up"].shape == (24, 48)
    for absent in ("l1.mix.k", "l1.mix.v.conv", "l3.mix.q.conv", "l2.mix.v", "l3.norm2", "l2.mlp.shared.up", "l1.mlp.e0.gate"):
        assert absent not in names
    needs = [n for n, _ in model.cache_needs()]
    assert needs[0] == CompositeNeed((PagedKVNeed(2, 10, 11, 14), StateNeed((2 * (60 + 20 + 28),))))
    assert needs[1] == CompositeNeed((PagedKVNeed(2, 10, 11, 14), StateNeed((60,))))
    assert needs[3] == PagedKVNeed(2, 10, 11, 14) and needs[2] == PagedKVNeed(2, 12, 13, 12)


@pytest.mark.parametrize("change, message", [
    (lambda d: d["layers"][0].update(type="conv"), "unknown layer type"),
    (lambda d: d["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda d: d["layers"][0]["mixer"].update(heads=5), "multiple"),
    (lambda d: d["layers"][0]["mixer"].update(conv=0), "conv"),
    (lambda d: d["layers"][0]["mixer"]["q_temp"].update(every=0), "every"),
    (lambda d: d["layers"][1]["mixer"].update(kv_from=3), "does not run before"),
    (lambda d: d["layers"][3]["mixer"].update(kv_from=1), "keeps no keys"),
    (lambda d: d["layers"][3]["mixer"].update(kv_from=2), "keeps no keys"),
    (lambda d: d["layers"][1]["mixer"].update(dim=12), "differs"),
    (lambda d: d["layers"][2]["mixer"].update(kv_from=0), "belongs to"),
    (lambda d: d["layers"][2]["mixer"].update(vdim=10), "vdim"),
    (lambda d: d["layers"][2]["mixer"]["rot"].update(dims=7), "even"),
    (lambda d: d["layers"][0]["mlp"].update(kind="routed"), "unknown kind"),
    (lambda d: d["layers"][1]["mlp"]["router"].update(top=5), "choices"),
    (lambda d: d["layers"][1]["mlp"]["router"]["groups"].update(count=4), "choices"),
    (lambda d: d["layers"][1]["mlp"].pop("expert"), "expert"),
    (lambda d: d.pop("norm"), "norm"),
])
def test_config_errors(change, message):
    d = copy.deepcopy(cases.MIXED)
    change(d)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(d)


def test_what_is_absent_does_not_exist():
    d = cases.config(50, 16, 1e-6, [cases.first(2, 1, 4, 6, 0.5), cases.second(2, 2, 4, 0.5)])
    spec = config_from_dict(d).model_spec()
    a, b = spec.layers[0].mixer.params, spec.layers[1].mixer.params
    assert a["window"] is None and a["cache_window"] is None and a["conv_taps"] == 0 and a["query_temperature"] is None
    assert b["position_encoding"] is None and b["window"] is None
    names = DecoderModel(spec).expected_tensors()
    assert "l0.mix.q.conv" not in names and "l0.norm2" not in names


def test_pages_read_from_another_entry_beside_a_state_of_ones_own():
    """A need of pages and a state that reads another entry: the pages are that entry's (read-only), the state is the
    reader's own and is zeroed at admission; pages that differ are refused."""
    pages, other = PagedKVNeed(2, 8, 5, 6), PagedKVNeed(2, 8, 7, 6)
    needs = [(CompositeNeed((pages, StateNeed((12,)))), None), (CompositeNeed((pages, StateNeed((4,)))), 0), (pages, 0)]
    cm = CacheManager(needs, page_size=4, num_pages=8, num_slots=2, max_seq_len=32, dtype=torch.float32, device=CPU)
    src, reader, plain_reader = cm.views
    assert reader.parts[0].pages["k"] is src.parts[0].pages["k"] and not reader.parts[0].write and reader.parts[1].write
    assert reader.parts[1].state.shape == (2, 4) and plain_reader.pages["v"] is src.parts[0].pages["v"]
    assert len(cm.groups) == 1
    reader.parts[1].state.fill_(3.0)
    slot = cm.admit("r")
    assert float(reader.parts[1].state[slot].abs().sum()) == 0.0
    with pytest.raises(CacheError, match="keeps none like"):
        CacheManager([needs[0], (CompositeNeed((other, StateNeed((4,)))), 0)], page_size=4, num_pages=8, num_slots=2,
                     max_seq_len=32, dtype=torch.float32, device=None)


# ------------------------------------------------------------------ mechanisms: the references against the plain functions
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("body", [mech.inputs_of_the_first_kind, mech.inputs_of_the_second_kind, mech.attention_edges,
                                  mech.gate_per_head, mech.experts_without_gate])
def test_reference_of_a_kernel(body, dtype):
    body(torch_ops, CPU, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_normed_embedding(cpu_ops, dtype):
    mech.normed_embedding(CPU, dtype)


def test_router_reference():
    mech.router_choice(torch_ops, CPU)


def test_inputs_with_other_taps():
    for taps in (0, 1, 2, 7):
        mech.inputs_of_the_first_kind(torch_ops, CPU, torch.float32, taps=taps)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_parts(cpu_ops, dtype):
    mech.first_kind_part(CPU, dtype)
    mech.second_kind_part(CPU, dtype)


# ------------------------------------------------------------------ the engine's host logic
@pytest.mark.parametrize("name", ["mixed", "only_first", "only_second"])
def test_cuts_match_plain(cpu_ops, tmp_path, name):
    cases.cuts_match_plain(tmp_path, CPU, name, "float32")


def test_windows_are_exact(cpu_ops, tmp_path):
    cases.windows_are_exact(tmp_path, CPU, "mixed", "float32")


def test_layers_match_plain(cpu_ops, tmp_path):
    cases.layers_match_plain(tmp_path, CPU, "mixed", "float32")


@pytest.mark.parametrize("name", ["mixed", "only_first"])
def test_batches_match_alone(cpu_ops, tmp_path, name):
    cases.batches_match_alone(tmp_path, CPU, name, "float32")


def test_bfloat16_run(cpu_ops, tmp_path):
    cases.cuts_match_plain(tmp_path, CPU, "only_second", "bfloat16", length=40)


@pytest.mark.parametrize("seed", range(4))
def test_drawn_configurations(cpu_ops, tmp_path, seed):
    cases.drawn_configuration_runs(tmp_path, CPU, seed, "float32")


def test_long_decoding(cpu_ops, tmp_path):
    cases.long_decoding(tmp_path, CPU, "mixed", "float32", steps=60, page_size=16)


def test_greedy_generation(cpu_ops, tmp_path):
    cases.greedy_generation(tmp_path, CPU, "mixed", "float32")
