"""Tabupel on the CPU: configuration and weights, every mechanism's plain torch reference against the plain
implementation's function, and the framework's host logic (model, parts, cache and state manager, step function,
scheduler) with the kernels replaced by those references."""
import json

import pytest
import torch

import plain_tabupel as plain
import tabupel_cases as cases
import tabupel_mechanisms as mech
import torch_ops
from simply_amd.config import ConfigError, TabupelConfig, config_from_dict, load_config
from simply_amd.models import DecoderModel
from simply_amd.weights import WeightsError

CPU = "cpu"


# ------------------------------------------------------------------ configuration, registry, weights
def test_config_round_trip_and_spec():
    cfg = config_from_dict(cases.MIXED)
    assert isinstance(cfg, TabupelConfig) and config_from_dict(cfg.to_dict()) == cfg
    spec = cfg.model_spec()
    # layers that run with another layer's tensors have none of their own: four layers, six schedule entries
    assert [l.mixer.kind for l in spec.layers] == ["rglru", "differential_attention", "latent_attention", "latent_attention"]
    assert [e.layer for e in spec.schedule] == [0, 1, 2, 0, 1, 3]
    assert all(l.block.kind == "pre_norm" and l.block.params["mult"] == 0.6 for l in spec.layers)
    assert [l.feed_forward is not None for l in spec.layers] == [True, True, False, True]
    assert spec.head.params["soft_cap"] == 12.0
    rope = spec.layers[2].mixer.params["position_encoding"]
    assert rope.kind == "pair_rope" and rope.params["scaling"]["kind"] == "ramp"
    assert spec.layers[1].mixer.params["position_encoding"].params["scaling"] == {"kind": "linear", "factor": 4.0}
    assert spec.layers[3].mixer.params["position_encoding"].params["scaling"] is None
    model = DecoderModel(spec)
    names = model.expected_tensors()
    assert names["l0.mix.ra"].shape == (3, 12, 12) and names["l2.mix.uq"].shape == (3 * 20, 20)
    assert names["l1.mix.q"].shape == (6 * 2 * 10, 48) and names["l1.mix.k"].shape == (2 * 2 * 10, 48)
    assert "l3.norm1" not in names and "l4.mix.q" not in names and "l5.mix.dkv" in names and "l2.norm2" not in names
    needs = [n for n, _ in model.cache_needs()]
    assert needs[0].shape == (36 * 3,) and needs[3] == needs[0]
    assert (needs[1].num_kv_heads, needs[1].head_dim, needs[1].value_dim, needs[1].window) == (2, 20, 14, 7)
    # a latent attention keeps one row [latent | rotated part] per token and the latent once more as its value
    assert (needs[2].num_kv_heads, needs[2].head_dim, needs[2].value_dim, needs[2].window) == (1, 24 + 8, 24, 13)
    assert needs[5].window is None


@pytest.mark.parametrize("change, message", [
    (lambda d: d["layers"][0].update(type="conv"), "unknown layer type"),
    (lambda d: d["layers"][1]["mixer"].pop("scale"), "scale"),
    (lambda d: d["layers"][1]["mixer"].pop("diff"), "diff"),
    (lambda d: d["layers"][1]["mixer"].update(heads=3, kv_heads=2), "multiple"),
    (lambda d: d["layers"][1]["mixer"]["rot"].update(dims=7), "even"),
    (lambda d: d["layers"][2]["mixer"]["rot"]["scaling"].pop("fast"), "fast"),
    (lambda d: d["layers"][2]["mixer"].pop("q_rank"), "q_rank"),
    (lambda d: d["layers"][0]["mixer"].update(blocks=5), "blocks"),
    (lambda d: d["layers"][0]["mixer"].update(conv=0), "conv"),
    (lambda d: d["layers"][0]["mlp"].update(kind="routed"), "unknown kind"),
    (lambda d: d["layers"][3].update(weights_of=1), "another type"),
    (lambda d: d["layers"][3].update(weights_of=9), "names layer"),
    (lambda d: d.pop("residual_mult"), "residual_mult"),
    (lambda d: d["norm"].pop("eps"), "eps"),
])
def test_config_errors(change, message):
    d = json.loads(json.dumps(cases.MIXED))
    change(d)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(d)


def test_folder_round_trip_missing_tensor_and_rank_from_shapes(tmp_path):
    d = cases.write_model("mixed", str(tmp_path / "m"))
    assert load_config(d).model_spec() == config_from_dict(cases.MIXED).model_spec()
    from safetensors.torch import load_file, save_file
    from simply_amd.engine.loading import load_model

    # a folder that leaves the query latent's size to the tensor
    raw = json.load(open(f"{d}/config.json"))
    raw["layers"][2]["mixer"].pop("q_rank")
    json.dump(raw, open(f"{d}/config.json", "w"))
    assert load_config(d).model_spec().layers[2].mixer.params["q_rank"] == 20
    tensors = load_file(f"{d}/model.safetensors")
    tensors["l2.norm2"] = torch.zeros(48)        # (the norm of a feed-forward that layer 2 does not have: left unread)
    tensors.pop("l1.mix.lq2")
    tensors["l3.mix.lam"] = torch.zeros(36)       # (layer 3 runs with layer 0's tensors: it stores none)
    save_file(tensors, f"{d}/model.safetensors")
    with pytest.raises(WeightsError) as e:
        load_model(d, torch.float32, "cpu")
    assert e.value.missing == ["l1.mix.lq2"] and e.value.unexpected == ["l3.mix.lam"]


def test_frequencies_of_the_rotation():
    """The position encoding's frequencies against the plain functions, for no scaling, a constant and the ramp."""
    from simply_amd.parts.rope import PairRoPE

    close = torch.testing.assert_close
    close(PairRoPE(8, 500.0).freq_host().double(), plain.linear_frequencies(8, 500.0), rtol=1e-6, atol=0)
    close(PairRoPE(8, 1e6, {"kind": "linear", "factor": 8.0}).freq_host().double(), plain.linear_frequencies(8, 1e6, 8.0),
          rtol=1e-6, atol=0)
    for dims, base, f, orig, fast, slow in ((32, 20000.0, 2.0, 2048, 32.0, 1.0), (8, 1000.0, 3.0, 64, 8.0, 1.0),
                                            (6, 50.0, 2.0, 16, 4.0, 0.5), (4, 100.0, 4.0, 16, 32.0, 0.5)):
        pe = PairRoPE(dims, base, {"kind": "ramp", "factor": f, "original": orig, "fast": fast, "slow": slow})
        want, mult = plain.ramp_frequencies(dims, base, f, orig, fast, slow)
        close(pe.freq_host().double(), want, rtol=1e-6, atol=0)
        assert pe.mult == mult
    # the ramp really blends: neither all frequencies as they are nor all divided
    f, _ = plain.ramp_frequencies(32, 20000.0, 2.0, 2048, 32.0, 1.0)
    ratio = f / plain.linear_frequencies(32, 20000.0)
    assert float(ratio[0]) == 1.0 and float(ratio[-1]) == 0.5 and ((ratio > 0.5) & (ratio < 1.0)).any()


# ------------------------------------------------------------------ the references of the kernels, one by one
@pytest.mark.parametrize("body", [mech.residual_add_next_norm, mech.norm_rotation_and_pages, mech.latent_rows_and_pages,
                                  mech.differential_attention_edges, mech.latent_attention_edges, mech.head_product,
                                  mech.short_convolution, mech.recurrence, mech.recurrence_of_unequal_requests])
def test_reference_of_a_kernel(body):
    body(torch_ops, CPU, torch.float32)


def test_reference_of_the_recurrence_in_portions_and_other_taps():
    mech.recurrence(torch_ops, CPU, torch.float32, cuts=(1, 2, 40, 1, 46))
    for n in (1, 2, 6):
        mech.short_convolution(torch_ops, CPU, torch.float32, n=n)


def test_differential_part(cpu_ops):
    mech.differential_part(CPU, torch.float32)


def test_latent_part(cpu_ops):
    mech.latent_part(CPU, torch.float32)


def test_rglru_part(cpu_ops):
    mech.rglru_part(CPU, torch.float32)
    mech.rglru_part(CPU, torch.float32, sizes=(24, 16, 1, 1), length=9, cuts=([9], [2, 2, 2, 2, 1]))


# ------------------------------------------------------------------ the engine's host logic
@pytest.mark.parametrize("name", ["only_rglru", "only_attention"])
def test_cuts_match_plain(tmp_path, cpu_ops, name):
    cases.cuts_match_plain(tmp_path, CPU, name)


def test_cuts_match_plain_and_windows_are_exact(tmp_path, cpu_ops):
    cases.windows_are_exact(tmp_path, CPU, "mixed")


def test_layers_match_plain(tmp_path, cpu_ops):
    cases.layers_match_plain(tmp_path, CPU, "mixed")


@pytest.mark.parametrize("name", ["mixed", "only_rglru"])
def test_batches_match_alone(tmp_path, cpu_ops, name):
    cases.batches_match_alone(tmp_path, CPU, name)


@pytest.mark.parametrize("seed", range(6))
def test_drawn_configurations(tmp_path, cpu_ops, seed):
    config_from_dict(cases.drawn_config(seed))    # (every drawn configuration is a valid one)
    cases.drawn_configuration_runs(tmp_path, CPU, seed)


def test_long_decoding(tmp_path, cpu_ops):
    cases.long_decoding(tmp_path, CPU, "mixed", steps=70, page_size=4)


def test_greedy_generation(tmp_path, cpu_ops):
    cases.greedy_generation(tmp_path, CPU)


def test_plain_portions_of_the_recurrence_and_the_convolution():
    """The plain implementation itself: carried over a cut, the recurrence gives what it gives in one piece, and the
    convolution's first results see zeros before the start."""
    T, C = 12, 6
    u, lam = mech.rand((T, C), 1), mech.rand((C,), 2)
    r, i = torch.sigmoid(mech.rand((T, C), 3)), torch.sigmoid(mech.rand((T, C), 4))
    whole = plain.gated_linear_recurrence(u, r, i, lam)
    a = plain.gated_linear_recurrence(u[:5], r[:5], i[:5], lam)
    b = plain.gated_linear_recurrence(u[5:], r[5:], i[5:], lam, a[-1])
    torch.testing.assert_close(torch.cat([a, b]), whole)
    a0 = torch.exp(-8.0 * r[0] * plain.softplus(lam))
    torch.testing.assert_close(whole[0], torch.sqrt(1 - a0 * a0) * i[0] * u[0])     # from S = 0, no special case
    x, taps, bias = mech.rand((9, 4), 6), mech.rand((4, 3), 7), mech.rand((4,), 8)
    y = plain.causal_conv(x, taps, bias)
    torch.testing.assert_close(y[0], x[0] * taps[:, 2] + bias)
    torch.testing.assert_close(y[4], x[4] * taps[:, 2] + x[3] * taps[:, 1] + x[2] * taps[:, 0] + bias)
