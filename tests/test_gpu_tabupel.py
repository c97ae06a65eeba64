"""Tabupel on the GPU: every kernel against the plain implementation's function for its mechanism, the mixers as
parts with a cache or a state of their own, and the engine (whole prompts, token-by-token decoding, portions down to
two tokens, unequal requests together in a tight pool, long decoding, recorded decode steps, greedy generation
through the scheduler, the trace runner as a child process) against the plain implementation, in 32-bit and in
bfloat16."""
import pytest
import torch

import plain_tabupel as plain
import tabupel_cases as cases
import tabupel_mechanisms as mech
from simply_amd.engine import StepEntry
from simply_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(autouse=True)
def _lib(gpu_lib):
    return gpu_lib


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("body", [mech.residual_add_next_norm, mech.norm_rotation_and_pages, mech.latent_rows_and_pages,
                                  mech.differential_attention_edges, mech.latent_attention_edges, mech.head_product,
                                  mech.short_convolution, mech.recurrence, mech.recurrence_of_unequal_requests])
def test_kernel(body, dtype):
    body(ops, DEV, dtype)


def test_kernels_on_pages_of_sixteen_keys():
    """Pages of 16 keys whose rows are a multiple of 32 entries are stored in operand blocks: the same tests in that
    layout, with windows and page borders that do not coincide."""
    mech.norm_rotation_and_pages(ops, DEV, torch.bfloat16, page_size=16, sizes=(4, 2, 16, 8, 8))
    mech.latent_rows_and_pages(ops, DEV, torch.bfloat16, page_size=16, sizes=(3, 24, 8))
    for dtype in DTYPES:
        mech.differential_attention_edges(ops, DEV, dtype, page_size=16, sizes=(4, 2, 16, 12))
        mech.latent_attention_edges(ops, DEV, dtype, page_size=16, sizes=(3, 24, 8))


def test_many_heads_over_one_key_head():
    """More query vectors over one key head than a workgroup's LDS holds: the heads are cut over workgroups."""
    mech.latent_attention_edges(ops, DEV, torch.bfloat16, page_size=16, sizes=(40, 416, 32))
    mech.differential_attention_edges(ops, DEV, torch.float32, page_size=16, sizes=(18, 1, 512, 40))


@pytest.mark.parametrize("sizes, differential", [((8, 2, 64, 128), True), ((4, 4, 32, 16), True), ((3, 1, 96, 80), True),
                                                 ((16, 1, 160, 128), False), ((40, 1, 576, 512), False),
                                                 ((6, 2, 64, 64), False)])
def test_attention_units_on_the_matrix_cores(sizes, differential):
    mech.attention_units_on_the_matrix_cores(ops, DEV, sizes=sizes, differential=differential)


def test_attention_of_many_units_on_the_matrix_cores():
    """Launches with thousands of units, as a prompt's portion makes them: a wave takes a unit of its own."""
    mech.attention_units_on_the_matrix_cores(ops, DEV, sizes=(40, 1, 576, 512), differential=False, last=700)
    mech.attention_units_on_the_matrix_cores(ops, DEV, sizes=(40, 1, 576, 128), differential=False, last=700)
    mech.attention_units_on_the_matrix_cores(ops, DEV, sizes=(8, 2, 64, 128), n=2400, differential=True, last=2400)
    mech.attention_units_on_the_matrix_cores(ops, DEV, sizes=(6, 2, 32, 48), n=1500, window=33, differential=False, last=1400)


def test_recurrence_in_portions_and_other_taps():
    mech.recurrence(ops, DEV, torch.float32, cuts=(1, 2, 40, 1, 46))
    mech.recurrence(ops, DEV, torch.bfloat16, T=400, cuts=(100, 1, 129, 64, 2, 104), block=16)
    for n in (1, 2, 6):
        mech.short_convolution(ops, DEV, torch.float32, n=n)
    # long portions run in segments: lengths at, just above and far from multiples of a segment, beside a single token
    mech.recurrence_of_unequal_requests(ops, DEV, torch.float32, lengths=(1, 641, 192))
    mech.recurrence_of_unequal_requests(ops, DEV, torch.bfloat16, lengths=(130, 129, 1000))
    mech.recurrence(ops, DEV, torch.float32, T=1500, cuts=(700, 1, 799))


@pytest.mark.parametrize("dtype", DTYPES)
def test_differential_part(dtype):
    mech.differential_part(DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_latent_part(dtype):
    mech.latent_part(DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_rglru_part(dtype):
    mech.rglru_part(DEV, dtype)
    mech.rglru_part(DEV, dtype, sizes=(24, 16, 1, 1), length=9, cuts=([9], [2, 2, 2, 2, 1]))


def test_parts_at_aligned_sizes():
    """Sizes in multiples of 32 and 64 in pages of 16 keys, bfloat16, 300 tokens: whatever fast kernels the parts
    choose at such sizes, whole, decoding behind a long portion, and in portions of 17."""
    cuts = ([300], [268] + [1] * 32, [17] * 17 + [11])
    mech.differential_part(DEV, torch.bfloat16, sizes=(128, 4, 2, 64, 128), window=48, page_size=16, length=300, cuts=cuts)
    mech.latent_part(DEV, torch.bfloat16, sizes=(128, 4, 64, 32, 64, 96, 128), window=80, page_size=16, length=300,
                     cuts=cuts, std=0.1)
    mech.rglru_part(DEV, torch.bfloat16, sizes=(128, 128, 2, 4), length=300, cuts=cuts)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "only_rglru", "only_attention", "aligned"])
def test_cuts_match_plain(tmp_path, name, dtype):
    cases.cuts_match_plain(tmp_path, DEV, name, dtype, length=45 if name != "aligned" else 70)


def test_windows_are_exact(tmp_path):
    cases.windows_are_exact(tmp_path, DEV, "mixed", "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_match_plain(tmp_path, dtype):
    cases.layers_match_plain(tmp_path, DEV, "mixed", dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "only_rglru", "aligned"])
def test_batches_match_alone(tmp_path, name, dtype):
    cases.batches_match_alone(tmp_path, DEV, name, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "only_attention"])
def test_long_portions(tmp_path, name, dtype):
    """A prompt of 171 tokens: whole, in long portions, in portions of two tokens and token by token."""
    cases.cuts_match_plain(tmp_path, DEV, name, dtype, length=171)


def test_pages_of_sixteen_keys(tmp_path):
    cases.cuts_match_plain(tmp_path, DEV, "aligned", "bfloat16", length=70, page_size=16)
    cases.batches_match_alone(tmp_path / "b", DEV, "aligned", "bfloat16", page_size=16)
    cases.long_decoding(tmp_path / "l", DEV, "aligned", "bfloat16", steps=150, page_size=16)


@pytest.mark.parametrize("seed", range(12))
def test_drawn_configurations(tmp_path, seed):
    cases.drawn_configuration_runs(tmp_path, DEV, seed, "float32")


@pytest.mark.parametrize("seed", [0, 2, 4, 6, 8, 10])
def test_drawn_configurations_bfloat16(tmp_path, seed):
    cases.drawn_configuration_runs(tmp_path, DEV, seed, "bfloat16")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding(tmp_path, dtype):
    cases.long_decoding(tmp_path, DEV, "mixed", dtype, steps=150, page_size=16)


@pytest.mark.parametrize("name, dtype, page_size", [("mixed", "float32", 4), ("mixed", "bfloat16", 4),
                                                   ("aligned", "bfloat16", 16)])
def test_recorded_decode_steps(tmp_path, name, dtype, page_size):
    """Decode-only steps are recorded in a HIP graph and replayed: three requests decode together for 40 steps, and
    each step's logits are those of the same step run eagerly by a second engine (states advance exactly once).  With
    the aligned sizes in pages of 16 keys the attentions run on the matrix cores, their keys cut into ranges."""
    d = cases.write_model(name, str(tmp_path / "m"))
    V = plain.load(d)[1]["vocab"]
    prompts = {r: cases.random_tokens(n, V, 70 + n) for r, n in (("a", 9), ("b", 3), ("c", 14))}
    follow = {r: cases.random_tokens(40, V, 90 + len(p)) for r, p in prompts.items()}
    engines = [cases.make_executor(d, DEV, dtype, page_size=page_size, num_pages=64, batch=4, max_len=64, graphs=g)
               for g in (True, False)]
    for ex in engines:
        for r, p in prompts.items():
            ex.add_request(r)
        ex.step([StepEntry(r, p, []) for r, p in prompts.items()])
    for k in range(40):
        outs = [ex.step([StepEntry(r, [follow[r][k]], [0]) for r in prompts]).clone() for ex in engines]
        torch.testing.assert_close(outs[0], outs[1], rtol=0, atol=0)


def test_greedy_generation(tmp_path):
    cases.greedy_generation(tmp_path, DEV, "mixed", "float32")


def test_trace_replay_child_process(tmp_path):
    """bin/trace_run as a user starts it: a folder, steps on standard input, logits in files; two live requests."""
    import json
    import os
    import subprocess

    import numpy as np

    d = cases.write_model("mixed", str(tmp_path / "m"), dtype=torch.bfloat16)
    w, cfg = plain.load(d)
    tx, ty = cases.random_tokens(30, cfg["vocab"], 5), cases.random_tokens(12, cfg["vocab"], 6)
    wx, wy = plain.forward(w, cfg, tx), plain.forward(w, cfg, ty)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": tx[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": tx[17:19], "want": []}, {"id": "y", "tokens": ty[:11], "want": [10]}],
              "end": []},
             {"step": 2, "entries": [{"id": "y", "tokens": ty[11:], "want": [0]}, {"id": "x", "tokens": tx[19:], "want": [10]}],
              "end": ["x", "y"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", d, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                       capture_output=True, timeout=600)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    got = [torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(n, -1)) for i, n in ((0, 2), (1, 1), (2, 2))]
    assert cases.rel_error(got[0], wx[[0, 16]]) <= cases.BOUND["float32"]
    assert cases.rel_error(got[1], wy[[10]]) <= cases.BOUND["float32"]
    assert cases.rel_error(got[2], torch.stack([wy[11], wx[29]])) <= cases.BOUND["float32"]
