"""Rudutar on the GPU: every kernel against the plain implementation's function for its mechanism, the mixers as
parts with a cache of their own, and the engine (whole prompts, token-by-token decoding, portions down to two tokens,
unequal requests together in a tight pool, long decoding, recorded decode steps, greedy generation through the
scheduler, the trace runner as a child process) against the plain implementation, in 32-bit and in bfloat16."""
import pytest
import torch

import plain_rudutar as plain
import rudutar_cases as cases
import rudutar_mechanisms as mech
from simply_amd.engine import StepEntry
from simply_amd.kernels import ops

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


@pytest.fixture(autouse=True)
def _lib(gpu_lib):
    return gpu_lib


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("body", [mech.inputs_of_the_first_kind, mech.inputs_of_the_second_kind, mech.attention_edges,
                                  mech.gate_per_head, mech.experts_without_gate])
def test_kernel(body, dtype):
    body(ops, DEV, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_normed_embedding(dtype):
    mech.normed_embedding(DEV, dtype)


def test_router():
    mech.router_choice(ops, DEV)
    mech.router_choice(ops, DEV, torch.bfloat16)    # (a correction stored in bfloat16)


def test_kernels_with_other_sizes():
    """No convolution, one tap (a factor per channel), two and seven; pages of 16 keys whose rows are a multiple of 32
    entries (stored in operand blocks); more heads over a key head than a workgroup holds; a single head."""
    for taps in (0, 1, 2, 7):
        mech.inputs_of_the_first_kind(ops, DEV, torch.float32, taps=taps)
    for dtype in DTYPES:
        mech.inputs_of_the_first_kind(ops, DEV, dtype, page_size=16, sizes=(4, 2, 32, 16))
        mech.inputs_of_the_second_kind(ops, DEV, dtype, page_size=16, sizes=(4, 4, 64), rot=(64, 10000.0), start=1000)
        mech.inputs_of_the_second_kind(ops, DEV, dtype, page_size=4, sizes=(1, 1, 6), rot=(0, 1.0), start=0)
        mech.attention_edges(ops, DEV, dtype, page_size=16, sizes=(4, 2, 32, 12), sharp=False)
        mech.attention_edges(ops, DEV, dtype, page_size=16, sizes=(1, 1, 6, 40), window=64, sharp=False)
    mech.attention_edges(ops, DEV, torch.float32, page_size=16, sizes=(18, 1, 512, 40), sharp=False)
    mech.inputs_of_the_first_kind(ops, DEV, torch.bfloat16, page_size=16, sizes=(32, 8, 128, 128))


@pytest.mark.parametrize("sizes", [(8, 2, 64, 64), (4, 4, 128, 128), (16, 1, 64, 64), (2, 1, 256, 256)])
def test_attention_on_the_matrix_cores(sizes):
    mech.attention_on_the_matrix_cores(ops, DEV, sizes=sizes)
    mech.attention_on_the_matrix_cores(ops, DEV, sizes=sizes, n=1500, window=None, last=32)


@pytest.mark.parametrize("dtype", DTYPES)
def test_parts(dtype):
    mech.first_kind_part(DEV, dtype)
    mech.second_kind_part(DEV, dtype)


def test_parts_at_aligned_sizes():
    """Sizes in multiples of 64 in pages of 16 keys, bfloat16, 300 tokens: the matrix-core kernels, whole, decoding
    behind a long portion, and in portions of 17."""
    cuts = ([300], [268] + [1] * 32, [17] * 17 + [11])
    mech.first_kind_part(DEV, torch.bfloat16, sizes=(128, 4, 2, 64, 64), window=48, taps=4, temp=(0.3, 16), page_size=16,
                         length=300, cuts=cuts, std=0.1)
    mech.second_kind_part(DEV, torch.bfloat16, sizes=(128, 4, 2, 128), window=80, rot=(64, 10000.0), page_size=16,
                          length=300, cuts=cuts, std=0.1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "only_first", "only_second", "aligned"])
def test_cuts_match_plain(tmp_path, name, dtype):
    cases.cuts_match_plain(tmp_path, DEV, name, dtype, length=45 if name != "aligned" else 70)


def test_windows_are_exact(tmp_path):
    cases.windows_are_exact(tmp_path, DEV, "mixed", "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layers_match_plain(tmp_path, dtype):
    cases.layers_match_plain(tmp_path, DEV, "mixed", dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "only_first", "aligned"])
def test_batches_match_alone(tmp_path, name, dtype):
    cases.batches_match_alone(tmp_path, DEV, name, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "only_second"])
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
    each step's logits are those of the same step run eagerly by a second engine (tails advance exactly once).  With
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
