"""Small Tabupel configurations, model folders with random weights, and the bodies of the tests that run the
framework against the plain implementation (tests/plain_tabupel.py).  A body takes the device; the CPU tests run it
with the kernels replaced by their plain torch references (the `cpu_ops` fixture), the GPU tests with the kernels
themselves.  Nothing here is read from outside the repository."""
from __future__ import annotations

import copy

import torch

import plain_tabupel as plain
from simply_amd.config import config_from_dict
from simply_amd.engine import StepEntry
from simply_amd.weights import write_random_model
from zenuzen_cases import (BOUND, make_executor, mixer_cache, one_request_ctx, random_tokens, rel_error,  # noqa: F401
                           run_cut, run_mixer)

#: bound on the average over a request's positions of the row error (as `zenuzen_cases.assert_close_logits` has it).
#: The bfloat16 figure is what these tiny models do to rounding alone: the kernels' plain torch references, run on the
#: CPU with bfloat16 roundings at the same places, are 0.043 off on average on the worst request of `MIXED` (0.087 at
#: its worst position), as the kernels are, position for position.  Faults of the logic show in 32-bit.
MEAN_BOUND = {"float32": 1e-4, "bfloat16": 6e-2}


def assert_close_logits(got: torch.Tensor, want: torch.Tensor, dtype: str, what=None) -> None:
    got, want = got.double().cpu(), want.double().cpu()
    assert torch.isfinite(got).all(), what
    rows = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()
    over = int((rows > BOUND[dtype]).sum())
    allowed = 0 if dtype == "float32" else max(1, len(rows) // 20)
    assert over <= allowed and float(rows.mean()) <= MEAN_BOUND[dtype], (what, over, float(rows.max()), float(rows.mean()))


def rot(dims, base, factor=None, ramp=None):
    r = {"dims": dims, "base": base}
    if ramp is not None:
        r["scaling"] = {"factor": factor, "original": ramp[0], "fast": ramp[1], "slow": ramp[2]}
    elif factor is not None:
        r["scaling"] = {"factor": factor}
    return r


def _mlp(ff):
    return None if ff is None else {"kind": "dense", "ff": ff}


def attention(heads, kv_heads, dim, vdim, scale, diff, window=None, rot=None, mlp=None, weights_of=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if window:
        m["mask"] = {"size": window}
    if rot:
        m["rot"] = rot
    l = {"type": "attention", "mixer": m, "mlp": _mlp(mlp)}
    if weights_of is not None:
        l["weights_of"] = weights_of
    return l


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, window=None, rot=None, mlp=None, weights_of=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if rot:
        m["rot"] = rot
    l = {"type": "latent_attention", "mixer": m, "mlp": _mlp(mlp)}
    if weights_of is not None:
        l["weights_of"] = weights_of
    return l


def rglru(width, blocks, conv, mlp=None, weights_of=None):
    l = {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}, "mlp": _mlp(mlp)}
    if weights_of is not None:
        l["weights_of"] = weights_of
    return l


def config(vocab, width, mult, eps, layers, cap=None):
    d = {"architecture": "Tabupel", "vocab": vocab, "width": width, "residual_mult": mult, "norm": {"eps": eps},
         "layers": layers}
    if cap is not None:
        d["logit_softcap"] = cap
    return d


#: odd sizes everywhere: windows shorter than the prompts, two key heads under six heads, values of a size of their
#: own, a latent attention whose three sizes differ, three blocks of gates, layers that run with another layer's
#: tensors (a recurrent one and an attention one: each needs a state or cache of its own), a layer without a
#: feed-forward, both kinds of frequency scaling
MIXED = config(97, 48, 0.6, 1e-5, [
    rglru(36, 3, 3, mlp=56),
    attention(6, 2, 10, 14, 0.33, 0.25, window=7, rot=rot(6, 500.0, factor=4.0), mlp=40),
    latent(3, 12, 8, 10, 20, 24, 0.3, window=13, rot=rot(8, 1000.0, factor=3.0, ramp=(64, 8.0, 1.0))),
    rglru(36, 3, 3, mlp=56, weights_of=0),
    attention(6, 2, 10, 14, 0.33, 0.25, window=7, rot=rot(6, 500.0, factor=4.0), mlp=40, weights_of=1),
    latent(2, 6, 4, 16, 9, 11, 0.5, rot=rot(4, 100.0), mlp=32),
], cap=12.0)
#: only recurrent layers: one block of gates, a single tap (no convolution state at all), five taps; no cap, m = 1
ONLY_RGLRU = config(61, 32, 1.0, 1e-6, [rglru(24, 1, 1, mlp=40), rglru(40, 4, 5), rglru(24, 1, 1, mlp=40, weights_of=0)])
#: only attention layers: as many key heads as heads, one head, no window, no rotation, rotation of everything,
#: a window of one token
ONLY_ATTENTION = config(70, 40, 0.8, 1e-5, [
    attention(4, 4, 8, 6, 0.5, 0.1, rot=rot(8, 100.0), mlp=30),
    latent(1, 8, 6, 8, 12, 10, 0.35, window=5, rot=rot(6, 50.0, factor=2.0, ramp=(16, 4.0, 0.5))),
    attention(1, 1, 12, 20, 0.3, 0.5, window=1),
    latent(4, 4, 2, 6, 8, 8, 0.6, window=1, mlp=24),
    attention(3, 1, 6, 9, 0.4, 0.35, window=40, rot=rot(2, 10.0, factor=8.0)),
], cap=30.0)
#: sizes in multiples of 32 and 64 (what fast kernels may take), still small
ALIGNED = config(256, 128, 0.7, 1e-5, [
    rglru(128, 2, 4, mlp=256),
    attention(4, 2, 64, 128, 0.125, 0.3, window=48, rot=rot(32, 1000000.0, factor=8.0), mlp=256),
    latent(4, 64, 32, 64, 96, 128, 0.1, window=80, rot=rot(32, 10000.0, factor=2.0, ramp=(64, 32.0, 1.0))),
    rglru(128, 2, 4, mlp=256, weights_of=0),
    attention(8, 1, 32, 64, 0.18, 0.2, rot=rot(32, 10000.0)),
], cap=15.0)
CONFIGS = {"mixed": (MIXED, 11), "only_rglru": (ONLY_RGLRU, 12), "only_attention": (ONLY_ATTENTION, 13),
           "aligned": (ALIGNED, 14)}


def drawn_config(seed: int) -> dict:
    """A configuration drawn at random: sizes, head counts, the order of the layers, which layers have a
    feed-forward, which run with another layer's tensors, windows, rotations and their scaling, taps, multiplier,
    eps and cap."""
    import random

    r = random.Random(1000 + seed)
    width = r.choice([24, 40, 56, 64, 96])

    def a_rot(most):
        if r.random() < 0.2:
            return None
        dims = r.choice([2, 4, most - most % 2])
        kind = r.random()
        if kind < 0.35:
            return rot(dims, r.choice([100.0, 10000.0, 1e6]))
        if kind < 0.7:
            return rot(dims, r.choice([100.0, 10000.0]), factor=r.choice([2.0, 8.0]))
        return rot(dims, r.choice([100.0, 20000.0]), factor=r.choice([2.0, 4.0]), ramp=(r.choice([16, 64, 2048]), r.choice([8.0, 32.0]), r.choice([0.5, 1.0])))

    layers = []
    for i in range(r.randint(2, 6)):
        mlp = r.choice([None, r.choice([32, 48, 100]), r.choice([32, 48, 100])])
        window = r.choice([None, 1, 3, 8, 17, 30])
        again = [j for j, l in enumerate(layers) if "weights_of" not in l]
        if again and r.random() < 0.25:
            j = r.choice(again)
            layers.append({**copy.deepcopy(layers[j]), "weights_of": j})
            continue
        kind = r.random()
        if kind < 0.33:
            kv, dim = r.choice([1, 2, 3]), r.choice([4, 8, 12, 16, 32])
            layers.append(attention(kv * r.choice([1, 2, 3]), kv, dim, r.choice([4, 8, 16, 24, 2 * dim]),
                                    r.choice([0.2, 0.5, dim ** -0.5]), r.choice([0.1, 0.3, 0.6]), window=window,
                                    rot=a_rot(dim), mlp=mlp))
        elif kind < 0.66:
            rd = r.choice([2, 4, 8, 16])
            layers.append(latent(r.choice([1, 2, 4, 5]), r.choice([4, 8, 12, 24]), rd, r.choice([4, 8, 20]),
                                 r.choice([6, 16, 40]), r.choice([8, 16, 36]), r.choice([0.2, 0.4]), window=window,
                                 rot=a_rot(rd), mlp=mlp))
        else:
            blocks = r.choice([1, 2, 3, 4])
            layers.append(rglru(blocks * r.choice([4, 8, 20]), blocks, r.choice([1, 2, 3, 4, 6]), mlp=mlp))
    return config(r.choice([50, 97, 130, 300]), width, r.choice([0.3, 0.7, 1.0, 1.4]), r.choice([1e-6, 1e-5, 1e-3]), layers,
                  cap=r.choice([None, 10.0, 30.0]))


def write_model(name: str, out_dir: str, dtype=torch.float32, std: float = 0.25, norm_std: float = 0.5) -> str:
    """Writes the configuration with random weights through the framework's random-weights mode.  Norm weights,
    biases and decays are drawn around 0 with norm_std."""
    d, seed = CONFIGS[name]
    return write_random_model(config_from_dict(d), out_dir, seed, dtype, std=std, norm_std=norm_std)


def plain_weights(model_dir, dtype):
    """The folder's weights as the engine holds them: a bfloat16 run rounds them first."""
    w, cfg = plain.load(model_dir)
    if dtype == "bfloat16":
        w = {k: (v.to(torch.bfloat16) if v.is_floating_point() else v) for k, v in w.items()}
    return w, cfg


# --------------------------------------------------------------------------- bodies


def cuts_match_plain(tmp_path, device, name, dtype="float32", length=45, page_size=4):
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    tokens = random_tokens(length, cfg["vocab"], 7)
    want = plain.forward(w, cfg, tokens)
    ex = make_executor(d, device, dtype, page_size=page_size)
    n = length
    for cuts in ([n], [n - 32] + [1] * 32, [7, 5, 3, 2, 11, 2, 2, n - 32], [2] * (n // 2) + [1] * (n % 2), [1] * n):
        got = run_cut(ex, "r", tokens, cuts)
        assert_close_logits(got, want, dtype, (name, cuts))
    return got, want, cfg, w, tokens


def windows_are_exact(tmp_path, device, name="mixed", dtype="float32"):
    """The test above would notice a window that is one token off: the plain implementation with every window one
    token longer, and one token shorter, is further from the engine than the bound by orders of magnitude."""
    got, want, cfg, w, tokens = cuts_match_plain(tmp_path, device, name, dtype)
    for delta in (1, -1):
        other = copy.deepcopy(cfg)
        for l in other["layers"]:
            if (l["mixer"].get("mask") or {}).get("size", 0) + delta >= 1 and l["mixer"].get("mask"):
                l["mixer"]["mask"]["size"] += delta
        off = plain.forward(w, other, tokens)
        assert rel_error(got, off) > 100 * BOUND[dtype], delta


def layers_match_plain(tmp_path, device, name="mixed", dtype="float32", length=21):
    """The residual stream behind every layer run against the plain implementation's."""
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    tokens = random_tokens(length, cfg["vocab"], 9)
    want: list = []
    plain.forward(w, cfg, tokens, layers_out=want)
    ex = make_executor(d, device, dtype, page_size=4)
    ex.add_request("r")
    T, R, ctx, rows, wants, _ = ex._prepare([StepEntry("r", tokens, [length - 1])])
    got: list = []
    ex.model.forward(ex._dev[:T], ctx, ex.cache.views, rows, after_layer=lambda i, h: got.append(h.double().cpu().clone()))
    assert len(got) == len(want) == len(cfg["layers"])
    for i, h in enumerate(want):
        err = float((got[i] - h).abs().max() / h.abs().max())
        assert err <= (2e-5 if dtype == "float32" else 1e-1), (i, cfg["layers"][i]["type"], err)


def batches_match_alone(tmp_path, device, name, dtype="float32", page_size=4):
    """Requests of unequal length run together, portions beside single tokens, in a pool so tight that pages and
    state slots are given back and used again (freed pages are filled with NaN): each request's logits are those of
    the request alone."""
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    V = cfg["vocab"]
    lengths = {"a": 37, "b": 9, "c": 1, "d": 22, "e": 30, "f": 2, "g": 17}
    toks = {r: random_tokens(n, V, 100 + i) for i, (r, n) in enumerate(lengths.items())}
    want = {r: plain.forward(w, cfg, t) for r, t in toks.items()}
    ex = make_executor(d, device, dtype, page_size=page_size, num_pages=26 if page_size == 4 else 8, batch=3, max_len=48,
                       poison=True)
    schedule = [
        [("a", 11), ("b", 3), ("c", 1)],          # c ends: its slot goes to d
        [("a", 2), ("b", 1), ("d", 5)],
        [("a", 1), ("b", 5), ("d", 1)],           # b ends
        [("a", 16), ("d", 2), ("e", 7)],
        [("a", 1), ("d", 1), ("e", 2)],
        [("d", 13), ("e", 1), ("a", 6)],          # a and d end
        [("e", 20), ("f", 2), ("g", 1)],          # e and f end
        [("g", 2)], [("g", 14)],
    ]
    run_schedule(ex, schedule, toks, want, dtype, name)


def run_schedule(ex, schedule, toks, want, dtype, what):
    done = {r: 0 for r in toks}
    got = {r: [] for r in toks}
    for step in schedule:
        entries = []
        for r, n in step:
            if not ex.has_request(r):
                ex.add_request(r)
            entries.append(StepEntry(r, toks[r][done[r]:done[r] + n], list(range(n))))
        logits = ex.step(entries).cpu()
        at = 0
        for r, n in step:
            got[r].append(logits[at:at + n])
            at += n
            done[r] += n
            if done[r] == len(toks[r]):
                ex.finish_request(r)
        ex.cache.check()
    for r in toks:
        assert done[r] == len(toks[r])
        assert_close_logits(torch.cat(got[r]), want[r], dtype, (what, r))


def drawn_configuration_runs(tmp_path, device, seed: int, dtype="float32"):
    """A drawn configuration, three requests of unequal length in portions beside single tokens, in a tight pool."""
    d = write_random_model(config_from_dict(drawn_config(seed)), str(tmp_path / f"m{seed}"), seed, torch.float32, std=0.3,
                           norm_std=0.4)
    w, cfg = plain_weights(d, dtype)
    toks = {r: random_tokens(n, cfg["vocab"], seed * 10 + i) for i, (r, n) in enumerate((("a", 41), ("b", 13), ("c", 26)))}
    want = {r: plain.forward(w, cfg, t) for r, t in toks.items()}
    ex = make_executor(d, device, dtype, page_size=4, num_pages=24, batch=2, max_len=44, poison=True)
    schedule = [[("a", 9), ("b", 2)], [("a", 1), ("b", 7)], [("a", 17), ("b", 1)], [("a", 2), ("b", 3)],   # b ends
                [("a", 1), ("c", 20)], [("a", 11), ("c", 1)], [("c", 2)], [("c", 3)]]
    run_schedule(ex, schedule, toks, want, dtype, seed)


def long_decoding(tmp_path, device, name, dtype="float32", prompt=5, steps=150, page_size=16):
    """A short prompt, then many tokens one by one: states, windows and the cache are carried over page borders."""
    d = write_model(name, str(tmp_path / name))
    w, cfg = plain_weights(d, dtype)
    tokens = random_tokens(prompt + steps, cfg["vocab"], 21)
    want = plain.forward(w, cfg, tokens)
    ex = make_executor(d, device, dtype, page_size=page_size, num_pages=-(-(prompt + steps) // page_size) + 1)
    got = run_cut(ex, "r", tokens, [prompt] + [1] * steps)
    assert_close_logits(got, want, dtype)


def greedy_generation(tmp_path, device, name="mixed", dtype="float32"):
    """Greedy generation through the framework's own entry point and scheduler: the plain implementation's tokens."""
    from simply_amd.engine.llm import LMInterface
    from simply_amd.sampling import SamplingParams

    d = write_model(name, str(tmp_path / name), std=0.4)
    w, cfg = plain.load(d)
    prompts = [random_tokens(n, cfg["vocab"], 50 + n) for n in (5, 11, 17, 3)]
    want = [plain.greedy(w, cfg, p, 6) for p in prompts]
    lm = LMInterface(d, activation_dtype=dtype, batch_size=3, max_seq_len=64, page_size=4, max_num_issue_tokens=16,
                     device=str(device))
    outs = lm.generate(prompts, sampling_params=SamplingParams(temperature=0.0, max_decode_steps=6))
    assert [o.output_token_ids for o in outs] == want
