"""Small Rudutar configurations, model folders with random weights, and the bodies of the tests that run the
framework against the plain implementation (tests/plain_rudutar.py).  A body takes the device; the CPU tests run it
with the kernels replaced by their plain torch references (the `cpu_ops` fixture), the GPU tests with the kernels
themselves.  Nothing here is read from outside the repository."""
from __future__ import annotations

import copy

import torch

import plain_rudutar as plain
from simply_amd.config import config_from_dict
from simply_amd.engine import StepEntry
from simply_amd.weights import write_random_model
from tabupel_cases import assert_close_logits, run_schedule  # noqa: F401
from zenuzen_cases import BOUND, make_executor, random_tokens, rel_error, run_cut  # noqa: F401


def _dense(ff):
    return None if ff is None else {"kind": "dense", "ff": ff}


def moe(experts, top, ff, scale=1.0, groups=None, shared=None):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups is not None:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    m = {"kind": "moe", "expert": {"ff": ff}, "router": r}
    if shared is not None:
        m["shared"] = {"ff": shared}
    return m


def first(heads, kv_heads, dim, vdim, scale, conv=None, window=None, temp=None, kv_from=None, mlp=None):
    """A layer of type "attention" (convolved, normed head by head, slopes, a sink)."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if conv is not None:
        m["conv"] = conv
    if window:
        m["mask"] = {"size": window}
    if temp is not None:
        m["q_temp"] = {"coef": temp[0], "every": temp[1]}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "attention", "mixer": m, "mlp": mlp if isinstance(mlp, dict) else _dense(mlp)}


def second(heads, kv_heads, dim, scale, window=None, rot=None, mlp=None):
    """A layer of type "attention_2" (biases, normed over the row, rotated, values = keys)."""
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if window:
        m["mask"] = {"size": window}
    if rot is not None:
        m["rot"] = {"dims": rot[0], "base": rot[1]}
    return {"type": "attention_2", "mixer": m, "mlp": mlp if isinstance(mlp, dict) else _dense(mlp)}


def config(vocab, width, eps, layers):
    return {"architecture": "Rudutar", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


#: odd sizes everywhere: windows shorter than the prompts, two key heads under six heads, values of another size than
#: the keys, a layer that reads another's keys and values through a longer window and with fewer taps, one that reads
#: them through a shorter one without a convolution or a temperature, groups of experts of which two of three stay,
#: one expert chosen of four without groups or a shared expert, a layer without a feed-forward
MIXED = config(97, 48, 1e-5, [
    first(6, 2, 10, 14, 0.33, conv=3, window=7, temp=(0.4, 5), mlp=56),
    first(6, 2, 10, 14, 0.3, conv=2, window=11, temp=(0.2, 3), kv_from=0,
          mlp=moe(6, 2, 20, scale=1.5, groups=(3, 2), shared=24)),
    second(4, 2, 12, 0.3, window=13, rot=(6, 500.0), mlp=moe(4, 1, 16, scale=0.7)),
    first(4, 2, 10, 14, 0.4, window=5, kv_from=0),
    second(3, 3, 8, 0.35, window=4, rot=(8, 100.0), mlp=40),
    first(2, 1, 16, 6, 0.25, conv=4, window=9, temp=(0.3, 7), mlp=moe(8, 3, 12, scale=2.0, groups=(2, 1), shared=10)),
])
#: only layers of the first kind: as many key heads as heads, one head, a convolution of one tap (a factor per
#: channel) and of six, a window of one token and none, a temperature that moves at every position
ONLY_FIRST = config(61, 32, 1e-6, [
    first(4, 4, 8, 8, 0.35, conv=1, temp=(0.5, 1), mlp=40),
    first(1, 1, 12, 20, 0.3, conv=6, window=1, mlp=moe(2, 2, 24, groups=(1, 1))),
    first(8, 4, 8, 8, 0.5, conv=3, window=6, kv_from=0),
    first(2, 2, 6, 4, 0.4, window=30, temp=(1.0, 16)),
])
#: only layers of the second kind: rotation of everything and of nothing, one head, no window, a window of one token
ONLY_SECOND = config(70, 40, 1e-5, [
    second(4, 4, 8, 0.5, rot=(8, 100.0), mlp=30),
    second(1, 1, 12, 0.3, window=5),
    second(6, 2, 6, 0.4, window=1, rot=(2, 10.0), mlp=moe(5, 2, 8, scale=1.2, shared=6)),
    second(3, 1, 10, 0.4, window=40, rot=(4, 50000.0)),
])
#: sizes in multiples of 32 and 64 (what fast kernels may take), still small
ALIGNED = config(256, 128, 1e-5, [
    first(4, 2, 64, 64, 0.125, conv=4, window=48, temp=(0.3, 16), mlp=256),
    first(4, 2, 64, 64, 0.125, conv=4, window=40, temp=(0.3, 16), kv_from=0, mlp=moe(8, 2, 64, scale=2.0, groups=(2, 1), shared=64)),
    second(4, 2, 128, 0.09, window=80, rot=(64, 10000.0), mlp=256),
    first(8, 1, 128, 128, 0.09, conv=2, mlp=128),
    second(8, 8, 64, 0.125, window=33, rot=(32, 1000000.0)),
])
CONFIGS = {"mixed": (MIXED, 11), "only_first": (ONLY_FIRST, 12), "only_second": (ONLY_SECOND, 13), "aligned": (ALIGNED, 14)}


def drawn_config(seed: int) -> dict:
    """A configuration drawn at random: sizes, head counts, the order of the layers, which layers have which
    feed-forward, which read another layer's keys and values, windows, taps, temperatures, rotations and eps."""
    import random

    r = random.Random(3000 + seed)
    width = r.choice([24, 40, 56, 64, 96])

    def a_mlp():
        kind = r.random()
        if kind < 0.25:
            return None
        if kind < 0.6:
            return r.choice([32, 48, 100])
        count = r.choice([1, 2, 3])
        per = r.choice([1, 2, 3])
        keep = r.randint(1, count)
        return moe(count * per, r.randint(1, keep * per), r.choice([8, 16, 24]), scale=r.choice([0.5, 1.0, 2.5]),
                   groups=None if count == 1 and r.random() < 0.5 else (count, keep), shared=r.choice([None, 8, 20]))

    layers = []
    for i in range(r.randint(2, 6)):
        window = r.choice([None, 1, 3, 8, 17, 30])
        if r.random() < 0.55:
            sources = [j for j, l in enumerate(layers) if l["type"] == "attention" and "kv_from" not in l["mixer"]]
            conv, temp = r.choice([None, 1, 2, 3, 4, 6]), r.choice([None, (r.choice([0.1, 0.5]), r.choice([1, 4, 9]))])
            if sources and r.random() < 0.4:
                j = r.choice(sources)
                m = layers[j]["mixer"]
                layers.append(first(m["kv_heads"] * r.choice([1, 2, 3]), m["kv_heads"], m["dim"], m["vdim"],
                                    r.choice([0.2, 0.5]), conv=conv, window=window, temp=temp, kv_from=j, mlp=a_mlp()))
                continue
            kv, dim = r.choice([1, 2, 3]), r.choice([4, 8, 12, 16, 32])
            layers.append(first(kv * r.choice([1, 2, 3]), kv, dim, r.choice([4, 8, 16, 24, dim]),
                                r.choice([0.2, 0.5, dim ** -0.5]), conv=conv, window=window, temp=temp, mlp=a_mlp()))
        else:
            kv, dim = r.choice([1, 2, 3]), r.choice([4, 8, 12, 16, 32])
            rot = r.choice([None, (r.choice([2, 4, dim]), r.choice([100.0, 10000.0, 1e6]))])
            layers.append(second(kv * r.choice([1, 2, 3]), kv, dim, r.choice([0.2, 0.5, dim ** -0.5]), window=window, rot=rot,
                                 mlp=a_mlp()))
    return config(r.choice([50, 97, 130, 300]), width, r.choice([1e-6, 1e-5, 1e-3]), layers)


def write_model(name: str, out_dir: str, dtype=torch.float32, std: float = 0.25, norm_std: float = 0.5) -> str:
    """Writes the configuration with random weights through the framework's random-weights mode.  Norm weights,
    biases and the routers' corrections are drawn around 0 with norm_std."""
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
    """Whole, a prompt and then token by token, portions of changing size, portions of two tokens, token by token."""
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
            if l["mixer"].get("mask") and l["mixer"]["mask"]["size"] + delta >= 1:
                l["mixer"]["mask"]["size"] += delta
        off = plain.forward(w, other, tokens)
        assert rel_error(got, off) > 100 * BOUND[dtype], delta


def layers_match_plain(tmp_path, device, name="mixed", dtype="float32", length=21):
    """The residual stream behind every layer against the plain implementation's."""
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
    """A short prompt, then many tokens one by one: tails, windows and the cache are carried over page borders."""
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
