"""Each mechanism of Rudutar alone against the plain implementation's function for it (tests/plain_rudutar.py), as
bodies that take the module of operations (`simply_amd.kernels.ops` on the GPU, `torch_ops` on the CPU) and the
device.  Inputs are made so that a fault shows: taps that differ by orders of magnitude, tails that are not zero, one
key whose score stands out just inside and just outside a window, at page borders and hundreds of tokens back,
queries whose scores are all so low that the sink takes the sum, choice scores below zero, groups whose best expert
is not in the best group."""
from __future__ import annotations

import torch

import plain_rudutar as plain
from simply_amd.config import PartSpec
from tabupel_mechanisms import _load_part, _meta, _pages_of
from zenuzen_cases import run_mixer
from zenuzen_mechanisms import close, rand, tol_of


# --------------------------------------------------------------------------- from the projection to the attention kernel


def inputs_of_the_first_kind(o, device, dtype, page_size=4, sizes=(4, 2, 10, 6), taps=4):
    """Convolution, norm head by head, temperature, pages: two requests of unequal length in two steps (so that the
    second step's first tokens read tails), with taps that differ by orders of magnitude."""
    import torch_ops

    H, K, dk, dv = sizes
    C = (H + K) * dk + K * dv
    lengths, cut = (23, 7), (9, 3)            # tokens of the two requests; how many of them run in the first step
    eps, coef, every = 1e-5, 0.4, 3
    w = (rand((C, taps), 1) * torch.tensor([10.0 ** (-j) for j in range(taps)][::-1], dtype=torch.float64)).to(dtype)
    qw, kw = rand((dk,), 2).to(dtype), rand((dk,), 3).to(dtype)
    xs = [rand((n, C + 5), 4 + i, 2.0).to(dtype) for i, n in enumerate(lengths)]    # (rows wider than the channels)
    want_q, want_k, want_v = [], [], []
    for x, n in zip(xs, lengths):
        y = plain.causal_conv(x[:, :C].double(), w.double()) if taps else x[:, :C].double()
        q = plain.rms_norm(y[:, :H * dk].view(n, H, dk), qw.double(), eps)
        want_q.append(q * plain.query_temperature(n, coef, every, torch.float64)[:, None, None])
        want_k.append(plain.rms_norm(y[:, H * dk:(H + K) * dk].view(n, K, dk), kw.double(), eps))
        want_v.append(y[:, (H + K) * dk:].view(n, K, dv))
    pages = sum(-(-n // page_size) for n in lengths)
    k_pages = torch.full((pages, K, page_size, dk), float("nan"), dtype=dtype, device=device)
    v_pages = torch.full((pages, K, dv, page_size), float("nan"), dtype=dtype, device=device)
    first_page = [0, -(-lengths[0] // page_size)]
    tails = torch.zeros((3, max(taps - 1, 0) * C + 2), dtype=torch.float32, device=device)
    got_q = [[], []]
    for step in range(2):
        spans = [(0, cut[i]) if step == 0 else (cut[i], lengths[i]) for i in range(2)]
        rows = torch.cat([xs[i][a:b] for i, (a, b) in enumerate(spans)]).to(device)
        meta, slots, at = [], [], 0
        for i, (a, b) in enumerate(spans):
            meta.append([i + 1, at, b - a, a])          # (state slots 1 and 2)
            slots += [first_page[i] * page_size + p for p in range(a, b)]
            at += b - a
        q = o.attention_inputs(rows, _meta(meta, device), 2, max(b - a for a, b in spans), H, K, dk, dv,
                               taps=w.to(device) if taps else None, tails=tails if taps > 1 else None, norm="head",
                               q_weight=qw.to(device), k_weight=kw.to(device), eps=eps, temp_coef=coef, temp_every=every,
                               slot_mapping=torch.tensor(slots, dtype=torch.int64, device=device), k_pages=k_pages,
                               v_pages=v_pages)
        at = 0
        for i, (a, b) in enumerate(spans):
            got_q[i].append(q[at:at + b - a])
            at += b - a
    krows = torch_ops.stored_keys_as_rows(k_pages.cpu())
    for i, n in enumerate(lengths):
        close(torch.cat(got_q[i]).view(n, H, dk), want_q[i], tol_of(dtype), f"queries of request {i}")
        pos = torch.arange(n)
        page, off = first_page[i] + pos // page_size, pos % page_size
        close(krows[page, :, off], want_k[i], tol_of(dtype), f"keys of request {i}")
        close(v_pages.cpu()[page, :, :, off], want_v[i], tol_of(dtype), f"values of request {i}")


def inputs_of_the_second_kind(o, device, dtype, page_size=4, sizes=(6, 2, 12), rot=(6, 500.0), start=37):
    """Norm over the whole row with a weight per entry, rotation of a head's first entries in halves, the keys as
    projected as the values; positions that do not start at 0."""
    import torch_ops

    H, K, dk = sizes
    n, eps = 11, 1e-4
    C = (H + K) * dk
    x = rand((n, C + 3), 11, 2.0).to(dtype)
    qw, kw = rand((H * dk,), 12).to(dtype), rand((K * dk,), 13).to(dtype)
    dims, base = rot
    inv_freq = (float(base) ** (-2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)).to(torch.float32)

    def at_positions(v):    # the plain rotation counts positions from 0: rotate a longer sequence, keep its end
        padded = torch.cat([torch.zeros((start,) + tuple(v.shape[1:]), dtype=v.dtype), v])
        return plain.rotate_half(padded, dims, base)[start:]

    bias = rand((C,), 14, 0.5).to(dtype)
    xd = x.double()
    xd[:, :C] += bias.double()
    want_q = at_positions(plain.rms_norm(xd[:, :H * dk], qw.double(), eps).view(n, H, dk))
    want_k = at_positions(plain.rms_norm(xd[:, H * dk:C], kw.double(), eps).view(n, K, dk))
    pages = -(-(start + n) // page_size)
    k_pages = torch.full((pages, K, page_size, dk), float("nan"), dtype=dtype, device=device)
    v_pages = torch.full((pages, K, dk, page_size), float("nan"), dtype=dtype, device=device)
    pos = torch.arange(start, start + n)
    q = o.attention_inputs(x.to(device), _meta([[0, 0, n, start]], device), 1, n, H, K, dk, dk, values_are_keys=True,
                           norm="row", q_weight=qw.to(device), k_weight=kw.to(device), eps=eps, in_bias=bias.to(device),
                           inv_freq=inv_freq.to(device), rot_dims=dims, q_mult=0.5,
                           slot_mapping=pos.to(torch.int64).to(device), k_pages=k_pages, v_pages=v_pages)
    tol = tol_of(dtype)
    close(q.view(n, H, dk), 0.5 * want_q, tol, "queries")
    close(torch_ops.stored_keys_as_rows(k_pages.cpu())[pos // page_size, :, pos % page_size], want_k, tol, "keys")
    close(v_pages.cpu()[pos // page_size, :, :, pos % page_size], xd[:, H * dk:C].view(n, K, dk), tol, "values")
    # a layer without keys and values of its own: queries only
    q2 = o.attention_inputs(x.to(device), _meta([[0, 0, n, start]], device), 1, n, H, K, dk, dk, norm="row",
                            q_weight=qw.to(device), eps=eps, inv_freq=inv_freq.to(device), rot_dims=dims,
                            in_bias=bias[:H * dk].contiguous().to(device))
    close(q2.view(n, H, dk), want_q, tol, "queries alone")


# --------------------------------------------------------------------------- attention with slopes and a sink


def _attention_case(dtype, sizes, n, window, page_size, seed=5):
    """Queries, keys and values in which, for the last queries, one key is made to stand out: just inside the window,
    just outside, at a page's first or last place, at the query itself, or far back (no window); every fourth of those
    queries instead points away from all keys, so that the sink takes nearly the whole sum."""
    H, K, dk, dv = sizes
    G = H // K
    g = torch.Generator().manual_seed(seed)
    keys = torch.randn((n, K, dk), generator=g, dtype=torch.float64)
    keys[..., 0] += 3.0      # (what all keys share: a query along minus that scores low against every key)
    values = torch.randn((n, K, dv), generator=g, dtype=torch.float64)
    q = torch.randn((n, H, dk), generator=g, dtype=torch.float64)
    picks = []
    for i in range(n - 16, n):
        w_ = window or n
        back = [w_ - 1, w_, 0, w_ - 2][i % 4] if window else [n - 19 + i % 3, 200, i % page_size, i][i % 4]
        j = i - back
        if j < 0:
            continue
        picks.append(i)
        if i % 5 == 0:
            q[i] = 0.0
            q[i, :, 0] = -10.0
            continue
        for h in range(H):
            keys[j, h // G] += q[i, h] * 8.0 / G
    return q.to(dtype), keys.to(dtype), values.to(dtype), picks


def attention_edges(o, device, dtype, page_size=4, n=300, window=37, sizes=(4, 2, 8, 6), scale=0.4, sharp=True):
    """The softmax with one more term exp(0), slopes by distance and a window, by the generic kernel: in a prompt's
    portion (many rows at once) and alone (one row), at the same positions; also without sink and slopes."""
    H, K, dk, dv = sizes
    for win in (window, None):
        q, keys, values, rows = _attention_case(dtype, sizes, n, win, page_size)
        for sink, sloped in ((True, True), (False, False), (True, False)):
            slopes = plain.distance_slopes(H, torch.float64) if sloped else None
            want = plain.softmax_attention(q.double(), keys.double(), values.double(), scale, win, slopes, sink)
            k_pages, v_pages, table = _pages_of(keys, values, page_size, dtype, device)
            pos = torch.tensor(rows, dtype=torch.int32, device=device)
            seq = torch.ones(len(rows), dtype=torch.int32, device=device)
            qrows = q[rows].reshape(len(rows), H * dk).to(device)
            kw = dict(scale=scale, window=win, sinks=torch.zeros(H, dtype=torch.float32, device=device) if sink else None,
                      slopes=slopes.to(torch.float32).to(device) if sloped else None)
            got = o.paged_attention_sink(qrows, k_pages, v_pages, table, seq, pos, H, **kw)
            tol = 2e-4 if dtype == torch.float32 else 6e-2
            close(got, want[rows], tol, f"portion, window {win}, sink {sink}, slopes {sloped}")
            for r, i in enumerate(rows):
                one = o.paged_attention_sink(qrows[r:r + 1], k_pages, v_pages, table, seq[:1], pos[r:r + 1], H, **kw)
                close(one, want[i:i + 1], tol, f"alone at {i}, window {win}, sink {sink}, slopes {sloped}")
            if sharp and sink and sloped and win is None:
                # the comparison is sharp: without the sink, or without the slopes, the answer is another
                for other in (plain.softmax_attention(q.double(), keys.double(), values.double(), scale, win, slopes, False),
                              plain.softmax_attention(q.double(), keys.double(), values.double(), scale, win, None, True)):
                    diff = (got.double().cpu() - other[rows]).norm(dim=-1) / other[rows].norm(dim=-1)
                    assert float(diff.max()) > 0.5 > tol


def _units_of(rows, per_unit, slot, device):
    """Consecutive positions `rows` of one request cut into units of per_unit tokens, in the layout of seq_meta."""
    units = []
    for a in range(0, len(rows), per_unit):
        part = rows[a:a + per_unit]
        units.append([slot, a, len(part), part[0]])
    return units


def attention_on_the_matrix_cores(o, device, sizes=(8, 2, 64, 64), n=700, window=100, last=24, scale=0.11):
    """The same attention on the MFMA kernels (bfloat16, pages of 16 keys): the last `last` positions as single
    decoded tokens (keys cut into ranges) and as a portion's units, with sink and slopes and without."""
    H, K, dk, dv = sizes
    dtype, page_size = torch.bfloat16, 16
    G = H // K
    q, keys, values, _ = _attention_case(dtype, sizes, n, window, page_size, seed=9)
    rows = list(range(n - last, n))
    k_pages, v_pages, table = _pages_of(keys, values, page_size, dtype, device)
    qs = (q[rows].double() * scale).to(dtype).reshape(last, H * dk).to(device)     # (these kernels have no factor)
    for sink, sloped in ((True, True), (False, False)):
        slopes = plain.distance_slopes(H, torch.float64) if sloped else None
        want = plain.softmax_attention((q.double() * scale).to(dtype).double(), keys.double(), values.double(), 1.0, window,
                                       slopes, sink)[rows]
        kw = dict(window=window, soft_cap=None, max_kv_len=n, sinks=torch.zeros(H, dtype=torch.float32, device=device) if sink else None,
                  slopes=slopes.to(torch.float32).to(device) if sloped else None)
        out = torch.zeros((last, H * dv), dtype=dtype, device=device)
        meta = _meta([[1, r, 1, rows[r]] for r in range(last)], device)
        o.paged_attention_decode(qs, k_pages, v_pages, table, meta, 0, last, H, max_q_len=1, out=out, **kw)
        close(out, want, 4e-2, f"decoded alone, sink {sink}")
        per = 16 // G
        group = o.prefill_units_per_group()
        units = _units_of(rows, per, 1, device)
        while len(units) % group:
            units.append([1, last, 0, rows[-1] + 1])
        out2 = torch.zeros((last, H * dv), dtype=dtype, device=device)
        o.paged_attention_prefill(qs, k_pages, v_pages, table, _meta(units, device), 0, len(units), H, max_q_len=per,
                                  out=out2, **kw)
        close(out2, want, 4e-2, f"units of a portion, sink {sink}")


# --------------------------------------------------------------------------- embedding, gates, router, experts


def normed_embedding(device, dtype):
    """The table's row through the norm with a weight of its own, 32-bit out."""
    from simply_amd import registry

    V, D, eps = 37, 24, 1e-3
    table, w = rand((V, D), 1, 3.0).to(dtype), rand((D,), 2).to(dtype)
    part = registry.EMBEDDINGS.build("normed_embedding", vocab_size=V, dim=D, eps=eps)
    part.load({"table": table.to(device), "norm": w.to(device)})
    tokens = torch.tensor([0, 36, 5, 5, 17], dtype=torch.int32, device=device)
    got = part.forward(tokens)
    assert got.dtype == torch.float32
    close(got, plain.rms_norm(table.double()[tokens.cpu().long()], w.double(), eps), 2e-6, "normed rows")



def gate_per_head(o, device, dtype):
    T, H, S = 5, 3, 20
    x, g = rand((T, H * S), 4, 2.0).to(dtype), rand((T, H + 7), 5, 2.0).to(dtype)
    gate = g[:, 3:3 + H]     # a view with a row stride, as the mixer hands it over
    want = (x.double().view(T, H, S) * torch.sigmoid(gate.double())[:, :, None]).reshape(T, H * S)
    got = o.gated_heads(x.to(device), g.to(device)[:, 3:3 + H], H, S, kind=0, out_dtype=dtype, per_head=True)
    close(got, want, tol_of(dtype), "one number per head")


def router_choice(o, device, dtype=torch.float32):
    """Sigmoid scores, a correction that pushes choice scores below zero, groups of which the best stay: made cases
    and drawn ones against the plain function, experts as sets and weights by expert."""
    # four groups of three; the single best expert (7) sits in a group whose two best sum below those of two others
    made = torch.full((1, 12), -3.0, dtype=torch.float64)
    made[0, [0, 1]] = torch.tensor([1.0, 0.9], dtype=torch.float64)    # group 0: two good ones
    made[0, 7] = 3.0                                                 # group 2: one very good one, the others bad
    made[0, [9, 10]] = torch.tensor([0.8, 0.7], dtype=torch.float64)   # group 3
    cases_ = [(made, torch.zeros(12, dtype=torch.float64), 3, 4, 2)]
    # every choice score below zero; shut-out experts must not win over them
    cases_.append((rand((7, 12), 3), torch.full((12,), -2.0, dtype=torch.float64) + 0.1 * rand((12,), 4), 4, 3, 2))
    for seed, (E, top, groups, keep) in enumerate([(8, 2, 2, 1), (6, 2, 3, 2), (16, 4, 4, 2), (5, 5, 1, 1), (9, 1, 9, 1),
                                                   (64, 6, 8, 3), (130, 3, 1, 1), (4, 1, 4, 4)]):
        cases_.append((rand((33, E), 10 + seed, 2.0), rand((E,), 30 + seed, 0.7), top, groups, keep))
    for z, corr, top, groups, keep in cases_:
        want_e, s = plain.choose_experts(z.float().double(), corr.to(dtype).double(), top, groups, keep)
        got_e, got_w = o.route_choice(z.float().to(device), top, 1.7, correction=corr.to(dtype).to(device), groups=groups,
                                      keep=keep)
        got_e, got_w = got_e.cpu().long(), got_w.cpu().double()
        for t in range(z.shape[0]):
            assert sorted(got_e[t].tolist()) == sorted(want_e[t].tolist()), (t, top, groups, keep)
        close(got_w, 1.7 * torch.gather(s, 1, got_e), 1e-5, "weights are scores without the correction")
    # the made case: expert 7's group is out although 7 has the largest score of all
    e, _ = o.route_choice(made.float().to(device), 3, 1.0, correction=None, groups=4, keep=2)
    assert sorted(e.cpu()[0].tolist()) == [0, 1, 9]


def experts_without_gate(o, device, dtype):
    """The chosen experts' results, weighted, plus the shared one: rows of few tokens and of many (both tile sizes)."""
    from simply_amd.kernels.packing import stack_experts

    D, F, E, top = 40, 24, 6, 2
    up = [rand((F, D), 100 + e, 0.3).to(dtype) for e in range(E)]
    down = [rand((D, F), 200 + e, 0.3).to(dtype) for e in range(E)]
    for T in (5, 130):
        x = rand((T, D), 7 + T).to(dtype)
        g = torch.Generator().manual_seed(T)
        experts = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
        weights = torch.rand((T, top), generator=g, dtype=torch.float32) * 2
        shared = rand((T, D), 9).to(dtype)
        want = shared.double().clone()
        for t in range(T):
            for k in range(top):
                e = int(experts[t, k])
                want[t] += weights[t, k].double() * plain.squared_relu_expert(x[t:t + 1].double(), up[e].double(), down[e].double())[0]
        got = o.routed_experts(x.to(device), experts.to(device), weights.to(device), None,
                               stack_experts(u.to(device) for u in up), stack_experts(d.to(device) for d in down), 2,
                               shared=shared.to(device), out_dtype=torch.float32)
        close(got, want, 2e-5 if dtype == torch.float32 else 3e-2, f"{T} tokens")


# --------------------------------------------------------------------------- the mixers as parts with a cache of their own

CUTS = ([61], [29] + [1] * 32, [7, 5, 3, 2, 11, 2, 2, 29], [2] * 30 + [1], [1] * 61)


def first_kind_part(device, dtype, sizes=(40, 6, 2, 10, 14), window=9, taps=3, temp=(0.4, 5), page_size=4, length=61,
                    cuts=CUTS, std=0.3):
    D, H, K, dk, dv = sizes
    m = {"heads": H, "kv_heads": K, "dim": dk, "vdim": dv, "scale": 0.35, "conv": taps, "mask": {"size": window},
         "q_temp": {"coef": temp[0], "every": temp[1]}}
    p = {"q": rand((H * dk, D), 50, std), "k": rand((K * dk, D), 51, std), "v": rand((K * dv, D), 52, std),
         "g": rand((H * dv, D), 53, std), "o": rand((D, H * dv), 54, std), "q.norm": rand((dk,), 55), "k.norm": rand((dk,), 56),
         "q.conv": rand((H * dk, taps), 57, 0.6), "k.conv": rand((K * dk, taps), 58, 0.6), "v.conv": rand((K * dv, taps), 59, 0.6)}
    p = {n: t.to(dtype).double() for n, t in p.items()}
    x = rand((length, D), 60).to(dtype)
    want = plain.conv_attention(x.double(), p, m, 1e-5)
    part = _load_part("gated_attention", {
        "hidden_size": D, "num_heads": H, "num_kv_heads": K, "key_dim": dk, "value_dim": dv, "scale": 0.35, "norm_eps": 1e-5,
        "qk_norm": "head", "conv_taps": taps, "query_temperature": temp, "slope_exponent": 8.0, "zero_sink": True,
        "output_gate": "element", "window": window,
    }, {"q_proj": p["q"], "k_proj": p["k"], "v_proj": p["v"], "gate_proj": p["g"], "o_proj": p["o"], "q_norm": p["q.norm"],
        "k_norm": p["k.norm"], "q_conv": p["q.conv"], "k_conv": p["k.conv"], "v_conv": p["v.conv"]}, dtype, device)
    for c in cuts:
        got = run_mixer(part, x.to(device), c, dtype, device, page_size)
        close(got, want, 2e-5 if dtype == torch.float32 else 6e-2, f"cuts {c[:4]}")


def second_kind_part(device, dtype, sizes=(40, 6, 2, 12), window=13, rot=(6, 500.0), page_size=4, length=61, cuts=CUTS,
                     std=0.3):
    D, H, K, dk = sizes
    m = {"heads": H, "kv_heads": K, "dim": dk, "vdim": dk, "scale": 0.3, "mask": {"size": window},
         "rot": {"dims": rot[0], "base": rot[1]}}
    p = {"q": rand((H * dk, D), 70, std), "k": rand((K * dk, D), 71, std), "q.b": rand((H * dk,), 72, 0.5),
         "k.b": rand((K * dk,), 73, 0.5), "g": rand((H, D), 74, std), "o": rand((D, H * dk), 75, std),
         "q.norm": rand((H * dk,), 76), "k.norm": rand((K * dk,), 77)}
    p = {n: t.to(dtype).double() for n, t in p.items()}
    x = rand((length, D), 80).to(dtype)
    want = plain.whole_norm_attention(x.double(), p, m, 1e-5)
    part = _load_part("gated_attention", {
        "hidden_size": D, "num_heads": H, "num_kv_heads": K, "key_dim": dk, "value_dim": dk, "scale": 0.3, "norm_eps": 1e-5,
        "qk_norm": "row", "bias": True, "values": "keys", "output_gate": "head", "window": window,
        "position_encoding": PartSpec("partial_rope", {"head_dim": dk, "dims": rot[0], "base": rot[1]}),
    }, {"q_proj": p["q"], "k_proj": p["k"], "q_bias": p["q.b"], "k_bias": p["k.b"], "gate_proj": p["g"], "o_proj": p["o"],
        "q_norm": p["q.norm"], "k_norm": p["k.norm"]}, dtype, device)
    for c in cuts:
        got = run_mixer(part, x.to(device), c, dtype, device, page_size)
        close(got, want, 2e-5 if dtype == torch.float32 else 6e-2, f"cuts {c[:4]}")
