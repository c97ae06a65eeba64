"""Each mechanism of Tabupel alone against the plain implementation's function for it (tests/plain_tabupel.py), as
bodies that take the module of operations (`simply_amd.kernels.ops` on the GPU, `torch_ops` on the CPU) and the
device.  Inputs are made so that a fault shows: one key whose score stands out, just inside and just outside a
window, at page borders and hundreds of tokens back; decays near 0 and near 1; taps that differ by an order of
magnitude; a second map that nearly cancels the first."""
from __future__ import annotations

import math

import torch

import plain_tabupel as plain
from simply_amd import registry
from simply_amd.config import PartSpec
from tabupel_cases import run_mixer
from zenuzen_mechanisms import close, rand, tol_of


def _meta(rows, device):
    return torch.tensor(rows, dtype=torch.int32, device=device)


# --------------------------------------------------------------------------- the block's sum and norm


def residual_add_next_norm(o, device, dtype):
    for T, D in ((5, 72), (3, 1500), (2, 4100)):
        y, h, w = rand((T, D), 1, 3.0).to(dtype), rand((T, D), 2).float(), rand((D,), 3).to(dtype)
        res = h.clone().to(device)
        out = o.residual_add_next_norm(y.to(device), res, w.to(device), eps=1e-3, mult=0.37, out_dtype=dtype)
        want = h.double() + 0.37 * y.double()
        close(res, want, 2e-6, "residual")
        close(out, plain.rms_norm(want, w.double(), 1e-3), tol_of(dtype), "normed")
        res2 = h.clone().to(device)     # nothing added: the norm alone, the stream untouched
        out = o.residual_add_next_norm(None, res2, w.to(device), eps=1e-3, plus_one=True, out_dtype=dtype)
        close(res2, h, 0.0)
        close(out, plain.rms_norm(h.double(), w.double() + 1.0, 1e-3), tol_of(dtype), "norm alone")


# --------------------------------------------------------------------------- norm, rotation, pages


def norm_rotation_and_pages(o, device, dtype, page_size=4, sizes=(4, 2, 10, 6, 6)):
    """Rows [H heads of two maps | K key heads of two maps | K values]: every map normed with a shared weight, its
    first entries rotated in neighbouring pairs; keys and values land where the slot mapping says.  Positions far
    from 0 and a page's last and first place are among them."""
    import torch_ops

    H, K, dk, dv, rd = sizes
    T, eps, mult = 6, 1e-5, 1.07
    width = (H + K) * 2 * dk + K * dv + 5
    proj = rand((T, width), 8).to(dtype)
    wq, wk = rand((dk,), 9).to(dtype), rand((dk,), 10).to(dtype)
    pos = torch.tensor([0, 1, 3, 4, 1000, 40000], dtype=torch.int32)
    slots = torch.tensor([0, 1, 3, 4, 23, 9], dtype=torch.int64)
    freq = plain.linear_frequencies(rd, 300.0, 4.0).float()
    ang_pos = pos   # (the plain rotation multiplies positions and frequencies in 64-bit; the bound allows for it)
    q = proj.double()[:, :H * 2 * dk].view(T, H, 2, dk)
    k = proj.double()[:, H * 2 * dk:(H + K) * 2 * dk].view(T, K, 2, dk)
    want_q = plain.rotate_pairs(plain.rms_norm(q, wq.double(), eps), ang_pos, freq.double(), mult)
    want_k = plain.rotate_pairs(plain.rms_norm(k, wk.double(), eps), ang_pos, freq.double(), mult)
    v = proj.double()[:, (H + K) * 2 * dk:(H + K) * 2 * dk + K * dv]
    k_pages = torch.zeros((6, K, page_size, 2 * dk), dtype=dtype, device=device)
    v_pages = torch.zeros((6, K, dv, page_size), dtype=dtype, device=device)
    p = proj.clone().to(device)
    o.norm_rope_cache_write(p, pos.to(device), freq.to(device), rd, H, K, 2 * dk, dv, rot_mult=mult, sub=2, eps=eps,
                            q_weight=wq.to(device), q_norm_dims=dk, k_weight=wk.to(device), k_norm_dims=dk,
                            slot_mapping=slots.to(device), k_pages=k_pages, v_pages=v_pages)
    # (angles are 32-bit products: at position 40000 they are a few 1e-3 from the 64-bit ones)
    tol = max(tol_of(dtype), 5e-3)
    close(p[:, :H * 2 * dk], want_q.reshape(T, -1), tol, "queries")
    close(p[:4, :H * 2 * dk], want_q[:4].reshape(4, -1), tol_of(dtype), "queries at small positions")
    close(p[:, H * 2 * dk:], proj[:, H * 2 * dk:], 0.0, "everything but the queries stays")
    krows = torch_ops.stored_keys_as_rows(k_pages.cpu())
    for t in range(T):
        page, off = int(slots[t]) // page_size, int(slots[t]) % page_size
        close(krows[page, :, off], want_k[t].reshape(K, 2 * dk), tol if t >= 4 else tol_of(dtype), f"key {t}")
        close(v_pages[page, :, :, off].cpu(), v[t].view(K, dv), tol_of(dtype), f"value {t}")


def latent_rows_and_pages(o, device, dtype, page_size=4, sizes=(3, 12, 8)):
    """The two uses of a latent attention: query vectors [R plain | dr rotated] without a norm, and one key row per
    token [R normed with a weight | dr rotated, not normed] written into key pages and, its latent part, transposed
    into value pages; the ramp's factor is on cos and sin."""
    import torch_ops

    H, R, dr = sizes
    T, eps = 5, 1e-4
    freq, mult = plain.ramp_frequencies(dr, 1000.0, 3.0, 64, 8.0, 1.0)
    assert mult == 0.1 * math.log(3.0) + 1.0
    pos = torch.tensor([0, 2, 3, 17, 300], dtype=torch.int32)
    slots = torch.tensor([0, 3, 4, 7, 13], dtype=torch.int64)
    qa = rand((T, H * (R + dr) + 3), 11).to(dtype)
    row = rand((T, 5 + R + dr + 2), 12).to(dtype)
    w = rand((R,), 13).to(dtype)
    qv = qa.double()[:, :H * (R + dr)].view(T, H, R + dr)
    want_q = torch.cat([qv[..., :R], plain.rotate_pairs(qv[..., R:], pos, freq, mult)], -1)
    kv = row.double()[:, 5:5 + R + dr]
    want_k = torch.cat([plain.rms_norm(kv[:, :R], w.double(), eps), plain.rotate_pairs(kv[:, R:], pos, freq, mult)], -1)
    f32 = freq.float().to(device)
    q_dev = qa.clone().to(device)
    o.norm_rope_cache_write(q_dev, pos.to(device), f32, dr, H, 0, R + dr, 0, rot_mult=mult, q_rot_at=R)
    close(q_dev[:, :H * (R + dr)], want_q.reshape(T, -1), tol_of(dtype), "queries")
    close(q_dev[:, H * (R + dr):], qa[:, H * (R + dr):], 0.0)
    k_pages = torch.zeros((4, 1, page_size, R + dr), dtype=dtype, device=device)
    v_pages = torch.zeros((4, 1, R, page_size), dtype=dtype, device=device)
    r_dev = row.clone().to(device)
    o.norm_rope_cache_write(r_dev[:, 5:5 + R + dr], pos.to(device), f32, dr, 0, 1, R + dr, 0, rot_mult=mult, eps=eps,
                            k_weight=w.to(device), k_norm_dims=R, k_rot_at=R, slot_mapping=slots.to(device),
                            k_pages=k_pages, v_pages=v_pages, key_values=R)
    close(r_dev, row, 0.0, "the row itself stays")
    krows = torch_ops.stored_keys_as_rows(k_pages.cpu())
    for t in range(T):
        page, off = int(slots[t]) // page_size, int(slots[t]) % page_size
        close(krows[page, 0, off], want_k[t], tol_of(dtype), f"row {t}")
        # the latent once more, transposed, as the token's value: the very numbers of the key row
        close(v_pages[page, 0, :, off].cpu(), krows[page, 0, off, :R], 0.0, f"value {t}")


# --------------------------------------------------------------------------- attention over pages


def _pages_of(keys, values, page_size, dtype, device, shuffle_seed=0):
    """keys [n, K, row], values [n, K, dv] or None -> (key pages in the kernels' layout, value pages, block table of
    one request whose pages lie in a shuffled order)."""
    import torch_ops

    n, K, row = keys.shape
    blocks = -(-n // page_size)
    order = torch.randperm(blocks + 3, generator=torch.Generator().manual_seed(shuffle_seed))[:blocks]
    krows = torch.full((blocks + 3, K, page_size, row), float("nan"), dtype=dtype)
    vp = None if values is None else torch.full((blocks + 3, K, values.shape[2], page_size), float("nan"), dtype=dtype)
    for j in range(n):
        krows[order[j // page_size], :, j % page_size] = keys[j].to(dtype)
        if values is not None:
            vp[order[j // page_size], :, :, j % page_size] = values[j].to(dtype)
    table = torch.full((2, blocks + 2), -1, dtype=torch.int32)
    table[1, :blocks] = order.to(torch.int32)
    return (torch_ops.rows_as_stored_keys(krows).to(device), None if vp is None else vp.to(device), table.to(device))


def differential_attention_edges(o, device, dtype, page_size=4, n=300, window=37, sizes=(4, 2, 8, 6)):
    """Two maps per head over the same values.  For every query a key is chosen: just inside the window, just
    outside, at a page's first or last place, or hundreds of tokens back (no window); that key's two vectors are made
    to point along the query's with a large factor, so that it takes nearly all of both softmax sums if it is seen,
    and a map that misses it or sees one too many gives another answer.  Queries run as a prompt's portion (many rows
    at once) and alone (one row), at the same positions."""
    H, K, dk, dv = sizes
    G = H // K
    scale, lam, eps, mult = 0.4, 0.6, 1e-5, 0.7
    g = torch.Generator().manual_seed(5)
    keys = torch.randn((n, K, 2, dk), generator=g, dtype=torch.float64)
    values = torch.randn((n, K, dv), generator=g, dtype=torch.float64)
    q = torch.randn((n, H, 2, dk), generator=g, dtype=torch.float64)
    for win in (window, None):
        kk, qq = keys.clone(), q.clone()
        picks = {}
        for i in range(n - 12, n):
            w_ = win or n
            back = [w_ - 1, w_, 1, w_ - 2][i % 4] if win else [n - 15 + i % 3, 200, i % page_size + 1, i][i % 4]
            j = i - back
            if j < 0:
                continue
            picks[i] = j
            for h in range(H):
                for m in range(2):
                    # the key at j points along query (i, h, m); map 2's is weaker, so the maps differ
                    kk[j, h // G, m] += qq[i, h, m] * (6.0 if m == 0 else 3.0) / H
        kd, vd, qd = kk.to(dtype).double(), values.to(dtype).double(), qq.to(dtype).double()
        want = torch.empty((n, H, dv), dtype=torch.float64)
        for h in range(H):
            a1 = plain.windowed_softmax_attention(qd[:, h, 0], kd[:, h // G, 0], vd[:, h // G], scale, win)
            a2 = plain.windowed_softmax_attention(qd[:, h, 1], kd[:, h // G, 1], vd[:, h // G], scale, win)
            want[:, h] = plain.rms_norm(a1 - lam * a2, None, eps) * mult
        k_pages, v_pages, table = _pages_of(kk.reshape(n, K, 2 * dk), values, page_size, dtype, device)
        rows = sorted(picks)
        pos = torch.tensor(rows, dtype=torch.int32, device=device)
        seq = torch.ones(len(rows), dtype=torch.int32, device=device)
        qrows = qq[rows].reshape(len(rows), H * 2 * dk).to(dtype).to(device)
        got = o.paged_attention_maps(qrows, k_pages, v_pages, table, seq, pos, H, scale=scale, maps=2, window=win,
                                     differential=(lam, eps, mult))
        tol = 2e-4 if dtype == torch.float32 else 6e-2
        close(got, want[rows].reshape(len(rows), -1), tol, f"portion, window {win}")
        for r, i in enumerate(rows):     # the same queries alone
            one = o.paged_attention_maps(qrows[r:r + 1], k_pages, v_pages, table, seq[:1], pos[r:r + 1], H, scale=scale,
                                         maps=2, window=win, differential=(lam, eps, mult))
            close(one, want[i].reshape(1, -1), tol, f"alone at {i}, window {win}")
        # without the combination the maps come out one by one
        both = o.paged_attention_maps(qrows, k_pages, v_pages, table, seq, pos, H, scale=scale, maps=2, window=win)
        assert tuple(both.shape) == (len(rows), H * 2 * dv)


def latent_attention_edges(o, device, dtype, page_size=4, n=260, window=33, sizes=(3, 12, 6)):
    """One key head whose rows are scored whole and whose first entries are the values: the chosen key stands out
    for its query just inside the window and is unseen just outside."""
    H, R, dr = sizes
    scale = 0.3
    g = torch.Generator().manual_seed(6)
    rows_ = torch.randn((n, 1, R + dr), generator=g, dtype=torch.float64)
    q = torch.randn((n, H, R + dr), generator=g, dtype=torch.float64)
    for win in (window, None):
        kk = rows_.clone()
        w_ = win or n
        chosen = list(range(n - 8, n))
        for i in chosen:
            back = [w_ - 1, w_, 0, w_ - 2][i % 4] if win else [n - 12, 130, i % page_size, i][i % 4]
            if i - back >= 0:
                kk[i - back, 0] += q[i].mean(0) * 5.0
        kd, qd = kk.to(dtype).double(), q.to(dtype).double()
        want = torch.stack([plain.windowed_softmax_attention(qd[:, h], kd[:, 0], kd[:, 0, :R], scale, win)
                            for h in range(H)], dim=1)
        k_pages, _, table = _pages_of(kk, None, page_size, dtype, device, shuffle_seed=3)
        pos = torch.tensor(chosen, dtype=torch.int32, device=device)
        seq = torch.ones(len(chosen), dtype=torch.int32, device=device)
        qrows = q[chosen].reshape(len(chosen), -1).to(dtype).to(device)
        got = o.paged_attention_maps(qrows, k_pages, None, table, seq, pos, H, scale=scale, value_dim=R, window=win)
        tol = 2e-4 if dtype == torch.float32 else 4e-2
        close(got, want[chosen].reshape(len(chosen), -1), tol, f"portion, window {win}")
        for r, i in enumerate(chosen):
            one = o.paged_attention_maps(qrows[r:r + 1], k_pages, None, table, seq[:1], pos[r:r + 1], H, scale=scale,
                                         value_dim=R, window=win)
            close(one, want[i].reshape(1, -1), tol, f"alone at {i}, window {win}")


# --------------------------------------------------------------------------- products per head


def head_product(o, device, dtype):
    T, H, I, O, tail = 21, 3, 70, 37, 5
    x, w, gate = rand((T, H * (I + tail) + 4), 14).to(dtype), rand((H, O, I), 15, 0.3).to(dtype), rand((T, H + 2), 16, 2.0).to(dtype)
    heads = x.double()[:, :H * (I + tail)].view(T, H, I + tail)
    prod = torch.einsum("thi,hoi->tho", heads[..., :I], w.double())
    got = o.head_product(x.to(device), w.to(device), tail=tail)
    close(got, torch.cat([prod, heads[..., I:]], -1).reshape(T, -1), tol_of(dtype), "with the tails copied")
    g_dev = gate.to(device)[:, 1:1 + H]      # a view with a row stride
    got = o.head_product(x.to(device), w.to(device), in_stride=I + tail, gate=g_dev, out_dtype=torch.float32)
    assert got.dtype == torch.float32
    close(got, (prod * torch.sigmoid(gate.double()[:, 1:1 + H])[:, :, None]).reshape(T, -1), tol_of(dtype), "gated")
    # one head, more outputs than a tile, float32 rows against weights of the activation type (the recurrence's gates)
    u, w1 = rand((9, 130), 17).float(), rand((1, 200, 130), 18, 0.2).to(dtype)
    got = o.head_product(u.to(device), w1.to(device), out_dtype=torch.float32)
    close(got, u.double() @ w1.double()[0].T, 2e-5, "32-bit rows")


# --------------------------------------------------------------------------- convolution and recurrence


def short_convolution(o, device, dtype, n=4):
    """Taps that differ by an order of magnitude, a bias on the input (kept in the tails) and one on the result; two
    requests of unequal length, in one piece and in portions whose tails carry over; zeros before the start."""
    C = 70
    lengths = (19, 3)
    x = [rand((L, C), 20 + i).to(dtype) for i, L in enumerate(lengths)]
    taps = (rand((C, n), 22) * torch.tensor([10.0 ** (j - n + 1) for j in range(n)], dtype=torch.float64)).to(dtype)
    b_in, b_out = rand((C,), 23).to(dtype), rand((C,), 24).to(dtype)
    want = [plain.causal_conv(xi.double() + b_in.double(), taps.double(), b_out.double()) for xi in x]
    for cuts in ((19,), (1, 2, 16), (5, 1, 1, 12)):
        tails = torch.zeros((3, (n - 1) * C + 2), dtype=torch.float32, device=device)
        at, got = 0, []
        for k, c in enumerate(cuts):
            second = k == 0       # the short request runs beside the first portion only
            rows = torch.cat([x[0][at:at + c]] + ([x[1]] if second else [])).to(device)
            meta = [[2, 0, c, at]] + ([[0, c, lengths[1], 0]] if second else [])
            y = o.short_conv(rows, taps.to(device), tails, _meta(meta, device), len(meta), max(m[2] for m in meta),
                             in_bias=b_in.to(device), out_bias=b_out.to(device))
            got.append(y[:c])
            if second:
                close(y[c:], want[1], 2e-5 if dtype == torch.float32 else 2e-2, "short request")
            at += c
        close(torch.cat(got), want[0], 2e-5 if dtype == torch.float32 else 2e-2, f"cuts {cuts}")
        if n > 1:
            close(tails[2, :(n - 1) * C].reshape(n - 1, C), (x[0].double() + b_in.double())[-(n - 1):], 1e-6, "tails")


def recurrence(o, device, dtype, T=90, cuts=(90,), block=5):
    """The real-gated recurrence with gate inputs so wide that decays run from nearly 0 to nearly 1 (where
    sqrt(1 - a^2) loses everything in a naive form), against the plain loop; in portions the state carries over."""
    C = 4 * block
    u = rand((T, C), 30, 2.0).float()
    gates = rand((T, 2 * C), 31, 4.0).float()
    rb, ib, lam, yb = (rand((C,), s, sc).to(dtype) for s, sc in ((32, 1.0), (33, 1.0), (34, 3.0), (35, 0.5)))
    y = rand((T, C + 3), 36).to(dtype)
    g4 = gates.double().view(T, C // block, 2, block)
    r = torch.sigmoid(g4[:, :, 0].reshape(T, C) + rb.double())
    i = torch.sigmoid(g4[:, :, 1].reshape(T, C) + ib.double())
    S = plain.gated_linear_recurrence(u.double(), r, i, lam.double())
    want = S * plain.gelu_tanh(y.double()[:, :C] + yb.double())
    state = torch.zeros((2, C + 7), dtype=torch.float32, device=device)
    at, got = 0, []
    for c in cuts:
        got.append(o.rglru_scan(u[at:at + c].contiguous().to(device), gates[at:at + c].contiguous().to(device), block,
                                rb.to(device), ib.to(device), lam.to(device), y.to(device)[at:at + c, :C], yb.to(device),
                                state[:, :C], _meta([[1, 0, c, at]], device), 1, c=8.0, out_dtype=torch.float32))
        at += c
    close(torch.cat(got), want, 3e-5, f"cuts {cuts}")
    close(state[1, :C], S[-1], 3e-5, "state")
    assert float(state[0].abs().max()) == 0.0 and float(state[1, C:].abs().max()) == 0.0


def recurrence_of_unequal_requests(o, device, dtype, lengths=(1, 40, 7)):
    """Three requests in one call (1, 40 and 7 tokens; or long ones, which run in segments of tokens side by side)
    from states that are not zero: each as alone."""
    C, block = 12, 3
    slots = (3, 0, 2)
    Tt = sum(lengths)
    u, gates = rand((Tt, C), 40).float(), rand((Tt, 2 * C), 41, 2.0).float()
    rb, ib, lam = (rand((C,), s).to(dtype) for s in (42, 43, 44))
    y = rand((Tt, C), 45).to(dtype)
    start = rand((4, C), 46).float()
    state = start.clone().to(device)
    meta, at = [], 0
    for L, s in zip(lengths, slots):
        meta.append([s, at, L, 5])
        at += L
    got = o.rglru_scan(u.to(device), gates.to(device), block, rb.to(device), ib.to(device), lam.to(device), y.to(device),
                       None, state, _meta(meta, device), 3, out_dtype=torch.float32, max_q_len=max(lengths))
    for s, first, L, _ in meta:
        sl = slice(first, first + L)
        g4 = gates[sl].double().view(L, C // block, 2, block)
        r = torch.sigmoid(g4[:, :, 0].reshape(L, C) + rb.double())
        i = torch.sigmoid(g4[:, :, 1].reshape(L, C) + ib.double())
        S = plain.gated_linear_recurrence(u[sl].double(), r, i, lam.double(), start[s].double())
        close(got[sl], S * plain.gelu_tanh(y[sl].double()), 3e-5, f"slot {s}")
        close(state[s], S[-1], 3e-5)
    close(state[1], start[1], 0.0, "a slot that no request has")


# --------------------------------------------------------------------------- the mixers as parts


def _load_part(kind, params, tensors, dtype, device):
    part = registry.MIXERS.build(kind, **params)
    specs = part.param_specs()
    assert set(specs) == set(tensors), (sorted(specs), sorted(tensors))
    loaded = {}
    for name, t in tensors.items():
        assert tuple(t.shape) == tuple(specs[name].shape), name
        loaded[name] = t.to(dtype if specs[name].role == "matrix" or dtype == torch.bfloat16 else torch.float32).to(device)
    part.load(loaded)
    return part


CUTS = ([61], [29] + [1] * 32, [7, 5, 3, 2, 11, 2, 2, 29], [2] * 30 + [1], [1] * 61)


def differential_part(device, dtype, sizes=(40, 6, 2, 10, 14), window=9, page_size=4, length=61, cuts=CUTS):
    D, H, K, dk, dv = sizes
    m = {"heads": H, "kv_heads": K, "dim": dk, "vdim": dv, "scale": 0.35, "diff": 0.3, "mask": {"size": window},
         "rot": {"dims": 6, "base": 500.0, "scaling": {"factor": 4.0}}}
    p = {"q": rand((H * 2 * dk, D), 50, 0.3), "k": rand((K * 2 * dk, D), 51, 0.3), "v": rand((K * dv, D), 52, 0.3),
         "o": rand((D, H * dv), 53, 0.3), "q.norm": rand((dk,), 54), "k.norm": rand((dk,), 55)}
    p.update({n: rand((dk,), 56 + i, 0.3) for i, n in enumerate(("lq1", "lk1", "lq2", "lk2"))})
    p = {n: t.to(dtype).double() for n, t in p.items()}
    x = rand((length, D), 60).to(dtype)
    want = plain.differential_attention(x.double(), p, m, 1e-5)
    part = _load_part("differential_attention", {
        "hidden_size": D, "num_heads": H, "num_kv_heads": K, "key_dim": dk, "value_dim": dv, "scale": 0.35, "diff": 0.3,
        "norm_eps": 1e-5, "window": window,
        "position_encoding": PartSpec("pair_rope", {"dims": 6, "base": 500.0, "scaling": {"kind": "linear", "factor": 4.0}}),
    }, {"q_proj": p["q"], "k_proj": p["k"], "v_proj": p["v"], "o_proj": p["o"], "q_norm": p["q.norm"],
        "k_norm": p["k.norm"], "lq1": p["lq1"], "lk1": p["lk1"], "lq2": p["lq2"], "lk2": p["lk2"]}, dtype, device)
    for c in cuts:
        got = run_mixer(part, x.to(device), c, dtype, device, page_size)
        close(got, want, 2e-5 if dtype == torch.float32 else 6e-2, f"cuts {c[:4]}")


def latent_part(device, dtype, sizes=(40, 3, 12, 8, 10, 20, 24), window=13, page_size=4, length=61, cuts=CUTS, std=0.3):
    """std: of the matrices (wide layers want smaller ones, or the scores grow so large that a bfloat16 run's rounding,
    the plain implementation's own with roundings at the same places included, moves whole softmax sums)."""
    D, H, dk, dr, dv, Rq, R = sizes
    sc = {"factor": 3.0, "original": 64, "fast": 8.0, "slow": 1.0}
    m = {"heads": H, "dim": dk, "rot_dim": dr, "vdim": dv, "q_rank": Rq, "kv_rank": R, "scale": 0.3,
         "mask": {"size": window}, "rot": {"dims": dr, "base": 1000.0, "scaling": sc}}
    p = {"dq": rand((Rq, D), 70, std), "dq.norm": rand((Rq,), 71), "uq": rand((H * (dk + dr), Rq), 72, std),
         "dkv": rand((R + dr, D), 73, std), "dkv.norm": rand((R,), 74), "uk": rand((H * dk, R), 75, std),
         "uv": rand((H * dv, R), 76, std), "g": rand((H, D), 77, std), "o": rand((D, H * dv), 78, std)}
    p = {n: t.to(dtype).double() for n, t in p.items()}
    x = rand((length, D), 79).to(dtype)
    want = plain.latent_attention(x.double(), p, m, 1e-5)
    part = _load_part("latent_attention", {
        "hidden_size": D, "num_heads": H, "key_dim": dk, "rot_dim": dr, "value_dim": dv, "q_rank": Rq, "kv_rank": R,
        "scale": 0.3, "norm_eps": 1e-5, "window": window, "output_gate": True,
        "position_encoding": PartSpec("pair_rope", {"dims": dr, "base": 1000.0, "scaling": {"kind": "ramp", **sc}}),
    }, {"dq_proj": p["dq"], "dq_norm": p["dq.norm"], "uq_proj": p["uq"], "dkv_proj": p["dkv"], "dkv_norm": p["dkv.norm"],
        "uk_proj": p["uk"], "uv_proj": p["uv"], "gate_proj": p["g"], "o_proj": p["o"]}, dtype, device)
    for c in cuts:
        got = run_mixer(part, x.to(device), c, dtype, device, page_size)
        close(got, want, 2e-5 if dtype == torch.float32 else 6e-2, f"cuts {c[:4]}")


def rglru_part(device, dtype, sizes=(40, 36, 3, 4), length=61, cuts=CUTS):
    D, C, B, n = sizes
    bs = C // B
    p = {"y": rand((C, D), 80, 0.3), "y.b": rand((C,), 81, 0.5), "x": rand((C, D), 82, 0.3), "x.b": rand((C,), 83, 0.5),
         "conv": rand((C, n), 84, 0.5), "conv.b": rand((C,), 85, 0.5), "ra": rand((B, bs, bs), 86, 0.5),
         "ra.b": rand((B, bs), 87), "ri": rand((B, bs, bs), 88, 0.5), "ri.b": rand((B, bs), 89), "lam": rand((C,), 90, 2.0),
         "o": rand((D, C), 91, 0.3)}
    p = {k: t.to(dtype).double() for k, t in p.items()}
    x = rand((length, D), 92).to(dtype)
    want = plain.rglru(x.double(), p, {})
    part = _load_part("rglru", {"hidden_size": D, "width": C, "blocks": B, "conv_taps": n, "decay_mult": 8.0},
                      {"y_proj": p["y"], "y_bias": p["y.b"], "x_proj": p["x"], "x_bias": p["x.b"], "conv": p["conv"],
                       "conv_bias": p["conv.b"], "r_gate": p["ra"], "r_bias": p["ra.b"], "i_gate": p["ri"],
                       "i_bias": p["ri.b"], "lam": p["lam"], "o_proj": p["o"]}, dtype, device)
    for c in cuts:
        got = run_mixer(part, x.to(device), c, dtype, device)
        close(got, want, 2e-5 if dtype == torch.float32 else 6e-2, f"cuts {c[:4]}")


# --------------------------------------------------------------------------- the same attention on the matrix cores


def _units_of(rows, per_unit, slot, device):
    """Consecutive positions of `rows` (sorted) grouped into units of at most per_unit tokens: (units, row of each)."""
    units, first = [], 0
    while first < len(rows):
        n = 1
        while n < per_unit and first + n < len(rows) and rows[first + n] == rows[first] + n:
            n += 1
        units.append([slot, first, n, rows[first]])
        first += n
    return torch.tensor(units, dtype=torch.int32, device=device)


def attention_units_on_the_matrix_cores(o, device, sizes=(8, 2, 64, 128), n=700, window=100, differential=True, last=24):
    """`paged_attention_maps_units` (bfloat16, pages of 16 keys) against the plain functions, with the chosen keys of
    `differential_attention_edges`: just inside and just outside the window, at page borders and far back; the
    queries as units of several tokens (a prompt's portion) and as units of one token (decoding), with the keys in
    one range and cut into several.  last: how many of the last positions are queries (hundreds: the launch has so
    many units that a wave takes a unit of its own; all of them: a sequence's first tokens are among them)."""
    dtype, page_size = torch.bfloat16, 16
    H, K, dk, dv = sizes
    maps = 2 if differential else 1
    G = H // K
    scale, lam, eps, mult = dk ** -0.5, 0.6, 1e-5, 0.7
    g = torch.Generator().manual_seed(15)
    keys = torch.randn((n, K, maps, dk), generator=g, dtype=torch.float64)
    values = torch.randn((n, K, dv), generator=g, dtype=torch.float64)
    q = torch.randn((n, H, maps, dk), generator=g, dtype=torch.float64)
    for win in (window, None):
        kk = keys.clone()
        w_ = win or n
        rows = list(range(n - last, n))
        for i in rows[-24:]:
            back = [w_ - 1, w_, 1, w_ - 2][i % 4] if win else [n - 30 + i % 3, 400, i % page_size + 1, i][i % 4]
            if i - back >= 0:
                for h in range(H):
                    for m in range(maps):
                        kk[i - back, h // G, m] += q[i, h, m] * (4.0 if m == 0 else 2.0) / G
        kd, vd, qd = kk.to(dtype).double(), values.to(dtype).double(), q.to(dtype).double()
        want = torch.empty((n, H, dv), dtype=torch.float64)
        for h in range(H):
            a = [plain.windowed_softmax_attention(qd[:, h, m], kd[:, h // G, m], vd[:, h // G], scale, win) for m in range(maps)]
            want[:, h] = plain.rms_norm(a[0] - lam * a[1], None, eps) * mult if differential else a[0]
        k_pages, v_pages, table = _pages_of(kk.reshape(n, K, maps * dk), values, page_size, dtype, device)
        qrows = q[rows].reshape(len(rows), H * maps * dk).to(dtype).to(device)
        per_unit = 16 // o.attention_maps_heads_per_unit(H, K)
        assert o.attention_maps_units_takes(qrows, k_pages, v_pages, H, maps)
        for tokens in (per_unit, 1):
            units = _units_of(rows, tokens, 1, device)
            got = o.paged_attention_maps_units(qrows, k_pages, v_pages, table, units, 0, units.shape[0], H, scale=scale,
                                               maps=maps, window=win, max_kv_len=n, max_q_len=tokens,
                                               differential=(lam, eps, mult) if differential else None)
            close(got, want[rows].reshape(len(rows), -1), 4e-2, f"units of {tokens}, window {win}")
        # a single request decoding: its keys are cut into ranges over the workgroups and merged
        units = _units_of(rows[-1:], 1, 1, device)
        got = o.paged_attention_maps_units(qrows[-1:], k_pages, v_pages, table, units, 0, 1, H, scale=scale, maps=maps,
                                           window=win, max_kv_len=n, max_q_len=1,
                                           differential=(lam, eps, mult) if differential else None)
        close(got, want[rows[-1]].reshape(1, -1), 4e-2, f"one request, window {win}")
