"""Plain torch versions of every kernel in `simply_amd.kernels.ops`, with the same signatures.

Two uses, both in tests only: the reference that each HIP kernel is compared with on the GPU, and
(patched in by the `cpu_ops` fixture) a stand-in that lets the engine's host logic (step function,
cache manager, scheduler) run on a machine without a GPU.  Internal arithmetic is float32 (or
float64 when `PRECISE` is set) whatever the storage type is.
"""
from __future__ import annotations

import math

import torch

PRECISE = False

EPILOGUE_NONE, EPILOGUE_GATED_GELU, EPILOGUE_SOFT_CAP = 0, 1, 2
ALGO_AUTO, ALGO_GENERIC, ALGO_SKINNY, ALGO_TILED = 0, 1, 2, 3


def _f(t) -> torch.Tensor:
    if hasattr(t, "rows"):   # a tiled weight
        from simply_amd.kernels.packing import unpack_tiles
        t = unpack_tiles(t)
    return t.to(torch.float64 if PRECISE else torch.float32)


def embed(table, tokens, scale, out=None):
    r = (_f(table)[tokens.long()] * scale).to(torch.float32)
    if out is not None:
        out.copy_(r)
        return out
    return r


def rmsnorm(x, weight, eps, plus_one, out_dtype, out=None):
    xf = _f(x)
    y = xf * torch.rsqrt((xf * xf).mean(-1, keepdim=True) + eps) * (_f(weight) + (1.0 if plus_one else 0.0))
    y = y.to(out_dtype)
    if out is not None:
        out.copy_(y)
        return out
    return y


def add_rmsnorm(y, residual, *, post_weight=None, post_eps=0.0, post_plus_one=True, next_weight=None, next_eps=0.0,
                next_plus_one=True, out_dtype=None, out=None):
    v = _f(y)
    if post_weight is not None:
        v = v * torch.rsqrt((v * v).mean(-1, keepdim=True) + post_eps) * (_f(post_weight) + (1.0 if post_plus_one else 0.0))
    residual.copy_((_f(residual) + v).to(torch.float32))
    if next_weight is None:
        return None
    return rmsnorm(residual, next_weight, next_eps, next_plus_one, out_dtype or y.dtype, out)


def _rotate(x, positions, timescale, scale_factor):
    """x: [T, n, hd] float; half-split pairs."""
    half = x.shape[-1] // 2
    angle = _f(positions)[:, None, None] / _f(timescale)[None, None, :] / scale_factor
    s, c = torch.sin(angle), torch.cos(angle)
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat([x1 * c - x2 * s, x2 * c + x1 * s], -1)


def rope_cache_write(qkv, positions, timescale, scale_factor, q_div, num_heads, num_kv_heads, head_dim,
                     slot_mapping=None, k_pages=None, v_pages=None):
    T = qkv.shape[0]
    H, K, hd = num_heads, num_kv_heads, head_dim
    x = _f(qkv).reshape(T, H + 2 * K, hd)
    q, k, v = x[:, :H], x[:, H:H + K], x[:, H + K:]
    if timescale is not None:
        q = _rotate(q, positions, timescale, scale_factor)
        k = _rotate(k, positions, timescale, scale_factor)
    q = q / q_div
    qkv[:, :H * hd] = q.reshape(T, H * hd).to(qkv.dtype)
    if k_pages is not None:
        P = k_pages.shape[2]
        page, off = slot_mapping[:T] // P, slot_mapping[:T] % P
        # element d of the key goes where the layout of a stored page puts it (key_element_index below)
        at = key_element_index(P, hd, off[:, None], torch.arange(hd, device=off.device)[None, :])    # [T, hd]
        flat = k_pages.view(k_pages.shape[0], K, P * hd)
        flat[page[:, None, None], torch.arange(K, device=off.device)[None, :, None], at[:, None, :]] = k.to(k_pages.dtype)
        v_pages[page, :, :, off] = v.to(v_pages.dtype)     # value pages are [page, head, hd, page_size]
    return qkv


def rope(x, positions, timescale, scale_factor, div, num_heads, head_dim):
    T = x.shape[0]
    v = _f(x[:, :num_heads * head_dim]).reshape(T, num_heads, head_dim)
    v = _rotate(v, positions, timescale, scale_factor) / div
    x[:, :num_heads * head_dim] = v.reshape(T, -1).to(x.dtype)


def gather_rows(x, index, out_dtype=None, out=None):
    r = x[index.long()].to(out_dtype or x.dtype)
    if out is not None:
        out.copy_(r)
        return out
    return r


def fill_(t, value_bits=0):
    t.view(torch.int32).fill_(value_bits if value_bits < 2**31 else value_bits - 2**32)


def gelu_tanh(x):
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * x ** 3)))


def silu(x):
    return x * torch.sigmoid(x)


def squared_relu(x):
    return torch.relu(x) ** 2


def gelu_erf(x):
    return 0.5 * x * (1.0 + torch.erf(x / math.sqrt(2.0)))


ACTIVATIONS = (gelu_tanh, silu, squared_relu, gelu_erf)   # by the kernels' activation codes


def gemm(a, w, *, w2=None, soft_cap=None, out_dtype=None, out=None, algo=0, shape=0, activation=0, defer_sum=False,
         activate=None):
    # (defer_sum: the kernels may leave a sum to the caller; this stand-in never cuts a product)
    out_dtype = out_dtype or a.dtype
    if getattr(w, "paired", False):
        from simply_amd.kernels.packing import unpack_gate_up
        w, w2 = unpack_gate_up(w)
    c = _f(a) @ _f(w).T
    if w2 is not None:
        up = _f(a) @ _f(w2).T
        c = ACTIVATIONS[activation](_f(c.to(out_dtype))) * _f(up.to(out_dtype))
    elif soft_cap:
        c = soft_cap * torch.tanh(c / soft_cap)
    elif activate is not None:
        c = ACTIVATIONS[activate](_f(c.to(out_dtype)))
    c = c.to(out_dtype)
    if out is not None:
        out.copy_(c)
        return out
    return c


def key_element_index(P: int, hd: int, key: torch.Tensor, d: torch.Tensor) -> torch.Tensor:
    """Where element d of key `key` (its offset inside a page) lies in a stored page of keys, by the layout's own
    definition (simply_amd/csrc/api.h, sa_paged_attention): row-major [P][hd], unless P % 16 == 0 and hd % 32 == 0;
    then in blocks of 16 keys x 32 dimensions, block (key // 16, d // 32) a contiguous 512 elements holding element
    [(d % 32) // 8 * 16 + key % 16][d % 8] of a [64][8] array, the blocks of a group of 16 keys one after the other.
    (Index arithmetic of the test's own: the product's re-layout functions are not used.)"""
    if P % 16 or hd % 32:
        return key * hd + d
    block = (key // 16) * (hd // 32) + d // 32
    return block * 512 + ((d % 32) // 8 * 16 + key % 16) * 8 + d % 8


def stored_keys_as_rows(k_pages: torch.Tensor) -> torch.Tensor:
    """Pages of keys as the kernels store them [pages, heads, P, hd] -> row-major [pages, heads, P, hd]."""
    n, Kh, P, hd = k_pages.shape
    key = torch.arange(P, device=k_pages.device)[:, None].expand(P, hd)
    d = torch.arange(hd, device=k_pages.device)[None, :].expand(P, hd)
    index = key_element_index(P, hd, key, d).reshape(-1)
    return k_pages.reshape(n, Kh, P * hd)[:, :, index].reshape(n, Kh, P, hd)


def rows_as_stored_keys(rows: torch.Tensor) -> torch.Tensor:
    """Row-major pages of keys [pages, heads, P, hd] -> the kernels' storage order (same shape)."""
    n, Kh, P, hd = rows.shape
    key = torch.arange(P, device=rows.device)[:, None].expand(P, hd)
    d = torch.arange(hd, device=rows.device)[None, :].expand(P, hd)
    index = key_element_index(P, hd, key, d).reshape(-1)
    out = torch.empty_like(rows).reshape(n, Kh, P * hd)
    out[:, :, index] = rows.reshape(n, Kh, P * hd)
    return out.reshape(n, Kh, P, hd)


def paged_attention(q, k_pages, v_pages, block_table, token_seq, positions, num_heads, *, window, soft_cap, out=None,
                    algo=0):
    T = q.shape[0]
    _, Kh, P, hd = k_pages.shape
    k_pages = stored_keys_as_rows(k_pages)
    H = num_heads
    G = H // Kh
    res = torch.empty((T, H * hd), dtype=q.dtype, device=q.device)
    for t in range(T):
        pos = int(positions[t])
        lo = max(pos - window + 1, 0) if window else 0
        keys = torch.arange(lo, pos + 1, device=q.device)
        pages = block_table[int(token_seq[t]), keys // P].long()
        assert (pages >= 0).all(), "attention reads a key that has no page"
        k = _f(k_pages[pages, :, keys % P])          # [n, Kh, hd]
        v = _f(v_pages[pages, :, :, keys % P])       # [n, Kh, hd]
        qt = _f(q[t, :H * hd]).reshape(Kh, G, hd)
        s = torch.einsum("kgd,nkd->kgn", qt, k)
        if soft_cap:
            s = soft_cap * torch.tanh(s / soft_cap)
        p = torch.softmax(s, -1)
        res[t] = torch.einsum("kgn,nkd->kgd", p, v).reshape(H * hd).to(q.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def decode_attention_takes(q, k_pages, num_heads, max_q_len):
    return False


def paged_attention_sink(q, k_pages, v_pages, block_table, token_seq, positions, num_heads, *, scale=1.0, sinks=None,
                         window=None, soft_cap=None, out=None, slopes=None):
    T = q.shape[0]
    _, Kh, P, dk = k_pages.shape
    dv = v_pages.shape[2]
    k_pages = stored_keys_as_rows(k_pages)
    H = num_heads
    G = H // Kh
    res = torch.empty((T, H * dv), dtype=q.dtype, device=q.device)
    for t in range(T):
        pos = int(positions[t])
        lo = max(pos - window + 1, 0) if window else 0
        keys = torch.arange(lo, pos + 1, device=q.device)
        pages = block_table[int(token_seq[t]), keys // P].long()
        assert (pages >= 0).all(), "attention reads a key that has no page"
        k = _f(k_pages[pages, :, keys % P])          # [n, Kh, dk]
        v = _f(v_pages[pages, :, :, keys % P])       # [n, Kh, dv]
        qt = _f(q[t, :H * dk]).reshape(Kh, G, dk)
        s = torch.einsum("kgd,nkd->kgn", qt, k) * scale
        if soft_cap:
            s = soft_cap * torch.tanh(s / soft_cap)
        if slopes is not None:
            s = s - _f(slopes).reshape(Kh, G, 1) * (pos - keys).to(s.dtype)[None, None, :]
        if sinks is not None:
            s = torch.cat([s, _f(sinks).reshape(Kh, G, 1)], dim=-1)
        p = torch.softmax(s, -1)[..., :len(keys)]
        res[t] = torch.einsum("kgn,nkd->kgd", p, v).reshape(H * dv).to(q.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def residual_add_norm(y, residual, *, weight=None, eps=0.0, plus_one=False, mult=1.0, out_dtype=None, out=None):
    if hasattr(y, "materialize"):
        y = y.materialize()
    if y is not None:
        v = _f(y)
        if weight is not None:
            v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * (_f(weight) + (1.0 if plus_one else 0.0))
        residual.copy_((_f(residual) + mult * v).to(torch.float32))
    if out is None and out_dtype is None:
        return None
    r = residual.to(out_dtype or out.dtype)
    if out is not None:
        out.copy_(r)
        return out
    return r


GATE_SIGMOID, GATE_SILU = 0, 1


def gated_heads(x, gate, num_heads, size, *, kind, weight=None, eps=0.0, out_dtype=None, out=None, per_head=False):
    T = x.shape[0]
    v = _f(x).reshape(T, num_heads, size)
    if weight is not None:
        v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * _f(weight)
    g = _f(gate).reshape(T, num_heads, 1 if per_head else size)
    g = torch.sigmoid(g) if kind == GATE_SIGMOID else g * torch.sigmoid(g)
    r = (v * g).reshape(T, num_heads * size).to(out_dtype or (out.dtype if out is not None else x.dtype))
    if out is not None:
        out.copy_(r)
        return out
    return r


def activation_(x, activation):
    x.copy_(ACTIVATIONS[activation](_f(x)).to(x.dtype))
    return x


def qk_norm_rope_cache_write(proj, positions, inv_freq, rot_dims, eps, num_heads, num_kv_heads, key_dim, value_dim, *,
                             v_first=None, v_mix=None, slot_mapping=None, k_pages=None, v_pages=None, q_mult=1.0):
    T = proj.shape[0]
    H, K, dk, dv = num_heads, num_kv_heads, key_dim, value_dim
    qk = _f(proj[:, :(H + K) * dk]).reshape(T, H + K, dk).clone()
    if rot_dims:
        half = rot_dims // 2
        ang = (positions.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]).to(qk.dtype)[:, None, :]
        s, c = torch.sin(ang), torch.cos(ang)
        a, b = qk[..., :half].clone(), qk[..., half:rot_dims].clone()
        qk[..., :half] = a * c - b * s
        qk[..., half:rot_dims] = b * c + a * s
    if eps is not None:
        qk = qk / torch.sqrt((qk * qk).mean(-1, keepdim=True) + eps)
    proj[:, :H * dk] = (qk[:, :H] * q_mult).reshape(T, H * dk).to(proj.dtype)
    if k_pages is None:
        return proj
    P = k_pages.shape[2]
    v = _f(proj[:, (H + K) * dk:(H + K) * dk + K * dv])
    if v_first is not None:
        lam = _f(v_mix).reshape(())
        v = (1.0 - lam) * v + lam * _f(v_first)
    page, off = (slot_mapping[:T] // P).long(), (slot_mapping[:T] % P).long()
    krows = stored_keys_as_rows(k_pages)
    krows[page, :, off] = qk[:, H:].to(k_pages.dtype)
    k_pages.copy_(rows_as_stored_keys(krows))
    v_pages[page, :, :, off] = v.reshape(T, K, dv).to(v_pages.dtype)
    return proj


def short_conv_silu(x, taps, tails, seq_meta, num_seqs, max_q_len, *, update_tails=True, out=None):
    T, C = x.shape
    n = taps.shape[1]
    y = torch.empty((T, C), dtype=torch.float32, device=x.device) if out is None else out
    w = _f(taps)
    for slot, first, count, _ in seq_meta[:num_seqs].tolist():
        old = _f(tails[slot, :(n - 1) * C]).reshape(n - 1, C)
        xs = torch.cat([old, _f(x[first:first + count])], dim=0)
        acc = sum(xs[j:j + count] * w[:, j][None, :] for j in range(n))
        y[first:first + count] = (acc * torch.sigmoid(acc)).to(torch.float32)
        if update_tails and n > 1:
            tails[slot, :(n - 1) * C] = xs[count:].reshape(-1).to(torch.float32)
    return y


def delta_prepare(qkv, ab, a_log, dt_bias, num_heads, num_qk_heads, key_dim):
    T, C = qkv.shape
    H, G, dk = num_heads, num_qk_heads, key_dim
    qk = _f(qkv[:, :2 * G * dk]).reshape(T, 2 * G, dk)
    qk = qk / torch.sqrt((qk * qk).sum(-1, keepdim=True) + 1e-6)
    qk[:, :G] = qk[:, :G] * dk ** -0.5
    qkv[:, :2 * G * dk] = qk.reshape(T, -1).to(torch.float32)
    a, b = _f(ab[:, :H]), _f(ab[:, H:2 * H])
    g = torch.exp(-torch.exp(_f(a_log)) * torch.nn.functional.softplus(a + _f(dt_bias), threshold=30.0))
    return torch.cat([torch.sigmoid(b), g], dim=1).to(torch.float32)


def delta_inputs(x, taps, tails, ab, a_log, dt_bias, seq_meta, num_seqs, max_q_len, num_heads, num_qk_heads, key_dim):
    qkv = short_conv_silu(x, taps, tails, seq_meta, num_seqs, max_q_len)
    return qkv, delta_prepare(qkv, ab, a_log, dt_bias, num_heads, num_qk_heads, key_dim)


def delta_rule(qkv, gates, state, seq_meta, num_seqs, num_heads, num_qk_heads, key_dim, value_dim):
    T, C = qkv.shape
    H, G, dk, dv = num_heads, num_qk_heads, key_dim, value_dim
    out = torch.empty((T, H * dv), dtype=torch.float32, device=qkv.device)
    x, gt = _f(qkv), _f(gates)
    for slot, first, count, _ in seq_meta[:num_seqs].tolist():
        S = _f(state[slot, :H * dk * dv]).reshape(H, dv, dk).transpose(1, 2).clone()   # stored column by column
        for t in range(first, first + count):
            for h in range(H):
                j = h // (H // G)
                q, k = x[t, j * dk:(j + 1) * dk], x[t, (G + j) * dk:(G + j + 1) * dk]
                v = x[t, 2 * G * dk + h * dv:2 * G * dk + (h + 1) * dv]
                S[h] = gt[t, H + h] * S[h]
                u = gt[t, h] * (v - S[h].T @ k)
                S[h] = S[h] + torch.outer(k, u)
                out[t, h * dv:(h + 1) * dv] = (S[h].T @ q).to(torch.float32)
        state[slot, :H * dk * dv] = S.transpose(1, 2).reshape(-1).to(torch.float32)
    return out


# ---- sampling: the same counter-based generator as the kernel, in integer arithmetic


def philox4x32_10(counter, key):
    M0, M1, W0, W1 = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85
    c0, c1, c2, c3 = counter
    k0, k1 = key
    mask = 0xFFFFFFFF
    for _ in range(10):
        p0, p1 = M0 * c0, M1 * c2
        c0, c1, c2, c3 = ((p1 >> 32) ^ c1 ^ k0) & mask, p1 & mask, ((p0 >> 32) ^ c3 ^ k1) & mask, p0 & mask
        k0, k1 = (k0 + W0) & mask, (k1 + W1) & mask
    return c0, c1, c2, c3


def gumbel_noise(seed: int, counter: int, vocab: int) -> torch.Tensor:
    """float64 Gumbel noise for every vocabulary entry, from the kernel's random stream."""
    import numpy as np

    idx = np.arange(vocab, dtype=np.uint64)
    blocks = (vocab + 3) // 4
    M0, M1, W0, W1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57), 0x9E3779B9, 0xBB67AE85
    m32 = np.uint64(0xFFFFFFFF)
    c0 = np.arange(blocks, dtype=np.uint64)
    c1 = np.full(blocks, counter & 0xFFFFFFFF, dtype=np.uint64)
    c2 = np.zeros(blocks, dtype=np.uint64)
    c3 = np.zeros(blocks, dtype=np.uint64)
    k0, k1 = seed & 0xFFFFFFFF, (seed >> 32) & 0xFFFFFFFF
    for _ in range(10):
        p0, p1 = M0 * c0, M1 * c2
        n0 = ((p1 >> np.uint64(32)) ^ c1 ^ np.uint64(k0)) & m32
        n1 = p1 & m32
        n2 = ((p0 >> np.uint64(32)) ^ c3 ^ np.uint64(k1)) & m32
        n3 = p0 & m32
        c0, c1, c2, c3 = n0, n1, n2, n3
        k0, k1 = (k0 + W0) & 0xFFFFFFFF, (k1 + W1) & 0xFFFFFFFF
    words = np.stack([c0, c1, c2, c3], axis=1).reshape(-1)[:vocab]
    u = ((words >> np.uint64(8)).astype(np.float64) + 0.5) / 16777216.0
    return torch.from_numpy(-np.log(-np.log(u)))


def sample(logits, temperature, top_k, top_p, seed, counter, tokens=None, logprobs=None, modes=7):
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    import plain_gemma2 as plain

    R, V = logits.shape
    toks = torch.empty(R, dtype=torch.int32)
    lps = torch.empty(R, dtype=torch.float32)
    for r in range(R):
        row = logits[r].double().cpu()
        t, k, p = float(temperature[r]), int(top_k[r]), float(top_p[r])
        if t == 0.0 or k == 1:
            toks[r], lps[r] = int(torch.argmax(row)), 0.0
            continue
        x = row / t
        keep = torch.ones(V, dtype=torch.bool)
        if k > 0:
            keep &= x >= torch.topk(x, min(k, V)).values[-1]
        if p < 1.0:
            xm = torch.where(keep, x, torch.full_like(x, -float("inf")))
            keep &= plain.top_p_mask(xm, p)
        xm = torch.where(keep, x, torch.full_like(x, -float("inf")))
        g = gumbel_noise(int(seed[r]) & (2**64 - 1), int(counter[r]), V)
        tok = int(torch.argmax(xm + g))
        toks[r] = tok
        lps[r] = float(torch.log_softmax(xm, -1)[tok])
    toks, lps = toks.to(logits.device), lps.to(logits.device)
    if tokens is not None:
        tokens[:R] = toks
        toks = tokens
    if logprobs is not None:
        logprobs[:R] = lps
        lps = logprobs
    return toks, lps


SCORE_MASKED = -0.5 * 3.4028234663852886e38


def score(logits, temperature, top_k, top_p, tokens, scores=None):
    """simply/utils/sampling_lib.py:540-601: the log-probability of a given token under temperature, top-k, top-p."""
    import sys, os
    sys.path.insert(0, os.path.dirname(__file__))
    import plain_gemma2 as plain

    R, V = logits.shape
    out = torch.empty(R, dtype=torch.float32)
    for r in range(R):
        row = logits[r].double().cpu()
        t, k, p, tok = float(temperature[r]), int(top_k[r]), float(top_p[r]), int(tokens[r])
        if t == 0.0 or k == 1:
            out[r] = 0.0 if int(torch.argmax(row)) == tok else SCORE_MASKED
            continue
        x = row / t
        keep = torch.ones(V, dtype=torch.bool)
        if k > 0:
            keep &= x >= torch.topk(x, min(k, V)).values[-1]
        if p < 1.0:
            xm = torch.where(keep, x, torch.full_like(x, -float("inf")))
            keep &= plain.top_p_mask(xm, p)
        xm = torch.where(keep, x, torch.full_like(x, -float("inf")))
        out[r] = float(torch.log_softmax(xm, -1)[tok]) if bool(keep[tok]) else SCORE_MASKED
    out = out.to(logits.device)
    if scores is not None:
        scores[:R] = out
        out = scores
    return out


# --------------------------------------------------------------------------- token tables, biases, sums of two mixers

def embed_sum(tokens, positions, seq_meta, num_seqs, max_q_len, table, *, pair=None, mul_prev=0, mul_cur=0, last=None,
              pos=None):
    T, D = tokens.shape[0], table.shape[1]
    out = torch.zeros((T, D), dtype=torch.float64 if PRECISE else torch.float32, device=table.device)
    for slot, first, count, _ in seq_meta[:num_seqs].tolist():
        for j in range(count):
            t = first + j
            tok, p = int(tokens[t]), int(positions[t])
            v = _f(table[tok])
            if pair is not None:
                buckets = pair.shape[0] - 1
                before = int(tokens[t - 1]) if j > 0 else int(last[slot, 0])
                row = (before * mul_prev + tok * mul_cur) % buckets if p > 0 else buckets
                v = v + _f(pair[row])
            if pos is not None:
                v = v + _f(pos[p])
            out[t] = v
        if pair is not None and count > 0:
            last[slot, 0] = int(tokens[first + count - 1])
    return out.to(torch.float32)


def _activation(code, x):
    return ACTIVATIONS[code](x)


def token_gate_(z, tokens, table, col0, activation):
    e = _f(table[tokens.long()][:, col0:col0 + z.shape[1]])
    z.copy_((_activation(activation, _f(z)) * e).to(z.dtype))
    return z


def bias_add_(x, bias):
    x.copy_((_f(x) + _f(bias)).to(x.dtype))
    return x


def weighted_sum(x, a, y, b, out=None):
    r = (a * _f(x) + b * _f(y)).to(x.dtype)
    if out is not None:
        out.copy_(r)
        return out
    return r


# --------------------------------------------------------------------------- matrix states that decay

def exp_gates(raw, bias, cap, num_heads, m_state, seq_meta, num_seqs):
    H = num_heads
    x = _f(raw) + (_f(bias) if bias is not None else 0.0)
    ig = cap * torch.tanh(x[:, :H] / cap)
    fg = torch.nn.functional.logsigmoid(cap * torch.tanh(x[:, H:] / cap))
    out = torch.zeros((raw.shape[0], 3 * H), dtype=x.dtype, device=raw.device)
    for slot, first, count, _ in seq_meta[:num_seqs].tolist():
        m = _f(m_state[slot])
        for t in range(first, first + count):
            new = torch.maximum(fg[t] + m, ig[t])
            out[t, :H], out[t, H:2 * H], out[t, 2 * H:] = torch.exp(fg[t] + m - new), torch.exp(ig[t] - new), torch.exp(-new)
            m = new
        if count > 0:
            m_state[slot] = m.to(torch.float32)
    return out.to(torch.float32)


def linear_state(proj, q_at, k_at, v_at, q_mult, gates, scalar, num_heads, key_dim, value_dim, ones, state, seq_meta,
                 num_seqs, *, decay_bias=None, tau=None):
    H, dk, dv = num_heads, key_dim, value_dim
    if tau is not None:   # the gates are z: a = sigmoid(z + bias)^(1 / tau)
        z = _f(gates) + (_f(decay_bias) if decay_bias is not None else 0.0)
        gates = torch.exp(torch.nn.functional.logsigmoid(z) / tau)
    CT = dv + int(bool(ones))
    T = proj.shape[0]
    p, g = _f(proj), _f(gates)
    out = torch.zeros((T, H * CT), dtype=p.dtype, device=proj.device)
    for slot, first, count, _ in seq_meta[:num_seqs].tolist():
        S = _f(state[slot, :H * dk * CT]).view(H, CT, dk).clone()   # column by column
        for t in range(first, first + count):
            q = p[t, q_at:q_at + H * dk].view(H, dk) * q_mult
            k = p[t, k_at:k_at + H * dk].view(H, dk)
            v = p[t, v_at:v_at + H * dv].view(H, dv)
            if ones:
                v = torch.cat([v, torch.ones((H, 1), dtype=v.dtype, device=v.device)], dim=1)
            if scalar:
                a, c = g[t, :H].view(H, 1, 1), g[t, H:2 * H].view(H, 1)
            else:
                a, c = g[t, :H * dk].view(H, 1, dk), 1.0
            S = a * S + (c * v)[:, :, None] * k[:, None, :]
            out[t] = torch.einsum("hcd,hd->hc", S, q).reshape(-1)
        if count > 0:
            state[slot, :H * dk * CT] = S.reshape(-1).to(torch.float32)
    return out.to(torch.float32)


def normalized_readout(x, floor, gate, weight, eps, num_heads, size, out_dtype):
    T, H = x.shape[0], num_heads
    xs = _f(x).view(T, H, size + 1)
    o = xs[:, :, :size] / (torch.maximum(xs[:, :, size:].abs(), _f(floor)[:, :, None]) + 1e-6)
    o = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + eps)
    o = o.reshape(T, H * size) * _f(weight) * torch.sigmoid(_f(gate))
    return o.to(out_dtype)


# --------------------------------------------------------------------------- routed experts

def route(logits, top, scale):
    s = torch.softmax(_f(logits), -1)
    best = torch.topk(s, top, dim=-1)
    return best.indices.to(torch.int32).contiguous(), (best.values * scale).to(torch.float32).contiguous()


def route_choice(logits, top, scale, *, correction=None, groups=1, keep=1):
    s = torch.sigmoid(_f(logits))
    T, E = s.shape
    c = s + _f(correction) if correction is not None else s.clone()
    if groups > 1:
        per = E // groups
        by_group = c.reshape(T, groups, per)
        score = torch.topk(by_group, min(2, per), dim=-1).values.sum(-1)
        stay = torch.zeros(T, groups, dtype=torch.bool, device=s.device)
        stay.scatter_(1, torch.topk(score, keep, dim=-1).indices, True)
        c = torch.where(stay[:, :, None].expand(T, groups, per).reshape(T, E), c, torch.full_like(c, float("-inf")))
    chosen = torch.topk(c, top, dim=-1).indices
    return chosen.to(torch.int32).contiguous(), (torch.gather(s, 1, chosen) * scale).to(torch.float32).contiguous()


def routed_experts(x, experts, weights, gate_w, up_w, down_w, activation, *, shared=None, shared_gate=None,
                   out_dtype=None):
    from simply_amd.kernels.packing import TiledWeight, unpack_tiles

    def matrix(stack, e):
        if stack.tiled:
            return _f(unpack_tiles(TiledWeight(stack.data[e], stack.rows, stack.cols)))
        return _f(stack.data[e])

    T, D = x.shape
    xf = _f(x)
    out = torch.zeros((T, D), dtype=xf.dtype, device=x.device)
    for t in range(T):
        for k in range(experts.shape[1]):
            e = int(experts[t, k])
            if gate_w is None:   # experts without a gate
                h = _activation(activation, (xf[t] @ matrix(up_w, e).T).to(x.dtype).to(xf.dtype))
            else:
                h = _activation(activation, (xf[t] @ matrix(gate_w, e).T).to(x.dtype).to(xf.dtype)) \
                    * (xf[t] @ matrix(up_w, e).T).to(x.dtype).to(xf.dtype)
            out[t] += _f(weights[t, k]) * (h.to(x.dtype).to(xf.dtype) @ matrix(down_w, e).T)
    if shared is not None:
        s = _f(shared)
        out = out + (s * torch.sigmoid(_f(shared_gate)[:, :1]) if shared_gate is not None else s)
    return out.to(out_dtype or x.dtype)


# --------------------------------------------------------------------------- attention with several maps, latents, rglru


def residual_add_next_norm(y, residual, weight, *, eps, plus_one=False, mult=1.0, out_dtype=None):
    if hasattr(y, "materialize"):
        y = y.materialize()
    if y is not None:
        residual.copy_((_f(residual) + mult * _f(y)).to(torch.float32))
    h = _f(residual)
    out = h / torch.sqrt((h * h).mean(-1, keepdim=True) + eps) * (_f(weight) + (1.0 if plus_one else 0.0))
    return out.to(out_dtype or (y.dtype if y is not None else torch.float32))


def paged_attention_maps(q, k_pages, v_pages, block_table, token_seq, positions, num_heads, *, scale, maps=1,
                         value_dim=None, window=None, differential=None, out=None):
    T = q.shape[0]
    _, Kh, P, row = k_pages.shape
    dk = row // maps
    krows = stored_keys_as_rows(k_pages)
    dv = v_pages.shape[2] if v_pages is not None else int(value_dim)
    H = num_heads
    G = H // Kh
    width = H * (1 if differential is not None else maps) * dv
    res = torch.empty((T, width), dtype=q.dtype, device=q.device)
    for t in range(T):
        pos = int(positions[t])
        lo = max(pos - window + 1, 0) if window else 0
        keys = torch.arange(lo, pos + 1, device=q.device)
        pages = block_table[int(token_seq[t]), keys // P].long()
        assert (pages >= 0).all(), "attention reads a key that has no page"
        k = _f(krows[pages, :, keys % P]).reshape(len(keys), Kh, maps, dk)
        v = _f(v_pages[pages, :, :, keys % P]) if v_pages is not None else _f(krows[pages, :, keys % P])[..., :dv]
        qt = _f(q[t, :H * maps * dk]).reshape(Kh, G, maps, dk)
        p = torch.softmax(torch.einsum("kgmd,nkmd->kgmn", qt, k) * scale, -1)
        a = torch.einsum("kgmn,nkd->kgmd", p, v)            # [Kh, G, maps, dv]
        if differential is not None:
            lam, eps, mult = differential
            o = a[:, :, 0] - lam * a[:, :, 1]
            a = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * mult
        res[t] = a.reshape(width).to(q.dtype)
    if out is not None:
        out.copy_(res)
        return out
    return res


def norm_rope_cache_write(proj, positions, freq, rot_dims, num_heads, num_kv_heads, key_dim, value_dim, *, rot_mult=1.0,
                          sub=1, eps=0.0, q_weight=None, q_norm_dims=0, q_rot_at=0, k_weight=None, k_norm_dims=0,
                          k_rot_at=0, slot_mapping=None, k_pages=None, v_pages=None, key_values=0):
    T = proj.shape[0]
    H, K, dk, dv = num_heads, num_kv_heads, key_dim, value_dim
    ds = dk // sub
    ang = None
    if rot_dims:
        ang = positions.to(torch.float32)[:, None] * freq.to(torch.float32)[None, :]       # 32-bit angles
        ang = ang.to(torch.float64 if PRECISE else torch.float32)[:, None, :]

    def treat(x, weight, norm_dims, rot_at):    # x [T, n, ds]
        x = x.clone()
        if weight is not None and norm_dims:
            part = x[..., :norm_dims]
            x[..., :norm_dims] = part / torch.sqrt((part * part).mean(-1, keepdim=True) + eps) * _f(weight)[:norm_dims]
        if rot_dims:
            s, c = torch.sin(ang) * rot_mult, torch.cos(ang) * rot_mult
            a = x[..., rot_at:rot_at + rot_dims:2].clone()
            b = x[..., rot_at + 1:rot_at + rot_dims:2].clone()
            x[..., rot_at:rot_at + rot_dims:2] = a * c - b * s
            x[..., rot_at + 1:rot_at + rot_dims:2] = b * c + a * s
        return x

    if H:
        q = treat(_f(proj[:, :H * dk]).reshape(T, H * sub, ds), q_weight, q_norm_dims, q_rot_at)
        proj[:, :H * dk] = q.reshape(T, H * dk).to(proj.dtype)
    if k_pages is None or K == 0:
        return proj
    k = treat(_f(proj[:, H * dk:(H + K) * dk]).reshape(T, K * sub, ds), k_weight, k_norm_dims, k_rot_at)
    P = k_pages.shape[2]
    page, off = (slot_mapping[:T] // P).long(), (slot_mapping[:T] % P).long()
    krows = stored_keys_as_rows(k_pages)
    krows[page, :, off] = k.reshape(T, K, dk).to(k_pages.dtype)
    k_pages.copy_(rows_as_stored_keys(krows))
    if key_values:
        v_pages[page, :, :, off] = k.reshape(T, K, dk)[..., :key_values].to(v_pages.dtype)
    if dv:
        v = proj[:, (H + K) * dk:(H + K) * dk + K * dv]
        v_pages[page, :, :, off] = v.reshape(T, K, dv).to(v_pages.dtype)
    return proj


def attention_maps_units_takes(q, k_pages, v_pages, num_heads, maps=1):
    return False


def short_conv(x, taps, tails, seq_meta, num_seqs, max_q_len, *, in_bias=None, out_bias=None, silu=False,
               update_tails=True):
    T, C = x.shape
    n = taps.shape[1]
    y = torch.empty((T, C), dtype=torch.float32, device=x.device)
    w = _f(taps)
    for slot, first, count, _ in seq_meta[:num_seqs].tolist():
        old = _f(tails[slot, :(n - 1) * C]).reshape(n - 1, C)
        new = _f(x[first:first + count])
        if in_bias is not None:
            new = new + _f(in_bias)[None, :]
        xs = torch.cat([old, new], dim=0)
        acc = sum(xs[j:j + count] * w[:, j][None, :] for j in range(n))
        if out_bias is not None:
            acc = acc + _f(out_bias)[None, :]
        y[first:first + count] = (acc * torch.sigmoid(acc) if silu else acc).to(torch.float32)
        if update_tails and n > 1:
            tails[slot, :(n - 1) * C] = xs[count:].reshape(-1).to(torch.float32)
    return y


def head_product(x, w, *, in_stride=None, tail=0, gate=None, out_dtype=None):
    T = x.shape[0]
    H, O, I = w.shape
    hs = in_stride if in_stride is not None else I + tail
    xf = _f(x)
    heads = torch.stack([xf[:, h * hs:h * hs + I + tail] for h in range(H)], dim=1)       # [T, H, I + tail]
    o = torch.einsum("thi,hoi->tho", heads[..., :I], _f(w))
    if gate is not None:
        o = o * torch.sigmoid(_f(gate))[:, :, None]
    return torch.cat([o, heads[..., I:]], dim=-1).reshape(T, H * (O + tail)).to(out_dtype or x.dtype)


def rglru_scan(u, gates, block, r_bias, i_bias, lam, y, y_bias, state, seq_meta, num_seqs, *, c=8.0, out_dtype=None,
               max_q_len=None):
    T, C = u.shape
    g = _f(gates).reshape(T, C // block, 2, block)
    r = torch.sigmoid(g[:, :, 0].reshape(T, C) + _f(r_bias))
    i = torch.sigmoid(g[:, :, 1].reshape(T, C) + _f(i_bias))
    lm = _f(lam)
    sp = torch.where(lm > 30.0, lm, torch.log1p(torch.exp(torch.clamp(lm, max=30.0))))
    log_a = -c * r * sp
    a, m = torch.exp(log_a), torch.sqrt(-torch.expm1(2.0 * log_a))
    z = _f(y) + (_f(y_bias) if y_bias is not None else 0.0)
    gy = gelu_tanh(z)
    uf = _f(u)
    out = torch.empty((T, C), dtype=out_dtype or y.dtype, device=u.device)
    for slot, first, count, _ in seq_meta[:num_seqs].tolist():
        S = _f(state[slot, :C])
        for t in range(first, first + count):
            S = a[t] * S + m[t] * (i[t] * uf[t])
            out[t] = (S * gy[t]).to(out.dtype)
        state[slot, :C] = S.to(torch.float32)
    return out


# --------------------------------------------------------------------------- what a windowed attention reads


def attention_inputs(proj, seq_meta, num_seqs, max_q_len, num_heads, num_kv_heads, key_dim, value_dim, *,
                     values_are_keys=False, taps=None, tails=None, norm=None, q_weight=None, k_weight=None, eps=0.0,
                     inv_freq=None, rot_dims=0, temp_coef=0.0, temp_every=0, q_mult=1.0, taps_by_tap=None, in_bias=None,
                     slot_mapping=None, k_pages=None, v_pages=None):
    H, K, dk, dv = num_heads, num_kv_heads, key_dim, value_dim
    own = k_pages is not None
    C = (H + K) * dk + (0 if values_are_keys else K * dv) if own else H * dk
    T = proj.shape[0]
    x = _f(proj[:, :C]).clone()
    if in_bias is not None:
        x = x + _f(in_bias)[:C]
    if taps is not None:
        n, w = taps.shape[1], _f(taps)
        for slot, first, count, _ in seq_meta[:num_seqs].tolist():
            new = x[first:first + count].clone()
            old = _f(tails[slot, :(n - 1) * C]).reshape(n - 1, C) if n > 1 else new[:0]
            xs = torch.cat([old, new], dim=0)
            x[first:first + count] = sum(xs[j:j + count] * w[:, j][None, :] for j in range(n))
            if n > 1:
                tails[slot, :(n - 1) * C] = xs[count:].reshape(-1).to(torch.float32)
    pos = torch.empty(T, dtype=torch.long, device=proj.device)
    for slot, first, count, start in seq_meta[:num_seqs].tolist():
        pos[first:first + count] = torch.arange(start, start + count, device=proj.device)

    def prepared(rows, heads, weight):
        v = rows.reshape(T, heads, dk)
        if norm == "head":
            v = v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps) * _f(weight)
        elif norm == "row":
            flat = v.reshape(T, heads * dk)
            v = (flat / torch.sqrt((flat * flat).mean(-1, keepdim=True) + eps) * _f(weight)).reshape(T, heads, dk)
        if rot_dims:
            half = rot_dims // 2
            a = pos.to(torch.float32)[:, None] * inv_freq.to(torch.float32)[None, :]
            cos, sin = torch.cos(a).to(v.dtype)[:, None, :], torch.sin(a).to(v.dtype)[:, None, :]
            u, w_ = v[..., :half], v[..., half:rot_dims]
            v = torch.cat([u * cos - w_ * sin, w_ * cos + u * sin, v[..., rot_dims:]], dim=-1)
        return v

    q = prepared(x[:, :H * dk], H, q_weight)
    if temp_every:
        q = q * (1.0 + temp_coef * torch.log(torch.floor((pos + 1) / temp_every) + 1.0)).to(q.dtype)[:, None, None]
    if own:
        k_raw = x[:, H * dk:(H + K) * dk]
        k = prepared(k_raw, K, k_weight)
        v = k_raw.reshape(T, K, dk) if values_are_keys else x[:, (H + K) * dk:C].reshape(T, K, dv)
        P = k_pages.shape[2]
        rows = stored_keys_as_rows(k_pages)
        keep = slot_mapping[:T] >= 0
        page, off = (slot_mapping[:T] // P)[keep], (slot_mapping[:T] % P)[keep]
        rows[page, :, off] = k[keep].to(k_pages.dtype)
        k_pages.copy_(rows_as_stored_keys(rows))
        v_pages[page, :, :, off] = v[keep].to(v_pages.dtype)
    return (q * q_mult).reshape(T, H * dk).to(proj.dtype)
