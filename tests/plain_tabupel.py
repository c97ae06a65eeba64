"""A plain, slow Tabupel decoder: whole sequences, no cache, one function per mechanism.

It shares no code with the `simply_amd` package: it reads `config.json` and `model.safetensors` itself and
computes with ordinary torch operations on the CPU in the dtype it is asked for (float64 for the tests).

The design, in this file's notation (x: residual stream [T, D]; rows of a weight are outputs):

  layer        x <- x + m * mixer(rms(x; norm1));  x <- x + m * ffn(rms(x; norm2))   (no second step without an ffn)
               rms(y; w) = y / sqrt(mean(y^2) + eps) * w;  a layer may use another layer's tensors
  attention    two score maps per head over the same values: q and k hold, per head, [map 1 | map 2]; every map of
               every head is normed (a weight shared by all), then its first dimensions are rotated in neighbouring
               pairs with frequencies divided by a constant; a_m = softmax(scale q_m.k_m over the window) v;
               o = a_1 - lambda a_2 with lambda = exp(lq1.lk1) - exp(lq2.lk2) + diff; o / rms(o) * (1 - diff)
  latent       c_q = rms(W_dq h; w) -> q = W_uq c_q, per head [plain | rotated]; W_dkv h -> [c | r]: c normed is the
               latent, r rotated is one key part for all heads; per head k = [W_uk c | r], v = W_uv c; softmax over the
               window; heads * sigmoid(W_g h); rotation with frequencies blended between f and f / factor by a ramp
               over the dimensions, cos and sin times 0.1 ln(factor) + 1
  rglru        y = gelu(W_y h + b), u = conv(W_x h + b); per block r = sigmoid(R u + b), i = sigmoid(I u + b);
               a = exp(-8 r softplus(lam)); S <- a S + sqrt(1 - a^2) i u; out = W_o (S y)
  ffn          down(silu(gate x) * up x)
  output       cap * tanh(head(rms(x; final.norm)) / cap)
"""
from __future__ import annotations

import json
import math
import os

import torch


def load(model_dir: str):
    """(weights by tensor name as stored, config.json as a dict)."""
    from safetensors import safe_open

    with open(os.path.join(model_dir, "config.json")) as f:
        cfg = json.load(f)
    w = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt", device="cpu") as h:
        for name in h.keys():
            w[name] = h.get_tensor(name)
    return w, cfg


# --------------------------------------------------------------------------- small functions


def rms_norm(x: torch.Tensor, weight: torch.Tensor | None, eps: float) -> torch.Tensor:
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


# --------------------------------------------------------------------------- rotation


def linear_frequencies(dims: int, base: float, factor: float = 1.0, dtype=torch.float64) -> torch.Tensor:
    """f_i = base^(-2 i / dims) / factor, i < dims / 2."""
    i = torch.arange(dims // 2, dtype=torch.float64)
    return ((float(base) ** (-2.0 * i / dims)) / float(factor)).to(dtype)


def ramp_frequencies(dims: int, base: float, factor: float, original: float, fast: float, slow: float,
                     dtype=torch.float64) -> tuple[torch.Tensor, float]:
    """Frequencies blended between f_i (where the ramp is 0) and f_i / factor (where it is 1), and the factor on
    cos and sin.  The ramp runs over the index i between the dimensions at which `fast` and `slow` turns fit into
    `original` positions."""
    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(fast)), 0)
    hi = min(math.ceil(dim_of(slow)), dims - 1)
    i = torch.arange(dims // 2, dtype=torch.float64)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    f = float(base) ** (-2.0 * i / dims)
    return (f / float(factor) * ramp + f * (1.0 - ramp)).to(dtype), 0.1 * math.log(float(factor)) + 1.0


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor, mult: float = 1.0) -> torch.Tensor:
    """x [T, ..., size]: entries (2i, 2i + 1), i < len(freq), turn by positions * freq[i]; cos and sin times `mult`;
    the other entries pass unchanged."""
    n = freq.numel()
    if n == 0:
        return x
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [n]
    ang = (positions.to(freq.dtype)[:, None] * freq[None, :]).to(x.dtype).reshape(shape)
    c, s = torch.cos(ang) * mult, torch.sin(ang) * mult
    a, b = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    rot = torch.stack([a * c - b * s, b * c + a * s], dim=-1).reshape(*x.shape[:-1], 2 * n)
    return torch.cat([rot, x[..., 2 * n:]], dim=-1)


def rot_of(rot: dict | None, dims_default: int | None = None, dtype=torch.float64):
    """(frequencies, factor on cos and sin) of a mixer's "rot" entry (None: no rotation)."""
    if rot is None:
        return torch.zeros(0, dtype=dtype), 1.0
    dims = int(rot.get("dims", dims_default))
    sc = rot.get("scaling")
    if sc is None:
        return linear_frequencies(dims, rot["base"], 1.0, dtype), 1.0
    if "original" in sc:
        return ramp_frequencies(dims, rot["base"], sc["factor"], sc["original"], sc["fast"], sc["slow"], dtype)
    return linear_frequencies(dims, rot["base"], sc["factor"], dtype), 1.0


# --------------------------------------------------------------------------- softmax over a window


def window_mask(T: int, window: int | None) -> torch.Tensor:
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    m = j <= i
    if window:
        m = m & (i - j < window)
    return m


def windowed_softmax_attention(q, k, v, scale: float, window: int | None) -> torch.Tensor:
    """q [T, dk], k [T, dk], v [T, dv] of one head -> [T, dv]."""
    s = (q @ k.T) * scale
    s = s.masked_fill(~window_mask(q.shape[0], window), float("-inf"))
    return torch.softmax(s, dim=-1) @ v


# --------------------------------------------------------------------------- mixers


def differential_attention(h, p, m, eps: float, positions=None):
    """h [T, D]; p: the mixer's tensors by their short names; m: its config entry."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    positions = torch.arange(T) if positions is None else positions
    q = (h @ p["q"].T).reshape(T, H, 2, dk)
    k = (h @ p["k"].T).reshape(T, G, 2, dk)
    v = (h @ p["v"].T).reshape(T, G, dv)
    q = rms_norm(q, p["q.norm"], eps)
    k = rms_norm(k, p["k.norm"], eps)
    freq, mult = rot_of(m.get("rot"), dtype=torch.float64)
    q = rotate_pairs(q, positions, freq, mult)
    k = rotate_pairs(k, positions, freq, mult)
    lam = float(torch.exp((p["lq1"] * p["lk1"]).sum()) - torch.exp((p["lq2"] * p["lk2"]).sum())) + m["diff"]
    window = (m.get("mask") or {}).get("size")
    out = []
    for hd in range(H):
        g = hd // (H // G)
        a1 = windowed_softmax_attention(q[:, hd, 0], k[:, g, 0], v[:, g], m["scale"], window)
        a2 = windowed_softmax_attention(q[:, hd, 1], k[:, g, 1], v[:, g], m["scale"], window)
        out.append(rms_norm(a1 - lam * a2, None, eps) * (1.0 - m["diff"]))
    return torch.cat(out, dim=-1) @ p["o"].T


def latent_attention(h, p, m, eps: float, positions=None):
    T = h.shape[0]
    H, dk, dr, dv, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    positions = torch.arange(T) if positions is None else positions
    cq = rms_norm(h @ p["dq"].T, p["dq.norm"], eps)
    q = (cq @ p["uq"].T).reshape(T, H, dk + dr)
    dkv = h @ p["dkv"].T
    c = rms_norm(dkv[:, :rank], p["dkv.norm"], eps)
    freq, mult = rot_of(m.get("rot"), dr, dtype=torch.float64)
    kr = rotate_pairs(dkv[:, rank:], positions, freq, mult)             # [T, dr], one for all heads
    qr = rotate_pairs(q[:, :, dk:], positions, freq, mult)
    kn = (c @ p["uk"].T).reshape(T, H, dk)
    v = (c @ p["uv"].T).reshape(T, H, dv)
    gate = torch.sigmoid(h @ p["g"].T)                                  # [T, H]
    window = (m.get("mask") or {}).get("size")
    out = []
    for hd in range(H):
        qh = torch.cat([q[:, hd, :dk], qr[:, hd]], dim=-1)
        kh = torch.cat([kn[:, hd], kr], dim=-1)
        out.append(windowed_softmax_attention(qh, kh, v[:, hd], m["scale"], window) * gate[:, hd:hd + 1])
    return torch.cat(out, dim=-1) @ p["o"].T


def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
    """x [T, C], taps [C, n]: y[t, c] = sum_j taps[c, j] * x[t - (n - 1 - j), c] (+ bias), zeros before the start."""
    T, C = x.shape
    n = taps.shape[1]
    padded = torch.cat([torch.zeros(n - 1, C, dtype=x.dtype), x], dim=0)
    y = torch.zeros_like(x) if bias is None else bias[None, :].expand(T, C).clone()
    for j in range(n):
        y = y + padded[j:j + T] * taps[:, j][None, :]
    return y


def block_gates(u, w, b):
    """u [T, C] cut into len(w) equal parts; part k goes through the square matrix w[k] ([out, in]) and bias b[k]."""
    B = w.shape[0]
    parts = u.reshape(u.shape[0], B, -1)
    return torch.sigmoid(torch.einsum("tbi,boi->tbo", parts, w) + b[None]).reshape(u.shape)


def gated_linear_recurrence(u, r, i, lam, state=None):
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with a_t = exp(-8 r_t softplus(lam)), from S = 0."""
    S = torch.zeros_like(u[0]) if state is None else state
    sp = softplus(lam)
    out = []
    for t in range(u.shape[0]):
        a = torch.exp(-8.0 * r[t] * sp)
        S = a * S + torch.sqrt(1.0 - a * a) * i[t] * u[t]
        out.append(S)
    return torch.stack(out)


def rglru(h, p, m, eps: float = 0.0, positions=None):
    y = gelu_tanh(h @ p["y"].T + p["y.b"])
    u = causal_conv(h @ p["x"].T + p["x.b"], p["conv"], p["conv.b"])
    r = block_gates(u, p["ra"], p["ra.b"])
    i = block_gates(u, p["ri"], p["ri.b"])
    S = gated_linear_recurrence(u, r, i, p["lam"])
    return (S * y) @ p["o"].T


def gated_ffn(x, p):
    return (silu(x @ p["gate"].T) * (x @ p["up"].T)) @ p["down"].T


MIXERS = {"attention": differential_attention, "latent_attention": latent_attention, "rglru": rglru}


# --------------------------------------------------------------------------- the model


def part_tensors(w, prefix: str, dtype) -> dict:
    return {name[len(prefix):]: t.to(dtype) for name, t in w.items() if name.startswith(prefix)}


def forward(w, cfg, tokens, dtype=torch.float64, layers_out: list | None = None) -> torch.Tensor:
    """tokens: a list of ids of one sequence -> logits [T, vocab] in `dtype`."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = w["embed"].to(dtype)[torch.as_tensor(tokens, dtype=torch.long)]
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        pre = f"l{src}."
        h = rms_norm(x, w[pre + "norm1"].to(dtype), eps)
        x = x + mult * MIXERS[layer["type"]](h, part_tensors(w, pre + "mix.", dtype), layer["mixer"], eps)
        if layer.get("mlp") is not None:
            h = rms_norm(x, w[pre + "norm2"].to(dtype), eps)
            x = x + mult * gated_ffn(h, part_tensors(w, pre + "mlp.", dtype))
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = rms_norm(x, w["final.norm"].to(dtype), eps) @ w["head"].to(dtype).T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits


def greedy(w, cfg, prompt, steps: int, dtype=torch.float64) -> list[int]:
    """`steps` tokens after `prompt`, each the largest logit's, the whole sequence run anew every time."""
    tokens = list(prompt)
    for _ in range(steps):
        tokens.append(int(forward(w, cfg, tokens, dtype)[-1].argmax()))
    return tokens[len(prompt):]
