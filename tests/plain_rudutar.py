"""A plain, slow Rudutar decoder: whole sequences, no cache, one function per mechanism.

It shares no code with the `simply_amd` package: it reads `config.json` and `model.safetensors` itself and
computes with ordinary torch operations on the CPU in the dtype it is asked for (float64 for the tests).

The design, in this file's notation (x: residual stream [T, D]; rows of a weight are outputs; positions from 0):

  embedding    x = rms(embed[token]; embed.norm)
  layer        x <- x + mixer(rms(x; norm1));  x <- x + ffn(rms(x; norm2))   (no second step without an ffn)
               rms(y; w) = y / sqrt(mean(y^2) + eps) * w
  attention    q, k, v = conv(W h): a causal convolution per channel, taps oldest first, zeros before the start;
               q and k normed head by head with a weight that the heads share; q_p times
               1 + coef ln(floor((p + 1) / every) + 1); s_ij = scale q_i.k_j - 2^(-8 (h + 1) / H) (i - j) for
               0 <= i - j < window; p_ij = exp(s_ij) / (1 + sum_j exp(s_ij)); heads * sigmoid(W_g h) entry by entry;
               a layer with "kv_from": j reads layer j's k (convolved, normed) and v (convolved) and has none itself
  attention_2  q = W_q h + b, k = W_k h + b, v = k; q and k normed over the whole row (all heads at once, a weight
               per entry), then the first `dims` entries of every head rotated in pairs (i, i + dims / 2) by
               p base^(-2 i / dims); softmax(scale q.k) over the window; head h times sigmoid(W_g h)_h
  ffn          dense: down(gelu(up x)) with the exact gelu;  moe: s = sigmoid(W_r x), choice c = s + correction;
               experts in equal groups of neighbours, a group's score the sum of its two largest c, only the `keep`
               best groups stay; the `top` largest c among them; sum of s_e * scale * down_e(relu(up_e x)^2) over the
               chosen, plus a shared expert of the same form
  output       head(rms(x; final.norm))
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


def gelu_exact(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def causal_conv(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """y_t = sum_j taps[:, j] * u_(t - n + 1 + j) over the n taps, u before the sequence's start being 0."""
    T, n = u.shape[0], taps.shape[1]
    y = torch.zeros_like(u)
    for j in range(n):
        back = n - 1 - j
        if back < T:
            y[back:] += taps[:, j] * u[:T - back]
    return y


def window_mask(T: int, window: int | None) -> torch.Tensor:
    """[T, T] True where query i sees key j: j <= i and, with a window, i - j < window."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = j <= i
    return seen if window is None else seen & (i - j < window)


def query_temperature(T: int, coef: float, every: int, dtype) -> torch.Tensor:
    """[T] factors 1 + coef ln(floor((p + 1) / every) + 1)."""
    p = torch.arange(T, dtype=torch.float64)
    return (1.0 + coef * torch.log(torch.floor((p + 1) / every) + 1.0)).to(dtype)


def distance_slopes(H: int, dtype) -> torch.Tensor:
    """[H] slopes 2^(-8 (h + 1) / H)."""
    return (2.0 ** (-8.0 * (torch.arange(H, dtype=torch.float64) + 1.0) / H)).to(dtype)


def rotate_half(x: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [T, heads, size]: the first `dims` entries of every head turn, entry i with entry i + dims / 2, by the angle
    p base^(-2 i / dims) at position p; the others pass."""
    if not dims:
        return x
    T, half = x.shape[0], dims // 2
    f = float(base) ** (-2.0 * torch.arange(half, dtype=torch.float64) / dims)
    a = torch.arange(T, dtype=torch.float64)[:, None] * f[None, :]
    cos, sin = torch.cos(a).to(x.dtype)[:, None, :], torch.sin(a).to(x.dtype)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def softmax_attention(q, k, v, scale: float, window: int | None, slopes=None, sink: bool = False) -> torch.Tensor:
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] -> [T, H * dv].  Query head h reads key head h // (H / G).  slopes
    [H]: slope_h (i - j) is taken off the scores.  sink: one more term exp(0) in every sum, without a value."""
    T, H, _ = q.shape
    G = k.shape[1]
    seen = window_mask(T, window)
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).to(q.dtype)
    out = []
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        if slopes is not None:
            s = s - slopes[h] * dist
        s = s.masked_fill(~seen, float("-inf"))
        m = s.max(dim=-1, keepdim=True).values
        if sink:
            m = torch.clamp(m, min=0.0)
        e = torch.exp(s - m)
        den = e.sum(dim=-1, keepdim=True)
        if sink:
            den = den + torch.exp(-m)
        out.append((e / den) @ v[:, g])
    return torch.cat(out, dim=-1)


# --------------------------------------------------------------------------- mixers


def conv_attention_keys_values(h, p, m, eps):
    """The keys (convolved, normed head by head) and values (convolved) of a layer that has them: what a layer that
    names it with "kv_from" reads too."""
    T, G, dk, dv = h.shape[0], m["kv_heads"], m["dim"], m["vdim"]
    k, v = h @ p["k"].T, h @ p["v"].T
    if m.get("conv"):
        k, v = causal_conv(k, p["k.conv"]), causal_conv(v, p["v.conv"])
    return rms_norm(k.view(T, G, dk), p["k.norm"], eps), v.view(T, G, dv)


def conv_attention(h, p, m, eps, kv=None):
    """kv: (keys, values) of the layer that "kv_from" names; None: this layer's own."""
    T, H, dk = h.shape[0], m["heads"], m["dim"]
    q = h @ p["q"].T
    if m.get("conv"):
        q = causal_conv(q, p["q.conv"])
    q = rms_norm(q.view(T, H, dk), p["q.norm"], eps)
    temp = m.get("q_temp")
    if temp is not None:
        q = q * query_temperature(T, temp["coef"], temp["every"], q.dtype)[:, None, None]
    k, v = kv if kv is not None else conv_attention_keys_values(h, p, m, eps)
    mask = m.get("mask")
    o = softmax_attention(q, k, v, m["scale"], mask["size"] if mask else None, distance_slopes(H, q.dtype), sink=True)
    return (o * torch.sigmoid(h @ p["g"].T)) @ p["o"].T


def whole_norm_attention(h, p, m, eps):
    T, H, G, dk = h.shape[0], m["heads"], m["kv_heads"], m["dim"]
    q, k = h @ p["q"].T + p["q.b"], h @ p["k"].T + p["k.b"]
    v = k.view(T, G, dk)
    q, k = rms_norm(q, p["q.norm"], eps).view(T, H, dk), rms_norm(k, p["k.norm"], eps).view(T, G, dk)
    rot = m.get("rot")
    if rot is not None:
        q, k = rotate_half(q, rot["dims"], rot["base"]), rotate_half(k, rot["dims"], rot["base"])
    mask = m.get("mask")
    o = softmax_attention(q, k, v, m["scale"], mask["size"] if mask else None)
    gate = torch.sigmoid(h @ p["g"].T)                      # [T, H]
    return (o.view(T, H, -1) * gate[:, :, None]).reshape(T, -1) @ p["o"].T


# --------------------------------------------------------------------------- feed-forwards


def dense_ffn(x, p):
    return gelu_exact(x @ p["up"].T) @ p["down"].T


def squared_relu_expert(x, up, down):
    return (torch.relu(x @ up.T) ** 2) @ down.T


def choose_experts(z: torch.Tensor, correction: torch.Tensor, top: int, groups: int, keep: int):
    """z [T, E] router logits -> (chosen [T, top] expert numbers, scores s [T, E])."""
    T, E = z.shape
    s = torch.sigmoid(z)
    c = s + correction
    if groups > 1:
        per = c.view(T, groups, E // groups)
        gs = per.topk(min(2, E // groups), dim=-1).values.sum(dim=-1)          # [T, groups]
        best = gs.topk(keep, dim=-1).indices
        allowed = torch.zeros(T, groups, dtype=torch.bool)
        allowed.scatter_(1, best, True)
        c = c.masked_fill(~allowed[:, :, None].expand(T, groups, E // groups).reshape(T, E), float("-inf"))
    return c.topk(top, dim=-1).indices, s


def moe_ffn(x, p, mlp):
    r = mlp["router"]
    E, top = r["experts"], r["top"]
    g = r.get("groups") or {"count": 1, "keep": 1}
    chosen, s = choose_experts(x @ p["router"].T, p["correction"], top, g["count"], g["keep"])
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e in chosen[t].tolist():
            y[t] += s[t, e] * r["scale"] * squared_relu_expert(x[t:t + 1], p[f"e{e}.up"], p[f"e{e}.down"])[0]
    if mlp.get("shared") is not None:
        y = y + squared_relu_expert(x, p["shared.up"], p["shared.down"])
    return y


# --------------------------------------------------------------------------- the model


def part_tensors(w, prefix: str, dtype) -> dict:
    return {name[len(prefix):]: t.to(dtype) for name, t in w.items() if name.startswith(prefix)}


def forward(w, cfg, tokens, dtype=torch.float64, layers_out: list | None = None) -> torch.Tensor:
    """tokens: a list of ids of one sequence -> logits [T, vocab] in `dtype`."""
    eps = cfg["norm"]["eps"]
    x = rms_norm(w["embed"].to(dtype)[torch.as_tensor(tokens, dtype=torch.long)], w["embed.norm"].to(dtype), eps)
    kept = {}   # layer -> its keys and values, for the layers that read them
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        h = rms_norm(x, w[pre + "norm1"].to(dtype), eps)
        p = part_tensors(w, pre + "mix.", dtype)
        if layer["type"] == "attention":
            src = m.get("kv_from")
            if src is None:
                kept[i] = conv_attention_keys_values(h, p, m, eps)
            x = x + conv_attention(h, p, m, eps, kept[i if src is None else src])
        elif layer["type"] == "attention_2":
            x = x + whole_norm_attention(h, p, m, eps)
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_norm(x, w[pre + "norm2"].to(dtype), eps)
            p = part_tensors(w, pre + "mlp.", dtype)
            x = x + (dense_ffn(h, p) if mlp["kind"] == "dense" else moe_ffn(h, p, mlp))
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"].to(dtype), eps) @ w["head"].to(dtype).T


def greedy(w, cfg, prompt, steps: int, dtype=torch.float64) -> list[int]:
    """`steps` tokens after `prompt`, each the largest logit's, the whole sequence run anew every time."""
    tokens = list(prompt)
    for _ in range(steps):
        tokens.append(int(forward(w, cfg, tokens, dtype)[-1].argmax()))
    return tokens[len(prompt):]
