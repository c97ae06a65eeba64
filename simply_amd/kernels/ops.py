"""Tensor-level calls of the gfx950 kernels.

Each function checks on the host that shapes, element types, strides and devices
are what the kernel assumes, then launches on torch's current stream.  Nothing
here computes on the CPU and nothing falls back to a library routine.
"""
from __future__ import annotations

import ctypes

import torch

from . import lib as _lib
from .lib import KernelError
from .packing import TiledWeight

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}

ALGO_AUTO, ALGO_GENERIC, ALGO_SKINNY, ALGO_TILED, ALGO_WIDE = 0, 1, 2, 3, 4


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"element type {t.dtype} is not supported by the kernels (float32, bfloat16)") from None


def _dev(*tensors) -> None:
    first = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelError("the kernels run on the GPU only: a tensor lies on " + str(t.device))
        if first is None:
            first = t.device
        elif t.device != first:
            raise KernelError(f"tensors lie on different devices: {first} and {t.device}")


def _ptr(t: torch.Tensor | None):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current torch stream's handle (through torch's own fast accessors where it has them: this is called once
    per kernel launch, and `torch.cuda.current_stream()` costs about as much as the launch)."""
    if _raw_stream is not None and _raw_device is not None:
        return ctypes.c_void_p(_raw_stream(_raw_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride of a 2-D tensor whose rows are contiguous."""
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1):
        raise KernelError(f"{what}: expected a 2-D tensor with contiguous rows, got shape {tuple(t.shape)} "
                          f"strides {t.stride()}")
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def _i32(t: torch.Tensor, what: str, n: int | None = None) -> None:
    if t.dtype != torch.int32 or not t.is_contiguous():
        raise KernelError(f"{what}: expected a contiguous int32 tensor, got {t.dtype}")
    if n is not None and t.numel() < n:
        raise KernelError(f"{what}: {t.numel()} entries, {n} needed")


# --------------------------------------------------------------------------- row-wise


def embed(table: "torch.Tensor | TiledWeight", tokens: torch.Tensor, scale: float,
          out: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = float32(table[tokens[t]]) * scale.  The table may be row-major or tiled."""
    packed = isinstance(table, TiledWeight)
    data = table.data if packed else table
    _dev(data, tokens, out)
    V, D = table.shape
    T = tokens.numel()
    _i32(tokens, "embed: tokens")
    if not data.is_contiguous():
        raise KernelError("embed: the table must be contiguous")
    if out is None:
        out = torch.empty((T, D), dtype=torch.float32, device=data.device)
    if out.dtype != torch.float32 or not out.is_contiguous() or tuple(out.shape) != (T, D):
        raise KernelError("embed: the output must be a contiguous float32 [T, D] tensor")
    _lib.call("sa_embed", _ptr(data), _code(data), _ptr(tokens), _ptr(out), T, D, V, float(scale), int(packed),
              _stream())
    return out


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, plus_one: bool, out_dtype: torch.dtype,
            out: torch.Tensor | None = None) -> torch.Tensor:
    _dev(x, weight, out)
    xs = _rows(x, "rmsnorm: x")
    T, D = x.shape
    if weight.numel() != D or not weight.is_contiguous():
        raise KernelError(f"rmsnorm: weight has {weight.numel()} entries for width {D}")
    if out is None:
        out = torch.empty((T, D), dtype=out_dtype, device=x.device)
    if tuple(out.shape) != (T, D):
        raise KernelError("rmsnorm: output shape differs from the input's")
    os_ = _rows(out, "rmsnorm: out")
    _lib.call("sa_rmsnorm", _ptr(x), _code(x), xs, _ptr(weight), _code(weight), _ptr(out), _code(out), os_, T, D,
              float(eps), int(plus_one), _stream())
    return out


class PartialSums:
    """A matrix product whose cuts of K have not been added up yet (`gemm(..., defer_sum=True)`): `planes`
    [cuts, M, N] float32 in the kernels' workspace, valid until the next kernel that is handed the workspace, and
    `out`, the tensor that the sum belongs in.  `add_rmsnorm` takes it in place of y and adds the planes up itself,
    which saves the sum kernel and its round trip; anyone else calls `materialize()`.  The planes remember how
    often the workspace had been handed out when they were written: whoever reads them after another kernel has
    been given the workspace is refused (`check_fresh`), instead of adding up someone else's partial results."""

    def __init__(self, planes: torch.Tensor, out: torch.Tensor):
        self.planes, self.out = planes, out
        self.shape, self.dtype, self.device = out.shape, out.dtype, out.device
        self._written_at = workspace_uses(out.device)

    def check_fresh(self) -> None:
        if self.planes is not None and workspace_uses(self.device) != self._written_at:
            raise KernelError(
                "partial sums of a matrix product were read after another kernel had been given the workspace that "
                "holds them: add them up (add_rmsnorm, rope_cache_write or materialize()) before anything else "
                "that uses the workspace runs (a product with K cut over workgroups, attention over key ranges, "
                "the sampler)")

    def materialize(self) -> torch.Tensor:
        """The product itself: the sum kernel, now."""
        if self.planes is not None:
            self.check_fresh()
            count, M, N = self.planes.shape
            _lib.call("sa_sum_planes", _ptr(self.planes), count, _ptr(self.out), _code(self.out), self.out.stride(0), M, N,
                      _stream())
            self.planes = None
        return self.out


def add_rmsnorm(y: "torch.Tensor | PartialSums", residual: torch.Tensor, *, post_weight: torch.Tensor | None = None,
                post_eps: float = 0.0, post_plus_one: bool = True, next_weight: torch.Tensor | None = None,
                next_eps: float = 0.0, next_plus_one: bool = True, out_dtype: torch.dtype | None = None,
                out: torch.Tensor | None = None) -> torch.Tensor | None:
    """residual += norm(y; post_weight) (or += y); returns norm(residual; next_weight) if asked."""
    T, D = residual.shape
    planes = None
    if isinstance(y, PartialSums):
        fits = (y.planes is not None and D % 4 == 0 and D <= 5120 and y.dtype == torch.bfloat16
                and tuple(y.shape) == (T, D) and all(w is None or w.data_ptr() % 16 == 0 for w in (post_weight, next_weight)))
        if fits:
            y.check_fresh()
            planes, y = y.planes, y.out   # (y stands for shape and type below; it is not read)
        else:
            y = y.materialize()
    _dev(y, residual, post_weight, next_weight, out)
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("add_rmsnorm: the residual stream must be contiguous float32")
    if tuple(y.shape) != (T, D) or not y.is_contiguous():
        raise KernelError(f"add_rmsnorm: y {tuple(y.shape)} does not match the residual {T, D}")
    for w in (post_weight, next_weight):
        if w is not None and (w.numel() != D or not w.is_contiguous()):
            raise KernelError("add_rmsnorm: a norm weight does not match the width")
    if next_weight is not None:
        if out is None:
            out = torch.empty((T, D), dtype=out_dtype or y.dtype, device=y.device)
        if tuple(out.shape) != (T, D) or not out.is_contiguous():
            raise KernelError("add_rmsnorm: bad output")
    else:
        out = None
    if planes is not None:
        _lib.call("sa_add_rmsnorm_planes", _ptr(planes), planes.shape[0], _ptr(post_weight),
                  _code(post_weight) if post_weight is not None else 0, float(post_eps), int(post_plus_one),
                  _ptr(residual), _ptr(next_weight), _code(next_weight) if next_weight is not None else 0,
                  float(next_eps), int(next_plus_one), _ptr(out), _code(out) if out is not None else 0, T, D, _stream())
        return out
    _lib.call("sa_add_rmsnorm", _ptr(y), _code(y), _ptr(post_weight),
              _code(post_weight) if post_weight is not None else 0, float(post_eps), int(post_plus_one),
              _ptr(residual), _ptr(next_weight), _code(next_weight) if next_weight is not None else 0,
              float(next_eps), int(next_plus_one), _ptr(out), _code(out) if out is not None else 0, T, D, _stream())
    return out


def add_rmsnorm_rows(y: torch.Tensor, residual: torch.Tensor, index: torch.Tensor, *, post_weight: torch.Tensor | None,
                     post_eps: float = 0.0, post_plus_one: bool = True, next_weight: torch.Tensor, next_eps: float,
                     next_plus_one: bool = True, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """out[r] = norm(residual[index[r]] + norm(y[index[r]]; post_weight); next_weight), the residual left as it is:
    `add_rmsnorm` followed by a gather of the rows that are wanted, in one kernel that touches those rows only."""
    _dev(y, residual, index, post_weight, next_weight)
    T, D = residual.shape
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("add_rmsnorm_rows: the residual stream must be contiguous float32")
    if tuple(y.shape) != (T, D) or not y.is_contiguous():
        raise KernelError(f"add_rmsnorm_rows: y {tuple(y.shape)} does not match the residual {T, D}")
    for w in (post_weight, next_weight):
        if w is not None and (w.numel() != D or not w.is_contiguous()):
            raise KernelError("add_rmsnorm_rows: a norm weight does not match the width")
    _i32(index, "add_rmsnorm_rows: index")
    R = index.numel()
    out = torch.empty((R, D), dtype=out_dtype or y.dtype, device=y.device)
    _lib.call("sa_add_rmsnorm_rows", _ptr(y), _code(y), _ptr(post_weight),
              _code(post_weight) if post_weight is not None else 0, float(post_eps), int(post_plus_one), _ptr(residual),
              _ptr(next_weight), _code(next_weight), float(next_eps), int(next_plus_one), _ptr(out), _code(out),
              _ptr(index), R, D, _stream())
    return out


def _check_pages(k_pages: torch.Tensor, v_pages: torch.Tensor, dtype: torch.dtype, what: str) -> int:
    """Key pages [pages, K, page_size, hd], value pages [pages, K, hd, page_size]; returns page_size."""
    if k_pages.dim() != 4 or v_pages.dim() != 4 or not k_pages.is_contiguous() or not v_pages.is_contiguous() \
            or k_pages.dtype != dtype or v_pages.dtype != dtype:
        raise KernelError(f"{what}: pages must be contiguous 4-D tensors of {dtype}")
    n, K, P, hd = k_pages.shape
    if tuple(v_pages.shape) != (n, K, hd, P):
        raise KernelError(f"{what}: key pages {tuple(k_pages.shape)} want value pages {(n, K, hd, P)}, "
                          f"got {tuple(v_pages.shape)}")
    return P


def rope_cache_write(qkv: "torch.Tensor | PartialSums", positions: torch.Tensor, timescale: torch.Tensor | None,
                     scale_factor: float, q_div: float, num_heads: int, num_kv_heads: int, head_dim: int,
                     slot_mapping: torch.Tensor | None = None, k_pages: torch.Tensor | None = None,
                     v_pages: torch.Tensor | None = None) -> torch.Tensor:
    """In place on the fused projection rows; writes keys and values into their pages.  A projection whose cuts of K
    are not added up yet is added up on the way (up to 256 tokens; its queries go to the tensor that it belongs in).
    Returns the projection's tensor, of which the queries are then the rotated and scaled ones."""
    planes = None
    if isinstance(qkv, PartialSums):
        if qkv.planes is not None and qkv.shape[0] <= 256 and qkv.dtype == torch.bfloat16:
            qkv.check_fresh()
            planes, qkv = qkv.planes, qkv.out
        else:
            qkv = qkv.materialize()
    _dev(qkv, positions, timescale, slot_mapping, k_pages, v_pages)
    stride = _rows(qkv, "rope_cache_write: qkv")
    T = qkv.shape[0]
    if qkv.shape[1] != (num_heads + 2 * num_kv_heads) * head_dim:
        raise KernelError(f"rope_cache_write: row width {qkv.shape[1]} is not (H + 2K) * hd = "
                          f"{(num_heads + 2 * num_kv_heads) * head_dim}")
    _i32(positions, "rope_cache_write: positions", T)
    if timescale is not None and (timescale.dtype != torch.float32 or timescale.numel() != head_dim // 2
                                  or not timescale.is_contiguous()):
        raise KernelError("rope_cache_write: timescale must be float32 [head_dim / 2]")
    page_size = 1
    if k_pages is not None:
        if v_pages is None or slot_mapping is None:
            raise KernelError("rope_cache_write: key pages, value pages and slots come together")
        page_size = _check_pages(k_pages, v_pages, qkv.dtype, "rope_cache_write")
        if k_pages.shape[1] != num_kv_heads or k_pages.shape[3] != head_dim:
            raise KernelError(f"rope_cache_write: pages {tuple(k_pages.shape)} do not match {num_kv_heads} heads of "
                              f"size {head_dim}")
        if slot_mapping.dtype != torch.int64 or slot_mapping.numel() < T or not slot_mapping.is_contiguous():
            raise KernelError("rope_cache_write: slot_mapping must be int64 [T]")
    if planes is not None:
        _lib.call("sa_rope_cache_write_planes", _ptr(planes), planes.shape[0], _ptr(qkv), stride, _ptr(positions),
                  _ptr(timescale), float(scale_factor), float(q_div), _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages),
                  T, num_heads, num_kv_heads, head_dim, page_size, _stream())
        return qkv
    _lib.call("sa_rope_cache_write", _ptr(qkv), _code(qkv), stride, _ptr(positions), _ptr(timescale),
              float(scale_factor), float(q_div), _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages), T, num_heads,
              num_kv_heads, head_dim, page_size, _stream())
    return qkv


def rope(x: torch.Tensor, positions: torch.Tensor, timescale: torch.Tensor, scale_factor: float, div: float,
         num_heads: int, head_dim: int) -> None:
    """In place: x[t, h, :] rotated by positions[t], then divided by div.  x: [T, >= num_heads * head_dim]."""
    _dev(x, positions, timescale)
    stride = _rows(x, "rope: x")
    T = x.shape[0]
    if x.shape[1] < num_heads * head_dim:
        raise KernelError("rope: rows are shorter than heads * head size")
    _i32(positions, "rope: positions", T)
    if timescale.dtype != torch.float32 or timescale.numel() != head_dim // 2 or not timescale.is_contiguous():
        raise KernelError("rope: timescale must be float32 [head_dim / 2]")
    _lib.call("sa_rope", _ptr(x), _code(x), stride, _ptr(positions), _ptr(timescale), float(scale_factor), float(div),
              T, num_heads, head_dim, _stream())


def gather_rows(x: torch.Tensor, index: torch.Tensor, out_dtype: torch.dtype | None = None,
                out: torch.Tensor | None = None) -> torch.Tensor:
    _dev(x, index, out)
    if x.dim() != 2 or not x.is_contiguous():
        raise KernelError("gather_rows: x must be contiguous 2-D")
    _i32(index, "gather_rows: index")
    R, D = index.numel(), x.shape[1]
    if out is None:
        out = torch.empty((R, D), dtype=out_dtype or x.dtype, device=x.device)
    if tuple(out.shape) != (R, D) or not out.is_contiguous():
        raise KernelError("gather_rows: bad output")
    _lib.call("sa_gather_rows", _ptr(x), _code(x), _ptr(index), _ptr(out), _code(out), R, D, _stream())
    return out


def fill_(t: torch.Tensor, value_bits: int = 0) -> None:
    """Sets every 32-bit word of `t` to `value_bits` with a kernel (safe inside a captured graph)."""
    _dev(t)
    nbytes = t.numel() * t.element_size()
    if not t.is_contiguous() or nbytes % 4:
        raise KernelError("fill_: needs a contiguous tensor of a multiple of 4 bytes")
    _lib.call("sa_fill_u32", _ptr(t), value_bits & 0xFFFFFFFF, nbytes // 4, _stream())


def decode_advance(step_counter: torch.Tensor, sampled_tokens: torch.Tensor, sampled_logprobs: torch.Tensor,
                   tokens_in: torch.Tensor, positions: torch.Tensor, seq_meta: torch.Tensor,
                   draw_counters: torch.Tensor, out_tokens: torch.Tensor, out_logprobs: torch.Tensor, *,
                   token_seq: torch.Tensor | None = None, page_size: int = 0,
                   groups: "list[tuple[torch.Tensor, torch.Tensor]] | None" = None) -> None:
    """Between two decode steps that the host does not see: what was drawn is recorded as row step_counter[0] of
    out_tokens / out_logprobs [max_steps, B] and becomes the next step's input; positions, the requests' first
    positions (seq_meta[:, 3]), their draw counters and the step counter go up by one.  groups: (block table, slot
    mapping) of up to four cache groups, whose slot mappings are set for the new positions in the same launch (what
    `decode_slots` does for one group): needs token_seq and page_size."""
    _dev(step_counter, sampled_tokens, sampled_logprobs, tokens_in, positions, seq_meta, draw_counters, out_tokens,
         out_logprobs)
    B = tokens_in.numel()
    for t, name in ((step_counter, "step_counter"), (sampled_tokens, "sampled_tokens"), (tokens_in, "tokens_in"),
                    (positions, "positions"), (seq_meta, "seq_meta"), (draw_counters, "draw_counters"),
                    (out_tokens, "out_tokens")):
        if t.dtype != torch.int32 or not t.is_contiguous():
            raise KernelError(f"decode_advance: {name} must be contiguous int32")
    for t, name in ((sampled_logprobs, "sampled_logprobs"), (out_logprobs, "out_logprobs")):
        if t.dtype != torch.float32 or not t.is_contiguous():
            raise KernelError(f"decode_advance: {name} must be contiguous float32")
    if out_tokens.dim() != 2 or out_tokens.shape[1] != B or tuple(out_logprobs.shape) != tuple(out_tokens.shape):
        raise KernelError("decode_advance: the records are [max_steps, B]")
    if min(sampled_tokens.numel(), sampled_logprobs.numel(), positions.numel(), draw_counters.numel()) < B \
            or seq_meta.numel() < 4 * B or step_counter.numel() < 1:
        raise KernelError("decode_advance: an array is shorter than the number of requests")
    if groups:
        if token_seq is None or page_size < 1 or len(groups) > 4:
            raise KernelError("decode_advance: slot mappings need token_seq, a page size and at most four groups")
        _i32(token_seq, "decode_advance: token_seq", B)
        n = len(groups)
        for table, slots in groups:
            _dev(table, slots)
            if table.dim() != 2 or table.dtype != torch.int32 or table.stride(1) != 1:
                raise KernelError("decode_advance: a block table must be int32 [sequences, blocks]")
            if slots.dtype != torch.int64 or slots.numel() < B or not slots.is_contiguous():
                raise KernelError("decode_advance: a slot mapping must be contiguous int64 with one entry per token")
        tables = (ctypes.c_void_p * n)(*[t.data_ptr() for t, _ in groups])
        strides = (ctypes.c_int * n)(*[t.stride(0) for t, _ in groups])
        mappings = (ctypes.c_void_p * n)(*[m.data_ptr() for _, m in groups])
        _lib.call("sa_decode_advance_slots", B, _ptr(step_counter), _ptr(sampled_tokens), _ptr(sampled_logprobs),
                  _ptr(tokens_in), _ptr(positions), _ptr(seq_meta), _ptr(draw_counters), _ptr(out_tokens),
                  _ptr(out_logprobs), out_tokens.shape[0], _ptr(token_seq), n, tables, strides, mappings, int(page_size),
                  _stream())
        return
    _lib.call("sa_decode_advance", B, _ptr(step_counter), _ptr(sampled_tokens), _ptr(sampled_logprobs), _ptr(tokens_in),
              _ptr(positions), _ptr(seq_meta), _ptr(draw_counters), _ptr(out_tokens), _ptr(out_logprobs),
              out_tokens.shape[0], _stream())


def decode_slots(positions: torch.Tensor, token_seq: torch.Tensor, block_table: torch.Tensor, page_size: int,
                 slot_mapping: torch.Tensor) -> None:
    """slot_mapping[b] = block_table[token_seq[b], positions[b] // page_size] * page_size + positions[b] % page_size."""
    _dev(positions, token_seq, block_table, slot_mapping)
    B = positions.numel()
    _i32(positions, "decode_slots: positions", B)
    _i32(token_seq, "decode_slots: token_seq", B)
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("decode_slots: block_table must be int32 [sequences, blocks]")
    if slot_mapping.dtype != torch.int64 or slot_mapping.numel() < B or not slot_mapping.is_contiguous():
        raise KernelError("decode_slots: slot_mapping must be contiguous int64 with one entry per token")
    _lib.call("sa_decode_slots", B, _ptr(positions), _ptr(token_seq), _ptr(block_table), block_table.stride(0),
              int(page_size), _ptr(slot_mapping), _stream())


# --------------------------------------------------------------------------- matrix products

EPILOGUE_NONE, EPILOGUE_GATED, EPILOGUE_SOFT_CAP, EPILOGUE_ACTIVATED = 0, 1, 2, 3
#: activations of the gated epilogue (simply_amd/csrc/activations.h); the epilogue argument is 1 + 16 * activation
ACT_GELU_TANH, ACT_SILU, ACT_SQUARED_RELU, ACT_GELU_ERF = 0, 1, 2, 3


def _gated(activation: int) -> int:
    if activation not in (ACT_GELU_TANH, ACT_SILU, ACT_SQUARED_RELU, ACT_GELU_ERF):
        raise KernelError(f"unknown activation code {activation!r}")
    return EPILOGUE_GATED + 16 * activation


#: scratch memory for partial results (attention over key ranges, products with K cut over workgroups), one per
#: device, allocated at first use; kernels on one stream use it one after the other
WORKSPACE_BYTES = 256 << 20
_scratch: dict = {}
_scratch_uses: dict = {}


def _workspace(device) -> torch.Tensor:
    """The device's workspace, for a kernel that is about to be launched with it: what an earlier kernel left there
    is lost from now on (`workspace_uses` counts these hand-outs)."""
    key = (device.type, device.index)
    if key not in _scratch:
        _scratch[key] = torch.empty(WORKSPACE_BYTES, dtype=torch.uint8, device=device)
    _scratch_uses[key] = _scratch_uses.get(key, 0) + 1
    return _scratch[key]


def workspace_uses(device) -> int:
    """How often the device's workspace has been handed to a kernel."""
    device = torch.device(device)
    return _scratch_uses.get((device.type, device.index), 0)


def gemm(a: torch.Tensor, w: "torch.Tensor | TiledWeight", *, w2: "torch.Tensor | TiledWeight | None" = None,
         soft_cap: float | None = None, out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None,
         algo: int = ALGO_AUTO, shape: int = 0, activation: int = ACT_GELU_TANH,
         defer_sum: bool = False, activate: int | None = None) -> "torch.Tensor | PartialSums":
    """a[M, K] . w[N, K]^T.  With w2 (row-major weights) or a paired `TiledWeight`: act(a.wg^T) * (a.wu^T) with
    the activation of that code.  With soft_cap: cap * tanh(. / cap).  With activate (an activation code): act(a.w^T),
    the product rounded to the output type first.  w is a row-major tensor or a `TiledWeight`.
    defer_sum: where the product is computed in cuts of K, leave their sum to the caller: the result is then a
    `PartialSums` (else the tensor as always)."""
    packed = isinstance(w, TiledWeight)
    wd = w.data if packed else w
    w2d = None
    paired = packed and w.paired
    if paired and (w2 is not None or soft_cap):
        raise KernelError("gemm: a paired tiled weight is the gated product by itself")
    if w2 is not None:
        if packed or isinstance(w2, TiledWeight):
            raise KernelError("gemm: tiled weights of a gated product come as one paired weight (pack_gate_up)")
        w2d = w2
    _dev(a, wd, w2d, out)
    lda = _rows(a, "gemm: a")
    M, K = a.shape
    if not wd.is_contiguous() or (not packed and w.dim() != 2) or w.shape[1] != K:
        raise KernelError(f"gemm: weight {tuple(w.shape)} does not match a {tuple(a.shape)} (expects [N, K] contiguous)")
    N = w.shape[0]
    if wd.dtype != a.dtype:
        raise KernelError(f"gemm: a is {a.dtype} but the weight is {wd.dtype}")
    epi, cap = EPILOGUE_NONE, 0.0
    if paired:
        epi = _gated(activation)
    elif w2 is not None:
        if soft_cap:
            raise KernelError("gemm: the gated and the soft-cap epilogue do not combine")
        if tuple(w2.shape) != tuple(w.shape) or w2d.dtype != wd.dtype or not w2d.is_contiguous():
            raise KernelError("gemm: the second weight must match the first")
        epi = _gated(activation)
    elif soft_cap:
        epi, cap = EPILOGUE_SOFT_CAP, float(soft_cap)
    if activate is not None:
        if epi != EPILOGUE_NONE or defer_sum:
            raise KernelError("gemm: an activation of the product combines with no other epilogue and no deferred sum")
        epi = _gated(activate) - EPILOGUE_GATED + EPILOGUE_ACTIVATED
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
    if tuple(out.shape) != (M, N):
        raise KernelError("gemm: bad output shape")
    ldc = _rows(out, "gemm: out")
    ws = _workspace(a.device)
    if defer_sum and epi == EPILOGUE_NONE and out.dtype == torch.bfloat16 and out.is_contiguous():
        count = ctypes.c_int(1)
        _lib.call("sa_gemm_planes", _ptr(a), _code(a), lda, _ptr(wd), _ptr(w2d), _code(wd), _ptr(out), _code(out), ldc, M, N,
                  K, epi, cap, algo, int(packed), int(shape), _ptr(ws), ws.numel(), ctypes.byref(count), _stream())
        if count.value > 1:
            words = count.value * M * N
            return PartialSums(ws.view(torch.float32)[:words].view(count.value, M, N), out)
        return out
    _lib.call("sa_gemm", _ptr(a), _code(a), lda, _ptr(wd), _ptr(w2d), _code(wd), _ptr(out), _code(out), ldc, M, N, K, epi,
              cap, algo, int(packed), int(shape), _ptr(ws), ws.numel(), _stream())
    return out


def gemm_plan(M: int, N: int, K: int, *, gated: bool = False, soft_cap: bool = False,
              out_dtype: torch.dtype = torch.bfloat16) -> tuple[int, dict[str, float]]:
    """Which kernel `gemm` would run for bfloat16 rows against a tiled [N, K] weight (ALGO_SKINNY, ALGO_TILED or
    ALGO_WIDE), and the microseconds that the library expects of each (negative: not eligible).  A host function:
    it needs no GPU."""
    us = (ctypes.c_double * 3)()
    epi = EPILOGUE_GATED if gated else (EPILOGUE_SOFT_CAP if soft_cap else EPILOGUE_NONE)
    kernel = _lib.load().sa_gemm_plan(int(M), int(N), int(K), epi, _CODES[out_dtype], WORKSPACE_BYTES, us)
    return kernel, {"skinny": us[0], "tiled": us[1], "wide": us[2]}


def gemm_normed_takes(M: int, w) -> bool:
    """Whether `gemm_normed` takes M rows against the weight `w`."""
    if not isinstance(w, TiledWeight) or not w.data.is_cuda:
        return False
    return bool(_lib.load().sa_gemm_normed_takes(int(M), int(w.rows), int(w.cols)))


def gemm_normed_pays(M: int, w) -> bool:
    """Whether `gemm_normed` takes M rows against the weight `w` and is expected to beat the separate norm and
    product kernels there (the library's own answer: it knows for which widths it has which prologue)."""
    if not isinstance(w, TiledWeight) or not w.data.is_cuda:
        return False
    return bool(_lib.load().sa_gemm_normed_pays(int(M), int(w.rows), int(w.cols)))


_few_rows: int | None = None


def few_rows_limit() -> int:
    """The most rows of a step for which the kernels that fuse the norms into the following product exist."""
    global _few_rows
    if _few_rows is None:
        _few_rows = int(_lib.load().sa_gemm_normed_max_rows())
    return _few_rows


def gemm_normed(y: torch.Tensor | None, h_in: torch.Tensor, h_out: torch.Tensor | None, w: TiledWeight, *,
                post_weight: torch.Tensor | None, post_eps: float, post_plus_one: bool, next_weight: torch.Tensor,
                next_eps: float, next_plus_one: bool, soft_cap: float | None = None,
                out_dtype: torch.dtype = torch.bfloat16, out: torch.Tensor | None = None,
                activation: int = ACT_GELU_TANH) -> torch.Tensor:
    """h_out = h_in + norm(y; post) (y None: the residual stays h_in); returns epilogue(norm(h_out; next) . w^T),
    in one kernel, for up to 16 rows.  The residual buffers are float32 [M, K] and must differ."""
    _dev(y, h_in, h_out, post_weight, next_weight, w.data)
    M, K = h_in.shape
    if h_in.dtype != torch.float32 or not h_in.is_contiguous() or w.cols != K:
        raise KernelError("gemm_normed: the residual must be contiguous float32 [M, K] with K the weight's width")
    if y is not None:
        if y.dtype != torch.bfloat16 or tuple(y.shape) != (M, K) or not y.is_contiguous():
            raise KernelError("gemm_normed: y must be contiguous bfloat16 [M, K]")
        if h_out is None or h_out.dtype != torch.float32 or tuple(h_out.shape) != (M, K) or not h_out.is_contiguous() \
                or h_out.data_ptr() == h_in.data_ptr():
            raise KernelError("gemm_normed: the updated residual needs its own contiguous float32 [M, K] buffer")
    for t in (post_weight, next_weight):
        if t is not None and (t.numel() != K or not t.is_contiguous()):
            raise KernelError("gemm_normed: a norm weight does not match the width")
    epi, cap = EPILOGUE_NONE, 0.0
    if w.paired:
        epi = _gated(activation)
    elif soft_cap:
        epi, cap = EPILOGUE_SOFT_CAP, float(soft_cap)
    if out is None:
        out = torch.empty((M, w.rows), dtype=out_dtype, device=h_in.device)
    if tuple(out.shape) != (M, w.rows) or out.stride(1) != 1 or out.device != h_in.device:
        raise KernelError(f"gemm_normed: the output must be [{M}, {w.rows}] with contiguous rows on the inputs' device")
    _lib.call("sa_gemm_normed", _ptr(y), _ptr(h_in), _ptr(h_out), _ptr(post_weight),
              _code(post_weight) if post_weight is not None else 0, float(post_eps), int(post_plus_one),
              _ptr(next_weight), _code(next_weight), float(next_eps), int(next_plus_one), _ptr(w.data), _ptr(out),
              _code(out), out.stride(0), M, w.rows, K, epi, cap, _stream())
    return out


def gemm_normed_rotary(y: torch.Tensor | None, h_in: torch.Tensor, h_out: torch.Tensor | None, w: TiledWeight, *,
                       post_weight: torch.Tensor | None, post_eps: float, post_plus_one: bool,
                       next_weight: torch.Tensor, next_eps: float, next_plus_one: bool, positions: torch.Tensor,
                       timescale: torch.Tensor | None, scale_factor: float, query_scale: float, num_heads: int,
                       num_kv_heads: int, head_dim: int, slot_mapping: torch.Tensor | None = None,
                       k_pages: torch.Tensor | None = None, v_pages: torch.Tensor | None = None) -> torch.Tensor:
    """`gemm_normed` for the fused q/k/v projection (w has (H + 2 K) * hd rows) followed by `rope_cache_write` in
    the same kernel.  Returns [M, (H + 2 K) * hd] of which only the query columns are written."""
    _dev(y, h_in, h_out, post_weight, next_weight, w.data, positions, timescale, slot_mapping, k_pages, v_pages)
    M, K = h_in.shape
    H, Kh, hd = num_heads, num_kv_heads, head_dim
    if w.paired or w.rows != (H + 2 * Kh) * hd or w.cols != K:
        raise KernelError("gemm_normed_rotary: the weight must have (H + 2 K) * hd rows of the residual's width")
    if h_in.dtype != torch.float32 or not h_in.is_contiguous():
        raise KernelError("gemm_normed_rotary: the residual must be contiguous float32 [M, K]")
    if y is not None:
        if y.dtype != torch.bfloat16 or tuple(y.shape) != (M, K) or not y.is_contiguous():
            raise KernelError("gemm_normed_rotary: y must be contiguous bfloat16 [M, K]")
        if h_out is None or h_out.dtype != torch.float32 or tuple(h_out.shape) != (M, K) or not h_out.is_contiguous() \
                or h_out.data_ptr() == h_in.data_ptr():
            raise KernelError("gemm_normed_rotary: the updated residual needs its own contiguous float32 [M, K] buffer")
    for t in (post_weight, next_weight):
        if t is not None and (t.numel() != K or not t.is_contiguous()):
            raise KernelError("gemm_normed_rotary: a norm weight does not match the width")
    _i32(positions, "gemm_normed_rotary: positions", M)
    if timescale is not None and (timescale.dtype != torch.float32 or timescale.numel() != hd // 2):
        raise KernelError("gemm_normed_rotary: timescale must be float32 [hd / 2]")
    page_size = 1
    if slot_mapping is not None:
        if k_pages is None or v_pages is None:
            raise KernelError("gemm_normed_rotary: slots come with key and value pages")
        _check_pages(k_pages, v_pages, torch.bfloat16, "gemm_normed_rotary")
        if k_pages.shape[1] != Kh or k_pages.shape[3] != hd:
            raise KernelError("gemm_normed_rotary: the pages do not match the heads")
        page_size = k_pages.shape[2]
        if slot_mapping.dtype != torch.int64 or slot_mapping.numel() < M or not slot_mapping.is_contiguous():
            raise KernelError("gemm_normed_rotary: slot_mapping must be contiguous int64 with one entry per row")
    out = torch.empty((M, w.rows), dtype=torch.bfloat16, device=h_in.device)
    _lib.call("sa_gemm_normed_rotary", _ptr(y), _ptr(h_in), _ptr(h_out), _ptr(post_weight),
              _code(post_weight) if post_weight is not None else 0, float(post_eps), int(post_plus_one),
              _ptr(next_weight), _code(next_weight), float(next_eps), int(next_plus_one), _ptr(w.data), _ptr(out),
              _code(out), out.stride(0), M, K, _ptr(positions), _ptr(timescale), float(scale_factor),
              float(query_scale), _ptr(slot_mapping), _ptr(k_pages) if slot_mapping is not None else None,
              _ptr(v_pages) if slot_mapping is not None else None, H, Kh, hd, int(page_size), _stream())
    return out


# --------------------------------------------------------------------------- attention


def paged_attention(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                    token_seq: torch.Tensor, positions: torch.Tensor, num_heads: int, *, window: int | None,
                    soft_cap: float | None, out: torch.Tensor | None = None, algo: int = ALGO_AUTO) -> torch.Tensor:
    """q: [T, >= H * hd] rows (a view into the fused projection is fine).  Returns [T, H * hd]."""
    _dev(q, k_pages, v_pages, block_table, token_seq, positions, out)
    q_stride = _rows(q, "paged_attention: q")
    T = q.shape[0]
    _check_pages(k_pages, v_pages, q.dtype, "paged_attention")
    num_pages, Kh, page_size, hd = k_pages.shape
    if q.shape[1] < num_heads * hd:
        raise KernelError("paged_attention: query rows are shorter than heads * head size")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("paged_attention: block_table must be int32 [sequences, blocks]")
    _i32(token_seq, "paged_attention: token_seq", T)
    _i32(positions, "paged_attention: positions", T)
    if out is None:
        out = torch.empty((T, num_heads * hd), dtype=q.dtype, device=q.device)
    if tuple(out.shape) != (T, num_heads * hd) or out.dtype != q.dtype:
        raise KernelError("paged_attention: bad output")
    out_stride = _rows(out, "paged_attention: out")
    _lib.call("sa_paged_attention", _ptr(q), _code(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
              block_table.stride(0), _ptr(token_seq), _ptr(positions), _ptr(out), out_stride, T, num_heads, Kh, hd,
              page_size, int(window or 0), float(soft_cap or 0.0), algo, _stream())
    return out


def decode_attention_takes(q: torch.Tensor, k_pages: torch.Tensor, num_heads: int, max_q_len: int) -> bool:
    """Whether `paged_attention_decode` takes requests of up to max_q_len tokens at these sizes."""
    _, Kh, page_size, hd = k_pages.shape
    return q.dtype == torch.bfloat16 and q.is_cuda and bool(_lib.load().sa_paged_attention_decode_takes(
        int(num_heads), int(Kh), int(hd), int(page_size), int(max_q_len), q.stride(0), _ptr(q)))


def _attention_units(entry: str, q, k_pages, v_pages, block_table, seq_meta, begin, count, num_heads, window, soft_cap,
                     max_kv_len, max_q_len, out, num_splits, sinks=None, slopes=None):
    _dev(q, k_pages, v_pages, block_table, seq_meta, out, sinks, slopes)
    name = entry[3:]
    if q.dtype != torch.bfloat16:
        raise KernelError(f"{name}: bfloat16 only")
    q_stride = _rows(q, f"{name}: q")
    _check_pages(k_pages, v_pages, q.dtype, name)
    _, Kh, page_size, hd = k_pages.shape
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError(f"{name}: block_table must be int32 [sequences, blocks]")
    if seq_meta.dtype != torch.int32 or seq_meta.dim() != 2 or seq_meta.shape[1] != 4 or not seq_meta.is_contiguous() \
            or begin < 0 or begin + count > seq_meta.shape[0]:
        raise KernelError(f"{name}: seq_meta must be int32 [S, 4] covering the requested range")
    if out.dtype != q.dtype or out.shape[0] != q.shape[0] or out.shape[1] != num_heads * hd:
        raise KernelError(f"{name}: bad output")
    out_stride = _rows(out, f"{name}: out")
    ws = _workspace(q.device)
    if sinks is not None or slopes is not None:
        # one more term exp(sinks[h]) in every softmax sum of query head h, without a value; slopes[h] times the
        # distance between query and key taken off the scores
        for per_head in (sinks, slopes):
            if per_head is not None and (per_head.dtype != torch.float32 or per_head.numel() != num_heads
                                         or not per_head.is_contiguous()):
                raise KernelError(f"{name}: sinks and slopes must be contiguous float32, one per query head")
        _lib.call(entry + "_sink", _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
                  block_table.stride(0), _ptr(seq_meta), begin, count, _ptr(out), out_stride, num_heads, Kh, hd,
                  page_size, int(window or 0), float(soft_cap or 0.0), int(max_kv_len), int(max_q_len), int(num_splits),
                  _ptr(ws), ws.numel(), _ptr(sinks), _ptr(slopes), _stream())
        return out
    _lib.call(entry, _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
              block_table.stride(0), _ptr(seq_meta), begin, count, _ptr(out), out_stride, num_heads, Kh, hd,
              page_size, int(window or 0), float(soft_cap or 0.0), int(max_kv_len), int(max_q_len), int(num_splits),
              _ptr(ws), ws.numel(), _stream())
    return out


def paged_attention_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                           seq_meta: torch.Tensor, seq_begin: int, seq_count: int, num_heads: int, *,
                           window: int | None, soft_cap: float | None, max_kv_len: int, max_q_len: int,
                           out: torch.Tensor, num_splits: int = 0, sinks: torch.Tensor | None = None,
                           slopes: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of requests seq_begin .. seq_begin + seq_count - 1 of seq_meta, each with few tokens
    ((heads per key head) * tokens <= 16).  q and out are the whole step's rows.  sinks: float32 [H], one more term
    exp(sinks[h]) in every softmax sum, without a value.  slopes: float32 [H], slopes[h] times the distance between
    query and key is taken off the scores."""
    return _attention_units("sa_paged_attention_decode", q, k_pages, v_pages, block_table, seq_meta, seq_begin,
                            seq_count, num_heads, window, soft_cap, max_kv_len, max_q_len, out, num_splits, sinks, slopes)


def prefill_units_per_group() -> int:
    """How many units one workgroup of the portion kernel takes (they must belong to one request)."""
    return int(_lib.load().sa_paged_attention_prefill_group())


def paged_attention_prefill(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                            units: torch.Tensor, unit_begin: int, unit_count: int, num_heads: int, *,
                            window: int | None, soft_cap: float | None, max_kv_len: int, max_q_len: int,
                            out: torch.Tensor, num_splits: int = 0, sinks: torch.Tensor | None = None,
                            slopes: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of portions of prompts cut into units of few tokens ((heads per key head) * tokens <= 16), rows
    unit_begin .. unit_begin + unit_count - 1 of `units` in the layout of seq_meta.  One workgroup takes a group of
    consecutive units, which must belong to one request (units without tokens fill up the last group), and
    reads the keys once for all of them."""
    if unit_count % prefill_units_per_group():
        raise KernelError(f"paged_attention_prefill: units come in groups of {prefill_units_per_group()}")
    return _attention_units("sa_paged_attention_prefill", q, k_pages, v_pages, block_table, units, unit_begin,
                            unit_count, num_heads, window, soft_cap, max_kv_len, max_q_len, out, num_splits, sinks, slopes)


def paged_attention_sink(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                         token_seq: torch.Tensor, positions: torch.Tensor, num_heads: int, *, scale: float = 1.0,
                         sinks: torch.Tensor | None = None, window: int | None = None, soft_cap: float | None = None,
                         out: torch.Tensor | None = None, slopes: torch.Tensor | None = None) -> torch.Tensor:
    """Attention whose values may have another size than its keys (key pages [pages, K, P, dk], value pages
    [pages, K, dv, P]), with scores times `scale` and, if `sinks` [H] is given, one more term exp(sinks[h]) in every
    softmax sum that has no value.  slopes (float32 [H]): slopes[h] * (query position - key position) is taken off
    the scaled scores.  q: [T, >= H * dk] rows.  Returns [T, H * dv]."""
    _dev(q, k_pages, v_pages, block_table, token_seq, positions, sinks, out, slopes)
    if slopes is not None and (slopes.dtype != torch.float32 or slopes.numel() != num_heads or not slopes.is_contiguous()):
        raise KernelError("paged_attention_sink: slopes must be contiguous float32, one per query head")
    q_stride = _rows(q, "paged_attention_sink: q")
    T = q.shape[0]
    if k_pages.dim() != 4 or v_pages.dim() != 4 or not k_pages.is_contiguous() or not v_pages.is_contiguous() \
            or k_pages.dtype != q.dtype or v_pages.dtype != q.dtype:
        raise KernelError(f"paged_attention_sink: pages must be contiguous 4-D tensors of {q.dtype}")
    num_pages, Kh, page_size, dk = k_pages.shape
    dv = v_pages.shape[2]
    if tuple(v_pages.shape) != (num_pages, Kh, dv, page_size):
        raise KernelError(f"paged_attention_sink: key pages {tuple(k_pages.shape)} do not go with value pages "
                          f"{tuple(v_pages.shape)}")
    if q.shape[1] < num_heads * dk:
        raise KernelError("paged_attention_sink: query rows are shorter than heads * key size")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("paged_attention_sink: block_table must be int32 [sequences, blocks]")
    _i32(token_seq, "paged_attention_sink: token_seq", T)
    _i32(positions, "paged_attention_sink: positions", T)
    if sinks is not None and (sinks.numel() != num_heads or not sinks.is_contiguous()):
        raise KernelError(f"paged_attention_sink: {sinks.numel()} sinks for {num_heads} heads")
    if out is None:
        out = torch.empty((T, num_heads * dv), dtype=q.dtype, device=q.device)
    if tuple(out.shape) != (T, num_heads * dv) or out.dtype != q.dtype:
        raise KernelError("paged_attention_sink: bad output")
    out_stride = _rows(out, "paged_attention_sink: out")
    _lib.call("sa_paged_attention_sink", _ptr(q), _code(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
              block_table.stride(0), _ptr(token_seq), _ptr(positions), _ptr(out), out_stride, T, num_heads, Kh, dk, dv,
              page_size, int(window or 0), float(soft_cap or 0.0), float(scale), _ptr(sinks),
              _code(sinks) if sinks is not None else 0, _ptr(slopes), _stream())
    return out


def paged_attention_maps(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor | None, block_table: torch.Tensor,
                         token_seq: torch.Tensor, positions: torch.Tensor, num_heads: int, *, scale: float,
                         maps: int = 1, value_dim: int | None = None, window: int | None = None,
                         differential: "tuple[float, float, float] | None" = None,
                         out: torch.Tensor | None = None) -> torch.Tensor:
    """Attention with `maps` score maps per query head, each a softmax of its own over the same values: q rows hold
    H * maps vectors of hd entries (head by head, map by map), key pages [pages, K, P, maps * hd].  With value pages
    [pages, K, dv, P]; v_pages None: a key's value is the first `value_dim` entries of its own row.  differential
    (lambda, eps, mult), for two maps: returns [T, H * dv] = (a_1 - lambda a_2) / sqrt(mean(.^2) + eps) * mult per
    head; else [T, H * maps * dv], every map's result."""
    _dev(q, k_pages, v_pages, block_table, token_seq, positions, out)
    q_stride = _rows(q, "paged_attention_maps: q")
    T = q.shape[0]
    if k_pages.dim() != 4 or not k_pages.is_contiguous() or k_pages.dtype != q.dtype:
        raise KernelError(f"paged_attention_maps: key pages must be a contiguous 4-D tensor of {q.dtype}")
    num_pages, Kh, page_size, row = k_pages.shape
    if maps not in (1, 2) or row % maps:
        raise KernelError(f"paged_attention_maps: key rows of {row} entries for {maps} maps")
    hd = row // maps
    if v_pages is not None:
        dv = v_pages.shape[2]
        if v_pages.dtype != q.dtype or not v_pages.is_contiguous() or tuple(v_pages.shape) != (num_pages, Kh, dv, page_size):
            raise KernelError(f"paged_attention_maps: key pages {tuple(k_pages.shape)} do not go with value pages "
                              f"{tuple(v_pages.shape)}")
    else:
        dv = int(value_dim or 0)
        if not 0 < dv <= row:
            raise KernelError(f"paged_attention_maps: {dv} values out of key rows of {row} entries")
    if q.shape[1] < num_heads * maps * hd:
        raise KernelError("paged_attention_maps: query rows are shorter than heads * maps * size")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("paged_attention_maps: block_table must be int32 [sequences, blocks]")
    _i32(token_seq, "paged_attention_maps: token_seq", T)
    _i32(positions, "paged_attention_maps: positions", T)
    if differential is not None and maps != 2:
        raise KernelError("paged_attention_maps: the differential combination needs two maps")
    width = num_heads * (1 if differential is not None else maps) * dv
    if out is None:
        out = torch.empty((T, width), dtype=q.dtype, device=q.device)
    if tuple(out.shape) != (T, width) or out.dtype != q.dtype:
        raise KernelError("paged_attention_maps: bad output")
    out_stride = _rows(out, "paged_attention_maps: out")
    lam, eps, mult = differential if differential is not None else (0.0, 0.0, 1.0)
    _lib.call("sa_paged_attention_maps", _ptr(q), _code(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
              block_table.stride(0), _ptr(token_seq), _ptr(positions), _ptr(out), out_stride, T, num_heads, Kh, hd, dv,
              page_size, int(window or 0), float(scale), int(maps), int(v_pages is None), int(differential is not None),
              float(lam), float(eps), float(mult), _stream())
    return out


def attention_maps_heads_per_unit(num_heads: int, num_kv_heads: int) -> int:
    """How many query heads of a key head share a unit of `paged_attention_maps_units` (a unit holds 16 rows: that
    many heads times 16 // that many tokens)."""
    return int(_lib.load().sa_attention_maps_heads_per_unit(int(num_heads), int(num_kv_heads)))


def attention_maps_units_takes(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor | None, num_heads: int,
                               maps: int = 1) -> bool:
    """Whether `paged_attention_maps_units` takes these sizes (bfloat16 on the GPU, pages of a multiple of 16 keys, key
    vectors of a multiple of 32 entries, values of a multiple of 16)."""
    if q.dtype != torch.bfloat16 or not q.is_cuda or v_pages is None or k_pages.dim() != 4:
        return False
    _, Kh, page_size, row = k_pages.shape
    if row % maps:
        return False
    return bool(_lib.load().sa_paged_attention_maps_units_takes(int(num_heads), int(Kh), int(maps), row // maps,
                                                                int(v_pages.shape[2]), int(page_size), q.stride(0), _ptr(q)))


def paged_attention_maps_units(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                               units: torch.Tensor, unit_begin: int, unit_count: int, num_heads: int, *, scale: float,
                               maps: int = 1, window: int | None = None,
                               differential: "tuple[float, float, float] | None" = None, max_kv_len: int, max_q_len: int,
                               out: torch.Tensor | None = None) -> torch.Tensor:
    """`paged_attention_maps` in bfloat16 on the matrix cores, over the units [unit_begin, unit_begin + unit_count) of
    `units` (int32 [U, 4]: slot, first row, tokens, first position; at most 16 // attention_maps_heads_per_unit tokens
    each).  Two maps come with their differential combination.  Returns [T, H * dv] (rows of no unit are not written)."""
    _dev(q, k_pages, v_pages, block_table, units, out)
    q_stride = _rows(q, "paged_attention_maps_units: q")
    if not attention_maps_units_takes(q, k_pages, v_pages, num_heads, maps):
        raise KernelError("paged_attention_maps_units does not take these sizes (attention_maps_units_takes)")
    if not k_pages.is_contiguous() or not v_pages.is_contiguous() or k_pages.dtype != q.dtype or v_pages.dtype != q.dtype:
        raise KernelError("paged_attention_maps_units: pages are contiguous and of the queries' type")
    num_pages, Kh, page_size, row = k_pages.shape
    dv = v_pages.shape[2]
    if tuple(v_pages.shape) != (num_pages, Kh, dv, page_size):
        raise KernelError(f"paged_attention_maps_units: key pages {tuple(k_pages.shape)} do not go with value pages "
                          f"{tuple(v_pages.shape)}")
    if (maps == 2) != (differential is not None):
        raise KernelError("paged_attention_maps_units: two maps come with their combination, one map has none")
    if block_table.dim() != 2 or block_table.dtype != torch.int32 or block_table.stride(1) != 1:
        raise KernelError("paged_attention_maps_units: block_table must be int32 [sequences, blocks]")
    if units.dtype != torch.int32 or units.dim() != 2 or units.shape[1] != 4 or not units.is_contiguous() \
            or unit_begin < 0 or unit_begin + unit_count > units.shape[0]:
        raise KernelError("paged_attention_maps_units: units must be int32 [U, 4] covering the requested range")
    if out is None:
        out = torch.empty((q.shape[0], num_heads * dv), dtype=q.dtype, device=q.device)
    if out.dtype != q.dtype or tuple(out.shape) != (q.shape[0], num_heads * dv):
        raise KernelError("paged_attention_maps_units: bad output")
    out_stride = _rows(out, "paged_attention_maps_units: out")
    lam, eps, mult = differential if differential is not None else (0.0, 0.0, 1.0)
    ws = _workspace(q.device)
    for at in range(0, int(unit_count), 32768):   # (a launch takes that many units)
        _lib.call("sa_paged_attention_maps_units", _ptr(q), q_stride, _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
                  block_table.stride(0), _ptr(units), int(unit_begin) + at, min(32768, int(unit_count) - at), _ptr(out),
                  out_stride, int(num_heads), Kh, row // maps, dv, page_size, int(window or 0), float(scale), int(maps),
                  int(differential is not None), float(lam), float(eps), float(mult), int(max_kv_len), int(max_q_len),
                  _ptr(ws), ws.numel(), _stream())
    return out


# --------------------------------------------------------------------------- norms behind parts, gates


def residual_add_norm(y: "torch.Tensor | PartialSums | None", residual: torch.Tensor, *,
                      weight: torch.Tensor | None = None, eps: float = 0.0, plus_one: bool = False, mult: float = 1.0,
                      out_dtype: torch.dtype | None = None, out: torch.Tensor | None = None) -> torch.Tensor | None:
    """residual += mult * norm(y; weight) (weight None: += mult * y; y None: nothing is added).  With out_dtype (or
    out) the updated residual is also returned in that type: what a next part without a norm in front reads."""
    if isinstance(y, PartialSums):
        y = y.materialize()
    _dev(y, residual, weight, out)
    T, D = residual.shape
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("residual_add_norm: the residual stream must be contiguous float32")
    ys = 0
    if y is not None:
        if tuple(y.shape) != (T, D):
            raise KernelError(f"residual_add_norm: y {tuple(y.shape)} does not match the residual {T, D}")
        ys = _rows(y, "residual_add_norm: y")
    if weight is not None and (weight.numel() != D or not weight.is_contiguous()):
        raise KernelError("residual_add_norm: the norm weight does not match the width")
    if out is None and out_dtype is not None:
        out = torch.empty((T, D), dtype=out_dtype, device=residual.device)
    if out is not None and (tuple(out.shape) != (T, D) or not out.is_contiguous()):
        raise KernelError("residual_add_norm: bad output")
    if y is None and out is None:
        return None
    _lib.call("sa_residual_add_norm", _ptr(y), _code(y) if y is not None else 0, ys, _ptr(weight),
              _code(weight) if weight is not None else 0, float(eps), int(plus_one), float(mult), _ptr(residual),
              _ptr(out), _code(out) if out is not None else 0, T, D, _stream())
    return out


def residual_add_next_norm(y: "torch.Tensor | PartialSums | None", residual: torch.Tensor, weight: torch.Tensor, *,
                           eps: float, plus_one: bool = False, mult: float = 1.0,
                           out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """residual += mult * y (y None: nothing is added); returns residual / sqrt(mean(residual^2) + eps) * (weight +
    plus_one) in out_dtype: one pass over the rows."""
    if isinstance(y, PartialSums):
        y = y.materialize()
    _dev(y, residual, weight)
    T, D = residual.shape
    if residual.dtype != torch.float32 or not residual.is_contiguous():
        raise KernelError("residual_add_next_norm: the residual stream must be contiguous float32")
    if weight.numel() != D or not weight.is_contiguous():
        raise KernelError("residual_add_next_norm: the norm weight does not match the width")
    ys = 0
    if y is not None:
        if tuple(y.shape) != (T, D):
            raise KernelError(f"residual_add_next_norm: y {tuple(y.shape)} does not match the residual {T, D}")
        ys = _rows(y, "residual_add_next_norm: y")
    if D > 8192:
        residual_add_norm(y, residual, mult=mult)
        return rmsnorm(residual, weight, eps, plus_one, out_dtype or (y.dtype if y is not None else torch.float32))
    out = torch.empty((T, D), dtype=out_dtype or (y.dtype if y is not None else torch.float32), device=residual.device)
    _lib.call("sa_residual_add_next_norm", _ptr(y), _code(y) if y is not None else 0, ys, float(mult), _ptr(residual),
              _ptr(weight), _code(weight), float(eps), int(plus_one), _ptr(out), _code(out), T, D, _stream())
    return out


GATE_SIGMOID, GATE_SILU = 0, 1


def gated_heads(x: torch.Tensor, gate: torch.Tensor, num_heads: int, size: int, *, kind: int,
                weight: torch.Tensor | None = None, eps: float = 0.0, out_dtype: torch.dtype | None = None,
                out: torch.Tensor | None = None, per_head: bool = False) -> torch.Tensor:
    """out[t, h] = (x[t, h] normed over the head's `size` entries and times weight [size], if a weight is given,
    else x[t, h]) * sigmoid(gate[t, h]) or * silu(gate[t, h]).  x, gate: rows of num_heads * size (views with a
    row stride are fine); per_head: gate rows of num_heads, one number for all entries of a head."""
    _dev(x, gate, weight, out)
    T = x.shape[0]
    width = num_heads * size
    xs, gs = _rows(x, "gated_heads: x"), _rows(gate, "gated_heads: gate")
    if x.shape[1] != width or tuple(gate.shape) != (T, num_heads if per_head else width):
        raise KernelError(f"gated_heads: rows of {width} expected, got x {tuple(x.shape)} gate {tuple(gate.shape)}")
    if weight is not None and (weight.numel() != size or not weight.is_contiguous()):
        raise KernelError("gated_heads: the norm weight has one entry per element of a head")
    if kind not in (GATE_SIGMOID, GATE_SILU):
        raise KernelError(f"gated_heads: unknown gate {kind!r}")
    if out is None:
        out = torch.empty((T, width), dtype=out_dtype or x.dtype, device=x.device)
    if tuple(out.shape) != (T, width):
        raise KernelError("gated_heads: bad output")
    os_ = _rows(out, "gated_heads: out")
    _lib.call("sa_gated_heads", _ptr(x), _code(x), xs, _ptr(gate), _code(gate), gs, _ptr(weight),
              _code(weight) if weight is not None else 0, float(eps), int(kind), _ptr(out), _code(out), os_, T,
              num_heads, size, int(bool(per_head)), _stream())
    return out


def activation_(x: torch.Tensor, activation: int) -> torch.Tensor:
    """x = act(x) in place (an activation code of the ACTIVATIONS registry)."""
    _dev(x)
    stride = _rows(x, "activation_: x")
    _lib.call("sa_activation", _ptr(x), _code(x), stride, x.shape[0], x.shape[1], int(activation), _stream())
    return x


def qk_norm_rope_cache_write(proj: torch.Tensor, positions: torch.Tensor, inv_freq: torch.Tensor | None, rot_dims: int,
                             eps: float | None, num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, *,
                             v_first: torch.Tensor | None = None, v_mix: torch.Tensor | None = None,
                             slot_mapping: torch.Tensor | None = None, k_pages: torch.Tensor | None = None,
                             v_pages: torch.Tensor | None = None, q_mult: float = 1.0) -> torch.Tensor:
    """In place on fused projection rows [H * dk | K * dk | K * dv | ...]: queries and keys rotated on their first
    rot_dims dimensions (angle position * inv_freq[i] for the pair (i, i + rot_dims / 2)), then divided by their root
    mean square (eps None: not); values mixed, (1 - v_mix) v + v_mix v_first (v_first [T, K * dv] rows of another
    layer, v_mix a tensor of one element), keys and values written into the pages.  q_mult: a factor on the
    queries (the scores' factor, for an attention kernel that has none of its own)."""
    _dev(proj, positions, inv_freq, v_first, v_mix, slot_mapping, k_pages, v_pages)
    stride = _rows(proj, "qk_norm_rope_cache_write: proj")
    T = proj.shape[0]
    H, K, dk, dv = num_heads, num_kv_heads, key_dim, value_dim
    if proj.shape[1] < (H + K) * dk + K * dv:
        raise KernelError(f"qk_norm_rope_cache_write: rows of {proj.shape[1]} are shorter than (H + K) dk + K dv")
    _i32(positions, "qk_norm_rope_cache_write: positions", T)
    if rot_dims:
        if inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rot_dims // 2 \
                or not inv_freq.is_contiguous() or rot_dims % 2 or rot_dims > dk:
            raise KernelError("qk_norm_rope_cache_write: inv_freq must be float32 [rot_dims / 2], rot_dims even, <= dk")
    page_size, vfs = 1, 0
    if k_pages is not None:
        if v_pages is None or slot_mapping is None:
            raise KernelError("qk_norm_rope_cache_write: key pages, value pages and slots come together")
        if k_pages.dim() != 4 or v_pages.dim() != 4 or not k_pages.is_contiguous() or not v_pages.is_contiguous() \
                or k_pages.dtype != proj.dtype or v_pages.dtype != proj.dtype:
            raise KernelError(f"qk_norm_rope_cache_write: pages must be contiguous 4-D tensors of {proj.dtype}")
        n, _, page_size, _ = k_pages.shape
        if tuple(k_pages.shape) != (n, K, page_size, dk) or tuple(v_pages.shape) != (n, K, dv, page_size):
            raise KernelError(f"qk_norm_rope_cache_write: pages {tuple(k_pages.shape)}, {tuple(v_pages.shape)} do not "
                              f"match {K} heads of key size {dk} and value size {dv}")
        if slot_mapping.dtype != torch.int64 or slot_mapping.numel() < T or not slot_mapping.is_contiguous():
            raise KernelError("qk_norm_rope_cache_write: slot_mapping must be int64 [T]")
    if v_first is not None:
        if v_mix is None or v_mix.numel() != 1 or v_first.dtype != proj.dtype or v_first.shape[0] != T \
                or v_first.shape[1] != K * dv:
            raise KernelError("qk_norm_rope_cache_write: mixed values need a factor of one element and rows "
                              "[T, K * dv] of the projection's type")
        vfs = _rows(v_first, "qk_norm_rope_cache_write: v_first")
    _lib.call("sa_qk_norm_rope_cache_write", _ptr(proj), _code(proj), stride, _ptr(positions), _ptr(inv_freq),
              int(rot_dims), float(eps) if eps is not None else -1.0, float(q_mult), _ptr(v_first), vfs, _ptr(v_mix),
              _code(v_mix) if v_mix is not None else 0, _ptr(slot_mapping), _ptr(k_pages), _ptr(v_pages), T, H, K, dk,
              dv, int(page_size), _stream())
    return proj


def attention_inputs(proj: torch.Tensor, seq_meta: torch.Tensor, num_seqs: int, max_q_len: int, num_heads: int,
                     num_kv_heads: int, key_dim: int, value_dim: int, *, values_are_keys: bool = False,
                     taps: torch.Tensor | None = None, tails: torch.Tensor | None = None, norm: str | None = None,
                     q_weight: torch.Tensor | None = None, k_weight: torch.Tensor | None = None, eps: float = 0.0,
                     inv_freq: torch.Tensor | None = None, rot_dims: int = 0, temp_coef: float = 0.0, temp_every: int = 0,
                     q_mult: float = 1.0, taps_by_tap: torch.Tensor | None = None, in_bias: torch.Tensor | None = None,
                     slot_mapping: torch.Tensor | None = None, k_pages: torch.Tensor | None = None,
                     v_pages: torch.Tensor | None = None) -> torch.Tensor:
    """From fused projection rows [H * dk queries | K * dk keys | K * dv values | ...] of a ragged step (seq_meta) to
    what an attention kernel reads.  taps [channels, n] with tails float32 [slots, (n - 1) * channels]: every channel
    passes a causal convolution first (taps oldest first; the tails are the rows that earlier steps projected last and
    are brought up to date).  norm 'head': queries and keys divided by each head's root mean square, times q_weight /
    k_weight [dk]; 'row': by the whole row's, times weights [H * dk] / [K * dk].  Then the first rot_dims entries of
    every head turn in pairs (i, i + rot_dims / 2) by position * inv_freq[i]; queries are multiplied by
    1 + temp_coef * ln(floor((position + 1) / temp_every) + 1) (temp_every 0: not) and by q_mult.  Keys go into k_pages, values
    (values_are_keys: the keys' columns as projected, and there are no value columns) into v_pages; without pages the
    rows hold queries only.  taps_by_tap: the taps once more as [n, channels] (what the kernel for aligned bfloat16 rows
    reads in pieces of eight channels).  in_bias (only without taps): a bias per channel that the projection has not
    had added yet.  Returns the queries [T, H * dk] in proj's type."""
    _dev(proj, seq_meta, taps, tails, q_weight, k_weight, inv_freq, slot_mapping, k_pages, v_pages)
    stride = _rows(proj, "attention_inputs: proj")
    T = proj.shape[0]
    H, K, dk, dv = int(num_heads), int(num_kv_heads), int(key_dim), int(value_dim)
    _seq_meta(seq_meta, num_seqs, "attention_inputs")
    own = k_pages is not None
    C = (H + K) * dk + (0 if values_are_keys else K * dv) if own else H * dk
    if proj.shape[1] < C:
        raise KernelError(f"attention_inputs: rows of {proj.shape[1]} are shorter than the {C} columns")
    code = {None: 0, "head": 1, "row": 2}.get(norm)
    if code is None:
        raise KernelError(f"attention_inputs: norm is None, 'head' or 'row', not {norm!r}")
    w_dtype = None
    if code:
        wanted = [(q_weight, dk if code == 1 else H * dk)] + ([(k_weight, dk if code == 1 else K * dk)] if own else [])
        for w, n in wanted:
            if w is None or not w.is_contiguous() or w.numel() != n or (w_dtype is not None and w.dtype != w_dtype):
                raise KernelError("attention_inputs: norm weights are contiguous, of one type, one entry per normed entry")
            w_dtype = w.dtype
    n_taps = 0
    if taps is not None:
        if taps.dim() != 2 or taps.shape[0] != C or not taps.is_contiguous():
            raise KernelError(f"attention_inputs: taps {tuple(taps.shape)} for {C} channels")
        n_taps = taps.shape[1]
        if n_taps > 1 and (tails is None or tails.dtype != torch.float32 or tails.dim() != 2 or tails.stride(1) != 1
                           or tails.shape[1] < (n_taps - 1) * C):
            raise KernelError("attention_inputs: tails must be float32 [slots, >= (taps - 1) * channels]")
    if taps_by_tap is not None and (taps is None or tuple(taps_by_tap.shape) != (n_taps, C) or taps_by_tap.dtype != taps.dtype
                                    or not taps_by_tap.is_contiguous()):
        raise KernelError("attention_inputs: taps_by_tap is the taps transposed, [taps, channels], contiguous")
    _dev(taps_by_tap, in_bias)
    if in_bias is not None and (taps is not None or in_bias.numel() < C or not in_bias.is_contiguous()):
        raise KernelError("attention_inputs: a bias (one entry per channel, contiguous) is added here only without a convolution")
    if rot_dims and (inv_freq is None or inv_freq.dtype != torch.float32 or inv_freq.numel() != rot_dims // 2
                     or not inv_freq.is_contiguous() or rot_dims % 2 or rot_dims > dk):
        raise KernelError("attention_inputs: inv_freq must be float32 [rot_dims / 2], rot_dims even, <= dk")
    page_size = 1
    if own:
        if v_pages is None or slot_mapping is None:
            raise KernelError("attention_inputs: key pages, value pages and slots come together")
        if k_pages.dim() != 4 or v_pages.dim() != 4 or not k_pages.is_contiguous() or not v_pages.is_contiguous() \
                or k_pages.dtype != proj.dtype or v_pages.dtype != proj.dtype:
            raise KernelError(f"attention_inputs: pages must be contiguous 4-D tensors of {proj.dtype}")
        n, _, page_size, _ = k_pages.shape
        if tuple(k_pages.shape) != (n, K, page_size, dk) or tuple(v_pages.shape) != (n, K, dv, page_size):
            raise KernelError(f"attention_inputs: pages {tuple(k_pages.shape)}, {tuple(v_pages.shape)} do not match "
                              f"{K} heads of key size {dk} and value size {dv}")
        if slot_mapping.dtype != torch.int64 or slot_mapping.numel() < T or not slot_mapping.is_contiguous():
            raise KernelError("attention_inputs: slot_mapping must be int64 [T]")
    q_out = torch.empty((T, H * dk), dtype=proj.dtype, device=proj.device)
    _lib.call("sa_attention_inputs", _ptr(proj), _code(proj), stride, H, K, dk, dv, H * dk, (H + K) * dk,
              int(bool(values_are_keys)), _ptr(taps), _code(taps) if taps is not None else 0, int(n_taps),
              _ptr(tails) if n_taps > 1 else None, tails.stride(0) if n_taps > 1 else 0, code, _ptr(q_weight),
              _ptr(k_weight) if own else None, _CODES[w_dtype] if w_dtype is not None else 0, float(eps), _ptr(inv_freq),
              int(rot_dims), float(temp_coef), int(temp_every), float(q_mult), _ptr(seq_meta), int(num_seqs), int(max_q_len),
              _ptr(slot_mapping) if own else None, _ptr(q_out), q_out.stride(0), _ptr(k_pages), _ptr(v_pages) if own else None,
              int(page_size), _ptr(taps_by_tap), _ptr(in_bias), _code(in_bias) if in_bias is not None else 0, _stream())
    return q_out


# --------------------------------------------------------------------------- recurrent mixers


def norm_rope_cache_write(proj: torch.Tensor, positions: torch.Tensor, freq: torch.Tensor | None, rot_dims: int,
                          num_heads: int, num_kv_heads: int, key_dim: int, value_dim: int, *, rot_mult: float = 1.0,
                          sub: int = 1, eps: float = 0.0, q_weight: torch.Tensor | None = None, q_norm_dims: int = 0,
                          q_rot_at: int = 0, k_weight: torch.Tensor | None = None, k_norm_dims: int = 0,
                          k_rot_at: int = 0, slot_mapping: torch.Tensor | None = None,
                          k_pages: torch.Tensor | None = None, v_pages: torch.Tensor | None = None,
                          key_values: int = 0) -> torch.Tensor:
    """In place on fused projection rows [H * dk | K * dk | K * dv | ...]: every query and key vector is `sub` equal
    parts; in each part the first *_norm_dims entries are divided by their root mean square (eps inside the root) and
    multiplied by *_weight (None: no norm), then the entries [*_rot_at, *_rot_at + rot_dims) turn in neighbouring pairs
    (2p, 2p + 1) by position * freq[p], cos and sin times rot_mult.  Queries go back in place, keys into k_pages
    [pages, K, P, dk], values (value_dim > 0) into v_pages [pages, K, dv, P]."""
    _dev(proj, positions, freq, q_weight, k_weight, slot_mapping, k_pages, v_pages)
    stride = _rows(proj, "norm_rope_cache_write: proj")
    T = proj.shape[0]
    H, K, dk, dv = int(num_heads), int(num_kv_heads), int(key_dim), int(value_dim)
    if proj.shape[1] < (H + K) * dk + K * dv:
        raise KernelError(f"norm_rope_cache_write: rows of {proj.shape[1]} are shorter than (H + K) dk + K dv")
    _i32(positions, "norm_rope_cache_write: positions", T)
    if rot_dims and (freq is None or freq.dtype != torch.float32 or freq.numel() != rot_dims // 2
                     or not freq.is_contiguous() or rot_dims % 2):
        raise KernelError("norm_rope_cache_write: freq must be float32 [rot_dims / 2], rot_dims even")
    w_dtype = None
    for w, n in ((q_weight, q_norm_dims), (k_weight, k_norm_dims)):
        if w is not None:
            if not w.is_contiguous() or w.numel() < n or (w_dtype is not None and w.dtype != w_dtype):
                raise KernelError("norm_rope_cache_write: norm weights are contiguous, of one type, one entry per normed entry")
            w_dtype = w.dtype
    page_size = 1
    if k_pages is not None:
        if slot_mapping is None or ((dv > 0 or key_values > 0) and v_pages is None):
            raise KernelError("norm_rope_cache_write: key pages come with slots and, if there are values, value pages")
        if key_values and (dv or not 0 < key_values <= dk):
            raise KernelError("norm_rope_cache_write: key_values goes with value_dim 0 and is at most the key size")
        if k_pages.dim() != 4 or not k_pages.is_contiguous() or k_pages.dtype != proj.dtype \
                or k_pages.shape[1] != K or k_pages.shape[3] != dk:
            raise KernelError(f"norm_rope_cache_write: key pages {tuple(k_pages.shape)} do not match {K} heads of {dk}")
        page_size = k_pages.shape[2]
        if (dv or key_values) and (v_pages.dtype != proj.dtype or not v_pages.is_contiguous()
                                   or tuple(v_pages.shape) != (k_pages.shape[0], K, dv or key_values, page_size)):
            raise KernelError(f"norm_rope_cache_write: value pages {tuple(v_pages.shape)} do not match")
        if slot_mapping.dtype != torch.int64 or slot_mapping.numel() < T or not slot_mapping.is_contiguous():
            raise KernelError("norm_rope_cache_write: slot_mapping must be int64 [T]")
    _lib.call("sa_norm_rope_cache_write", _ptr(proj), _code(proj), stride, _ptr(positions), _ptr(freq), int(rot_dims),
              float(rot_mult), _ptr(q_weight), int(q_norm_dims), int(q_rot_at), _ptr(k_weight), int(k_norm_dims),
              int(k_rot_at), _CODES[w_dtype] if w_dtype is not None else 0, float(eps), int(sub), _ptr(slot_mapping),
              _ptr(k_pages), _ptr(v_pages) if (dv > 0 or key_values > 0) and k_pages is not None else None, T, H, K, dk, dv,
              int(page_size), int(key_values) if k_pages is not None else 0, _stream())
    return proj


def short_conv(x: torch.Tensor, taps: torch.Tensor, tails: torch.Tensor, seq_meta: torch.Tensor, num_seqs: int,
               max_q_len: int, *, in_bias: torch.Tensor | None = None, out_bias: torch.Tensor | None = None,
               silu: bool = False, update_tails: bool = True) -> torch.Tensor:
    """`short_conv_silu` with the activation optional and two biases: y = act(sum_j taps[c, j] (x + in_bias)[t - ...]
    + out_bias); the tails hold x + in_bias.  Returns float32 [T, C]."""
    _dev(x, taps, tails, seq_meta, in_bias, out_bias)
    stride = _rows(x, "short_conv: x")
    T, C = x.shape
    if taps.dim() != 2 or taps.shape[0] != C or not taps.is_contiguous():
        raise KernelError(f"short_conv: taps {tuple(taps.shape)} for {C} channels")
    n = taps.shape[1]
    if tails.dtype != torch.float32 or tails.dim() != 2 or tails.stride(1) != 1 or tails.shape[1] < (n - 1) * C:
        raise KernelError("short_conv: tails must be float32 [slots, >= (taps - 1) * channels]")
    _seq_meta(seq_meta, num_seqs, "short_conv")
    b_dtype = None
    for b in (in_bias, out_bias):
        if b is not None:
            if b.numel() != C or not b.is_contiguous() or (b_dtype is not None and b.dtype != b_dtype):
                raise KernelError("short_conv: biases are contiguous, of one type, one entry per channel")
            b_dtype = b.dtype
    out = torch.empty((T, C), dtype=torch.float32, device=x.device)
    _lib.call("sa_short_conv", _ptr(x), _code(x), stride, _ptr(in_bias), _ptr(taps), _code(taps), n, _ptr(out_bias),
              _CODES[b_dtype] if b_dtype is not None else 0, int(silu), _ptr(tails), tails.stride(0), _ptr(seq_meta),
              int(num_seqs), int(max_q_len), _ptr(out), C, int(update_tails), _stream())
    return out


def head_product(x: torch.Tensor, w: torch.Tensor, *, in_stride: int | None = None, tail: int = 0,
                 gate: torch.Tensor | None = None, out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """A product per head: out[t, h, :O] = w[h] x[t, h, :I] with w [H, O, I], summed in 32-bit.  x rows hold the
    heads `in_stride` entries apart (default I + tail).  tail: the entries behind a head's inputs are copied behind its
    outputs.  gate [T, H] (a view is fine): the outputs are multiplied by sigmoid(gate).  Returns [T, H * (O + tail)]."""
    _dev(x, w, gate)
    xs = _rows(x, "head_product: x")
    T = x.shape[0]
    if w.dim() != 3 or not w.is_contiguous():
        raise KernelError("head_product: the weights are a contiguous [heads, outputs, inputs] tensor")
    H, O, I = w.shape
    hs = int(in_stride) if in_stride is not None else I + tail
    if hs < I + tail or x.shape[1] < (H - 1) * hs + I + tail:
        raise KernelError(f"head_product: rows of {x.shape[1]} do not hold {H} heads {hs} apart with {I + tail} entries")
    gs = 0
    if gate is not None:
        gs = _rows(gate, "head_product: gate")
        if gate.shape[0] != T or gate.shape[1] != H:
            raise KernelError(f"head_product: gates {tuple(gate.shape)} are not [T, H]")
    out = torch.empty((T, H * (O + tail)), dtype=out_dtype or x.dtype, device=x.device)
    _lib.call("sa_head_product", _ptr(x), _code(x), xs, hs, _ptr(w), _code(w), _ptr(out), _code(out), out.stride(0),
              O + tail, T, H, I, O, int(tail), _ptr(gate), _code(gate) if gate is not None else 0, gs, _stream())
    return out


def rglru_scan(u: torch.Tensor, gates: torch.Tensor, block: int, r_bias: torch.Tensor, i_bias: torch.Tensor,
               lam: torch.Tensor, y: torch.Tensor, y_bias: torch.Tensor | None, state: torch.Tensor,
               seq_meta: torch.Tensor, num_seqs: int, *, c: float = 8.0, out_dtype: torch.dtype | None = None,
               max_q_len: int | None = None) -> torch.Tensor:
    """The real-gated linear recurrence, channel by channel over each request's tokens, from and into state [slots, C]
    float32 (a view is fine): r = sigmoid(gr + r_bias), i = sigmoid(gi + i_bias), a = exp(-c r softplus(lam)),
    S <- a S + sqrt(1 - a^2) i u; returns S * gelu_tanh(y + y_bias) in out_dtype.  u float32 [T, C]; gates float32
    [T, 2 C], per block of `block` channels [gr | gi]; y [T, C] rows of the activation type.  max_q_len: the most
    tokens of a request (None: T); long portions run in segments of 64 tokens side by side."""
    _dev(u, gates, r_bias, i_bias, lam, y, y_bias, state, seq_meta)
    T, C = u.shape
    if u.dtype != torch.float32 or not u.is_contiguous() or gates.dtype != torch.float32 or not gates.is_contiguous() \
            or tuple(gates.shape) != (T, 2 * C):
        raise KernelError("rglru_scan: u is contiguous float32 [T, C], gates contiguous float32 [T, 2 C]")
    if block < 1 or C % block:
        raise KernelError(f"rglru_scan: blocks of {block} do not divide {C} channels")
    vecs = [r_bias, i_bias, lam] + ([y_bias] if y_bias is not None else [])
    if any(v.numel() != C or not v.is_contiguous() or v.dtype != lam.dtype for v in vecs):
        raise KernelError("rglru_scan: biases and lam are contiguous, of one type, one entry per channel")
    ys = _rows(y, "rglru_scan: y")
    if tuple(y.shape) != (T, C):
        raise KernelError(f"rglru_scan: y {tuple(y.shape)} is not [T, C]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < C:
        raise KernelError("rglru_scan: the state must be float32 [slots, >= channels]")
    _seq_meta(seq_meta, num_seqs, "rglru_scan")
    out = torch.empty((T, C), dtype=out_dtype or y.dtype, device=u.device)
    q = max(1, min(int(max_q_len if max_q_len is not None else T), T))
    scratch = None
    if q > 128:   # (the segments' summaries and the requests' states at the step's start)
        scratch = torch.empty((int(num_seqs) * (2 * -(-q // 64) + 1) * C,), dtype=torch.float32, device=u.device)
    _lib.call("sa_rglru_scan", _ptr(u), _ptr(gates), int(block), _ptr(r_bias), _ptr(i_bias), _ptr(lam), _code(lam),
              float(c), _ptr(y), _code(y), ys, _ptr(y_bias), _ptr(state), state.stride(0), _ptr(seq_meta), int(num_seqs),
              q, _ptr(scratch), scratch.numel() if scratch is not None else 0, _ptr(out), _code(out), C, _stream())
    return out


def short_conv_silu(x: torch.Tensor, taps: torch.Tensor, tails: torch.Tensor, seq_meta: torch.Tensor, num_seqs: int,
                    max_q_len: int, *, update_tails: bool = True, out: torch.Tensor | None = None) -> torch.Tensor:
    """y[t, c] = silu(sum_j taps[c, j] x[t - (n - 1 - j), c]) along each request's tokens (seq_meta rows: state slot,
    first row, rows, first position); inputs before the step come from tails [slots, (n - 1) * C] float32, which
    afterwards hold each request's last n - 1 inputs.  x: [T, C] rows (a view is fine).  Returns float32 [T, C]."""
    _dev(x, taps, tails, seq_meta, out)
    stride = _rows(x, "short_conv_silu: x")
    T, C = x.shape
    if taps.dim() != 2 or taps.shape[0] != C or not taps.is_contiguous():
        raise KernelError(f"short_conv_silu: taps {tuple(taps.shape)} for {C} channels")
    n = taps.shape[1]
    if tails.dtype != torch.float32 or tails.dim() != 2 or tails.stride(1) != 1 or tails.shape[1] < (n - 1) * C:
        raise KernelError("short_conv_silu: tails must be float32 [slots, >= (taps - 1) * channels]")
    if seq_meta.dtype != torch.int32 or seq_meta.dim() != 2 or seq_meta.shape[1] != 4 or not seq_meta.is_contiguous() \
            or seq_meta.shape[0] < num_seqs:
        raise KernelError("short_conv_silu: seq_meta must be int32 [S, 4]")
    if out is None:
        out = torch.empty((T, C), dtype=torch.float32, device=x.device)
    if out.dtype != torch.float32 or tuple(out.shape) != (T, C) or not out.is_contiguous():
        raise KernelError("short_conv_silu: the output must be contiguous float32 [T, C]")
    _lib.call("sa_short_conv_silu", _ptr(x), _code(x), stride, _ptr(taps), _code(taps), n, _ptr(tails), tails.stride(0),
              _ptr(seq_meta), int(num_seqs), int(max_q_len), _ptr(out), C, int(update_tails), _stream())
    return out


def delta_prepare(qkv: torch.Tensor, ab: torch.Tensor, a_log: torch.Tensor, dt_bias: torch.Tensor, num_heads: int,
                  num_qk_heads: int, key_dim: int) -> torch.Tensor:
    """In place on qkv float32 [T, C] = [G q heads | G k heads | values]: q and k heads to unit length, q also times
    key_dim ** -0.5.  Returns gates float32 [T, 2 H]: beta = sigmoid(b), then g = exp(-exp(a_log) softplus(a +
    dt_bias)), from ab [T, 2 H] = [a | b]."""
    _dev(qkv, ab, a_log, dt_bias)
    T, C = qkv.shape
    H, G = num_heads, num_qk_heads
    if qkv.dtype != torch.float32 or not qkv.is_contiguous():
        raise KernelError("delta_prepare: qkv must be contiguous float32")
    abs_ = _rows(ab, "delta_prepare: ab")
    if ab.shape[0] != T or ab.shape[1] != 2 * H:
        raise KernelError(f"delta_prepare: ab {tuple(ab.shape)} is not [T, 2 H]")
    if a_log.numel() != H or dt_bias.numel() != H or a_log.dtype != dt_bias.dtype or not a_log.is_contiguous() \
            or not dt_bias.is_contiguous():
        raise KernelError("delta_prepare: a_log and dt_bias have one entry per head, of one type")
    gates = torch.empty((T, 2 * H), dtype=torch.float32, device=qkv.device)
    _lib.call("sa_delta_prepare", _ptr(qkv), T, C, G, key_dim, _ptr(ab), _code(ab), abs_, _ptr(a_log), _ptr(dt_bias),
              _code(a_log), H, _ptr(gates), _stream())
    return gates


def delta_inputs(x: torch.Tensor, taps: torch.Tensor, tails: torch.Tensor, ab: torch.Tensor, a_log: torch.Tensor,
                 dt_bias: torch.Tensor, seq_meta: torch.Tensor, num_seqs: int, max_q_len: int, num_heads: int,
                 num_qk_heads: int, key_dim: int) -> tuple[torch.Tensor, torch.Tensor]:
    """`short_conv_silu` (the tails updated) followed by `delta_prepare`: returns (qkv float32 [T, C], gates float32
    [T, 2 H]).  One launch where no request of the step brings more than a handful of tokens (decoding), the two
    kernels otherwise."""
    if x.dtype != taps.dtype or not bool(_lib.load().sa_delta_inputs_few_takes(int(max_q_len), int(key_dim))):
        qkv = short_conv_silu(x, taps, tails, seq_meta, num_seqs, max_q_len)
        return qkv, delta_prepare(qkv, ab, a_log, dt_bias, num_heads, num_qk_heads, key_dim)
    _dev(x, taps, tails, ab, a_log, dt_bias, seq_meta)
    stride = _rows(x, "delta_inputs: x")
    T, C = x.shape
    H, G = num_heads, num_qk_heads
    if taps.dim() != 2 or taps.shape[0] != C or not taps.is_contiguous():
        raise KernelError(f"delta_inputs: taps {tuple(taps.shape)} for {C} channels")
    n = taps.shape[1]
    if tails.dtype != torch.float32 or tails.dim() != 2 or tails.stride(1) != 1 or tails.shape[1] < (n - 1) * C:
        raise KernelError("delta_inputs: tails must be float32 [slots, >= (taps - 1) * channels]")
    if seq_meta.dtype != torch.int32 or seq_meta.dim() != 2 or seq_meta.shape[1] != 4 or not seq_meta.is_contiguous() \
            or seq_meta.shape[0] < num_seqs:
        raise KernelError("delta_inputs: seq_meta must be int32 [S, 4]")
    abs_ = _rows(ab, "delta_inputs: ab")
    if ab.shape[0] != T or ab.shape[1] != 2 * H or C < 2 * G * key_dim:
        raise KernelError(f"delta_inputs: ab {tuple(ab.shape)} is not [T, 2 H], or too few channels")
    if a_log.numel() != H or dt_bias.numel() != H or a_log.dtype != dt_bias.dtype or not a_log.is_contiguous() \
            or not dt_bias.is_contiguous():
        raise KernelError("delta_inputs: a_log and dt_bias have one entry per head, of one type")
    qkv = torch.empty((T, C), dtype=torch.float32, device=x.device)
    gates = torch.empty((T, 2 * H), dtype=torch.float32, device=x.device)
    _lib.call("sa_delta_inputs_few", _ptr(x), _code(x), stride, _ptr(taps), _code(taps), n, _ptr(tails), tails.stride(0),
              _ptr(seq_meta), int(num_seqs), int(max_q_len), _ptr(qkv), C, G, int(key_dim), _ptr(ab), _code(ab), abs_,
              _ptr(a_log), _ptr(dt_bias), _code(a_log), H, _ptr(gates), _stream())
    return qkv, gates


def delta_rule(qkv: torch.Tensor, gates: torch.Tensor, state: torch.Tensor, seq_meta: torch.Tensor, num_seqs: int,
               num_heads: int, num_qk_heads: int, key_dim: int, value_dim: int) -> torch.Tensor:
    """The gated delta rule along each request's tokens, from and into state [slots, >= H * dk * dv] float32 (per
    slot and head the matrix S [dk, dv], stored column by column: [H][dv][dk]).  qkv float32 [T, C] as `delta_prepare` left it, gates [T, 2 H].  Returns float32 [T, H * dv]."""
    _dev(qkv, gates, state, seq_meta)
    T, C = qkv.shape
    H, G, dk, dv = num_heads, num_qk_heads, key_dim, value_dim
    if qkv.dtype != torch.float32 or not qkv.is_contiguous() or C < 2 * G * dk + H * dv:
        raise KernelError("delta_rule: qkv must be contiguous float32 [T, >= 2 G dk + H dv]")
    if gates.dtype != torch.float32 or tuple(gates.shape) != (T, 2 * H) or not gates.is_contiguous():
        raise KernelError("delta_rule: gates must be contiguous float32 [T, 2 H]")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < H * dk * dv:
        raise KernelError("delta_rule: the state must be float32 [slots, >= H * dk * dv]")
    if seq_meta.dtype != torch.int32 or seq_meta.dim() != 2 or seq_meta.shape[1] != 4 or not seq_meta.is_contiguous() \
            or seq_meta.shape[0] < num_seqs:
        raise KernelError("delta_rule: seq_meta must be int32 [S, 4]")
    out = torch.empty((T, H * dv), dtype=torch.float32, device=qkv.device)
    _lib.call("sa_delta_rule", _ptr(qkv), C, G, dk, dv, _ptr(gates), H, _ptr(state), state.stride(0), _ptr(seq_meta),
              int(num_seqs), _ptr(out), _stream())
    return out


# --------------------------------------------------------------------------- measurements of the machine


def probe_hbm_read(buffer: torch.Tensor, order: torch.Tensor | None = None) -> None:
    """All CUs read `buffer` (whole 8 KiB pieces) once from memory, piece after piece or in the order given (int32
    piece numbers): the caller times it.  What the decode step's kernels, which are bound by reading weights and
    cache, can reach at most."""
    _dev(buffer, order)
    nbytes = buffer.numel() * buffer.element_size()
    if not buffer.is_contiguous() or nbytes % 8192:
        raise KernelError("probe_hbm_read: a contiguous buffer of whole 8 KiB pieces")
    if order is not None:
        _i32(order, "probe_hbm_read: order", nbytes // 8192)
    sink = _workspace(buffer.device)
    _lib.call("sa_probe_hbm_read", _ptr(buffer), nbytes, _ptr(order), _ptr(sink), _stream())


def probe_mfma(operands: torch.Tensor, iters: int, workgroups: int = 256) -> float:
    """`workgroups` workgroups of eight waves each retire 16 * iters bfloat16 MFMA instructions per wave on the
    16 KiB of `operands`; returns the floating-point operations that this is (the caller times it).  The rate
    depends on the operands' bits: the clock that the GPU holds under this load does."""
    _dev(operands)
    if operands.numel() * operands.element_size() < 16384 or not operands.is_contiguous():
        raise KernelError("probe_mfma: 16 KiB of operands")
    sink = _workspace(operands.device)
    _lib.call("sa_probe_mfma", _ptr(operands), int(iters), int(workgroups), _ptr(sink), _stream())
    return 2.0 * 16 * 16 * 32 * 16 * iters * 8 * workgroups


# --------------------------------------------------------------------------- sampling


SAMPLE_DRAWN, SAMPLE_TOP_K, SAMPLE_TOP_P = 1, 2, 4


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           seed: torch.Tensor, counter: torch.Tensor, tokens: torch.Tensor | None = None,
           logprobs: torch.Tensor | None = None, modes: int = 7) -> tuple[torch.Tensor, torch.Tensor]:
    """One token per row.  All per-row parameter tensors are on the device, [R].  modes: what some row may ask
    for (SAMPLE_DRAWN + SAMPLE_TOP_K + SAMPLE_TOP_P); the kernels for what no row asks for are left out."""
    _dev(logits, temperature, top_k, top_p, seed, counter, tokens, logprobs)
    if logits.dtype != torch.float32:
        raise KernelError("sample: logits must be float32")
    stride = _rows(logits, "sample: logits")
    R, V = logits.shape
    for t, dt, name in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"),
                        (top_p, torch.float32, "top_p"), (seed, torch.int64, "seed"), (counter, torch.int32, "counter")):
        if t.dtype != dt or t.numel() < R or not t.is_contiguous():
            raise KernelError(f"sample: {name} must be a contiguous {dt} tensor with one entry per row")
    if tokens is None:
        tokens = torch.empty(R, dtype=torch.int32, device=logits.device)
    if logprobs is None:
        logprobs = torch.empty(R, dtype=torch.float32, device=logits.device)
    _i32(tokens, "sample: tokens", R)
    ws = _workspace(logits.device)
    _lib.call("sa_sample", _ptr(logits), stride, R, V, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(seed),
              _ptr(counter), _ptr(tokens), _ptr(logprobs), int(modes), _ptr(ws), ws.numel(), _stream())
    return tokens, logprobs


#: what `score` gives for a token that is left out (the reference's neg_inf for float32)
SCORE_MASKED = -0.5 * 3.4028234663852886e38


def score(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
          tokens: torch.Tensor, scores: torch.Tensor | None = None) -> torch.Tensor:
    """The log-probability of tokens[r] under row r's temperature, top-k and top-p, as `sample` reports it for the
    token it draws: greedy rows give 0 for the argmax and SCORE_MASKED otherwise, a token that the masks leave out
    gives SCORE_MASKED."""
    _dev(logits, temperature, top_k, top_p, tokens, scores)
    if logits.dtype != torch.float32:
        raise KernelError("score: logits must be float32")
    stride = _rows(logits, "score: logits")
    R, V = logits.shape
    for t, dt, name in ((temperature, torch.float32, "temperature"), (top_k, torch.int32, "top_k"),
                        (top_p, torch.float32, "top_p")):
        if t.dtype != dt or t.numel() < R or not t.is_contiguous():
            raise KernelError(f"score: {name} must be a contiguous {dt} tensor with one entry per row")
    _i32(tokens, "score: tokens", R)
    if scores is None:
        scores = torch.empty(R, dtype=torch.float32, device=logits.device)
    if scores.dtype != torch.float32 or scores.numel() < R or not scores.is_contiguous():
        raise KernelError("score: scores must be a contiguous float32 tensor with one entry per row")
    _lib.call("sa_score", _ptr(logits), stride, R, V, _ptr(temperature), _ptr(top_k), _ptr(top_p), _ptr(tokens),
              _ptr(scores), _stream())
    return scores


def philox4x32_10(counter: tuple[int, int, int, int], key: tuple[int, int]) -> tuple[int, int, int, int]:
    """Host function: one block of the generator that `sample` uses."""
    c = (ctypes.c_uint32 * 4)(*counter)
    k = (ctypes.c_uint32 * 2)(*key)
    o = (ctypes.c_uint32 * 4)()
    _lib.load().sa_philox4x32_10(c, k, o)
    return tuple(int(v) for v in o)


# --------------------------------------------------------------------------- token tables, biases, sums of two mixers

def _seq_meta(seq_meta: torch.Tensor, num_seqs: int, what: str) -> None:
    if seq_meta.dtype != torch.int32 or seq_meta.dim() != 2 or seq_meta.shape[1] != 4 or not seq_meta.is_contiguous() \
            or seq_meta.shape[0] < num_seqs:
        raise KernelError(f"{what}: seq_meta must be int32 [S, 4]")


def embed_sum(tokens: torch.Tensor, positions: torch.Tensor, seq_meta: torch.Tensor, num_seqs: int, max_q_len: int,
              table: torch.Tensor, *, pair: torch.Tensor | None = None, mul_prev: int = 0, mul_cur: int = 0,
              last: torch.Tensor | None = None, pos: torch.Tensor | None = None) -> torch.Tensor:
    """float32 [T, D]: table[token] + pair[(previous * mul_prev + token * mul_cur) mod buckets] + pos[position].  pair
    [buckets + 1, D]: its last row is a request's first token's; `last` int32 [slots, 1] holds every slot's last
    token and is brought up to date.  pair, pos: None to leave them out."""
    _dev(tokens, positions, seq_meta, table, pair, last, pos)
    T = tokens.shape[0]
    _i32(tokens, "embed_sum: tokens")
    _i32(positions, "embed_sum: positions", T)
    _seq_meta(seq_meta, num_seqs, "embed_sum")
    V, D = table.shape
    for name, t in (("table", table), ("pair", pair), ("pos", pos)):
        if t is not None and (t.dim() != 2 or t.shape[1] != D or not t.is_contiguous()):
            raise KernelError(f"embed_sum: {name} must be a contiguous table of rows of {D}")
    if pair is not None:
        if last is None or last.dtype != torch.int32 or last.dim() != 2 or last.stride(1) != 1:
            raise KernelError("embed_sum: a table of pairs needs the slots' last tokens, int32 [slots, >= 1]")
        if pair.shape[0] < 2:
            raise KernelError("embed_sum: the table of pairs has at least one bucket and the first token's row")
    out = torch.empty((T, D), dtype=torch.float32, device=tokens.device)
    _lib.call("sa_embed_sum", _ptr(tokens), _ptr(positions), _ptr(seq_meta), int(num_seqs), int(max_q_len), _ptr(table),
              _code(table), V, _ptr(pair), _code(pair) if pair is not None else 0,
              (pair.shape[0] - 1) if pair is not None else 0, int(mul_prev), int(mul_cur), _ptr(last),
              last.stride(0) if last is not None else 0, _ptr(pos), _code(pos) if pos is not None else 0,
              pos.shape[0] if pos is not None else 0, _ptr(out), D, _stream())
    return out


def token_gate_(z: torch.Tensor, tokens: torch.Tensor, table: torch.Tensor, col0: int, activation: int) -> torch.Tensor:
    """z[t, j] = act(z[t, j]) * table[tokens[t], col0 + j], in place."""
    _dev(z, tokens, table)
    T, N = z.shape
    _i32(tokens, "token_gate_: tokens", T)
    if table.dim() != 2 or table.stride(1) != 1 or col0 < 0 or col0 + N > table.shape[1]:
        raise KernelError(f"token_gate_: columns {col0}..{col0 + N} of a table {tuple(table.shape)}")
    _lib.call("sa_token_gate", _ptr(z), _code(z), _rows(z, "token_gate_: z"), _ptr(tokens), _ptr(table), _code(table),
              table.stride(0), int(col0), T, N, int(activation), _stream())
    return z


def bias_add_(x: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x[t, :] += bias, in place (the sum in 32-bit)."""
    _dev(x, bias)
    T, N = x.shape
    if bias.numel() != N or not bias.is_contiguous():
        raise KernelError(f"bias_add_: {bias.numel()} biases for rows of {N}")
    _lib.call("sa_bias_add", _ptr(x), _code(x), _rows(x, "bias_add_: x"), _ptr(bias), _code(bias), T, N, _stream())
    return x


def weighted_sum(x: torch.Tensor, a: float, y: torch.Tensor, b: float, out: torch.Tensor | None = None) -> torch.Tensor:
    """a * x + b * y."""
    _dev(x, y, out)
    if x.shape != y.shape or x.dtype != y.dtype:
        raise KernelError("weighted_sum: the two terms differ in shape or type")
    if out is None:
        out = torch.empty_like(x, memory_format=torch.contiguous_format)
    if out.shape != x.shape or out.dtype != x.dtype:
        raise KernelError("weighted_sum: bad output")
    T, N = x.shape
    _lib.call("sa_weighted_sum", _ptr(x), _rows(x, "weighted_sum: x"), float(a), _ptr(y), _rows(y, "weighted_sum: y"),
              float(b), _code(x), _ptr(out), _rows(out, "weighted_sum: out"), T, N, _stream())
    return out


# --------------------------------------------------------------------------- matrix states that decay

def exp_gates(raw: torch.Tensor, bias: torch.Tensor | None, cap: float, num_heads: int, m_state: torch.Tensor,
              seq_meta: torch.Tensor, num_seqs: int) -> torch.Tensor:
    """The gates of a matrix memory with exponential gates.  raw float32 [T, 2 H] (input gates' projections, then forget
    gates'), bias [2 H] or None, m_state float32 [slots, H] (a view with a row stride): every slot's running maximum,
    brought up to date.  Returns float32 [T, 3 H]: decay, input factor, exp(-maximum)."""
    _dev(raw, bias, m_state, seq_meta)
    T, H = raw.shape[0], int(num_heads)
    if raw.dtype != torch.float32 or raw.shape[1] != 2 * H:
        raise KernelError("exp_gates: raw must be float32 [T, 2 H]")
    if bias is not None and (bias.numel() != 2 * H or not bias.is_contiguous()):
        raise KernelError("exp_gates: one bias per gate and head")
    if m_state.dtype != torch.float32 or m_state.dim() != 2 or m_state.shape[1] != H or m_state.stride(1) != 1:
        raise KernelError("exp_gates: the maxima must be float32 [slots, H]")
    _seq_meta(seq_meta, num_seqs, "exp_gates")
    out = torch.empty((T, 3 * H), dtype=torch.float32, device=raw.device)
    _lib.call("sa_exp_gates", _ptr(raw), _rows(raw, "exp_gates: raw"), _ptr(bias), _code(bias) if bias is not None else 0,
              float(cap), H, _ptr(m_state), m_state.stride(0), _ptr(seq_meta), int(num_seqs), _ptr(out), _stream())
    return out


def linear_state(proj: torch.Tensor, q_at: int, k_at: int, v_at: int, q_mult: float, gates: torch.Tensor, scalar: bool,
                 num_heads: int, key_dim: int, value_dim: int, ones: bool, state: torch.Tensor, seq_meta: torch.Tensor,
                 num_seqs: int, *, decay_bias: torch.Tensor | None = None, tau: float | None = None) -> torch.Tensor:
    """S <- diag(a) S + c k v^T, o = S^T (q * q_mult) along each request's tokens, from and into state float32 [slots,
    >= H * dk * (dv + ones)] (per head [dv + ones][dk]).  q, k, v: columns q_at, k_at, v_at of proj's rows, H heads
    each.  scalar: gates float32 [T, >= 2 H] hold a and c per head; else [T, H * dk] hold a per key channel, c = 1;
    with `tau` these hold z instead, and a = sigmoid(z + decay_bias)^(1 / tau) (decay_bias [H * dk] or None).
    ones: one more column whose value is always 1 (a normalizer).  Returns float32 [T, H * (dv + ones)]."""
    _dev(proj, gates, state, seq_meta)
    T = proj.shape[0]
    H, dk, dv, CT = int(num_heads), int(key_dim), int(value_dim), int(value_dim) + int(bool(ones))
    if gates.dtype != torch.float32 or gates.shape[0] != T:
        raise KernelError("linear_state: gates must be float32 with one row per token")
    if state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < H * dk * CT:
        raise KernelError("linear_state: the state must be float32 [slots, >= H * dk * (dv + ones)]")
    _seq_meta(seq_meta, num_seqs, "linear_state")
    if (tau is not None or decay_bias is not None) and (scalar or tau is None or tau <= 0):
        raise KernelError("linear_state: tau (positive) and a bias belong to decays per channel")
    if decay_bias is not None and (decay_bias.numel() != H * dk or not decay_bias.is_contiguous()):
        raise KernelError("linear_state: one bias per key channel")
    _dev(decay_bias)
    out = torch.empty((T, H * CT), dtype=torch.float32, device=proj.device)
    _lib.call("sa_linear_state", _ptr(proj), _code(proj), _rows(proj, "linear_state: proj"), int(q_at), int(k_at), int(v_at),
              float(q_mult), _ptr(gates), _rows(gates, "linear_state: gates"), _ptr(decay_bias),
              _code(decay_bias) if decay_bias is not None else 0, float(tau or 0.0), int(bool(scalar)), H, dk, dv,
              int(bool(ones)), _ptr(state), state.stride(0), _ptr(seq_meta), int(num_seqs), _ptr(out), _stream())
    return out


def normalized_readout(x: torch.Tensor, floor: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, eps: float,
                       num_heads: int, size: int, out_dtype: torch.dtype) -> torch.Tensor:
    """x float32 [T, H * (size + 1)] (per head its `size` outputs and the normalizer's product with the query), floor
    float32 [T, H] (a view): out[t, h] = unit_rms(x / (max(|n . q|, floor) + 1e-6)) * weight[h] * sigmoid(gate[t, h])."""
    _dev(x, floor, gate, weight)
    T, H, size = x.shape[0], int(num_heads), int(size)
    if x.dtype != torch.float32 or not x.is_contiguous() or x.shape[1] != H * (size + 1):
        raise KernelError("normalized_readout: x must be contiguous float32 [T, H * (size + 1)]")
    if floor.dtype != torch.float32 or tuple(floor.shape) != (T, H):
        raise KernelError("normalized_readout: floor must be float32 [T, H]")
    if tuple(gate.shape) != (T, H * size) or weight.numel() != H * size or not weight.is_contiguous():
        raise KernelError("normalized_readout: gate [T, H * size] and weight [H * size] expected")
    out = torch.empty((T, H * size), dtype=out_dtype, device=x.device)
    _lib.call("sa_normalized_readout", _ptr(x), _ptr(floor), _rows(floor, "normalized_readout: floor"), _ptr(gate),
              _code(gate), _rows(gate, "normalized_readout: gate"), _ptr(weight), _code(weight), float(eps), _ptr(out),
              _code(out), H * size, T, H, size, _stream())
    return out


# --------------------------------------------------------------------------- routed experts

def route(logits: torch.Tensor, top: int, scale: float) -> tuple[torch.Tensor, torch.Tensor]:
    """softmax over the experts' logits (float32 [T, E]); returns (experts int32 [T, top], weights float32 [T, top] =
    score * scale) of the `top` largest scores, largest first."""
    _dev(logits)
    T, E = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("route: the router's logits are float32")
    experts = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    _lib.call("sa_route", _ptr(logits), _rows(logits, "route: logits"), T, E, int(top), float(scale), _ptr(experts),
              _ptr(weights), _stream())
    return experts, weights


def route_choice(logits: torch.Tensor, top: int, scale: float, *, correction: torch.Tensor | None = None,
                 groups: int = 1, keep: int = 1) -> tuple[torch.Tensor, torch.Tensor]:
    """Scores are sigmoids of the logits (float32 [T, E]); the `top` experts with the largest score + correction[e] are
    chosen, among the `keep` groups (of `groups` equal groups of neighbouring experts) whose two largest choice scores
    have the largest sums.  Returns (experts int32 [T, top], weights float32 [T, top] = score * scale, the score
    without the correction), largest choice first."""
    _dev(logits, correction)
    T, E = logits.shape
    if logits.dtype != torch.float32:
        raise KernelError("route_choice: the router's logits are float32")
    if correction is not None and (correction.numel() != E or not correction.is_contiguous()):
        raise KernelError(f"route_choice: a correction of {correction.numel()} entries for {E} experts")
    experts = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    _lib.call("sa_route_choice", _ptr(logits), _rows(logits, "route_choice: logits"), T, E, int(top), float(scale),
              _ptr(correction), _code(correction) if correction is not None else 0, int(groups), int(keep),
              _ptr(experts), _ptr(weights), _stream())
    return experts, weights


def routed_experts(x: torch.Tensor, experts: torch.Tensor, weights: torch.Tensor, gate_w, up_w, down_w, activation: int,
                   *, shared: torch.Tensor | None = None, shared_gate: torch.Tensor | None = None,
                   out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """sum_k weights[t, k] * down[e](act(gate[e] x) * (up[e] x)) with e = experts[t, k], plus sigmoid(shared_gate[t]) *
    shared[t] (shared None: nothing; shared_gate None: shared as it is).  gate_w, up_w, down_w: `packing.ExpertStack`s
    (every expert's matrix, tiled if bfloat16).  x [T, D] in the weights' type; shared_gate float32 [T, 1].
    gate_w None: experts without a gate, down[e](act(up[e] x))."""
    _dev(x, experts, weights, gate_w.data if gate_w is not None else None, up_w.data, down_w.data, shared, shared_gate)
    T, D = x.shape
    top, E, F = experts.shape[1], up_w.experts, up_w.rows
    if up_w.cols != D or (gate_w is not None and (gate_w.experts, gate_w.rows, gate_w.cols) != (E, F, D)) \
            or (down_w.experts, down_w.rows, down_w.cols) != (E, D, F):
        raise KernelError("routed_experts: the experts' matrices do not go together")
    if x.dtype != up_w.data.dtype or up_w.tiled != (x.dtype == torch.bfloat16):
        raise KernelError("routed_experts: bfloat16 rows go with tiled weights, float32 rows with row-major ones")
    if experts.dtype != torch.int32 or not experts.is_contiguous() or tuple(weights.shape) != (T, top) \
            or weights.dtype != torch.float32 or not weights.is_contiguous():
        raise KernelError("routed_experts: experts int32 [T, top] and weights float32 [T, top] expected")
    P = T * top
    dev = x.device
    # tiles of 64 rows share the weights' operands between four sub-tiles: for steps that bring an expert many rows
    tile_rows = 64 if P >= 32 * E else 16
    max_tiles = _lib.load().sa_expert_tiles_max(P, E, tile_rows)
    sorted_ = torch.empty(P, dtype=torch.int32, device=dev)
    plan = torch.empty(1 + 2 * max_tiles, dtype=torch.int32, device=dev)
    _lib.call("sa_expert_sort", _ptr(experts), P, E, tile_rows, _ptr(sorted_), _ptr(plan), plan.numel(), _stream())
    h = torch.empty((P, F), dtype=x.dtype, device=dev)
    first, second = (gate_w.data, up_w.data) if gate_w is not None else (up_w.data, None)
    _lib.call("sa_expert_product", _ptr(x), _code(x), _rows(x, "routed_experts: x"), 1, top, _ptr(first),
              _ptr(second), F, D, _ptr(sorted_), _ptr(plan), P, E, tile_rows, int(activation), _ptr(h), F, 0,
              int(gate_w is None), _stream())
    y = torch.empty((P, D), dtype=torch.float32, device=dev)
    _lib.call("sa_expert_product", _ptr(h), _code(h), F, 0, top, _ptr(down_w.data), None, D, F, _ptr(sorted_), _ptr(plan), P,
              E, tile_rows, 0, _ptr(y), D, 1, 0, _stream())
    out = torch.empty((T, D), dtype=out_dtype or x.dtype, device=dev)
    if shared is not None and tuple(shared.shape) != (T, D):
        raise KernelError("routed_experts: the shared expert's rows do not match")
    if shared_gate is not None and (shared_gate.dtype != torch.float32 or shared_gate.shape[0] != T):
        raise KernelError("routed_experts: the shared expert's gate is float32 [T, 1]")
    _lib.call("sa_expert_combine", _ptr(y), _ptr(weights), top, _ptr(shared), _code(shared) if shared is not None else 0,
              _rows(shared, "routed_experts: shared") if shared is not None else 0, _ptr(shared_gate),
              shared_gate.stride(0) if shared_gate is not None else 0, _ptr(out), _code(out), D, T, D, _stream())
    return out
