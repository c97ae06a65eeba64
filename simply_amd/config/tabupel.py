"""Typed configuration of Tabupel, read from the model folder's `config.json`.

A decoder whose layers are listed one by one.  A layer is a pre-norm block with a residual multiplier m,
x += m * mixer(norm(x)), x += m * ff(norm(x)), and one of three mixers: "attention" (two softmax maps per head over
the same values whose difference is normed head by head; queries and keys normed with a shared weight and rotated in
neighbouring pairs), "latent_attention" (queries and keys/values through normed latents, one rotated key part for all
heads, a sigmoid gate per head; only the latent and the rotated part are cached) and "rglru" (two branches, a short
causal convolution, block-diagonal gates, a real-gated linear recurrence with one number of state per channel).  A
layer that says "weights_of": j runs with layer j's tensors and a cache or state of its own.  The feed-forward is the
gated one with silu, or none.  The head's logits are soft-capped.

Keys: "architecture", "vocab", "width", "residual_mult", "norm": {"eps"}, "logit_softcap", "layers": [{"type",
"mixer": {...}, "mlp": {"kind": "dense", "ff"} | null, "weights_of"}].  attention: heads, kv_heads, dim, vdim, scale,
diff, mask {size}, rot {dims, base, scaling}.  latent_attention: heads, dim, rot_dim, vdim, q_rank, kv_rank, scale,
mask {size}, rot {dims, base, scaling}.  rot.scaling is {factor} (every frequency divided by it) or {factor,
original, fast, slow} (a ramp between the two, cos and sin times 0.1 ln factor + 1).  rglru: width, blocks, conv.
Whatever is absent (mask, rot, scaling, mlp, logit_softcap) does not exist in the model.  Tensors: "embed",
"l<i>.norm1", "l<i>.norm2", "l<i>.mix.*", "l<i>.mlp.{gate,up,down}", "final.norm", "head"; matrices are [out, in].
"""
from __future__ import annotations

import copy
import dataclasses
from typing import Any, Mapping

from ..registry import ARCHITECTURES
from .gemma2 import ConfigError
from .nemidra import _positive
from .spec import LayerSpec, ModelSpec, PartSpec, ScheduleEntry
from .zenuzen import _get

LAYER_TYPES = ("attention", "latent_attention", "rglru")
MLP_KINDS = ("dense",)
#: the recurrence's decay is exp(-DECAY_MULT * r * softplus(lam)): fixed by the design
DECAY_MULT = 8.0


def _window(m: Mapping[str, Any], where: str):
    mask = m.get("mask")
    return None if mask is None else _positive(_get(mask, "size", where + ".mask", int), "mask.size")


def _rotation(m: Mapping[str, Any], where: str, most: int, default_dims: int | None = None) -> "PartSpec | None":
    """The mixer's "rot" entry as a `pair_rope` spec (None: nothing is rotated)."""
    rot = m.get("rot")
    if rot is None:
        return None
    rw = where + ".rot"
    dims = rot.get("dims", default_dims)
    if dims is None:
        dims = _get(rot, "dims", rw, int)
    if isinstance(dims, bool) or not isinstance(dims, int) or dims % 2 or not 0 <= dims <= most:
        raise ConfigError(f"config.json: {rw}: dims {dims!r} must be even and at most {most}")
    base = _get(rot, "base", rw, float)
    if base <= 0:
        raise ConfigError(f"config.json: {rw}: base must be positive")
    sc, scaling = rot.get("scaling"), None
    if sc is not None:
        sw = rw + ".scaling"
        if any(k in sc for k in ("original", "fast", "slow")):
            scaling = {"kind": "ramp", **{k: _positive(_get(sc, k, sw, float), k) for k in ("factor", "original", "fast", "slow")}}
        else:
            scaling = {"kind": "linear", "factor": _positive(_get(sc, "factor", sw, float), "factor")}
    return PartSpec("pair_rope", {"dims": dims, "base": base, "scaling": scaling})


@dataclasses.dataclass(frozen=True)
class TabupelConfig:
    #: the dictionary of config.json, as read (`to_dict` gives it back)
    raw: Mapping[str, Any]
    vocab: int
    width: int
    residual_mult: float
    norm_eps: float
    num_layers: int
    #: not part of the design: the longest sequence that the engine plans for when --max_seq_len does not say
    max_position: int = 8192
    eos_token_ids: tuple[int, ...] = ()
    initializer_range: float = 0.02

    architecture = "Tabupel"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any], check: bool = True) -> "TabupelConfig":
        layers = _get(d, "layers", "top level")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError('config.json: "layers" must be a non-empty list')
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        eps = _get(_get(d, "norm", "top level"), "eps", "norm", float)
        if eps < 0:
            raise ConfigError("config.json: norm.eps must not be negative")
        cfg = cls(raw=copy.deepcopy(dict(d)), vocab=_positive(_get(d, "vocab", "top level", int), "vocab"),
                  width=_positive(_get(d, "width", "top level", int), "width"),
                  residual_mult=_get(d, "residual_mult", "top level", float), norm_eps=eps, num_layers=len(layers),
                  max_position=int(d.get("max_position", 8192)), eos_token_ids=eos_ids,
                  initializer_range=float(d.get("initializer_range", 0.02)))
        if check:
            cfg.model_spec()   # (reads every key: whatever is missing or wrong is said now)
        return cfg

    @classmethod
    def from_dict_open(cls, d: Mapping[str, Any]) -> "TabupelConfig":
        """The configuration of a model folder before `resolve_shapes` has read the sizes that the tensors give."""
        return cls.from_dict(d, check=False)

    def to_dict(self) -> dict[str, Any]:
        return copy.deepcopy(dict(self.raw))

    def resolve_shapes(self, shapes: Mapping[str, tuple]) -> "TabupelConfig":
        """Sizes that config.json may leave to the tensors: the rank of a latent attention's query latent."""
        raw = copy.deepcopy(dict(self.raw))
        for i, l in enumerate(raw["layers"]):
            name = f"l{self.weights_layer(i)}.mix.dq"
            if l.get("type") == "latent_attention" and "q_rank" not in l.get("mixer", {}) and name in shapes:
                l["mixer"]["q_rank"] = int(shapes[name][0])
        return type(self).from_dict(raw)

    # ------------------------------------------------------------------ layers that share tensors
    def weights_layer(self, i: int) -> int:
        """The layer whose tensors layer i runs with (itself, unless it says "weights_of")."""
        layers, seen = self.raw["layers"], set()
        while layers[i].get("weights_of") is not None:
            if i in seen:
                raise ConfigError(f"config.json: layers[{i}]: \"weights_of\" goes round in a circle")
            seen.add(i)
            j = layers[i]["weights_of"]
            if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < len(layers):
                raise ConfigError(f"config.json: layers[{i}]: \"weights_of\" names layer {j!r} of {len(layers)}")
            if layers[j].get("type") != layers[i].get("type"):
                raise ConfigError(f"config.json: layers[{i}]: \"weights_of\" names a layer of another type")
            i = j
        return i

    # ------------------------------------------------------------------ parts
    def _mixer(self, i: int, l: Mapping[str, Any]) -> PartSpec:
        D, eps, p, where = self.width, self.norm_eps, f"l{i}.mix.", f"layers[{i}].mixer"
        m = _get(l, "mixer", f"layers[{i}]")
        kind = l["type"]
        if kind == "attention":
            dim = _positive(_get(m, "dim", where, int), "dim")
            heads, kv = _positive(_get(m, "heads", where, int), "heads"), _positive(_get(m, "kv_heads", where, int), "kv_heads")
            if heads % kv:
                raise ConfigError(f"config.json: {where}: heads {heads} is not a multiple of kv_heads {kv}")
            return PartSpec("differential_attention", {
                "hidden_size": D, "num_heads": heads, "num_kv_heads": kv, "key_dim": dim,
                "value_dim": _positive(_get(m, "vdim", where, int), "vdim"), "scale": _get(m, "scale", where, float),
                "diff": _get(m, "diff", where, float), "norm_eps": eps, "qk_norm": True, "window": _window(m, where),
                "position_encoding": _rotation(m, where, dim),
            }, {"q_proj": p + "q", "k_proj": p + "k", "v_proj": p + "v", "o_proj": p + "o", "q_norm": p + "q.norm",
                "k_norm": p + "k.norm", "lq1": p + "lq1", "lk1": p + "lk1", "lq2": p + "lq2", "lk2": p + "lk2"})
        if kind == "latent_attention":
            rot_dim = _positive(_get(m, "rot_dim", where, int), "rot_dim")
            q_rank = m.get("q_rank")
            if q_rank is None:
                raise ConfigError(f"config.json: {where}: the query latent's size is given neither by \"q_rank\" nor by "
                                  f"the tensor {p}dq of a model folder")
            return PartSpec("latent_attention", {
                "hidden_size": D, "num_heads": _positive(_get(m, "heads", where, int), "heads"),
                "key_dim": _positive(_get(m, "dim", where, int), "dim"), "rot_dim": rot_dim,
                "value_dim": _positive(_get(m, "vdim", where, int), "vdim"), "q_rank": _positive(int(q_rank), "q_rank"),
                "kv_rank": _positive(_get(m, "kv_rank", where, int), "kv_rank"), "scale": _get(m, "scale", where, float),
                "norm_eps": eps, "window": _window(m, where), "output_gate": True,
                "position_encoding": _rotation(m, where, rot_dim, default_dims=rot_dim),
            }, {"dq_proj": p + "dq", "dq_norm": p + "dq.norm", "uq_proj": p + "uq", "dkv_proj": p + "dkv",
                "dkv_norm": p + "dkv.norm", "uk_proj": p + "uk", "uv_proj": p + "uv", "gate_proj": p + "g",
                "o_proj": p + "o"})
        width, blocks = _positive(_get(m, "width", where, int), "width"), _positive(_get(m, "blocks", where, int), "blocks")
        if width % blocks:
            raise ConfigError(f"config.json: {where}: width {width} does not split into {blocks} blocks")
        return PartSpec("rglru", {"hidden_size": D, "width": width, "blocks": blocks,
                                  "conv_taps": _positive(_get(m, "conv", where, int), "conv"), "decay_mult": DECAY_MULT},
                        {"y_proj": p + "y", "y_bias": p + "y.b", "x_proj": p + "x", "x_bias": p + "x.b", "conv": p + "conv",
                         "conv_bias": p + "conv.b", "r_gate": p + "ra", "r_bias": p + "ra.b", "i_gate": p + "ri",
                         "i_bias": p + "ri.b", "lam": p + "lam", "o_proj": p + "o"})

    def model_spec(self) -> ModelSpec:
        D, d = self.width, self.raw

        def norm(name: str) -> PartSpec:
            return PartSpec("rmsnorm", {"dim": D, "eps": self.norm_eps, "scale_plus_one": False}, {"scale": name})

        layers, at, ignorable = [], {}, []   # at: config layer -> index among the layers that have tensors of their own
        for i, l in enumerate(d["layers"]):
            p, where = f"l{i}.", f"layers[{i}]"
            kind = _get(l, "type", where)
            if kind not in LAYER_TYPES:
                raise ConfigError(f"config.json: {where}: unknown layer type {kind!r}; known: {', '.join(LAYER_TYPES)}")
            if l.get("weights_of") is not None:
                self.weights_layer(i)
                continue
            norms = {"pre_mixer": norm(p + "norm1")}
            ffn = None
            mlp = l.get("mlp")
            if mlp is not None:
                mk = _get(mlp, "kind", where + ".mlp")
                if mk not in MLP_KINDS:
                    raise ConfigError(f"config.json: {where}.mlp: unknown kind {mk!r}; known: {', '.join(MLP_KINDS)}")
                ffn = PartSpec("gated_dense", {"hidden_size": D, "activation": "silu",
                                               "intermediate_size": _positive(_get(mlp, "ff", where + ".mlp", int), "ff")},
                               {"gate_proj": p + "mlp.gate", "up_proj": p + "mlp.up", "down_proj": p + "mlp.down"})
                norms["pre_ffn"] = norm(p + "norm2")
            else:
                ignorable.append(p + "norm2")   # (a folder may hold the norm of a feed-forward that is not there)
            at[i] = len(layers)
            layers.append(LayerSpec(block=PartSpec("pre_norm", {"mult": self.residual_mult}), mixer=self._mixer(i, l),
                                    feed_forward=ffn, norms=norms))
        cap = d.get("logit_softcap")
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=D, vocab_size=self.vocab,
            embedding=PartSpec("scaled_embedding", {"vocab_size": self.vocab, "dim": D, "scale": 1.0}, {"table": "embed"}),
            layers=tuple(layers), schedule=tuple(ScheduleEntry(at[self.weights_layer(i)]) for i in range(self.num_layers)),
            final_norm=norm("final.norm"),
            head=PartSpec("linear_head", {"vocab_size": self.vocab, "dim": D, "soft_cap": float(cap) if cap else None},
                          {"weight": "head"}),
            max_position=self.max_position, eos_token_ids=self.eos_token_ids, initializer_range=self.initializer_range,
            ignorable=tuple(ignorable))
        spec.validate()
        return spec


ARCHITECTURES.register("Tabupel", TabupelConfig)
