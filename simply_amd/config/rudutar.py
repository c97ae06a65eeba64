"""Typed configuration of Rudutar, read from the model folder's `config.json`.

A decoder whose layers are listed one by one.  The embedding is normed before the first layer.  A layer is a pre-norm
block, x += mixer(norm(x)), x += ff(norm(x)), with one of two windowed attentions, both with grouped key heads and a
sigmoid gate on the heads from a projection of the mixer's input:

  "attention"    q, k and v pass a short causal convolution per channel; q and k are normed head by head with a weight
                 that the heads share; no rotation: a query is multiplied by a temperature that grows with the logarithm
                 of its position, and the scores lose a slope per head times the distance to the key; the softmax has one
                 more term exp(0) without a value; the gate has an entry per entry of the heads.  A layer that says
                 "kv_from": j has queries only and reads the keys and values that layer j keeps.
  "attention_2"  q and k have biases and are normed over the whole projection with a weight per entry, then rotated on
                 the first entries of every head; the values are the keys as projected; ordinary softmax; one gate
                 number per head.

The feed-forward is dense (exact GELU), a mixture of experts without gates (square of relu; sigmoid router with a
correction per expert for the choice, groups of experts of which the best stay, weights not renormalized, a shared
expert), or none.

Keys: "architecture", "vocab", "width", "norm": {"eps"}, "layers": [{"type", "mixer": {...}, "mlp": {...} | null}].
Mixer: heads, kv_heads, dim, vdim, scale, mask {size}; attention: conv, q_temp {coef, every}, kv_from; attention_2:
rot {dims, base}.  mlp: {"kind": "dense", "ff"} or {"kind": "moe", "expert": {"ff"}, "router": {"experts", "top",
"scale", "groups": {"count", "keep"}}, "shared": {"ff"}}.  Whatever is absent (mask, conv, q_temp, rot, groups, shared,
mlp) does not exist in the model.  Tensors: "embed", "embed.norm", "l<i>.norm1", "l<i>.norm2", "l<i>.mix.{q,k,v,g,o}"
with ".b", ".norm" and ".conv" behind a projection's name, "l<i>.mlp.{up,down}", "l<i>.mlp.{router,correction}",
"l<i>.mlp.e<n>.{up,down}", "l<i>.mlp.shared.{up,down}", "final.norm", "head"; matrices are [out, in].
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

LAYER_TYPES = ("attention", "attention_2")
MLP_KINDS = ("dense", "moe")
#: head h of H loses 2^(-SLOPE_EXPONENT (h + 1) / H) per position of distance: fixed by the design
SLOPE_EXPONENT = 8.0


def _window(m: Mapping[str, Any], where: str):
    mask = m.get("mask")
    return None if mask is None else _positive(_get(mask, "size", where + ".mask", int), "mask.size")


@dataclasses.dataclass(frozen=True)
class RudutarConfig:
    #: the dictionary of config.json, as read (`to_dict` gives it back)
    raw: Mapping[str, Any]
    vocab: int
    width: int
    norm_eps: float
    num_layers: int
    #: not part of the design: the longest sequence that the engine plans for when --max_seq_len does not say
    max_position: int = 8192
    eos_token_ids: tuple[int, ...] = ()
    initializer_range: float = 0.02

    architecture = "Rudutar"

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "RudutarConfig":
        layers = _get(d, "layers", "top level")
        if not isinstance(layers, (list, tuple)) or not layers:
            raise ConfigError('config.json: "layers" must be a non-empty list')
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in (eos if isinstance(eos, (list, tuple)) else [eos]))
        eps = _get(_get(d, "norm", "top level"), "eps", "norm", float)
        if eps < 0:
            raise ConfigError("config.json: norm.eps must not be negative")
        cfg = cls(raw=copy.deepcopy(dict(d)), vocab=_positive(_get(d, "vocab", "top level", int), "vocab"),
                  width=_positive(_get(d, "width", "top level", int), "width"), norm_eps=eps, num_layers=len(layers),
                  max_position=int(d.get("max_position", 8192)), eos_token_ids=eos_ids,
                  initializer_range=float(d.get("initializer_range", 0.02)))
        cfg.model_spec()   # (reads every key: whatever is missing or wrong is said now)
        return cfg

    def to_dict(self) -> dict[str, Any]:
        return copy.deepcopy(dict(self.raw))

    # ------------------------------------------------------------------ layers that read another layer's keys and values
    def kv_source(self, i: int) -> "int | None":
        """The layer whose keys and values layer i reads (None: its own)."""
        layers = self.raw["layers"]
        m = layers[i].get("mixer") or {}
        j = m.get("kv_from")
        if j is None:
            return None
        where = f"layers[{i}].mixer"
        if layers[i].get("type") != "attention":
            raise ConfigError(f"config.json: {where}: \"kv_from\" belongs to layers of type \"attention\"")
        if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < i:
            raise ConfigError(f"config.json: {where}: \"kv_from\" names layer {j!r}, which does not run before layer {i}")
        src = layers[j].get("mixer") or {}
        if layers[j].get("type") != "attention" or src.get("kv_from") is not None:
            raise ConfigError(f"config.json: {where}: \"kv_from\" names layer {j}, which keeps no keys and values of this kind")
        for key in ("kv_heads", "dim", "vdim"):
            if src.get(key) != m.get(key):
                raise ConfigError(f"config.json: {where}: \"{key}\" differs from that of layer {j}, whose keys and values "
                                  f"it reads")
        return j

    def _kept_window(self, i: int, own: "int | None") -> "int | None | str":
        """How many tokens back layer i keeps its pages: the largest window among itself and the layers that read its
        keys and values (None: all of them)."""
        windows = [own]
        for k, l in enumerate(self.raw["layers"]):
            if k > i and l.get("type") == "attention" and (l.get("mixer") or {}).get("kv_from") == i:
                windows.append(_window(l["mixer"], f"layers[{k}].mixer"))
        return None if any(w is None for w in windows) else max(windows)

    # ------------------------------------------------------------------ parts
    def _mixer(self, i: int, l: Mapping[str, Any]) -> PartSpec:
        D, eps, p, where = self.width, self.norm_eps, f"l{i}.mix.", f"layers[{i}].mixer"
        m = _get(l, "mixer", f"layers[{i}]")
        dim = _positive(_get(m, "dim", where, int), "dim")
        heads, kv = _positive(_get(m, "heads", where, int), "heads"), _positive(_get(m, "kv_heads", where, int), "kv_heads")
        if heads % kv:
            raise ConfigError(f"config.json: {where}: heads {heads} is not a multiple of kv_heads {kv}")
        vdim = _positive(_get(m, "vdim", where, int), "vdim")
        window = _window(m, where)
        common = {"hidden_size": D, "num_heads": heads, "num_kv_heads": kv, "key_dim": dim, "value_dim": vdim,
                  "scale": _get(m, "scale", where, float), "norm_eps": eps, "window": window}
        if l["type"] == "attention":
            source = self.kv_source(i)
            own = source is None
            taps = m.get("conv")
            if taps is not None:
                taps = _positive(_get(m, "conv", where, int), "conv")
            temp = m.get("q_temp")
            if temp is not None:
                temp = (_get(temp, "coef", where + ".q_temp", float),
                        _positive(_get(temp, "every", where + ".q_temp", int), "q_temp.every"))
            tensors = {"q_proj": p + "q", "q_norm": p + "q.norm", "gate_proj": p + "g", "o_proj": p + "o"}
            if own:
                tensors.update(k_proj=p + "k", v_proj=p + "v", k_norm=p + "k.norm")
            if taps:
                tensors.update({s + "_conv": p + s + ".conv" for s in (("q", "k", "v") if own else ("q",))})
            return PartSpec("gated_attention", {
                **common, "qk_norm": "head", "conv_taps": taps or 0, "query_temperature": temp,
                "slope_exponent": SLOPE_EXPONENT, "zero_sink": True, "output_gate": "element", "own_keys_values": own,
                # (a layer that reads another's pages names the same need: what that layer keeps)
                "cache_window": self._kept_window(i, window) if own else self._kept_window(
                    source, _window(self.raw["layers"][source]["mixer"], f"layers[{source}].mixer"))}, tensors)
        if m.get("kv_from") is not None:
            self.kv_source(i)   # (says why not)
        if vdim != dim:
            raise ConfigError(f"config.json: {where}: the values of this layer are its keys: vdim {vdim} must equal dim {dim}")
        rot, pe = m.get("rot"), None
        if rot is not None:
            rw = where + ".rot"
            dims = _get(rot, "dims", rw, int)
            if isinstance(dims, bool) or dims % 2 or not 0 <= dims <= dim:
                raise ConfigError(f"config.json: {rw}: dims {dims!r} must be even and at most {dim}")
            base = _get(rot, "base", rw, float)
            if base <= 0:
                raise ConfigError(f"config.json: {rw}: base must be positive")
            pe = PartSpec("partial_rope", {"head_dim": dim, "dims": dims, "base": base})
        return PartSpec("gated_attention", {
            **common, "qk_norm": "row", "bias": True, "values": "keys", "position_encoding": pe, "output_gate": "head"},
            {"q_proj": p + "q", "q_bias": p + "q.b", "k_proj": p + "k", "k_bias": p + "k.b", "q_norm": p + "q.norm",
             "k_norm": p + "k.norm", "gate_proj": p + "g", "o_proj": p + "o"})

    def _feed_forward(self, i: int, mlp: Mapping[str, Any]) -> PartSpec:
        D, p, where = self.width, f"l{i}.mlp.", f"layers[{i}].mlp"
        kind = _get(mlp, "kind", where)
        if kind not in MLP_KINDS:
            raise ConfigError(f"config.json: {where}: unknown kind {kind!r}; known: {', '.join(MLP_KINDS)}")
        if kind == "dense":
            return PartSpec("dense", {"hidden_size": D, "activation": "gelu_erf",
                                      "intermediate_size": _positive(_get(mlp, "ff", where, int), "ff")},
                            {"up_proj": p + "up", "down_proj": p + "down"})
        r = _get(mlp, "router", where)
        rw = where + ".router"
        E, top = _positive(_get(r, "experts", rw, int), "experts"), _positive(_get(r, "top", rw, int), "top")
        groups = r.get("groups")
        count = keep = 1
        if groups is not None:
            count = _positive(_get(groups, "count", rw + ".groups", int), "groups.count")
            keep = _positive(_get(groups, "keep", rw + ".groups", int), "groups.keep")
        if top > E or E % count or keep > count or top > keep * (E // count):
            raise ConfigError(f"config.json: {rw}: {E} experts in {count} groups of which {keep} stay do not give {top} "
                              f"choices")
        shared = mlp.get("shared")
        tensors = {"router": p + "router", "correction": p + "correction"}
        for e in range(E):
            tensors.update({f"e{e}.up": f"{p}e{e}.up", f"e{e}.down": f"{p}e{e}.down"})
        if shared is not None:
            tensors.update({"shared.up_proj": p + "shared.up", "shared.down_proj": p + "shared.down"})
        return PartSpec("routed_experts", {
            "hidden_size": D, "num_experts": E, "top": top, "router_scale": _get(r, "scale", rw, float),
            "expert_size": _positive(_get(_get(mlp, "expert", where), "ff", where + ".expert", int), "expert.ff"),
            "activation": "squared_relu", "gated": False, "router": "sigmoid", "correction": True, "num_groups": count,
            "keep_groups": keep, "shared_gate": False,
            "shared_size": None if shared is None else _positive(_get(shared, "ff", where + ".shared", int), "shared.ff"),
        }, tensors)

    def model_spec(self) -> ModelSpec:
        D, d = self.width, self.raw

        def norm(name: str) -> PartSpec:
            return PartSpec("rmsnorm", {"dim": D, "eps": self.norm_eps, "scale_plus_one": False}, {"scale": name})

        layers, schedule, ignorable = [], [], []
        for i, l in enumerate(d["layers"]):
            p, where = f"l{i}.", f"layers[{i}]"
            kind = _get(l, "type", where)
            if kind not in LAYER_TYPES:
                raise ConfigError(f"config.json: {where}: unknown layer type {kind!r}; known: {', '.join(LAYER_TYPES)}")
            norms = {"pre_mixer": norm(p + "norm1")}
            ffn = None
            mlp = l.get("mlp")
            if mlp is not None:
                ffn = self._feed_forward(i, mlp)
                norms["pre_ffn"] = norm(p + "norm2")
            else:
                ignorable.append(p + "norm2")   # (a folder may hold the norm of a feed-forward that is not there)
            layers.append(LayerSpec(block=PartSpec("pre_norm", {"mult": 1.0}), mixer=self._mixer(i, l), feed_forward=ffn,
                                    norms=norms))
            schedule.append(ScheduleEntry(i, cache_from=self.kv_source(i) if kind == "attention" else None))
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=D, vocab_size=self.vocab,
            embedding=PartSpec("normed_embedding", {"vocab_size": self.vocab, "dim": D, "eps": self.norm_eps},
                               {"table": "embed", "norm": "embed.norm"}),
            layers=tuple(layers), schedule=tuple(schedule), final_norm=norm("final.norm"),
            head=PartSpec("linear_head", {"vocab_size": self.vocab, "dim": D, "soft_cap": None}, {"weight": "head"}),
            max_position=self.max_position, eos_token_ids=self.eos_token_ids, initializer_range=self.initializer_range,
            ignorable=tuple(ignorable))
        spec.validate()
        return spec


ARCHITECTURES.register("Rudutar", RudutarConfig)
