"""Typed view of a Legavik ``config.json``.

The file names the design under ``architecture`` and describes every layer on its own::

    {"architecture": "Legavik", "vocab": V, "width": W, "norm": {"eps": e}, "logit_softcap": c,
     "layers": [{"type": "attention",
                 "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": s,
                           "mask": {"size": w, "keep_first": n},
                           "rot": {"base": b, "dims": d,
                                   "scaling": {"factor": f, "original": n, "fast": a, "slow": c}}},
                 "mlp": {"kind": "moe", "expert": {"ff": I},
                         "router": {"experts": E, "top": k, "groups": {"count": n, "keep": m}}} | null},
                {"type": "parallel",
                 "mixer": {"left": {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": s, "conv": K,
                                    "q_temp": {"coef": c, "every": n}},
                           "right": {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "conv": K},
                           "left_scale": a, "right_scale": b},
                 "mlp": ...}, ...]}

Every size and constant a model of the design can choose comes from here; what is absent or null (a
mask, kept first tokens, a rotation or its scaling, a query temperature, groups of experts, the cap on
the logits) does not exist in that model.  The widths of the low-rank inputs of a ``right`` mixer's decay
and gate come from the tensors themselves unless ``decay_rank`` / ``gate_rank`` name them (a folder of
random weights needs that).  What the design fixes lives where the plan is put together.
"""

from __future__ import annotations

from collections.abc import Mapping
from dataclasses import dataclass
from typing import Any

from turboserve_amd.config.dovudra_config import RotationScaling
from turboserve_amd.config.model_config import UnsupportedModelError
from turboserve_amd.config.sisisun_config import _count, _mapping, _real

ARCHITECTURE = "Legavik"
MIXER_TYPES = ("attention", "parallel")


def _optional(where: str, data: Mapping[str, Any], key: str) -> Mapping[str, Any] | None:
    return None if data.get(key) is None else _mapping(where, data, key)


def _heads(where: str, data: Mapping[str, Any]) -> tuple[int, int]:
    heads, kv_heads = _count(where, data, "heads"), _count(where, data, "kv_heads")
    if heads % kv_heads != 0:
        raise UnsupportedModelError(f"config.json: {where}: {heads} heads are not a multiple of {kv_heads} kv_heads")
    return heads, kv_heads


@dataclass(frozen=True)
class KeyedAttentionSizes:
    """Attention whose values are its keys: rotation of a head's first elements, a norm without gain behind
    it, a window that keeps the first tokens, a gate per head."""

    heads: int
    kv_heads: int
    dim: int
    scale: float
    window: int | None
    keep_first: int
    rot_base: float | None
    rot_dims: int
    rot_scaling: RotationScaling | None

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "KeyedAttentionSizes":
        heads, kv_heads = _heads(where, data)
        dim = _count(where, data, "dim")
        if data.get("vdim") is not None and _count(where, data, "vdim") != dim:
            raise UnsupportedModelError(f"config.json: {where}.vdim {data['vdim']} must be dim {dim}: the values are the keys")
        mask = _optional(where, data, "mask")
        window = keep = None
        if mask is not None:
            window = _count(f"{where}.mask", mask, "size")
            keep = 0 if mask.get("keep_first") is None else _count(f"{where}.mask", mask, "keep_first", least=0)
        rot = _optional(where, data, "rot")
        base, dims, scaling = None, 0, None
        if rot is not None:
            base, dims = _real(f"{where}.rot", rot, "base"), _count(f"{where}.rot", rot, "dims", least=2)
            if dims > dim or dims % 2 != 0:
                raise UnsupportedModelError(f"config.json: {where}.rot.dims {dims} must be even and at most dim {dim}")
            if rot.get("scaling") is not None:
                scaling = RotationScaling.read(f"{where}.rot.scaling", _mapping(f"{where}.rot", rot, "scaling"))
        return cls(heads, kv_heads, dim, _real(where, data, "scale"), window, keep or 0, base, dims, scaling)

    def cached_elements(self) -> int:
        return 2 * self.kv_heads * self.dim


@dataclass(frozen=True)
class ConvolvedAttentionSizes:
    """The left mixer of a parallel layer: biased projections, a short convolution, q/k norm, causal."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    taps: int | None
    temp_coef: float | None
    temp_every: int

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "ConvolvedAttentionSizes":
        heads, kv_heads = _heads(where, data)
        temp = _optional(where, data, "q_temp")
        coef, every = None, 1
        if temp is not None:
            coef, every = _real(f"{where}.q_temp", temp, "coef", positive=False), _count(f"{where}.q_temp", temp, "every")
        taps = None if data.get("conv") is None else _count(where, data, "conv")
        return cls(heads, kv_heads, _count(where, data, "dim"), _count(where, data, "vdim"), _real(where, data, "scale"),
                   taps, coef, every)

    def cached_elements(self) -> int:
        return self.kv_heads * (self.dim + self.vdim)


@dataclass(frozen=True)
class DeltaRuleSizes:
    """The right mixer of a parallel layer: the gated delta rule."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    taps: int
    decay_rank: int | None
    gate_rank: int | None

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "DeltaRuleSizes":
        heads, kv_heads = _heads(where, data)
        ranks = [None if data.get(key) is None else _count(where, data, key) for key in ("decay_rank", "gate_rank")]
        return cls(heads, kv_heads, _count(where, data, "dim"), _count(where, data, "vdim"), _count(where, data, "conv"), *ranks)


@dataclass(frozen=True)
class ParallelSizes:
    left: ConvolvedAttentionSizes
    right: DeltaRuleSizes
    left_scale: float
    right_scale: float

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "ParallelSizes":
        return cls(ConvolvedAttentionSizes.read(f"{where}.left", _mapping(where, data, "left")),
                   DeltaRuleSizes.read(f"{where}.right", _mapping(where, data, "right")),
                   _real(where, data, "left_scale", positive=False), _real(where, data, "right_scale", positive=False))

    def cached_elements(self) -> int:
        return self.left.cached_elements()


@dataclass(frozen=True)
class RoutedSizes:
    ff: int
    experts: int
    top: int
    groups: int
    keep: int

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "RoutedSizes":
        if data.get("kind") != "moe":
            raise UnsupportedModelError(f"config.json: {where}.kind {data.get('kind')!r} is not implemented; supported: ['moe']")
        router = _mapping(where, data, "router")
        experts, top = _count(f"{where}.router", router, "experts"), _count(f"{where}.router", router, "top")
        groups = _optional(f"{where}.router", router, "groups")
        count = keep = 1
        if groups is not None:
            count = _count(f"{where}.router.groups", groups, "count")
            keep = _count(f"{where}.router.groups", groups, "keep")
        if experts % count != 0 or keep > count or top > (experts // count) * keep:
            raise UnsupportedModelError(f"config.json: {where}.router: {top} of {experts} experts cannot be taken from {keep} of "
                                        f"{count} equal groups")
        return cls(_count(f"{where}.expert", _mapping(where, data, "expert"), "ff"), experts, top, count, keep)


@dataclass(frozen=True)
class LegavikLayer:
    type: str
    mixer: KeyedAttentionSizes | ParallelSizes
    mlp: RoutedSizes | None


@dataclass(frozen=True)
class LegavikConfig:
    """One checkpoint's numbers (frozen: model, cache sizing and runner share it)."""

    architecture: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    logit_softcap: float | None
    layers: tuple[LegavikLayer, ...]
    eos_token_ids: tuple[int, ...] = ()
    name_or_path: str = ""

    def kv_bytes_per_token(self, dtype) -> int:
        """Bytes one token takes in the pages of all layers."""
        return sum(layer.mixer.cached_elements() for layer in self.layers) * dtype.itemsize

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], *, name_or_path: str = "") -> "LegavikConfig":
        if str(data.get("architecture")) != ARCHITECTURE:
            raise UnsupportedModelError(f"architecture {data.get('architecture')!r} is not {ARCHITECTURE}")
        listed = data.get("layers")
        if not isinstance(listed, (list, tuple)) or not listed:
            raise UnsupportedModelError("config.json: layers must be a non-empty list")
        readers = {"attention": KeyedAttentionSizes, "parallel": ParallelSizes}
        layers = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            if not isinstance(entry, Mapping):
                raise UnsupportedModelError(f"config.json: {where} must be an object")
            kind = entry.get("type")
            if kind not in readers:
                raise UnsupportedModelError(f"config.json: {where}.type {kind!r} is not implemented; supported: {list(MIXER_TYPES)}")
            mixer = readers[kind].read(f"{where}.mixer", _mapping(where, entry, "mixer"))
            mlp = None if entry.get("mlp") is None else RoutedSizes.read(f"{where}.mlp", _mapping(where, entry, "mlp"))
            layers.append(LegavikLayer(kind, mixer, mlp))
        named = data.get("eos_token_id")
        eos = () if named is None else (int(named),) if isinstance(named, int) else tuple(int(t) for t in named)
        cap = None if data.get("logit_softcap") is None else _real("config", data, "logit_softcap")
        return cls(
            architecture=ARCHITECTURE, vocab_size=_count("config", data, "vocab"), hidden_size=_count("config", data, "width"),
            norm_eps=_real("norm", _mapping("config", data, "norm"), "eps"), logit_softcap=cap, layers=tuple(layers),
            eos_token_ids=eos, name_or_path=name_or_path,
        )
