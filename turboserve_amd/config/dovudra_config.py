"""Typed view of a Dovudra ``config.json``.

The file names the design under ``architecture`` and describes every layer on its own::

    {"architecture": "Dovudra", "vocab": V, "width": W, "norm": {"eps": e}, "residual_mult": m,
     "layers": [{"type": "attention",
                 "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": Dv, "scale": s, "bias_max": M,
                           "mask": {"size": w}, "v_mix": true},
                 "mlp": {"kind": "dense", "ff": I} | null},
                {"type": "latent_attention",
                 "mixer": {"heads": H, "dim": D, "rot_dim": R, "vdim": Dv, "kv_rank": C, "scale": s,
                           "mask": {"size": w},
                           "rot": {"base": b, "dims": d,
                                   "scaling": {"factor": f, "original": n, "fast": a, "slow": c}}},
                 "mlp": ...}, ...]}

Every size and constant a model of the design can choose comes from here; the number of rows of an
attention layer's table of distance biases comes from the tensor itself unless ``mixer.bias_rows``
names it (a folder of random weights needs that).  What the design fixes lives where the plan is
put together.
"""

from __future__ import annotations

from collections.abc import Mapping
from dataclasses import dataclass
from typing import Any

from turboserve_amd.config.model_config import UnsupportedModelError
from turboserve_amd.config.sisisun_config import _count, _mapping, _real

ARCHITECTURE = "Dovudra"
MIXER_TYPES = ("attention", "latent_attention")


def _window(where: str, data: Mapping[str, Any]) -> int | None:
    if data.get("mask") is None:
        return None
    return _count(f"{where}.mask", _mapping(where, data, "mask"), "size")


@dataclass(frozen=True)
class BiasedAttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    bias_max: float
    bias_rows: int | None  # None: from the tensor
    window: int | None
    v_mix: bool

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "BiasedAttentionSizes":
        mix = data.get("v_mix", False)
        if not isinstance(mix, bool):
            raise UnsupportedModelError(f"config.json: {where}.v_mix must be true or false, got {mix!r}")
        sizes = cls(heads=_count(where, data, "heads"), kv_heads=_count(where, data, "kv_heads"), dim=_count(where, data, "dim"),
                    vdim=_count(where, data, "vdim"), scale=_real(where, data, "scale"), bias_max=_real(where, data, "bias_max"),
                    bias_rows=None if data.get("bias_rows") is None else _count(where, data, "bias_rows", least=2),
                    window=_window(where, data), v_mix=mix)
        if sizes.heads % sizes.kv_heads != 0:
            raise UnsupportedModelError(f"config.json: {where}: {sizes.heads} heads are not a multiple of {sizes.kv_heads} kv_heads")
        return sizes

    def cached_elements(self) -> int:
        return self.kv_heads * (self.dim + self.vdim)


@dataclass(frozen=True)
class RotationScaling:
    factor: float
    original: float
    fast: float
    slow: float

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "RotationScaling":
        return cls(factor=_real(where, data, "factor"), original=_real(where, data, "original"),
                   fast=_real(where, data, "fast"), slow=_real(where, data, "slow"))

    def as_mapping(self) -> dict[str, float]:
        return {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}


@dataclass(frozen=True)
class GatedLatentSizes:
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int | None
    rot_base: float
    rot_dims: int
    rot_scaling: RotationScaling | None

    @classmethod
    def read(cls, where: str, data: Mapping[str, Any]) -> "GatedLatentSizes":
        rot = _mapping(where, data, "rot")
        scaling = None
        if rot.get("scaling") is not None:
            scaling = RotationScaling.read(f"{where}.rot.scaling", _mapping(f"{where}.rot", rot, "scaling"))
        sizes = cls(heads=_count(where, data, "heads"), dim=_count(where, data, "dim"), rot_dim=_count(where, data, "rot_dim"),
                    vdim=_count(where, data, "vdim"), kv_rank=_count(where, data, "kv_rank"), scale=_real(where, data, "scale"),
                    window=_window(where, data), rot_base=_real(f"{where}.rot", rot, "base"),
                    rot_dims=_count(f"{where}.rot", rot, "dims", least=2), rot_scaling=scaling)
        if sizes.rot_dims > sizes.rot_dim or sizes.rot_dims % 2 != 0:
            raise UnsupportedModelError(f"config.json: {where}.rot.dims {sizes.rot_dims} must be even and at most rot_dim {sizes.rot_dim}")
        return sizes

    def cached_elements(self) -> int:
        return self.kv_rank + self.rot_dim


@dataclass(frozen=True)
class DenseSizes:
    ff: int


@dataclass(frozen=True)
class DovudraLayer:
    type: str
    mixer: BiasedAttentionSizes | GatedLatentSizes
    mlp: DenseSizes | None


@dataclass(frozen=True)
class DovudraConfig:
    """One checkpoint's numbers (frozen: model, cache sizing and runner share it)."""

    architecture: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    residual_mult: float
    layers: tuple[DovudraLayer, ...]
    eos_token_ids: tuple[int, ...] = ()
    name_or_path: str = ""

    def kv_bytes_per_token(self, dtype) -> int:
        """Bytes one token takes in the pages of all layers."""
        return sum(layer.mixer.cached_elements() for layer in self.layers) * dtype.itemsize

    def first_value_mixer(self) -> int | None:
        """The first layer whose values the later ``v_mix`` layers mix into their own."""
        for index, layer in enumerate(self.layers):
            if isinstance(layer.mixer, BiasedAttentionSizes) and layer.mixer.v_mix:
                return index
        return None

    @classmethod
    def from_dict(cls, data: Mapping[str, Any], *, name_or_path: str = "") -> "DovudraConfig":
        if str(data.get("architecture")) != ARCHITECTURE:
            raise UnsupportedModelError(f"architecture {data.get('architecture')!r} is not {ARCHITECTURE}")
        listed = data.get("layers")
        if not isinstance(listed, (list, tuple)) or not listed:
            raise UnsupportedModelError("config.json: layers must be a non-empty list")
        readers = {"attention": BiasedAttentionSizes, "latent_attention": GatedLatentSizes}
        layers = []
        for index, entry in enumerate(listed):
            where = f"layers[{index}]"
            if not isinstance(entry, Mapping):
                raise UnsupportedModelError(f"config.json: {where} must be an object")
            kind = entry.get("type")
            if kind not in readers:
                raise UnsupportedModelError(f"config.json: {where}.type {kind!r} is not implemented; supported: {list(MIXER_TYPES)}")
            mixer = readers[kind].read(f"{where}.mixer", _mapping(where, entry, "mixer"))
            mlp = entry.get("mlp")
            if mlp is not None:
                mlp = _mapping(where, entry, "mlp")
                if mlp.get("kind") != "dense":
                    raise UnsupportedModelError(f"config.json: {where}.mlp.kind {mlp.get('kind')!r} is not implemented; supported: ['dense']")
                mlp = DenseSizes(ff=_count(f"{where}.mlp", mlp, "ff"))
            layers.append(DovudraLayer(kind, mixer, mlp))
        mixing = [layer.mixer for layer in layers if isinstance(layer.mixer, BiasedAttentionSizes) and layer.mixer.v_mix]
        if any((m.kv_heads, m.vdim) != (mixing[0].kv_heads, mixing[0].vdim) for m in mixing):
            raise UnsupportedModelError("config.json: layers that mix their values need the same kv_heads and vdim")
        named = data.get("eos_token_id")
        eos = () if named is None else (int(named),) if isinstance(named, int) else tuple(int(t) for t in named)
        mult = 1.0 if data.get("residual_mult") is None else _real("config", data, "residual_mult")
        return cls(
            architecture=ARCHITECTURE, vocab_size=_count("config", data, "vocab"), hidden_size=_count("config", data, "width"),
            norm_eps=_real("norm", _mapping("config", data, "norm"), "eps"), residual_mult=mult, layers=tuple(layers),
            eos_token_ids=eos, name_or_path=name_or_path,
        )
