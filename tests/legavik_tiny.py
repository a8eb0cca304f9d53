"""Small Legavik configurations that differ in every size, constant and layer order, and helpers that
write their random model folders and compute the plain implementation's logits."""

from __future__ import annotations

import json
from pathlib import Path

import torch

from plain import legavik_plain as plain


def keyed(heads, kv_heads, dim, scale=None, window=None, keep=None, rot=None, stretch=None, base=10000.0):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": dim ** -0.5 if scale is None else scale}
    if window is not None:
        mixer["mask"] = {"size": window} if keep is None else {"size": window, "keep_first": keep}
    if rot is not None:
        mixer["rot"] = {"base": base, "dims": rot}
        if stretch is not None:
            mixer["rot"]["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
    return {"type": "attention", "mixer": mixer}


def left(heads, kv_heads, dim, vdim, taps, scale=None, temp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale}
    if taps is not None:
        mixer["conv"] = taps
    if temp is not None:
        mixer["q_temp"] = {"coef": temp[0], "every": temp[1]}
    return mixer


def right(heads, kv_heads, dim, vdim, taps, decay_rank, gate_rank):
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": taps, "decay_rank": decay_rank,
            "gate_rank": gate_rank}


def parallel(left_sizes, right_sizes, left_scale, right_scale):
    return {"type": "parallel", "mixer": {"left": left_sizes, "right": right_sizes, "left_scale": left_scale,
                                          "right_scale": right_scale}}


def moe(ff, experts, top, groups=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff}, "router": router}


def layer(mixer, mlp):
    return {**mixer, "mlp": mlp}


#: A: a parallel layer first; a window shorter than two pages with kept first tokens that end inside a
#: page; a head rotated in part, with stretched frequencies whose ramp lies inside the pairs; a layer
#: without a feed-forward; experts in groups; values wider than keys on the left, narrower on the right.
CONFIG_A = {
    "architecture": "Legavik", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "logit_softcap": 12.0,
    "layers": [
        layer(parallel(left(4, 2, 16, 24, 3, scale=0.3, temp=(0.4, 8)), right(4, 2, 16, 8, 4, 6, 5), 0.7, 1.2), moe(24, 6, 2, (3, 2))),
        layer(keyed(4, 2, 16, scale=0.5, window=20, keep=5, rot=8, stretch=(4.0, 64, 8.0, 1.0), base=1000.0), None),
        layer(parallel(left(2, 2, 8, 8, 2, temp=(0.2, 30)), right(2, 1, 8, 16, 2, 3, 7), 1.0, 0.5), moe(40, 4, 1)),
        layer(keyed(3, 1, 24, window=120, keep=17, rot=24), moe(16, 4, 3, (2, 2))),
    ],
}
PAGE_A = 16

#: B: sizes that 16-byte accesses do not divide; one head; as many key heads as query heads; a window
#: of one token with kept tokens, a window without kept tokens, no window; no rotation at all in one
#: layer; no cap on the logits; convolutions of one tap and of five; no query temperature; every expert
#: a group of its own; one expert taken.
CONFIG_B = {
    "architecture": "Legavik", "vocab": 97, "width": 52, "norm": {"eps": 1e-6},
    "layers": [
        layer(keyed(1, 1, 12, scale=0.4, window=1, keep=3, rot=4, base=50.0), moe(28, 3, 1, (3, 1))),
        layer(parallel(left(5, 5, 12, 12, 1, scale=0.5), right(3, 3, 12, 20, 5, 4, 4), 0.45, 1.3), moe(20, 5, 2, (5, 3))),
        layer(keyed(2, 2, 6, window=7, rot=6, stretch=(2.0, 16, 4.0, 0.5), base=300.0), None),
        layer(keyed(3, 3, 20, scale=0.3), moe(12, 2, 2)),
        layer(parallel(left(1, 1, 20, 36, 4, temp=(1.0, 1)), right(1, 1, 20, 12, 1, 2, 9), -0.8, 1.0), None),
    ],
}
PAGE_B = 8

#: C: heads on the matrix-core path, windows of several pages, kept tokens of more than a page, key
#: channels beyond 64 on the right, pages of 32.
CONFIG_C = {
    "architecture": "Legavik", "vocab": 160, "width": 96, "norm": {"eps": 1e-6}, "logit_softcap": 25.0,
    "layers": [
        layer(keyed(6, 2, 32, window=70, keep=40, rot=16, stretch=(6.0, 128, 24.0, 2.0), base=200000.0), moe(48, 10, 4, (5, 3))),
        layer(parallel(left(4, 4, 32, 64, 3, temp=(0.25, 48)), right(4, 2, 96, 32, 4, 8, 8), 0.8, 0.55), moe(64, 8, 2, (2, 1))),
        layer(keyed(8, 1, 64, window=33, keep=1, rot=64), None),
        layer(parallel(left(8, 2, 16, 16, 3), right(2, 2, 40, 72, 3, 16, 4), 1.0, 1.0), moe(32, 6, 6)),
    ],
}
PAGE_C = 32

TINY = {"A": (CONFIG_A, 21, PAGE_A), "B": (CONFIG_B, 22, PAGE_B), "C": (CONFIG_C, 23, PAGE_C)}


def draw_tensors(config: dict, seed: int, dtype: torch.dtype, std: float) -> dict[str, torch.Tensor]:
    """Random tensors by the names and shapes the engine's own description of the model gives (the plain
    implementation reads them by name): matrices N(0, std); norm weights around one with biases and an
    ``alpha`` that leave the tanh neither linear nor saturated; convolution taps, gates, decay rates and
    biases wide enough to matter (decays of the delta rule from a few tokens to hundreds)."""
    from turboserve_amd.weights.random_init import describe_model

    _, model = describe_model(config)
    generator = torch.Generator().manual_seed(seed)
    tensors = {}
    for name, spec in model.tensor_specs().items():
        values = torch.randn(spec.shape, generator=generator)
        leaf = name.rsplit(".", 1)[-1]
        if name.endswith(".alpha"):
            values = 0.8 + 0.2 * values
        elif leaf in ("norm", "norm1", "norm2") or name == "final.norm":
            values = 1.0 + 0.3 * values
        elif leaf == "b" and name.count(".") >= 2 and name.rsplit(".", 2)[-2] in ("norm1", "norm2", "norm"):
            values = 0.2 * values
        elif name == "embed":
            values = 0.9 * values
        elif leaf == "conv":
            values = 0.6 * values
        elif leaf == "A_log":
            values = -2.0 + 1.5 * values
        elif leaf == "dt_bias":
            values = -1.0 + values
        elif leaf in ("a2", "g2"):
            values = 0.5 * values
        elif leaf == "router":
            values = 4.0 * std * values
        elif leaf == "b":
            values = 0.3 * values  # a projection's bias, or the delta rule's beta matrix
        else:
            values = std * values
        tensors[name] = values.to(dtype).contiguous()
    return tensors


def make_model_dir(folder: Path, config: dict, seed: int, dtype: torch.dtype = torch.float32, std: float = 0.15,
                   tensors: dict[str, torch.Tensor] | None = None) -> Path:
    from safetensors.torch import save_file

    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(config, indent=1))
    save_file(tensors if tensors is not None else draw_tensors(config, seed, dtype, std), str(folder / "model.safetensors"))
    return folder


def without_ranks(config: dict) -> dict:
    """The configuration as a checkpoint's own file has it: the low-rank widths are not named."""
    out = json.loads(json.dumps(config))
    for entry in out["layers"]:
        if entry["type"] == "parallel":
            entry["mixer"]["right"].pop("decay_rank", None)
            entry["mixer"]["right"].pop("gate_rank", None)
    return out


def read_model_dir(folder: Path) -> tuple[dict, dict[str, torch.Tensor]]:
    from safetensors.torch import load_file

    config = json.loads((Path(folder) / "config.json").read_text())
    tensors = {name: t.to(torch.float32) for name, t in load_file(str(Path(folder) / "model.safetensors")).items()}
    return config, tensors


def plain_logits(folder: Path, tokens: list[int]) -> torch.Tensor:
    config, tensors = read_model_dir(folder)
    return plain.forward(config, tensors, tokens)


def greedy(config: dict, tensors: dict[str, torch.Tensor], prompt: list[int], new: int) -> list[int]:
    tokens = list(prompt)
    for _ in range(new):
        tokens.append(int(plain.forward(config, tensors, tokens)[-1].argmax()))
    return tokens[len(prompt):]
