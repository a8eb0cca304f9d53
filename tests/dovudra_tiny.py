"""Small Dovudra configurations that differ in every size, constant and layer order, and helpers
that write their random model folders and compute the plain implementation's logits."""

from __future__ import annotations

import json
from pathlib import Path

import torch

from plain import dovudra_plain as plain


def attention(heads, kv_heads, dim, vdim, window, rows, farthest, scale=None, v_mix=False):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5 if scale is None else scale,
             "bias_max": farthest, "bias_rows": rows, "v_mix": v_mix}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "attention", "mixer": mixer}


def latent(heads, dim, rot_dim, vdim, rank, window, turned=None, base=10000.0, scale=None, stretch=None):
    rot = {"base": base, "dims": rot_dim if turned is None else turned}
    if stretch is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), stretch))
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
             "scale": (dim + rot_dim) ** -0.5 if scale is None else scale, "rot": rot}
    if window is not None:
        mixer["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mixer}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def layer(mixer, mlp):
    return {**mixer, "mlp": mlp}


#: A: attention first; three layers mix their values (the first is the source); values narrower than
#: keys; a window shorter than two pages and one longer than most requests; a layer without a
#: feed-forward; stretched frequencies whose ramp lies inside the pairs.
CONFIG_A = {
    "architecture": "Dovudra", "vocab": 211, "width": 64, "norm": {"eps": 1e-5}, "residual_mult": 0.5,
    "layers": [
        layer(attention(4, 2, 16, 8, 20, 8, 40, scale=0.3, v_mix=True), dense(96)),
        layer(latent(3, 16, 8, 12, 24, 50, base=1000.0, stretch=(4.0, 64, 8.0, 1.0)), None),
        layer(attention(2, 2, 24, 8, 120, 12, 90.0, v_mix=True), dense(40)),
        layer(attention(4, 2, 16, 8, 9, 6, 7, v_mix=True), None),
    ],
}
PAGE_A = 16

#: B: sizes that 16-byte accesses do not divide; one head; as many key heads as query heads; a
#: window of one token and one shorter than a page; fewer turned elements than rotated ones; no
#: stretch; no mixing; a multiplier of one (the key left out); a table with an odd number of rows.
CONFIG_B = {
    "architecture": "Dovudra", "vocab": 97, "width": 52, "norm": {"eps": 1e-6},
    "layers": [
        layer(latent(1, 12, 12, 20, 10, 5, turned=4, base=50.0, scale=0.4), dense(28)),
        layer(attention(5, 5, 12, 12, 7, 5, 30, scale=0.5), dense(44)),
        layer(latent(2, 6, 4, 10, 18, 1, base=300.0, stretch=(2.0, 16, 4.0, 0.5)), dense(20)),
        layer(attention(1, 1, 20, 36, 33, 9, 400), None),
    ],
}
PAGE_B = 8

#: C: larger heads on the matrix-core path, windows of several pages and none at all, one mixing
#: layer alone (a source nobody reads), values wider than keys, pages of 32.
CONFIG_C = {
    "architecture": "Dovudra", "vocab": 160, "width": 96, "norm": {"eps": 1e-6}, "residual_mult": 0.25,
    "layers": [
        layer(latent(4, 32, 32, 16, 64, 70, base=200000.0, stretch=(6.0, 128, 24.0, 2.0)), dense(160)),
        layer(attention(6, 2, 32, 48, 100, 16, 64, v_mix=True), dense(64)),
        layer(latent(2, 64, 16, 32, 48, None, base=10000.0), dense(96)),
        layer(attention(8, 4, 16, 16, None, 32, 128, scale=0.2), dense(128)),
    ],
}
PAGE_C = 32

TINY = {"A": (CONFIG_A, 21, PAGE_A), "B": (CONFIG_B, 22, PAGE_B), "C": (CONFIG_C, 23, PAGE_C)}


def draw_tensors(config: dict, seed: int, dtype: torch.dtype, std: float) -> dict[str, torch.Tensor]:
    """Random tensors by the names and shapes the engine's own description of the model gives (the
    plain implementation reads them by name): matrices N(0, std), gains around one, bias tables, sinks,
    gates and mixing weights wide enough to matter.  The first mixing layer's weight, which nobody
    reads, is in the folder too."""
    from turboserve_amd.weights.random_init import describe_model

    _, model = describe_model(config)
    generator = torch.Generator().manual_seed(seed)
    tensors = {}
    names = dict(model.tensor_specs())
    for name in model.ignorable_names():
        if name.endswith(".vmix"):
            names[name] = None
    for name, spec in names.items():
        values = torch.randn(() if spec is None else spec.shape, generator=generator)
        if name.endswith(("norm", "norm1", "norm2", "norm1b", "norm2b")):
            values = 1.0 + 0.3 * values
        elif name == "embed":
            values = 0.7 * values
        elif name.endswith(".rel"):
            values = 1.5 * values
        elif name.endswith(".sink"):
            values = 1.0 + values
        elif name.endswith(".vmix"):
            values = 0.35 + 0.1 * values
        elif name.endswith(".g"):
            values = 4.0 * std * values
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


def without_rows(config: dict) -> dict:
    """The configuration as a checkpoint's own file has it: the bias tables' rows are not named."""
    out = json.loads(json.dumps(config))
    for entry in out["layers"]:
        entry["mixer"].pop("bias_rows", None)
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
