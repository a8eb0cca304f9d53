"""Dovudra restated from its equations: whole sequences, no cache, no batching, one function per
mechanism, written with explicit loops where that makes the rule plain.  It shares no code with the
engine; the tests compare the engine with it.

Notation: ``x [T, W]`` is the stream of one sequence, position ``i`` sees position ``j`` of the same
sequence.  ``config`` is the mapping a ``config.json`` holds, ``tensors`` the checkpoint by name.
Everything is computed in the dtype of the tensors handed in (the tests hand in float32 or float64).
"""

from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps) * gain`` over the last dimension."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * gain


# -- attention with bucketed distance biases, a window, a learned sink ---------------------------


def bucket(distance: int, rows: int, farthest: float) -> int:
    """Row of the bias table for a key ``distance`` back: below ``rows // 2`` a row each, then rows
    spaced evenly in ``ln(distance)`` up to ``farthest``, the last row for all beyond."""
    near = rows // 2
    if distance < near:
        return distance
    return min(rows - 1, near + math.floor(math.log(distance / near) / math.log(farthest / near) * (rows - near)))


def sink_softmax_row(scores: torch.Tensor, sink: torch.Tensor) -> torch.Tensor:
    """Weights ``exp(s_j) / (exp(sink) + sum_k exp(s_k))``: the sink is in the denominator only."""
    top = torch.maximum(scores.max(), sink)
    weights = torch.exp(scores - top)
    return weights / (weights.sum() + torch.exp(sink - top))


def biased_attention(prefix: str, sizes: dict, tensors: dict, h: torch.Tensor, eps: float, first_values: list) -> torch.Tensor:
    """``first_values``: an empty list at the first layer that mixes values; it leaves its own there,
    and every later mixing layer blends them into its own."""
    T = h.shape[0]
    H, G, D, Dv = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]
    q = (h @ tensors[prefix + ".q"].T).view(T, H, D)
    k = (h @ tensors[prefix + ".k"].T).view(T, G, D)
    v = (h @ tensors[prefix + ".v"].T).view(T, G, Dv)
    q = rms(q, tensors[prefix + ".q.norm"], eps)
    k = rms(k, tensors[prefix + ".k.norm"], eps)
    if sizes.get("v_mix"):
        if not first_values:
            first_values.append(v)
        else:
            lam = tensors[prefix + ".vmix"]
            v = (1 - lam) * v + lam * first_values[0]
    rel, sink = tensors[prefix + ".rel"], tensors[prefix + ".sink"]
    window = sizes["mask"]["size"] if sizes.get("mask") else T
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        for i in range(T):
            seen = range(max(0, i - window + 1), i + 1)
            scores = torch.stack([(q[i, head] @ k[j, g]) * sizes["scale"] + rel[bucket(i - j, rel.shape[0], sizes["bias_max"]), head]
                                  for j in seen])
            weights = sink_softmax_row(scores, sink[head])
            out[i, head] = weights @ v[seen.start:i + 1, g]
    return out.reshape(T, H * Dv) @ tensors[prefix + ".o"].T


# -- latent attention with rotated neighbours, stretched frequencies, a window, an output gate -----


def frequencies(rot: dict) -> tuple[torch.Tensor, float]:
    """``f_i`` of the pairs and the factor on cosine and sine."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = base ** (-2.0 * i / dims)
    stretch = rot.get("scaling")
    if not stretch:
        return f, 1.0

    def where(turns: float) -> float:
        return dims * math.log(stretch["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(where(stretch["fast"])), 0)
    hi = min(math.ceil(where(stretch["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return f / stretch["factor"] * ramp + f * (1 - ramp), 0.1 * math.log(stretch["factor"]) + 1.0


def turn(x: torch.Tensor, rot: dict) -> torch.Tensor:
    """``x [T, ..., R]``: the pair ``(2i, 2i + 1)`` of the first ``rot.dims`` elements at position ``p``
    becomes ``(u cos a - v sin a, v cos a + u sin a)``, ``a = p f_i``; the rest pass."""
    f, magnitude = frequencies(rot)
    out = x.clone()
    for p in range(x.shape[0]):
        for i in range(rot["dims"] // 2):
            a = p * float(f[i])
            c, s = math.cos(a) * magnitude, math.sin(a) * magnitude
            u, v = x[p, ..., 2 * i], x[p, ..., 2 * i + 1]
            out[p, ..., 2 * i] = u * c - v * s
            out[p, ..., 2 * i + 1] = v * c + u * s
    return out


def gated_latent_attention(prefix: str, sizes: dict, tensors: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, R, Dv, C = sizes["heads"], sizes["dim"], sizes["rot_dim"], sizes["vdim"], sizes["kv_rank"]
    q = (h @ tensors[prefix + ".q"].T).view(T, H, D + R)
    down = h @ tensors[prefix + ".dkv"].T
    latent = rms(down[:, :C], tensors[prefix + ".dkv.norm"], eps)
    shared = turn(down[:, C:], sizes["rot"])
    q_plain, q_turned = q[..., :D], turn(q[..., D:], sizes["rot"])
    keys = (latent @ tensors[prefix + ".uk"].T).view(T, H, D)
    values = (latent @ tensors[prefix + ".uv"].T).view(T, H, Dv)
    window = sizes["mask"]["size"] if sizes.get("mask") else T
    gate = torch.sigmoid(h @ tensors[prefix + ".g"].T)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for head in range(H):
        for i in range(T):
            lo = max(0, i - window + 1)
            scores = torch.stack([(q_plain[i, head] @ keys[j, head] + q_turned[i, head] @ shared[j]) * sizes["scale"]
                                  for j in range(lo, i + 1)])
            out[i, head] = torch.softmax(scores, dim=0) @ values[lo:i + 1, head] * gate[i, head]
    return out.reshape(T, H * Dv) @ tensors[prefix + ".o"].T


# -- feed-forward, layers, the model ---------------------------------------------------------------


def squared_relu_mlp(prefix: str, tensors: dict, h: torch.Tensor) -> torch.Tensor:
    return torch.relu(h @ tensors[prefix + ".up"].T) ** 2 @ tensors[prefix + ".down"].T


def layers(config: dict, tensors: dict, tokens: list[int]) -> list[torch.Tensor]:
    """The stream after every layer."""
    eps, mult = config["norm"]["eps"], config.get("residual_mult", 1.0)
    x = tensors["embed"][torch.tensor(tokens)]
    first_values: list = []
    after = []
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}"
        h = rms(x, tensors[p + ".norm1"], eps)
        if layer["type"] == "attention":
            mixed = biased_attention(p + ".mix", layer["mixer"], tensors, h, eps, first_values)
        else:
            mixed = gated_latent_attention(p + ".mix", layer["mixer"], tensors, h, eps)
        x = x + mult * rms(mixed, tensors[p + ".norm1b"], eps)
        if layer["mlp"] is not None:
            h = rms(x, tensors[p + ".norm2"], eps)
            x = x + mult * rms(squared_relu_mlp(p + ".mlp", tensors, h), tensors[p + ".norm2b"], eps)
        after.append(x)
    return after


def forward(config: dict, tensors: dict, tokens: list[int]) -> torch.Tensor:
    """``[T, V]`` logits: the final norm, then the embedding table as the output matrix."""
    x = layers(config, tensors, tokens)[-1]
    return rms(x, tensors["final.norm"], config["norm"]["eps"]) @ tensors["embed"].T
