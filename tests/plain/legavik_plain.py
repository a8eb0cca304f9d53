"""Legavik restated from its equations: whole sequences, no cache, no batching, one function per
mechanism, written with explicit loops where that makes the rule plain.  It shares no code with the
engine; the tests compare the engine with it.

Notation: ``x [T, W]`` is the stream of one sequence, position ``i`` sees position ``j`` of the same
sequence.  ``config`` is the mapping a ``config.json`` holds, ``tensors`` the checkpoint by name.
Everything is computed in the dtype of the tensors handed in (the tests hand in float32 or float64).
"""

from __future__ import annotations

import math

import torch


def squash_norm(x: torch.Tensor, tensors: dict, name: str) -> torch.Tensor:
    """A norm without statistics: ``tanh(alpha x) * w + b`` with a scalar ``alpha``."""
    return torch.tanh(tensors[name + ".alpha"] * x) * tensors[name] + tensors[name + ".b"]


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """``x / sqrt(mean(x^2) + eps)`` over the last dimension."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def short_conv(u: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """``u [T, C]``, ``taps [C, K]``: ``y_t = sum_j taps[:, j] u_(t - K + 1 + j)``, zeros before the start."""
    T, K = u.shape[0], taps.shape[1]
    y = torch.zeros_like(u)
    for t in range(T):
        for j in range(K):
            s = t - K + 1 + j
            if s >= 0:
                y[t] += taps[:, j] * u[s]
    return y


# -- rotation in halves with stretched frequencies -------------------------------------------------


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


def turn_halves(x: torch.Tensor, rot: dict) -> torch.Tensor:
    """``x [T, heads, D]``: element ``i`` and element ``i + dims/2`` of the first ``dims`` form a pair;
    at position ``p`` the pair ``(u, v)`` becomes ``(u cos a - v sin a, v cos a + u sin a)``."""
    f, magnitude = frequencies(rot)
    half = rot["dims"] // 2
    out = x.clone()
    for p in range(x.shape[0]):
        for i in range(half):
            a = p * float(f[i])
            c, s = math.cos(a) * magnitude, math.sin(a) * magnitude
            u, v = x[p, ..., i], x[p, ..., i + half]
            out[p, ..., i] = u * c - v * s
            out[p, ..., i + half] = v * c + u * s
    return out


# -- attention whose values are its keys, a window that keeps the first tokens ---------------------


def sees(i: int, j: int, mask: dict | None) -> bool:
    if j > i:
        return False
    if not mask:
        return True
    return i - j < mask["size"] or j < mask.get("keep_first", 0)


def head_gate(prefix: str, tensors: dict, h: torch.Tensor) -> torch.Tensor:
    """One number per token and head: ``sigmoid(Wg h)``."""
    return torch.sigmoid(h @ tensors[prefix + ".g"].T)


def softmax_heads(q, k, v, scale: float, mask: dict | None, gate: torch.Tensor) -> torch.Tensor:
    """``q [T, H, D]``, ``k [T, G, D]``, ``v [T, G, Dv]`` -> ``[T, H * Dv]``, every head's output times
    its gate."""
    T, H, G = q.shape[0], q.shape[1], k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for head in range(H):
        g = head // (H // G)
        for i in range(T):
            seen = [j for j in range(i + 1) if sees(i, j, mask)]
            scores = (k[seen, g] @ q[i, head]) * scale
            out[i, head] = torch.softmax(scores, dim=0) @ v[seen, g] * gate[i, head]
    return out.reshape(T, -1)


def keyed_attention(prefix: str, sizes: dict, tensors: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, D = sizes["heads"], sizes["kv_heads"], sizes["dim"]
    q = (h @ tensors[prefix + ".q"].T).view(T, H, D)
    k = (h @ tensors[prefix + ".k"].T).view(T, G, D)
    v = k
    if sizes.get("rot"):
        q, k = turn_halves(q, sizes["rot"]), turn_halves(k, sizes["rot"])
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    mixed = softmax_heads(q, k, v, sizes["scale"], sizes.get("mask"), head_gate(prefix, tensors, h))
    return mixed @ tensors[prefix + ".o"].T


# -- the two mixers of a parallel layer ------------------------------------------------------------


def convolved_attention(prefix: str, sizes: dict, tensors: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    """Biased projections, a short convolution on each, q/k norm with a shared gain, a query
    temperature that grows with the position, causal softmax, gate, output projection with bias."""
    T = h.shape[0]
    H, G, D, Dv = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]

    def project(name):
        projected = h @ tensors[f"{prefix}.{name}"].T + tensors[f"{prefix}.{name}.b"]
        return short_conv(projected, tensors[f"{prefix}.{name}.conv"]) if sizes.get("conv") else projected

    q, k, v = project("q").view(T, H, D), project("k").view(T, G, D), project("v").view(T, G, Dv)
    q = unit_rms(q, eps) * tensors[prefix + ".q.norm"]
    k = unit_rms(k, eps) * tensors[prefix + ".k.norm"]
    temp = sizes.get("q_temp")
    if temp:
        for p in range(T):
            q[p] = q[p] * (1 + temp["coef"] * math.log(math.floor((p + 1) / temp["every"]) + 1))
    mixed = softmax_heads(q, k, v, sizes["scale"], None, head_gate(prefix, tensors, h))
    return mixed @ tensors[prefix + ".o"].T + tensors[prefix + ".o.b"]


def delta_rule(prefix: str, sizes: dict, tensors: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    """Per head a state ``S [D, Dv]``: decay its rows, correct what the key reads by ``beta``, read."""
    T = h.shape[0]
    H, G, D, Dv = sizes["heads"], sizes["kv_heads"], sizes["dim"], sizes["vdim"]

    def project(name):
        return torch.nn.functional.silu(short_conv(h @ tensors[f"{prefix}.{name}"].T, tensors[f"{prefix}.{name}.conv"]))

    q, k, v = project("q").view(T, G, D), project("k").view(T, G, D), project("v").view(T, H, Dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ tensors[prefix + ".b"].T)
    step = torch.nn.functional.softplus((h @ tensors[prefix + ".a1"].T) @ tensors[prefix + ".a2"].T + tensors[prefix + ".dt_bias"])
    decay = torch.exp(-torch.exp(tensors[prefix + ".A_log"])[:, None] * step.view(T, H, D))
    gate = torch.sigmoid((h @ tensors[prefix + ".g1"].T) @ tensors[prefix + ".g2"].T).view(T, H, Dv)
    out = torch.zeros(T, H, Dv, dtype=h.dtype)
    for head in range(H):
        g = head // (H // G)
        S = torch.zeros(D, Dv, dtype=h.dtype)
        for t in range(T):
            S = decay[t, head][:, None] * S
            u = beta[t, head] * (v[t, head] - S.T @ k[t, g])
            S = S + torch.outer(k[t, g], u)
            out[t, head] = S.T @ q[t, g]
    out = unit_rms(out, eps) * tensors[prefix + ".norm"] * gate
    return out.reshape(T, H * Dv) @ tensors[prefix + ".o"].T


def side_by_side(prefix: str, sizes: dict, tensors: dict, h: torch.Tensor, eps: float) -> torch.Tensor:
    left = convolved_attention(prefix + ".left", sizes["left"], tensors, h, eps)
    right = delta_rule(prefix + ".right", sizes["right"], tensors, h, eps)
    return sizes["left_scale"] * left + sizes["right_scale"] * right


# -- routed experts ----------------------------------------------------------------------------------


def choose(scores: torch.Tensor, router: dict) -> list[int]:
    """The ``top`` best experts among those of the ``keep`` groups whose best expert scores highest
    (equal scores: the lower index)."""
    E = scores.shape[0]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    size = E // groups["count"]
    marks = [max(float(scores[g * size + e]) for e in range(size)) for g in range(groups["count"])]
    kept = sorted(range(groups["count"]), key=lambda g: (-marks[g], g))[:groups["keep"]]
    allowed = [e for e in range(E) if e // size in kept]
    return sorted(allowed, key=lambda e: (-float(scores[e]), e))[:router["top"]]


def routed(prefix: str, mlp: dict, tensors: dict, h: torch.Tensor) -> torch.Tensor:
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        scores = torch.softmax(h[t] @ tensors[prefix + ".router"].T, dim=0)
        taken = choose(scores, mlp["router"])
        total = sum(scores[e] for e in taken) + 1e-20
        for e in taken:
            p = f"{prefix}.e{e}"
            inner = torch.nn.functional.silu(tensors[p + ".gate"] @ h[t]) * (tensors[p + ".up"] @ h[t])
            out[t] += scores[e] / total * (tensors[p + ".down"] @ inner)
    return out


# -- layers, the model -----------------------------------------------------------------------------


def layers(config: dict, tensors: dict, tokens: list[int]) -> list[torch.Tensor]:
    """The stream after every layer."""
    eps = config["norm"]["eps"]
    x = tensors["embed"][torch.tensor(tokens)]
    after = []
    for index, layer in enumerate(config["layers"]):
        p = f"l{index}"
        h = squash_norm(x, tensors, p + ".norm1")
        if layer["type"] == "attention":
            x = x + keyed_attention(p + ".mix", layer["mixer"], tensors, h, eps)
        else:
            x = x + side_by_side(p + ".mix", layer["mixer"], tensors, h, eps)
        if layer["mlp"] is not None:
            x = x + routed(p + ".mlp", layer["mlp"], tensors, squash_norm(x, tensors, p + ".norm2"))
        after.append(x)
    return after


def forward(config: dict, tensors: dict, tokens: list[int]) -> torch.Tensor:
    """``[T, V]`` logits: the final norm, the output matrix, then ``c tanh(z / c)``."""
    x = layers(config, tensors, tokens)[-1]
    logits = squash_norm(x, tensors, "final.norm") @ tensors["head"].T
    cap = config.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
