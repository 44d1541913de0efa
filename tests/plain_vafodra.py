"""The Vafodra design written out plainly: float64, whole sequences, no cache, one function per mechanism.

Nothing here is shared with the library: the tests compare the engine (any cutting of a sequence into steps,
any batch) with these functions run over the whole sequence at once.  A model is a dict of the configuration
(the keys of its config.json) and a dict name -> tensor.

Notation: T tokens, H heads, G key/value heads or groups, N state size, P value size of a head.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

F = torch.float64


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.logaddexp(z, torch.zeros_like(z))


def rms_divide(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def dynamic_tanh(x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor, alpha: torch.Tensor) -> torch.Tensor:
    """tanh(alpha x) w + b: no mean, no variance."""
    return torch.tanh(alpha * x) * weight + bias


def causal_conv(x: torch.Tensor, taps: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x [T, C], taps [C, K]: y[t, c] = sum_j taps[c, j] x[t - (K - 1) + j, c], zeros before the start;
    the last column of `taps` meets the current token."""
    T, C = x.shape
    K = taps.shape[1]
    padded = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], 0)
    y = torch.zeros_like(x)
    for j in range(K):
        y = y + padded[j : j + T] * taps[:, j]
    return y if bias is None else y + bias


def visible(i: int, j: int, window: int, keep_first: int) -> bool:
    """Whether position i sees position j: causal, inside the window, or among the kept first tokens."""
    return j <= i and (i - j < window or j < keep_first)


def sink_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, window: int,
                   keep_first: int) -> torch.Tensor:
    """q [T, H, D], k [T, G, D], v [T, G, P] -> [T, H, P].  Scores are (q . k) scale without any position
    encoding; the softmax has one more term in its denominator, a sink of score 0 that carries no value."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    mask = (j <= i) & ((i - j < window) | (j < keep_first))  # `visible`, for all pairs at once
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        e = torch.where(mask, torch.exp(s), torch.zeros_like(s))
        out[:, h] = (e / (1.0 + e.sum(-1, keepdim=True))) @ v[:, g]
    return out


def left_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, c: dict) -> torch.Tensor:
    """The attention side: projections, sink attention, a gate per head, output projection."""
    T = h.shape[0]
    H, G, D, P = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = (h @ w[p + ".q"].T).view(T, H, D)
    k = (h @ w[p + ".k"].T).view(T, G, D)
    v = (h @ w[p + ".v"].T).view(T, G, P)
    o = sink_attention(q, k, v, c["scale"], c["mask"]["size"], c["mask"]["keep_first"])
    gate = torch.sigmoid(h @ w[p + ".g"].T)  # [T, H]
    o = o * gate[:, :, None]
    return o.reshape(T, H * P) @ w[p + ".o"].T


def ssd_scan(x: torch.Tensor, B: torch.Tensor, C: torch.Tensor, dt: torch.Tensor, A_log: torch.Tensor,
             D: torch.Tensor) -> torch.Tensor:
    """x [T, H, P], B and C [T, G, N], dt [T, H] (after its softplus) -> y [T, H, P].
    S_t = exp(-exp(A_log) dt_t) S_(t-1) + dt_t B_t x_t^T,  y_t = S_t^T C_t + D x_t."""
    T, H, P = x.shape
    G, N = B.shape[1], B.shape[2]
    y = torch.zeros_like(x)
    for h in range(H):
        g = h // (H // G)
        S = torch.zeros(N, P, dtype=x.dtype)
        for t in range(T):
            S = torch.exp(-torch.exp(A_log[h]) * dt[t, h]) * S + dt[t, h] * torch.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + D[h] * x[t, h]
    return y


def right_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, c: dict, eps: float) -> torch.Tensor:
    """The state-space side."""
    T = h.shape[0]
    H, P, N, G = c["heads"], c["vdim"], c["state"], c["groups"]
    inner = H * P
    u = h @ w[p + ".in"].T
    z, xbc, dt = u[:, :inner], u[:, inner : 2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N :]
    xbc = silu(causal_conv(xbc, w[p + ".conv"], w[p + ".conv.b"]))
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner : inner + G * N].view(T, G, N)
    C = xbc[:, inner + G * N :].view(T, G, N)
    dt = softplus(dt + w[p + ".dt_bias"])
    y = ssd_scan(x, B, C, dt, w[p + ".A_log"], w[p + ".D"]).reshape(T, inner)
    y = y * silu(z)
    parts = c["norm_groups"]
    y = rms_divide(y.view(T, parts, inner // parts), eps).reshape(T, inner) * w[p + ".norm"]
    return y @ w[p + ".o"].T


def parallel_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, c: dict, eps: float) -> torch.Tensor:
    """Both sides read h; each result is RMS-normed over the width with its own weight; half their sum."""
    left = rms_divide(left_mixer(h, w, p + ".left", c["left"]), eps) * w[p + ".left.out"]
    right = rms_divide(right_mixer(h, w, p + ".right", c["right"], eps), eps) * w[p + ".right.out"]
    return 0.5 * (left + right)


def delta_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """q, k [T, G, D], v [T, H, P], beta and g [T, H] -> o [T, H, P].  Per head:
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q."""
    T, H, P = v.shape
    G, D = k.shape[1], k.shape[2]
    o = torch.zeros_like(v)
    for h in range(H):
        j = h // (H // G)
        S = torch.zeros(D, P, dtype=v.dtype)
        for t in range(T):
            S = g[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, j])
            S = S + torch.outer(k[t, j], u)
            o[t, h] = S.T @ q[t, j]
    return o


def delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str, c: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, P = c["heads"], c["kv_heads"], c["dim"], c["vdim"]
    q = silu(causal_conv(h @ w[p + ".q"].T, w[p + ".q.conv"])).view(T, G, D)
    k = silu(causal_conv(h @ w[p + ".k"].T, w[p + ".k.conv"])).view(T, G, D)
    v = silu(causal_conv(h @ w[p + ".v"].T, w[p + ".v.conv"])).view(T, H, P)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + ".b"].T)
    g = torch.exp(-torch.exp(w[p + ".A_log"]) * softplus(h @ w[p + ".a"].T + w[p + ".dt_bias"]))
    o = delta_scan(q, k, v, beta, g)
    o = rms_divide(o, eps) * w[p + ".norm"]
    o = o * silu(h @ w[p + ".g"].T).view(T, H, P)
    return o.reshape(T, H * P) @ w[p + ".o"].T


def feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], p: str) -> torch.Tensor:
    return (torch.relu(h @ w[p + ".gate"].T) * (h @ w[p + ".up"].T)) @ w[p + ".down"].T


def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  `streams`, if a list, receives the residual stream after
    every layer run."""
    w = {n: t.to(F) for n, t in weights.items()}
    eps = float(config["norm"]["eps"])
    m = float(config["residual_mult"])
    x = w["embed"][torch.tensor(tokens)] * float(config["embedding"]["scale"])
    for i, layer in enumerate(config["layers"]):
        p = f"l{layer.get('weights_of', i)}"
        h = dynamic_tanh(x, w[p + ".norm1"], w[p + ".norm1.b"], w[p + ".norm1.alpha"])
        if layer["type"] == "parallel":
            mixed = parallel_mixer(h, w, p + ".mix", layer["mixer"], eps)
        elif layer["type"] == "delta":
            mixed = delta_mixer(h, w, p + ".mix", layer["mixer"], eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            mixed = mixed + feed_forward(h, w, p + ".mlp")
        x = x + m * mixed
        if streams is not None:
            streams.append(x.clone())
    x = dynamic_tanh(x, w["final.norm"], w["final.norm.b"], w["final.norm.alpha"])
    return x @ w["head"].T
