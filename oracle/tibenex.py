"""Plain CPU statement of the Tibenex decoder (TEST INFRASTRUCTURE ONLY, like oracle/model.py).

One function per mechanism, fp32 torch on the host, no cache, no state pool and no batching: a sequence is always
recomputed whole, attention is a dense [T, T] matrix per head, keys and values of the latent layers are expanded for
every head, and the state-space recurrence is a Python loop over the tokens, so nothing here can share a fault with the
engine's pools, kernels or scheduler.  Weights arrive as a dict of tensors under the checkpoint's own names (`embed`,
`l<i>.norm1`, `l<i>.ls1`, `l<i>.shift`, `l<i>.mix.q`, `l<i>.mix.conv`, `l<i>.mlp.gate`, ..., `final.norm`, `head`); the
configuration is the checkpoint's config.json as a dict.

Notation: T tokens, W the model width, H heads, G key/value heads (attention) or groups (state space), D the key size,
E the value size, P the rotated size, R the latent size, N the state size.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch


def rms_norm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    x = x.float()
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight.float()


def pair_frequencies(rot: dict):
    """(frequency of every pair, the factor on cos and sin): base^(-2i / dims), and with rot['scaling'] the stretched low
    frequencies of YaRN."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=torch.float64)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def where(turns):
        return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo, hi = max(math.floor(where(sc["fast"])), 0), min(math.ceil(where(sc["slow"])), dims - 1)
    ramp = torch.tensor([min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(dims // 2)], dtype=torch.float64)
    return f / sc["factor"] * ramp + f * (1 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x: torch.Tensor, rot: dict, halves: bool) -> torch.Tensor:
    """x [T, heads, size]: the first rot['dims'] elements of every head are turned by position * frequency_i, pair i being
    elements (i, i + dims / 2) with `halves` and (2i, 2i + 1) without; the rest passes."""
    T, dims = x.shape[0], int(rot["dims"])
    f, m = pair_frequencies(rot)
    ang = torch.arange(T, dtype=torch.float32).view(T, 1) * f.float().view(1, -1)
    c, s = (torch.cos(ang) * m).view(T, 1, -1), (torch.sin(ang) * m).view(T, 1, -1)
    x = x.float().clone()
    if halves:
        a, b = x[..., : dims // 2].clone(), x[..., dims // 2: dims].clone()
        x[..., : dims // 2] = a * c - b * s
        x[..., dims // 2: dims] = b * c + a * s
    else:
        a, b = x[..., 0:dims:2].clone(), x[..., 1:dims:2].clone()
        x[..., 0:dims:2] = a * c - b * s
        x[..., 1:dims:2] = b * c + a * s
    return x


def causal_softmax(scores: torch.Tensor) -> torch.Tensor:
    """scores [H, T, T] -> weights, key j visible to query i when j <= i."""
    T = scores.shape[-1]
    hidden = torch.arange(T).view(1, 1, T) > torch.arange(T).view(1, T, 1)
    return torch.softmax(scores.float().masked_fill(hidden, float("-inf")), dim=-1)


def token_shift(h: torch.Tensor, mu: torch.Tensor) -> torch.Tensor:
    """h_t + (h_(t-1) - h_t) * mu, zeros in front of the first token."""
    h = h.float()
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu.float()


def latent_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, P, E, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    h = h.float()
    cq = rms_norm(h @ w[pre + "dq"].float().t(), w[pre + "dq.norm"], eps)
    q = (cq @ w[pre + "uq"].float().t()).view(T, H, D + P)
    down = h @ w[pre + "dkv"].float().t()
    c = rms_norm(down[:, :R], w[pre + "dkv.norm"], eps)
    k_rot = rotate(down[:, R:].view(T, 1, P), m["rot"], halves=True)
    q_rot = rotate(q[..., D:], m["rot"], halves=True)
    k = (c @ w[pre + "uk"].float().t()).view(T, H, D)
    v = (c @ w[pre + "uv"].float().t()).view(T, H, E)
    s = (torch.einsum("ihd,jhd->hij", q[..., :D], k) + torch.einsum("ihd,jd->hij", q_rot, k_rot[:, 0])) * m["scale"]
    o = causal_softmax(s) @ v.transpose(0, 1)                        # [H, T, T] x [H, T, E]
    o = o.transpose(0, 1) * torch.sigmoid(h @ w[pre + "g"].float().t()).view(T, H, 1)
    return o.reshape(T, H * E) @ w[pre + "o"].float().t()


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    h = h.float()
    q = rms_norm(h @ w[pre + "q"].float().t(), w[pre + "q.norm"], eps).view(T, H, D)
    k = rms_norm(h @ w[pre + "k"].float().t(), w[pre + "k.norm"], eps).view(T, G, D)
    v = (h @ w[pre + "v"].float().t()).view(T, G, E)
    q, k = rotate(q, m["rot"], halves=False), rotate(k, m["rot"], halves=False)
    of = torch.arange(H) // (H // G)                                  # key/value head of every query head
    s = torch.einsum("ihd,jhd->hij", q, k[:, of]) * m["scale"] * w[pre + "temp"].float().view(H, 1, 1)
    p = causal_softmax(s)
    p = torch.einsum("hg,gij->hij", w[pre + "talk"].float(), p)       # the heads' weights mixed after the softmax
    o = p @ v[:, of].transpose(0, 1)
    return o.transpose(0, 1).reshape(T, H * E) @ w[pre + "o"].float().t()


def causal_conv_silu(x: torch.Tensor, taps: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, n]: y_t = bias + sum_i taps[:, n - 1 - i] * x_(t - i), zeros in front of the sequence; then silu."""
    T, n = x.shape[0], taps.shape[1]
    y = bias.float().expand_as(x).clone()
    for i in range(min(n, T)):
        y[i:] += taps[:, n - 1 - i].float() * x[: T - i]
    return torch.nn.functional.silu(y)


def state_space_scan(x, dt, decay_rate, B, C, skip):
    """x [T, H, E]; dt [T, H]; decay_rate, skip [H]; B, C [T, H, N] -> [T, H, E].  Per head a matrix S [N, E] from zero:
    S <- exp(-decay_rate dt) S + dt B x^T;  y = S^T C + skip x."""
    T, H, E = x.shape
    S = torch.zeros(H, B.shape[-1], E)
    out = torch.zeros(T, H, E)
    for t in range(T):
        S = S * torch.exp(-decay_rate * dt[t]).view(H, 1, 1) + torch.einsum("hn,he->hne", B[t] * dt[t].view(H, 1), x[t])
        out[t] = torch.einsum("hne,hn->he", S, C[t]) + skip.view(H, 1) * x[t]
    return out


def mamba2_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, E, N, G, parts = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = H * E
    p = h.float() @ w[pre + "in"].float().t()
    z, xbc, dt = p[:, :inner], p[:, inner: 2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    xbc = causal_conv_silu(xbc, w[pre + "conv"], w[pre + "conv.b"])
    x = xbc[:, :inner].view(T, H, E)
    of = torch.arange(H) // (H // G)
    B = xbc[:, inner: inner + G * N].view(T, G, N)[:, of]
    C = xbc[:, inner + G * N:].view(T, G, N)[:, of]
    dt = torch.nn.functional.softplus(dt + w[pre + "dt_bias"].float())
    y = state_space_scan(x, dt, torch.exp(w[pre + "A_log"].float()), B, C, w[pre + "D"].float()).reshape(T, inner)
    y = y * torch.nn.functional.silu(z)
    y = rms_norm(y.view(T, parts, inner // parts), None, eps).reshape(T, inner) * w[pre + "norm"].float()
    return y @ w[pre + "o"].float().t()


def dense_feed_forward(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str) -> torch.Tensor:
    h = h.float()
    a, b = h @ w[pre + "gate"].float().t(), h @ w[pre + "up"].float().t()
    return (torch.nn.functional.silu(a) * b) @ w[pre + "down"].float().t()


MIXERS = {"latent_attention": latent_attention_mixer, "attention": attention_mixer, "mamba2": mamba2_mixer}


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], streams: Optional[list] = None) -> torch.Tensor:
    """Logits [T, vocab] of one sequence; `streams` collects the stream after every layer.  A layer norms AFTER each sum:
    x <- norm1(alpha x + ls1 * mixer(shifted x)), x <- norm2(alpha x + ls2 * ff(x))."""
    eps, alpha = float(cfg["norm"]["eps"]), float(cfg["postln_alpha"])
    x = w["embed"][torch.tensor(tokens)].float() * float(cfg["embedding"]["scale"])
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        y = MIXERS[layer["type"]](token_shift(x, w[pre + "shift"]), w, pre + "mix.", layer["mixer"], eps)
        x = rms_norm(alpha * x + y * w[pre + "ls1"].float(), w[pre + "norm1"], eps)
        if layer.get("mlp") is not None:
            y = dense_feed_forward(x, w, pre + "mlp.")
            x = rms_norm(alpha * x + y * w[pre + "ls2"].float(), w[pre + "norm2"], eps)
        if streams is not None:
            streams.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].float().t()


def forward_layers(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int]):
    """(logits, the stream after every layer)."""
    streams: list = []
    return forward(cfg, w, tokens, streams), streams


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Random bf16 weights under the checkpoint's names, scaled so that every sublayer matters and nothing saturates."""
    gen = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(n_out, n_in, gain=1.0):
        return (torch.randn(n_out, n_in, generator=gen) * gain / math.sqrt(n_in)).to(torch.bfloat16)

    def vec(n, scale=0.1, shift=0.0):
        return (torch.randn(n, generator=gen) * scale + shift).to(torch.bfloat16)

    w = {"embed": torch.randn(V, W, generator=gen).to(torch.bfloat16), "final.norm": vec(W, 0.1, 1.0), "head": mat(V, W)}
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        w[pre + "norm1"] = vec(W, 0.1, 1.0)
        w[pre + "ls1"] = vec(W, 0.2, 1.0)
        w[pre + "shift"] = (torch.rand(W, generator=gen) * 0.8).to(torch.bfloat16)
        if layer["type"] == "latent_attention":
            H, D, P, E, R, Rq = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            w[pre + "mix.dq"] = mat(Rq, W)
            w[pre + "mix.dq.norm"] = vec(Rq, 0.1, 1.0)
            w[pre + "mix.uq"] = mat(H * (D + P), Rq)
            w[pre + "mix.dkv"] = mat(R + P, W)
            w[pre + "mix.dkv.norm"] = vec(R, 0.1, 1.0)
            w[pre + "mix.uk"] = mat(H * D, R)
            w[pre + "mix.uv"] = mat(H * E, R)
            w[pre + "mix.g"] = mat(H, W)
            w[pre + "mix.o"] = mat(W, H * E)
        elif layer["type"] == "attention":
            H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w[pre + "mix.q"] = mat(H * D, W)
            w[pre + "mix.k"] = mat(G * D, W)
            w[pre + "mix.v"] = mat(G * E, W)
            w[pre + "mix.q.norm"] = vec(H * D, 0.2, 1.0)
            w[pre + "mix.k.norm"] = vec(G * D, 0.2, 1.0)
            w[pre + "mix.talk"] = (torch.eye(H) + 0.4 * torch.randn(H, H, generator=gen)).to(torch.bfloat16)
            w[pre + "mix.temp"] = (0.5 + 1.5 * torch.rand(H, generator=gen)).to(torch.bfloat16)
            w[pre + "mix.o"] = mat(W, H * E)
        else:
            H, E, N, G, n = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
            C = H * E + 2 * G * N
            w[pre + "mix.in"] = mat(2 * H * E + 2 * G * N + H, W)
            w[pre + "mix.conv"] = (torch.randn(C, n, generator=gen) * 0.5).to(torch.bfloat16)
            w[pre + "mix.conv.b"] = vec(C, 0.2)
            w[pre + "mix.dt_bias"] = vec(H, 0.5, -1.0)
            w[pre + "mix.A_log"] = vec(H, 0.5, -1.0)
            w[pre + "mix.D"] = vec(H, 0.5, 1.0)
            w[pre + "mix.norm"] = vec(H * E, 0.1, 1.0)
            w[pre + "mix.o"] = mat(W, H * E)
        mlp = layer.get("mlp")
        if mlp is not None:
            w[pre + "norm2"] = vec(W, 0.1, 1.0)
            w[pre + "ls2"] = vec(W, 0.2, 1.0)
            w[pre + "mlp.gate"] = mat(mlp["ff"], W)
            w[pre + "mlp.up"] = mat(mlp["ff"], W)
            w[pre + "mlp.down"] = mat(W, mlp["ff"])
    return w
