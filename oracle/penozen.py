"""Plain CPU statement of the Penozen decoder (TEST INFRASTRUCTURE ONLY, like oracle/model.py).

One function per mechanism, fp32 torch on the host, no cache, no state pool and no batching: a sequence is always
recomputed whole, keys and values are expanded from the latent for every head, and the delta rule is a Python loop over
the tokens, so nothing here can share a fault with the engine's pools, kernels or scheduler.  Weights arrive as a dict
of tensors under the checkpoint's own names (`embed`, `bigram`, `l<i>.norm1`, `l<i>.mix.q`, `l<i>.mix.q.conv`,
`l<i>.mlp.e<j>.gate`, ..., `final.norm`, `head`); the configuration is the checkpoint's config.json as a dict.

Notation: T tokens, W the model width, H heads, G key heads of the delta rule, D the key size, E the value size, P the
rotated size, R the latent size, X experts of which each token takes K.
"""
from __future__ import annotations

import math
from typing import Dict, List

import torch


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float, around_zero: bool) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) times the weight; a weight stored around zero stands for 1 + weight."""
    x = x.float()
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y * (weight.float() + 1.0 if around_zero else weight.float())


def embed_tokens(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int]) -> torch.Tensor:
    """embed[token] * scale + bigram[hash(previous token, token)]; the first token of a sequence takes the table's last row."""
    e, bg = cfg["embedding"], cfg["embedding"]["bigram"]
    rows = []
    for t, tok in enumerate(tokens):
        r = bg["buckets"] if t == 0 else (tokens[t - 1] * bg["mul_prev"] + tok * bg["mul_cur"]) % bg["buckets"]
        rows.append(w["embed"][tok].float() * e["scale"] + w["bigram"][r].float())
    return torch.stack(rows)


def yarn_frequencies(rot: dict):
    """(frequency of every pair, the factor on cos and sin) of a rotation over rot['dims'] elements with the stretched
    low frequencies of YaRN."""
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


def rotate_pairs(x: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, heads, P]: the first rot['dims'] elements are neighbouring pairs (2i, 2i + 1) turned by position * frequency_i."""
    T, dims = x.shape[0], int(rot["dims"])
    f, m = yarn_frequencies(rot)
    ang = (torch.arange(T, dtype=torch.float32).view(T, 1) * f.float().view(1, -1))
    c, s = (torch.cos(ang) * m).view(T, 1, -1), (torch.sin(ang) * m).view(T, 1, -1)
    x = x.float().clone()
    a, b = x[..., 0:dims:2].clone(), x[..., 1:dims:2].clone()
    x[..., 0:dims:2] = a * c - b * s
    x[..., 1:dims:2] = b * c + a * s
    return x


def sink_softmax(scores: torch.Tensor, sink: torch.Tensor) -> torch.Tensor:
    """scores [H, Tq, Tk], the queries being the LAST Tq positions of the Tk keys' sequence: causal softmax over the keys whose
    denominator also holds exp(sink) of the head (a term without key or value, counted once)."""
    H, Tq, Tk = scores.shape
    qpos = torch.arange(Tk - Tq, Tk).view(1, Tq, 1)
    s = scores.float().masked_fill(torch.arange(Tk).view(1, 1, Tk) > qpos, float("-inf"))
    sink = sink.float().view(H, 1, 1)
    top = torch.maximum(s.max(-1, keepdim=True).values, sink)
    p = torch.exp(s - top)
    return p / (p.sum(-1, keepdim=True) + torch.exp(sink - top))


def latent_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, P, E, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    h = h.float()
    q = (h @ w[pre + "q"].float().t()).view(T, H, D + P)
    down = h @ w[pre + "dkv"].float().t()
    c = rms_norm(down[:, :R], w[pre + "dkv.norm"], eps, around_zero=False)
    k_rot = rotate_pairs(down[:, R:].view(T, 1, P), m["rot"])
    q_rot = rotate_pairs(q[..., D:], m["rot"])
    k = (c @ w[pre + "uk"].float().t()).view(T, H, D)
    v = (c @ w[pre + "uv"].float().t()).view(T, H, E)
    s = (torch.einsum("ihd,jhd->hij", q[..., :D], k) + torch.einsum("ihd,jd->hij", q_rot, k_rot[:, 0])) * m["scale"]
    o = sink_softmax(s, w[pre + "sink"]) @ v.transpose(0, 1)         # [H, T, T] x [H, T, E]
    o = o.transpose(0, 1).reshape(T, H * E)
    o = o * torch.sigmoid(h @ w[pre + "g"].float().t())
    return o @ w[pre + "o"].float().t()


def short_conv_silu(x: torch.Tensor, taps: torch.Tensor) -> torch.Tensor:
    """x [T, C], taps [C, n]: y_t = sum_i taps[:, n - 1 - i] * x_(t - i), zeros in front of the sequence; then silu."""
    T, n = x.shape[0], taps.shape[1]
    y = torch.zeros_like(x)
    for i in range(n):
        y[i:] += taps[:, n - 1 - i].float() * x[: T - i] if i else taps[:, n - 1].float() * x
    return torch.nn.functional.silu(y)


def delta_rule(q, k, v, beta, g):
    """q, k [T, H, D]; v [T, H, E]; beta, g [T, H] -> [T, H, E].  Per head, a matrix S [D, E] from zero:
    S <- g S;  S <- S + k (beta (v - S^T k))^T;  out = S^T q."""
    T, H, D = q.shape
    E = v.shape[-1]
    S = torch.zeros(H, D, E)
    out = torch.zeros(T, H, E)
    for t in range(T):
        S = S * g[t].view(H, 1, 1)
        u = beta[t].view(H, 1) * (v[t] - torch.einsum("hde,hd->he", S, k[t]))
        S = S + torch.einsum("hd,he->hde", k[t], u)
        out[t] = torch.einsum("hde,hd->he", S, q[t])
    return out


def delta_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, G, D, E = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    h = h.float()
    q = short_conv_silu(h @ w[pre + "q"].float().t(), w[pre + "q.conv"]).view(T, G, D)
    k = short_conv_silu(h @ w[pre + "k"].float().t(), w[pre + "k.conv"]).view(T, G, D)
    v = short_conv_silu(h @ w[pre + "v"].float().t(), w[pre + "v.conv"]).view(T, H, E)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    q, k = q.repeat_interleave(H // G, 1), k.repeat_interleave(H // G, 1)
    beta = torch.sigmoid(h @ w[pre + "b"].float().t())
    g = torch.exp(-torch.exp(w[pre + "A_log"].float()) * torch.nn.functional.softplus(h @ w[pre + "a"].float().t()
                                                                                    + w[pre + "dt_bias"].float()))
    o = delta_rule(q, k, v, beta, g)
    o = rms_norm(o, w[pre + "norm"], eps, around_zero=False)
    o = o.reshape(T, H * E) * torch.nn.functional.silu(h @ w[pre + "g"].float().t())
    return o @ w[pre + "o"].float().t()


def router_margin(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, mlp: dict) -> torch.Tensor:
    """Per token, the gap between the smallest router logit that is chosen and the largest that is not (infinite when every
    expert is chosen): a comparison in reduced precision may only be held against positions where this is not small."""
    X, K = mlp["router"]["experts"], mlp["router"]["top"]
    z = (h.float() @ w[pre + "router"].float().t()).sort(-1, descending=True).values
    return z[:, K - 1] - z[:, K] if K < X else torch.full((h.shape[0],), float("inf"))


def expert_mixture(h: torch.Tensor, w: Dict[str, torch.Tensor], pre: str, mlp: dict) -> torch.Tensor:
    """Sigmoid scores of all experts, the K largest kept and divided by their sum; expert = down(act(gate, up)) with
    act(a, b) = a' sigmoid(1.702 a') (b' + 1), a' = min(a, limit), b' = clamp(b, -limit, limit)."""
    X, K, limit = mlp["router"]["experts"], mlp["router"]["top"], float(mlp["expert"]["limit"])
    h = h.float()
    s = torch.sigmoid(h @ w[pre + "router"].float().t())
    top_s, top_i = torch.topk(s, K, dim=-1)
    top_s = top_s / (top_s.sum(-1, keepdim=True) + 1e-20)
    out = torch.zeros(h.shape[0], w[pre + "e0.down"].shape[0])
    for e in range(X):
        a = torch.clamp(h @ w[pre + f"e{e}.gate"].float().t(), max=limit)
        b = torch.clamp(h @ w[pre + f"e{e}.up"].float().t(), -limit, limit)
        y = (a * torch.sigmoid(1.702 * a) * (b + 1)) @ w[pre + f"e{e}.down"].float().t()
        weight = (top_s * (top_i == e)).sum(-1, keepdim=True)
        out += weight * y
    return out


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], return_layers: bool = False, margins: list = None):
    """Logits [T, vocab] of one sequence (and the stream after every layer).  `margins`, a list, receives the router margin
    [T] of every layer with experts."""
    eps = float(cfg["norm"]["eps"])
    x = embed_tokens(cfg, w, tokens)
    layers = []
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        hn = rms_norm(x, w[pre + "norm1"], eps, around_zero=True)
        if layer["type"] == "latent_attention":
            x = x + latent_attention_mixer(hn, w, pre + "mix.", layer["mixer"], eps)
        elif layer["type"] == "delta":
            x = x + delta_mixer(hn, w, pre + "mix.", layer["mixer"], eps)
        else:
            raise ValueError(f"layer {i}: mixer type {layer['type']!r}")
        if layer.get("mlp") is not None:
            hn = rms_norm(x, w[pre + "norm2"], eps, around_zero=True)
            if margins is not None:
                margins.append(router_margin(hn, w, pre + "mlp.", layer["mlp"]))
            x = x + expert_mixture(hn, w, pre + "mlp.", layer["mlp"])
        layers.append(x.clone())
    hn = rms_norm(x, w["final.norm"], eps, around_zero=True)
    logits = hn @ w["head"].float().t()
    cap = float(cfg.get("logit_softcap") or 0.0)
    if cap > 0:
        logits = cap * torch.tanh(logits / cap)
    return (logits, layers) if return_layers else logits


def random_weights(cfg: dict, seed: int = 0) -> Dict[str, torch.Tensor]:
    """Random bf16 weights under the checkpoint's names, scaled so that every sublayer matters and nothing saturates."""
    gen = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def mat(n_out, n_in, gain=1.0):
        return (torch.randn(n_out, n_in, generator=gen) * gain / math.sqrt(n_in)).to(torch.bfloat16)

    def vec(n, scale=0.1, shift=0.0):
        return (torch.randn(n, generator=gen) * scale + shift).to(torch.bfloat16)

    w = {"embed": (torch.randn(V, W, generator=gen) / cfg["embedding"]["scale"]).to(torch.bfloat16),
         "bigram": (torch.randn(cfg["embedding"]["bigram"]["buckets"] + 1, W, generator=gen) * 0.5).to(torch.bfloat16),
         "final.norm": vec(W), "head": mat(V, W)}
    for i, layer in enumerate(cfg["layers"]):
        pre, m = f"l{i}.", layer["mixer"]
        w[pre + "norm1"] = vec(W)
        if layer["type"] == "latent_attention":
            H, D, P, E, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            w[pre + "mix.q"] = mat(H * (D + P), W, 2.0)
            w[pre + "mix.dkv"] = mat(R + P, W, 2.0)
            w[pre + "mix.dkv.norm"] = vec(R, 0.1, 1.0)
            w[pre + "mix.uk"] = mat(H * D, R, 2.0)
            w[pre + "mix.uv"] = mat(H * E, R)
            w[pre + "mix.sink"] = vec(H, 1.0)
            w[pre + "mix.g"] = mat(H * E, W)
            w[pre + "mix.o"] = mat(W, H * E)
        else:
            H, G, D, E, n = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            for name, rows in (("q", G * D), ("k", G * D), ("v", H * E)):
                w[pre + "mix." + name] = mat(rows, W, 2.0)
                w[pre + f"mix.{name}.conv"] = (torch.randn(rows, n, generator=gen) * 0.5).to(torch.bfloat16)
            w[pre + "mix.b"] = mat(H, W)
            w[pre + "mix.a"] = mat(H, W)
            w[pre + "mix.A_log"] = vec(H, 0.5, -1.0)
            w[pre + "mix.dt_bias"] = vec(H, 0.5, -1.0)
            w[pre + "mix.norm"] = vec(E, 0.1, 1.0)
            w[pre + "mix.g"] = mat(H * E, W)
            w[pre + "mix.o"] = mat(W, H * E, 2.0)
        mlp = layer.get("mlp")
        if mlp is not None:
            w[pre + "norm2"] = vec(W)
            w[pre + "mlp.router"] = mat(mlp["router"]["experts"], W, 4.0)
            for e in range(mlp["router"]["experts"]):
                w[pre + f"mlp.e{e}.gate"] = mat(mlp["expert"]["ff"], W, 2.0)
                w[pre + f"mlp.e{e}.up"] = mat(mlp["expert"]["ff"], W, 2.0)
                w[pre + f"mlp.e{e}.down"] = mat(W, mlp["expert"]["ff"])
    return w
