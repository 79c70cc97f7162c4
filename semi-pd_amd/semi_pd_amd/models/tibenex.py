"""Tibenex: a decoder whose layers norm AFTER each sum, scale each sublayer's result per channel, read a token-shifted
stream in the mixer, and mix tokens by latent attention, by attention whose heads talk after the softmax, or by a
state-space recurrence; a dense gated feed-forward behind the mixer.

On an fp32 stream x (n(v) = v / sqrt(mean(v^2) + eps) * w):
    x = embed[token] * scale
    h = x + (x_prev - x) * mu                                   (x_prev: the previous token's x, zeros at position 0)
    x <- n_1(alpha x + ls_1 * mixer(h));   x <- n_2(alpha x + ls_2 * ff(x))   (a layer may have no ff);   logits = head n_f(x)
latent_attention, H heads, query [D unrotated | P rotated] per head, latent sizes Rq and R, value size E:
    q = W_uq n(W_dq h);  c = n(W_dkv h [:R]),  r = W_dkv h [R:] turned by the position: ONE pool row [c | r] per token;
    key of head h = [W_uk,h c | r], value = W_uv,h c.  Scores (q_u . W_uk,h c + q_r . r) * scale = ([W_uk,h^T q_u | q_r] .
    [c | r]) * scale: every head attends over the pool rows themselves with the query folded through W_uk, takes the
    weighted sum of latents and expands it with W_uv afterwards; causal softmax; head h times sigmoid((W_g h)_h); W_o.
    Rotation: pairs (i, i + dims / 2), frequencies stretched as in YaRN, cos and sin times its factor.
attention, H heads over G key/value heads, key size D, value size E:
    q, k normed over the whole projection (all heads at once), the first rot dims of every head turned in pairs
    (2i, 2i + 1); scores q . k * scale * temp_h; causal softmax; the heads' weights mixed, w'_h = sum_g talk[h, g] w_g, and
    applied to the values of h's own key/value head.  The sum over keys is linear, so every head's weights are applied to
    the values of all G key/value heads in one attention call (value row = the G heads side by side) and the mix is a small
    launch on the results: out_h = sum_g talk[h, g] (w_g V_c(h)).
mamba2, H heads of E values, state N per head, G groups: csrc/state_space.hip.

Launches per layer: [token shift, prompt batches and the first layer; decode batches get it from the seam in front],
GEMM(s) of the mixer's input, its preparation, attention or the recurrence, [up-projection, gate | mix], GEMM(o), seam
(norm after the sum, copy for the feed-forward), GEMM(gate | up) + silu * up, GEMM(down), seam (+ the next layer's shift
in decode batches).
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch
from torch import nn

from semi_pd_amd import ops
from semi_pd_amd.distributed import get_tensor_model_parallel_world_size
from semi_pd_amd.layers.attention_backend import RadixAttention
from semi_pd_amd.layers.basic import (LogitsProcessor, MergedColumnParallelLinear, ParallelLMHead, RowParallelLinear, SiluAndMul,
                                      VocabParallelEmbedding, dense_linear, gate_up_silu)
from semi_pd_amd.models.penozen import EXPAND_MIN_TOKENS, context_rows, stretched_frequencies


@dataclass
class RotationConfig:
    dims: int                     # leading elements of a head (or of the rotated part) that are turned
    base: float
    scaling: Optional[Dict[str, float]] = None      # {factor, original, fast, slow} or None

    @classmethod
    def from_dict(cls, rot: Optional[dict], default_dims: int, where: str) -> "RotationConfig":
        rot = rot or {}
        unknown = set(rot) - {"base", "dims", "scaling"}
        if unknown:
            raise ValueError(f"{where}: rotation keys {sorted(unknown)} are not supported")
        sc = rot.get("scaling")
        if sc is not None and set(sc) != {"factor", "original", "fast", "slow"}:
            raise ValueError(f"{where}: rotation scaling needs factor, original, fast and slow, got {sorted(sc)}")
        r = cls(int(rot.get("dims", default_dims)), float(rot.get("base", 10000.0)), {k: float(v) for k, v in sc.items()} if sc else None)
        if r.dims % 2 or r.dims < 0:
            raise ValueError(f"{where}: {r.dims} turned elements")
        return r


@dataclass
class TibenexLatentConfig:
    heads: int
    dim: int                      # unrotated query / key elements per head
    rot_dim: int                  # rotated query / key elements per head (the key part is shared by the heads)
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot: RotationConfig


@dataclass
class TibenexAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: RotationConfig


@dataclass
class TibenexStateSpaceConfig:
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int                     # taps of the short convolution


@dataclass
class TibenexLayerConfig:
    kind: str                     # "latent_attention" | "attention" | "mamba2"
    mixer: Any
    ff: int = 0                   # 0: the layer has no feed-forward


@dataclass
class TibenexConfig:
    vocab_size: int = 32000
    hidden_size: int = 1024
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    postln_alpha: float = 1.0
    layers: List[TibenexLayerConfig] = field(default_factory=list)
    architectures: tuple = ("Tibenex",)
    supports_float32 = True       # every kernel of its path is templated on the element type (ServerArgs --dtype float32)

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "TibenexConfig":
        """The checkpoint's config.json: vocab, width, norm.eps, embedding.scale, postln_alpha and one entry per layer
        (type, mixer {...}, mlp {kind: dense, ff} or null)."""
        layers = []
        for i, entry in enumerate(d["layers"]):
            kind, m = entry.get("type"), entry["mixer"]
            where = f"Tibenex layer {i}"
            if kind == "latent_attention":
                mixer: Any = TibenexLatentConfig(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                                                 kv_rank=int(m["kv_rank"]), q_rank=int(m["q_rank"]), scale=float(m["scale"]),
                                                 rot=RotationConfig.from_dict(m.get("rot"), int(m["rot_dim"]), where))
                if mixer.rot.dims > mixer.rot_dim:
                    raise ValueError(f"{where}: {mixer.rot.dims} turned elements of a rotated part of {mixer.rot_dim}")
            elif kind == "attention":
                mixer = TibenexAttentionConfig(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                                               vdim=int(m["vdim"]), scale=float(m["scale"]),
                                               rot=RotationConfig.from_dict(m.get("rot"), int(m["dim"]), where))
                if mixer.heads % mixer.kv_heads:
                    raise ValueError(f"{where}: {mixer.heads} heads over {mixer.kv_heads} key/value heads")
                if mixer.rot.dims > mixer.dim:
                    raise ValueError(f"{where}: {mixer.rot.dims} turned elements of a head of {mixer.dim}")
            elif kind == "mamba2":
                mixer = TibenexStateSpaceConfig(heads=int(m["heads"]), vdim=int(m["vdim"]), state=int(m["state"]),
                                                groups=int(m.get("groups", 1)), norm_groups=int(m.get("norm_groups", 1)),
                                                conv=int(m["conv"]))
                if mixer.heads % mixer.groups or (mixer.heads * mixer.vdim) % mixer.norm_groups or mixer.conv < 1:
                    raise ValueError(f"{where}: {mixer.heads} heads over {mixer.groups} groups, {mixer.norm_groups} norm groups, "
                                     f"{mixer.conv} taps")
            else:
                raise ValueError(f"{where}: mixer type {kind!r} is not supported (latent_attention, attention, mamba2)")
            mlp = entry.get("mlp")
            if mlp is None:
                layers.append(TibenexLayerConfig(kind, mixer))
                continue
            if mlp.get("kind") != "dense":
                raise ValueError(f"{where}: feed-forward kind {mlp.get('kind')!r} is not supported (dense only)")
            layers.append(TibenexLayerConfig(kind, mixer, ff=int(mlp["ff"])))
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                   embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)), postln_alpha=float(d.get("postln_alpha", 1.0)),
                   layers=layers)


def tibenex_uniform(vocab_size: int, hidden_size: int, pattern: str, ff: int, heads: int, kv_heads: int, dim: int, vdim: int,
                    rot_dim: int, kv_rank: int, q_rank: int, ssm_heads: int, ssm_vdim: int, state: int, groups: int,
                    norm_groups: int = 1, conv: int = 4, alpha: float = 2.0, norm_eps: float = 1e-6, latent_heads: int = 0,
                    latent_dim: int = 0, latent_vdim: int = 0) -> TibenexConfig:
    """A configuration from a pattern of layer kinds: 'l' latent attention (latent_heads / latent_dim / latent_vdim, by default
    the attention layers' sizes), 'a' attention, 'm' state space (benchmarks, tests)."""
    lh, ld, lv = latent_heads or heads, latent_dim or dim, latent_vdim or vdim
    layers = []
    for ch in pattern:
        if ch == "l":
            layers.append(TibenexLayerConfig("latent_attention", TibenexLatentConfig(
                lh, ld, rot_dim, lv, kv_rank, q_rank, (ld + rot_dim) ** -0.5, RotationConfig(rot_dim, 10000.0)), ff))
        elif ch == "a":
            layers.append(TibenexLayerConfig("attention", TibenexAttentionConfig(
                heads, kv_heads, dim, vdim, dim ** -0.5, RotationConfig(dim, 10000.0)), ff))
        else:
            layers.append(TibenexLayerConfig("mamba2", TibenexStateSpaceConfig(ssm_heads, ssm_vdim, state, groups, norm_groups, conv), ff))
    return TibenexConfig(vocab_size=vocab_size, hidden_size=hidden_size, norm_eps=norm_eps, embedding_scale=1.0, postln_alpha=alpha,
                         layers=layers)


def _portions(forward_batch):
    """(q_start, q_len) of an extend batch, (None, None) of a decode batch: how the kernels find a row's request."""
    if forward_batch.forward_mode.is_decode():
        return None, None
    return forward_batch.extend_start_loc, forward_batch.extend_seq_lens


class TibenexLatentAttention(nn.Module):
    def __init__(self, hidden_size: int, mc: TibenexLatentConfig, eps: float, region: int, dtype):
        super().__init__()
        self.mc, self.eps = mc, eps
        H, D, P, E, R = mc.heads, mc.dim, mc.rot_dim, mc.vdim, mc.kv_rank
        self.c_size = R + P
        # rows of the merged weight: the query latent, the key/value latent with the shared rotated key part, the heads' gates
        self.in_proj = MergedColumnParallelLinear(hidden_size, [mc.q_rank, self.c_size, H], params_dtype=dtype)
        self.q_norm = nn.Parameter(torch.ones(mc.q_rank, dtype=dtype), requires_grad=False)
        self.q_up = nn.Parameter(torch.empty(H * (D + P), mc.q_rank, dtype=dtype), requires_grad=False)
        self.out_proj = RowParallelLinear(H * E, hidden_size, params_dtype=dtype)
        self.latent_norm = nn.Parameter(torch.ones(R, dtype=dtype), requires_grad=False)
        self.w_uk = nn.Parameter(torch.empty(H, D, R, dtype=dtype), requires_grad=False)     # key up-projection [H * D, R] by head
        self.w_uv = nn.Parameter(torch.empty(H, E, R, dtype=dtype), requires_grad=False)     # value up-projection [H * E, R] by head
        freq, self.mscale = stretched_frequencies(mc.rot.dims, mc.rot.base, mc.rot.scaling) if mc.rot.dims else (torch.zeros(0), 1.0)
        self.register_buffer("freq", freq, persistent=False)
        # the pool row [latent | rotated key part] is the one key/value head of every query head; its first R elements the value
        self.attn = RadixAttention(H, R + P, mc.scale, 1, region, v_head_dim=R)
        # prompt batches: keys [W_uk,h c | r] of all heads from the latent rows in one GEMM, W = [[W_uk,h, 0], [0, I]] per head
        self.register_buffer("w_key_rows", torch.empty(0, dtype=dtype), persistent=False)
        self.register_buffer("w_val_rows", torch.empty(0, dtype=dtype), persistent=False)     # [W_uv | 0]: values from the same rows

    def post_load_weights(self):
        mc = self.mc
        H, D, P, R = mc.heads, mc.dim, mc.rot_dim, mc.kv_rank
        w = torch.zeros(H, D + P, R + P, dtype=self.w_uk.dtype, device=self.w_uk.device)
        w[:, :D, :R] = self.w_uk
        w[:, D:, R:] = torch.eye(P, dtype=w.dtype, device=w.device)
        self.w_key_rows = w.view(H * (D + P), R + P)
        wv = torch.zeros(H * mc.vdim, R + P, dtype=self.w_uv.dtype, device=self.w_uv.device)
        wv[:, :R] = self.w_uv.view(H * mc.vdim, R)
        self.w_val_rows = wv

    def expands_keys(self, forward_batch) -> bool:
        """Whether a batch expands the keys and values of its requests' tokens from the latent rows and attends head by head
        (fewer multiply-adds per query-key pair: D + P + E against 2 R + P) instead of attending over the latent rows: prompt
        batches whose context is not much longer than their new tokens.  SEMIPD_LATENT_EXPAND: 0 never, 2 every extend batch."""
        knob = os.environ.get("SEMIPD_LATENT_EXPAND", "1")
        if knob == "0" or not forward_batch.forward_mode.is_extend() or self.w_key_rows.numel() == 0:
            return False
        new = forward_batch.extend_num_tokens
        ctx = new + sum(forward_batch.extend_prefix_lens_cpu)
        return knob == "2" or (new >= EXPAND_MIN_TOKENS and ctx <= 4 * new)

    def _forward_expanded(self, p: torch.Tensor, q: torch.Tensor, forward_batch) -> torch.Tensor:
        mc = self.mc
        H, D, P, E, R = mc.heads, mc.dim, mc.rot_dim, mc.vdim, mc.kv_rank
        T = p.shape[0]
        pool = forward_batch.token_to_kv_pool.get_key_buffer(self.attn.layer_id)
        pool = pool.view(pool.shape[0], -1)
        ops.latent_prep(q, p[:, mc.q_rank: mc.q_rank + self.c_size], H, D, P, R, self.latent_norm, self.eps, forward_batch.positions,
                        self.freq if mc.rot.dims else None, mc.rot.dims, self.mscale, pool, forward_batch.out_cache_loc, halves=True)
        slots, table, rows = context_rows(forward_batch)
        ctx = ops.gather_rows(pool, slots)                                    # [N, R + P]: every request's tokens, in order
        keys = dense_linear(ctx, self.w_key_rows)                             # [N, H * (D + P)]
        vals = dense_linear(ctx, self.w_val_rows)                             # [N, H * E]
        out = torch.empty((T, H * E), dtype=p.dtype, device=p.device)
        ops.local_attention_fwd(q, out, keys.view(-1, H, D + P), vals.view(-1, H, E), table, rows, forward_batch.seq_lens,
                                forward_batch.extend_start_loc, forward_batch.extend_seq_lens, max(forward_batch.extend_seq_lens_cpu),
                                mc.scale, 0.0, 0, None, None, form=int(os.environ.get("SEMIPD_LOCAL_ATTN_FORM", "0")))
        return self.out_proj(ops.sigmoid_gate_heads_(out, p[:, mc.q_rank + self.c_size:]))

    def forward(self, h: torch.Tensor, forward_batch) -> torch.Tensor:
        mc = self.mc
        H, D, P, E, R = mc.heads, mc.dim, mc.rot_dim, mc.vdim, mc.kv_rank
        T = h.shape[0]
        p = self.in_proj(h)
        cq = ops.rmsnorm(p[:, : mc.q_rank], self.q_norm, self.eps)
        q = dense_linear(cq, self.q_up)                                            # [T, H * (D + P)]
        if self.expands_keys(forward_batch):
            return self._forward_expanded(p, q, forward_batch)
        pool = forward_batch.token_to_kv_pool.get_key_buffer(self.attn.layer_id)
        q_in = torch.empty((T, H * (R + P)), dtype=p.dtype, device=p.device)
        ops.latent_prep(q, p[:, mc.q_rank: mc.q_rank + self.c_size], H, D, P, R, self.latent_norm, self.eps, forward_batch.positions,
                        self.freq if mc.rot.dims else None, mc.rot.dims, self.mscale, pool.view(pool.shape[0], -1),
                        forward_batch.out_cache_loc, q_in, halves=True)
        # the unrotated query part through the key up-projection, head by head: [H, T, D] x [H, D, R] -> q_in[:, h, :R]
        q_u = q.view(T, H, D + P)[..., :D]
        torch.bmm(q_u.transpose(0, 1), self.w_uk, out=q_in.view(T, H, R + P)[..., :R].transpose(0, 1))
        o_lat = forward_batch.attn_backend.forward_latent(q_in, self.attn, forward_batch, sink=None)
        # the weighted sums of latents through the value up-projection: [H, T, R] x [H, R, E]
        o = torch.empty((T, H, E), dtype=p.dtype, device=p.device)
        torch.bmm(o_lat.view(T, H, R).transpose(0, 1), self.w_uv.transpose(1, 2), out=o.transpose(0, 1))
        o = ops.sigmoid_gate_heads_(o.view(T, H * E), p[:, mc.q_rank + self.c_size:])
        return self.out_proj(o)


class TibenexTalkingAttention(nn.Module):
    def __init__(self, hidden_size: int, mc: TibenexAttentionConfig, eps: float, region: int, dtype):
        super().__init__()
        self.mc, self.eps = mc, eps
        H, G, D, E = mc.heads, mc.kv_heads, mc.dim, mc.vdim
        self.k_off, self.v_off = H * D, (H + G) * D
        self.in_proj = MergedColumnParallelLinear(hidden_size, [H * D, G * D, G * E], params_dtype=dtype)
        self.out_proj = RowParallelLinear(H * E, hidden_size, params_dtype=dtype)
        self.q_norm = nn.Parameter(torch.ones(H * D, dtype=dtype), requires_grad=False)
        self.k_norm = nn.Parameter(torch.ones(G * D, dtype=dtype), requires_grad=False)
        self.talk = nn.Parameter(torch.eye(H, dtype=torch.float32), requires_grad=False)
        self.temp = nn.Parameter(torch.ones(H, dtype=torch.float32), requires_grad=False)
        freq, self.mscale = stretched_frequencies(mc.rot.dims, mc.rot.base, mc.rot.scaling) if mc.rot.dims else (torch.zeros(0), 1.0)
        self.register_buffer("freq", freq, persistent=False)
        self.attn = RadixAttention(H, D, mc.scale, G, region, v_head_dim=E)

    def forward(self, h: torch.Tensor, forward_batch) -> torch.Tensor:
        mc = self.mc
        H, G, D, E = mc.heads, mc.kv_heads, mc.dim, mc.vdim
        p = self.in_proj(h)
        k_buf, v_buf = forward_batch.token_to_kv_pool.get_kv_buffer(self.attn.layer_id)
        ops.qk_norm_rope_kv_store(p, H, G, D, E, self.k_off, self.v_off, self.q_norm, self.k_norm, self.eps, forward_batch.positions,
                                  self.freq if mc.rot.dims else None, mc.rot.dims, False, self.mscale, self.temp, k_buf, v_buf,
                                  forward_batch.out_cache_loc)
        parts = forward_batch.attn_backend.forward_shared_values(p[:, : H * D], self.attn, forward_batch)     # [T, H * G * E]
        return self.out_proj(ops.talk_mix(parts, self.talk, G))


class TibenexStateSpace(nn.Module):
    def __init__(self, hidden_size: int, mc: TibenexStateSpaceConfig, eps: float, state_ids, dtype):
        super().__init__()
        self.mc, self.eps = mc, eps
        self.state_id, self.conv_id = state_ids
        inner, gn = mc.heads * mc.vdim, mc.groups * mc.state
        self.channels = inner + 2 * gn
        # z | x | B | C | dt, the order of the checkpoint's rows
        self.in_proj = MergedColumnParallelLinear(hidden_size, [inner, inner, gn, gn, mc.heads], params_dtype=dtype)
        self.out_proj = RowParallelLinear(inner, hidden_size, params_dtype=dtype)
        self.conv = nn.Parameter(torch.empty(self.channels, mc.conv, dtype=dtype), requires_grad=False)
        self.conv_bias = nn.Parameter(torch.zeros(self.channels, dtype=dtype), requires_grad=False)
        self.a_log = nn.Parameter(torch.zeros(mc.heads, dtype=torch.float32), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(mc.heads, dtype=torch.float32), requires_grad=False)
        self.d_skip = nn.Parameter(torch.ones(mc.heads, dtype=torch.float32), requires_grad=False)
        self.out_norm = nn.Parameter(torch.ones(inner, dtype=dtype), requires_grad=False)

    @staticmethod
    def state_widths(mc: TibenexStateSpaceConfig):
        """(the matrices S of all heads, the last taps - 1 inputs of all convolution channels) in fp32 elements."""
        return mc.heads * mc.state * mc.vdim, (mc.conv - 1) * (mc.heads * mc.vdim + 2 * mc.groups * mc.state)

    def forward(self, h: torch.Tensor, forward_batch) -> torch.Tensor:
        mc = self.mc
        inner = mc.heads * mc.vdim
        p = self.in_proj(h)
        q_start, q_len = _portions(forward_batch)
        sp = forward_batch.state_pool
        o = ops.state_space(p, 0, inner, inner + self.channels, self.conv, self.conv_bias, self.dt_bias, self.a_log, self.d_skip,
                            self.out_norm, mc.norm_groups, self.eps, sp.get_state_buffer(self.state_id),
                            sp.get_state_buffer(self.conv_id) if mc.conv > 1 else None, forward_batch.state_indices,
                            forward_batch.seq_lens, q_start, q_len, mc.heads, mc.groups, mc.state, mc.vdim)
        return self.out_proj(o)


class TibenexMLP(nn.Module):
    def __init__(self, hidden_size: int, ff: int, dtype):
        super().__init__()
        self.gate_up_proj = MergedColumnParallelLinear(hidden_size, [ff, ff], params_dtype=dtype)
        self.down_proj = RowParallelLinear(ff, hidden_size, params_dtype=dtype)
        self.act_fn = SiluAndMul(any_width=True)

    def forward(self, x):
        return self.down_proj(gate_up_silu(x, self.gate_up_proj, self.act_fn))


class PostNorm(nn.Module):
    """The joint behind a sublayer of a block that norms after the sum, on an fp32 stream (csrc/layernorm.hip:
    semipd_postnorm_stream): stream <- rms_norm(alpha * stream + layer_scale * y) * weight."""

    def __init__(self, hidden_size: int, eps: float, alpha: float, dtype=None):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(hidden_size, dtype=dtype), requires_grad=False)
        self.layer_scale = nn.Parameter(torch.ones(hidden_size, dtype=dtype), requires_grad=False)
        self.eps, self.alpha = float(eps), float(alpha)

    def forward(self, y: torch.Tensor, stream: torch.Tensor, want_out: bool = True, shift: Optional["TokenShift"] = None,
                forward_batch=None) -> Optional[torch.Tensor]:
        """Returns the new stream in the activation type, with `shift` (one row per request) the next mixer's shifted input."""
        if shift is None:
            return ops.postnorm_stream(y, self.layer_scale, stream, self.alpha, self.weight, self.eps, want_out=want_out)
        return ops.postnorm_stream(y, self.layer_scale, stream, self.alpha, self.weight, self.eps, shift_mu=shift.mu,
                                   prev=forward_batch.state_pool.get_state_buffer(shift.state_id),
                                   state_indices=forward_batch.state_indices, seq_lens=forward_batch.seq_lens)


class TokenShift(nn.Module):
    """What a mixer reads: s_t + (s_(t-1) - s_t) * mu over the fp32 stream; the previous token's stream is a column range of
    the request's state row (csrc/layernorm.hip: semipd_token_shift)."""

    def __init__(self, hidden_size: int, state_id: int, dtype=None):
        super().__init__()
        self.mu = nn.Parameter(torch.zeros(hidden_size, dtype=dtype), requires_grad=False)
        self.state_id = state_id

    def forward(self, stream: torch.Tensor, forward_batch) -> torch.Tensor:
        q_start, q_len = _portions(forward_batch)
        return ops.token_shift(stream, self.mu, forward_batch.state_pool.get_state_buffer(self.state_id), forward_batch.state_indices,
                               forward_batch.seq_lens, q_start, q_len)


class TibenexDecoderLayer(nn.Module):
    def __init__(self, config: TibenexConfig, layer_id: int, region: Optional[int], shift_id: int, state_ids, dtype):
        super().__init__()
        lc = config.layers[layer_id]
        W = config.hidden_size
        if lc.kind == "latent_attention":
            self.mix = TibenexLatentAttention(W, lc.mixer, config.norm_eps, region, dtype)
        elif lc.kind == "attention":
            self.mix = TibenexTalkingAttention(W, lc.mixer, config.norm_eps, region, dtype)
        else:
            self.mix = TibenexStateSpace(W, lc.mixer, config.norm_eps, state_ids, dtype)
        self.shift = TokenShift(W, shift_id, dtype)
        self.norm1 = PostNorm(W, config.norm_eps, config.postln_alpha, dtype)
        self.mlp = TibenexMLP(W, lc.ff, dtype) if lc.ff else None
        self.norm2 = PostNorm(W, config.norm_eps, config.postln_alpha, dtype) if lc.ff else None

    def forward(self, x: torch.Tensor, h: torch.Tensor, forward_batch, next_shift: Optional[TokenShift]) -> Optional[torch.Tensor]:
        """x: the fp32 stream (updated in place); h: the shifted stream in the activation type.  Returns the next layer's
        shifted input when `next_shift` is given (decode batches: it comes out of the last seam), else None."""
        y = self.mix(h, forward_batch)
        if self.mlp is None:
            return self.norm1(y, x, want_out=next_shift is not None, shift=next_shift, forward_batch=forward_batch)
        y = self.mlp(self.norm1(y, x))
        return self.norm2(y, x, want_out=next_shift is not None, shift=next_shift, forward_batch=forward_batch)


class TibenexForCausalLM(nn.Module):
    def __init__(self, config: TibenexConfig, dtype=torch.bfloat16):
        super().__init__()
        if get_tensor_model_parallel_world_size() != 1:
            raise ValueError("Tibenex runs on one GPU per replica (tensor parallelism over its per-layer head counts and its "
                             "recurrent state is not implemented)")
        if not config.layers:
            raise ValueError("Tibenex: the configuration lists no layers")
        self.config = config
        W = config.hidden_size
        self.embed = VocabParallelEmbedding(config.vocab_size, W, params_dtype=dtype)
        # pool regions: one per attention layer of either kind; state columns: per layer the previous token's stream, and for
        # a state-space layer the matrices S and the convolution's last inputs
        self._regions: List[Any] = []
        self._state_widths: List[int] = []
        layers = []
        for i, lc in enumerate(config.layers):
            shift_id = len(self._state_widths)
            self._state_widths.append(W)
            region, ids = None, None
            if lc.kind == "mamba2":
                s_w, c_w = TibenexStateSpace.state_widths(lc.mixer)
                ids = (len(self._state_widths), len(self._state_widths) + 1)
                self._state_widths += [s_w, max(c_w, 1)]
            else:
                region = len(self._regions)
                self._regions.append(lc.mixer)
            layers.append(TibenexDecoderLayer(config, i, region, shift_id, ids, dtype))
        self.layers = nn.ModuleList(layers)
        self.final_norm_weight = nn.Parameter(torch.ones(W, dtype=dtype), requires_grad=False)
        self.head = ParallelLMHead(config.vocab_size, W, params_dtype=dtype)
        self.logits_processor = LogitsProcessor(config.vocab_size)
        self.layer_probe = None      # tests: a callable (layer index, fp32 stream) run after every layer
        # SEMIPD_TIBENEX_FUSED_SHIFT=0: decode batches take the separate token-shift launch too
        self.fused_shift = os.environ.get("SEMIPD_TIBENEX_FUSED_SHIFT", "1") != "0"
        for p in self.parameters():
            p.requires_grad_(False)

    def post_load_weights(self):
        for layer in self.layers:
            if isinstance(layer.mix, TibenexLatentAttention):
                layer.mix.post_load_weights()

    @property
    def kv_geometry(self):
        """A latent-attention layer keeps one row [latent | shared rotated key part] per token whose first kv_rank elements
        are the values; an attention layer keeps G key heads and G value heads (a model without such layers keeps one
        token-sized dummy region)."""
        ms = self._regions
        if not ms:
            return dict(kind="mha", num_kv_heads=[1], head_dim=[8], v_head_dim=[8], num_heads=[1], num_layers=1, values_in_keys=[True])
        latent = [isinstance(m, TibenexLatentConfig) for m in ms]
        return dict(kind="mha", num_kv_heads=[1 if f else m.kv_heads for m, f in zip(ms, latent)],
                    head_dim=[m.kv_rank + m.rot_dim if f else m.dim for m, f in zip(ms, latent)],
                    v_head_dim=[m.kv_rank if f else m.vdim for m, f in zip(ms, latent)],
                    num_heads=[m.heads for m in ms], num_layers=len(ms), values_in_keys=latent)

    @property
    def state_geometry(self) -> List[int]:
        """Columns of a request's state row: per layer the previous token's stream [width], and for a state-space layer the
        matrices S and the convolution's last inputs."""
        return list(self._state_widths)

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch):
        x = ops.embed_stream(input_ids, self.embed.weight, self.config.embedding_scale)
        fused = self.fused_shift and forward_batch.forward_mode.is_decode()
        n = len(self.layers)
        h = None
        for i, layer in enumerate(self.layers):
            if h is None:
                h = layer.shift(x, forward_batch)
            h = layer(x, h, forward_batch, self.layers[i + 1].shift if (fused and i + 1 < n) else None)
            if self.layer_probe is not None:
                self.layer_probe(i, x)
        h = ops.rms_stream(None, x, self.final_norm_weight, self.config.norm_eps)
        return self.logits_processor(input_ids, h, self.head, forward_batch)
