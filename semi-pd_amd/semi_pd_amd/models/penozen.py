"""Penozen: a pre-norm decoder whose layers mix tokens either by latent attention or by a gated delta rule, with a mixture
of clamped gated experts behind the mixer, a hashed bigram table beside the token embedding and soft-capped logits.

On an fp32 residual stream x, n(v) = v / sqrt(mean(v^2) + eps) * (1 + w):
    x = embed[token] * scale + bigram[(previous token * a + token * b) mod buckets]     (the table's last row at position 0)
    x <- x + mixer(n_1(x));   x <- x + experts(n_2(x))   (a layer may have no experts);   logits = cap * tanh(head n_f(x) / cap)
latent_attention, H heads, query [D unrotated | P rotated] per head, latent size R, value size E:
    c = rms_norm(W_dkv h [:R]) (plain weight), r = W_dkv h [R:] turned by the position: ONE pool row [c | r] per token;
    key of head h = [W_uk,h c | r], value = W_uv,h c.  Scores (q_u . W_uk,h c + q_r . r) * scale = ([W_uk,h^T q_u | q_r] . [c | r])
    * scale, so every head attends over the pool rows themselves with the query folded through W_uk, takes the weighted sum of
    latents and expands it with W_uv afterwards; softmax over the causal keys with exp(sink_h) in the denominator; the heads
    times sigmoid(W_g h); W_o.  Rotation: neighbouring pairs, frequencies stretched as in YaRN, cos and sin times its factor.
delta, H heads over G query/key heads of size D, values of size E:
    q, k, v through a short causal convolution per channel and silu; q, k to unit length (q times D^-1/2);
    beta = sigmoid(W_b h), g = exp(-exp(A_log) softplus(W_a h + dt_bias));
    S <- g S;  S <- S + k (beta (v - S^T k))^T;  o = S^T q   per head, S [D, E] fp32 in the request's state row together
    with the last taps - 1 inputs of the convolutions; o / rms(o) * weight * silu(W_g h); W_o.
experts: sigmoid of the router logits (fp32), the top-k kept and divided by their sum, expert = down(a sigmoid(1.702 a) (b + 1)),
    a = min(gate h, limit), b = clamp(up h, -limit, limit).

Launches per layer: GEMM(q | dkv | g) or GEMM(q | k | v | g | a | b), the mixer's preparation (norm of the latent, rotation,
pool store / convolution, unit norms, gates), [q_u x W_uk], attention or the recurrence, [x W_uv, gate], GEMM(o), seam (stream
+= y; next input = norm(stream)), router (fp32), top-k, expert GEMMs + activation + sum, seam.
"""
from __future__ import annotations

import math
import os
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

import torch
from torch import nn

from semi_pd_amd import ops
from semi_pd_amd.distributed import get_tensor_model_parallel_world_size
from semi_pd_amd.layers.attention_backend import RadixAttention
from semi_pd_amd.layers.basic import (BigramEmbedding, LogitsProcessor, MergedColumnParallelLinear, ParallelLMHead,
                                      RowParallelLinear, StreamRMSNorm, dense_linear)
from semi_pd_amd.layers.moe import ClampedGatedMoE


@dataclass
class LatentAttentionConfig:
    heads: int
    dim: int                      # unrotated query / key elements per head
    rot_dim: int                  # rotated query / key elements per head (the key part is shared by the heads)
    vdim: int
    kv_rank: int
    scale: float
    rot_dims: int                 # leading elements of the rotated part that are turned
    rot_base: float
    rot_scaling: Optional[Dict[str, float]] = None      # {factor, original, fast, slow} or None


@dataclass
class DeltaConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int                     # taps of the short convolutions


@dataclass
class PenozenLayerConfig:
    kind: str                     # "latent_attention" | "delta"
    mixer: Any
    experts: int = 0              # 0: the layer has no feed-forward
    top: int = 0
    ff: int = 0
    limit: float = 0.0


@dataclass
class PenozenConfig:
    vocab_size: int = 32000
    hidden_size: int = 1024
    norm_eps: float = 1e-5
    embedding_scale: float = 1.0
    bigram_buckets: int = 1
    bigram_mul_prev: int = 1
    bigram_mul_cur: int = 1
    logit_softcap: float = 0.0
    layers: List[PenozenLayerConfig] = field(default_factory=list)
    architectures: tuple = ("Penozen",)
    supports_float32 = True       # every kernel of its path is templated on the element type (ServerArgs --dtype float32)

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "PenozenConfig":
        """The checkpoint's config.json: vocab, width, norm.eps, embedding {scale, bigram {buckets, mul_prev, mul_cur}},
        logit_softcap and one entry per layer (type, mixer {...}, mlp {kind, expert {ff, limit}, router {experts, top}} or null)."""
        layers = []
        for i, entry in enumerate(d["layers"]):
            kind, m = entry.get("type"), entry["mixer"]
            if kind == "latent_attention":
                rot = m.get("rot") or {}
                unknown = set(rot) - {"base", "dims", "scaling"}
                if unknown:
                    raise ValueError(f"Penozen layer {i}: rotation keys {sorted(unknown)} are not supported")
                sc = rot.get("scaling")
                if sc is not None and set(sc) != {"factor", "original", "fast", "slow"}:
                    raise ValueError(f"Penozen layer {i}: rotation scaling needs factor, original, fast and slow, got {sorted(sc)}")
                mixer = LatentAttentionConfig(heads=int(m["heads"]), dim=int(m["dim"]), rot_dim=int(m["rot_dim"]), vdim=int(m["vdim"]),
                                              kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                                              rot_dims=int(rot.get("dims", m["rot_dim"])), rot_base=float(rot.get("base", 10000.0)),
                                              rot_scaling={k: float(v) for k, v in sc.items()} if sc else None)
                if mixer.rot_dims % 2 or mixer.rot_dims > mixer.rot_dim:
                    raise ValueError(f"Penozen layer {i}: {mixer.rot_dims} turned elements of a rotated part of {mixer.rot_dim}")
            elif kind == "delta":
                mixer = DeltaConfig(heads=int(m["heads"]), kv_heads=int(m.get("kv_heads", m["heads"])), dim=int(m["dim"]),
                                    vdim=int(m["vdim"]), conv=int(m["conv"]))
                if mixer.heads % mixer.kv_heads:
                    raise ValueError(f"Penozen layer {i}: {mixer.heads} heads over {mixer.kv_heads} query/key heads")
                if mixer.conv < 1:
                    raise ValueError(f"Penozen layer {i}: a convolution of {mixer.conv} taps")
            else:
                raise ValueError(f"Penozen layer {i}: mixer type {kind!r} is not supported (latent_attention, delta)")
            mlp = entry.get("mlp")
            if mlp is None:
                layers.append(PenozenLayerConfig(kind, mixer))
                continue
            if mlp.get("kind") != "moe":
                raise ValueError(f"Penozen layer {i}: feed-forward kind {mlp.get('kind')!r} is not supported (moe only)")
            lc = PenozenLayerConfig(kind, mixer, experts=int(mlp["router"]["experts"]), top=int(mlp["router"]["top"]),
                                    ff=int(mlp["expert"]["ff"]), limit=float(mlp["expert"]["limit"]))
            if not 0 < lc.top <= lc.experts:
                raise ValueError(f"Penozen layer {i}: top {lc.top} of {lc.experts} experts")
            layers.append(lc)
        emb = d["embedding"]
        bg = emb["bigram"]
        return cls(vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), norm_eps=float(d["norm"]["eps"]),
                   embedding_scale=float(emb.get("scale", 1.0)), bigram_buckets=int(bg["buckets"]), bigram_mul_prev=int(bg["mul_prev"]),
                   bigram_mul_cur=int(bg["mul_cur"]), logit_softcap=float(d.get("logit_softcap") or 0.0), layers=layers)


def penozen_uniform(vocab_size: int, hidden_size: int, pattern: str, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                    delta_heads: int, delta_kv_heads: int, delta_dim: int, delta_vdim: int, experts: int, top: int, ff: int,
                    conv: int = 4, limit: float = 7.0, norm_eps: float = 1e-5) -> PenozenConfig:
    """A configuration from a pattern of layer kinds, 'a' = latent attention, 'd' = delta (benchmarks, tests)."""
    layers = []
    for ch in pattern:
        if ch == "a":
            mixer: Any = LatentAttentionConfig(heads, dim, rot_dim, vdim, kv_rank, (dim + rot_dim) ** -0.5, rot_dim, 10000.0, None)
        else:
            mixer = DeltaConfig(delta_heads, delta_kv_heads, delta_dim, delta_vdim, conv)
        layers.append(PenozenLayerConfig("latent_attention" if ch == "a" else "delta", mixer, experts, top, ff, limit))
    return PenozenConfig(vocab_size=vocab_size, hidden_size=hidden_size, norm_eps=norm_eps, embedding_scale=math.sqrt(hidden_size),
                         bigram_buckets=4093, bigram_mul_prev=1009, bigram_mul_cur=31, logit_softcap=50.0, layers=layers)


def stretched_frequencies(dims: int, base: float, scaling: Optional[Dict[str, float]]):
    """(fp32 frequency of every neighbouring pair, factor on cos and sin).  Without scaling: base^(-2i / dims) and 1.  With
    {factor, original, fast, slow} (YaRN): pairs that turn fewer than `slow` times over `original` positions are slowed by
    `factor`, pairs that turn more than `fast` times are kept, a linear ramp over the pair index between; cos and sin are
    multiplied by 0.1 ln(factor) + 1."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return torch.tensor(f, dtype=torch.float64).float(), 1.0

    def pair_of(turns: float) -> float:
        return dims * math.log(scaling["original"] / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(pair_of(scaling["fast"])), 0)
    hi = min(math.ceil(pair_of(scaling["slow"])), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / scaling["factor"] * ramp + fi * (1 - ramp))
    return torch.tensor(out, dtype=torch.float64).float(), 0.1 * math.log(scaling["factor"]) + 1.0


EXPAND_MIN_TOKENS = 256      # new tokens from which a prompt batch expands keys and values from the latent rows


def context_rows(forward_batch):
    """For an extend batch: (pool slots of every request's tokens, request after request, int64 [N]; a table [B, longest] whose
    row b numbers request b's tokens 0-based within that order, int32; the rows' numbers, int64 [B]).  Built once per batch
    and shared by its layers."""
    cached = getattr(forward_batch, "_context_rows", None)
    if cached is not None:
        return cached
    from semi_pd_amd.managers.schedule_batch import host_list_to_device
    lens = [p + e for p, e in zip(forward_batch.extend_prefix_lens_cpu, forward_batch.extend_seq_lens_cpu)]
    dev = forward_batch.seq_lens.device
    r2t = forward_batch.req_to_token_pool.req_to_token.index_select(0, forward_batch.req_pool_indices)
    slots = torch.cat([r2t[b, :n] for b, n in enumerate(lens)]).long()
    longest = max(lens)
    starts, at = [], 0
    for n in lens:
        starts.append(at)
        at += n
    base = host_list_to_device(starts, torch.int32, dev)
    table = (torch.arange(longest, dtype=torch.int32, device=dev).unsqueeze(0) + base.unsqueeze(1)).contiguous()
    rows = torch.arange(len(lens), dtype=torch.int64, device=dev)
    forward_batch._context_rows = (slots, table, rows)
    return forward_batch._context_rows


class PenozenLatentAttention(nn.Module):
    def __init__(self, hidden_size: int, mc: LatentAttentionConfig, eps: float, region: int, dtype):
        super().__init__()
        self.mc, self.eps = mc, eps
        H, D, P, E, R = mc.heads, mc.dim, mc.rot_dim, mc.vdim, mc.kv_rank
        self.q_size, self.c_size, self.o_size = H * (D + P), R + P, H * E
        # rows of the merged weight: the queries, the latent and the shared rotated key part, the output gate
        self.in_proj = MergedColumnParallelLinear(hidden_size, [self.q_size, self.c_size, self.o_size], params_dtype=dtype)
        self.out_proj = RowParallelLinear(self.o_size, hidden_size, params_dtype=dtype)
        self.latent_norm = nn.Parameter(torch.ones(R, dtype=dtype), requires_grad=False)
        self.w_uk = nn.Parameter(torch.empty(H, D, R, dtype=dtype), requires_grad=False)     # key up-projection [H * D, R] by head
        self.w_uv = nn.Parameter(torch.empty(H, E, R, dtype=dtype), requires_grad=False)     # value up-projection [H * E, R] by head
        self.sink = nn.Parameter(torch.zeros(H, dtype=torch.float32), requires_grad=False)
        freq, self.mscale = stretched_frequencies(mc.rot_dims, mc.rot_base, mc.rot_scaling) if mc.rot_dims else (torch.zeros(0), 1.0)
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

    def _forward_expanded(self, p: torch.Tensor, forward_batch) -> torch.Tensor:
        mc = self.mc
        H, D, P, E, R = mc.heads, mc.dim, mc.rot_dim, mc.vdim, mc.kv_rank
        T = p.shape[0]
        pool = forward_batch.token_to_kv_pool.get_key_buffer(self.attn.layer_id)
        pool = pool.view(pool.shape[0], -1)
        ops.latent_prep(p, p[:, self.q_size: self.q_size + self.c_size], H, D, P, R, self.latent_norm, self.eps,
                        forward_batch.positions, self.freq if mc.rot_dims else None, mc.rot_dims, self.mscale, pool,
                        forward_batch.out_cache_loc)
        slots, table, rows = context_rows(forward_batch)
        ctx = ops.gather_rows(pool, slots)                                    # [N, R + P]: every request's tokens, in order
        keys = dense_linear(ctx, self.w_key_rows)                             # [N, H * (D + P)]
        vals = dense_linear(ctx, self.w_val_rows)                             # [N, H * E]
        out = torch.empty((T, H * E), dtype=p.dtype, device=p.device)
        ops.local_attention_fwd(p[:, : self.q_size], out, keys.view(-1, H, D + P), vals.view(-1, H, E), table, rows,
                                forward_batch.seq_lens, forward_batch.extend_start_loc, forward_batch.extend_seq_lens,
                                max(forward_batch.extend_seq_lens_cpu), mc.scale, 0.0, 0, self.sink,
                                p[:, self.q_size + self.c_size:], form=int(os.environ.get("SEMIPD_LOCAL_ATTN_FORM", "0")))
        return self.out_proj(out)

    def forward(self, h: torch.Tensor, forward_batch) -> torch.Tensor:
        mc = self.mc
        H, D, P, E, R = mc.heads, mc.dim, mc.rot_dim, mc.vdim, mc.kv_rank
        T = h.shape[0]
        p = self.in_proj(h)
        if self.expands_keys(forward_batch):
            return self._forward_expanded(p, forward_batch)
        pool = forward_batch.token_to_kv_pool.get_key_buffer(self.attn.layer_id)
        q_in = torch.empty((T, H * (R + P)), dtype=p.dtype, device=p.device)
        ops.latent_prep(p, p[:, self.q_size: self.q_size + self.c_size], H, D, P, R, self.latent_norm, self.eps,
                        forward_batch.positions, self.freq if mc.rot_dims else None, mc.rot_dims, self.mscale,
                        pool.view(pool.shape[0], -1), forward_batch.out_cache_loc, q_in)
        # the unrotated query part through the key up-projection, head by head: [H, T, D] x [H, D, R] -> q_in[:, h, :R]
        q_u = p[:, : self.q_size].view(T, H, D + P)[..., :D]
        torch.bmm(q_u.transpose(0, 1), self.w_uk, out=q_in.view(T, H, R + P)[..., :R].transpose(0, 1))
        o_lat = forward_batch.attn_backend.forward_latent(q_in, self.attn, forward_batch, sink=self.sink)
        # the weighted sums of latents through the value up-projection: [H, T, R] x [H, R, E]
        o = torch.empty((T, H, E), dtype=p.dtype, device=p.device)
        torch.bmm(o_lat.view(T, H, R).transpose(0, 1), self.w_uv.transpose(1, 2), out=o.transpose(0, 1))
        gate = p[:, self.q_size + self.c_size:]
        o = ops.sigmoid_gate_(o.view(T, H * E), gate)
        return self.out_proj(o)


class PenozenDelta(nn.Module):
    def __init__(self, hidden_size: int, mc: DeltaConfig, eps: float, state_ids, dtype):
        super().__init__()
        self.mc, self.eps = mc, eps
        self.state_id, self.conv_id = state_ids
        H, G, D, E = mc.heads, mc.kv_heads, mc.dim, mc.vdim
        gd, hv = G * D, H * E
        sizes = [gd, gd, hv, hv, H, H]            # q | k | v | gate | a | b
        self.offsets = [sum(sizes[:i]) for i in range(6)]
        self.in_proj = MergedColumnParallelLinear(hidden_size, sizes, params_dtype=dtype)
        self.out_proj = RowParallelLinear(hv, hidden_size, params_dtype=dtype)
        self.conv_q = nn.Parameter(torch.empty(gd, mc.conv, dtype=dtype), requires_grad=False)
        self.conv_k = nn.Parameter(torch.empty(gd, mc.conv, dtype=dtype), requires_grad=False)
        self.conv_v = nn.Parameter(torch.empty(hv, mc.conv, dtype=dtype), requires_grad=False)
        self.a_log = nn.Parameter(torch.zeros(H, dtype=torch.float32), requires_grad=False)
        self.dt_bias = nn.Parameter(torch.zeros(H, dtype=torch.float32), requires_grad=False)
        self.out_norm = nn.Parameter(torch.ones(E, dtype=dtype), requires_grad=False)

    @staticmethod
    def state_widths(mc: DeltaConfig):
        """(the matrices S of all heads, the last taps - 1 inputs of all convolution channels) in fp32 elements."""
        return mc.heads * mc.dim * mc.vdim, (mc.conv - 1) * (2 * mc.kv_heads * mc.dim + mc.heads * mc.vdim)

    def forward(self, h: torch.Tensor, forward_batch) -> torch.Tensor:
        mc = self.mc
        p = self.in_proj(h)
        if forward_batch.forward_mode.is_decode():
            q_start = q_len = None
        else:
            q_start, q_len = forward_batch.extend_start_loc, forward_batch.extend_seq_lens
        sp = forward_batch.state_pool
        o = ops.delta_rule(p, self.offsets, self.conv_q, self.conv_k, self.conv_v, self.a_log, self.dt_bias, self.out_norm, self.eps,
                           sp.get_state_buffer(self.state_id), sp.get_state_buffer(self.conv_id) if mc.conv > 1 else None,
                           forward_batch.state_indices, forward_batch.seq_lens, q_start, q_len, mc.heads, mc.kv_heads, mc.dim,
                           mc.vdim)
        return self.out_proj(o)


class PenozenDecoderLayer(nn.Module):
    def __init__(self, config: PenozenConfig, layer_id: int, region: Optional[int], state_ids, dtype):
        super().__init__()
        lc = config.layers[layer_id]
        W = config.hidden_size
        if lc.kind == "latent_attention":
            self.mix = PenozenLatentAttention(W, lc.mixer, config.norm_eps, region, dtype)
        else:
            self.mix = PenozenDelta(W, lc.mixer, config.norm_eps, state_ids, dtype)
        self.norm1 = StreamRMSNorm(W, config.norm_eps, 1.0, dtype)
        self.mlp = ClampedGatedMoE(lc.experts, lc.top, W, lc.ff, lc.limit, params_dtype=dtype) if lc.experts else None
        self.norm2 = StreamRMSNorm(W, config.norm_eps, 1.0, dtype) if lc.experts else None

    def forward(self, x: torch.Tensor, h: torch.Tensor, forward_batch, next_norm: StreamRMSNorm) -> torch.Tensor:
        """x: the fp32 stream (updated in place); h = norm1(x) in the activation type.  Returns next_norm(x)."""
        y = self.mix(h, forward_batch)
        if self.mlp is None:
            return StreamRMSNorm.seam(y, x, next_norm)
        h = StreamRMSNorm.seam(y, x, self.norm2)
        return StreamRMSNorm.seam(self.mlp(h), x, next_norm)


class PenozenForCausalLM(nn.Module):
    def __init__(self, config: PenozenConfig, dtype=torch.bfloat16):
        super().__init__()
        if get_tensor_model_parallel_world_size() != 1:
            raise ValueError("Penozen runs on one GPU per replica (tensor parallelism over its per-layer head counts and its "
                             "recurrent state is not implemented)")
        if not config.layers:
            raise ValueError("Penozen: the configuration lists no layers")
        self.config = config
        W = config.hidden_size
        self.embed = BigramEmbedding(config.vocab_size, W, config.bigram_buckets, config.bigram_mul_prev, config.bigram_mul_cur,
                                     config.embedding_scale, params_dtype=dtype)
        # pool regions: one per latent-attention layer; state columns: the previous token, then (S, convolution inputs) per delta layer
        self._regions: List[LatentAttentionConfig] = []
        self._state_widths: List[int] = [1]
        layers = []
        for i, lc in enumerate(config.layers):
            if lc.kind == "latent_attention":
                layers.append(PenozenDecoderLayer(config, i, len(self._regions), None, dtype))
                self._regions.append(lc.mixer)
            else:
                s_w, c_w = PenozenDelta.state_widths(lc.mixer)
                ids = (len(self._state_widths), len(self._state_widths) + 1)
                self._state_widths += [s_w, max(c_w, 1)]
                layers.append(PenozenDecoderLayer(config, i, None, ids, dtype))
        self.layers = nn.ModuleList(layers)
        self.final_norm = StreamRMSNorm(W, config.norm_eps, 1.0, dtype)
        self.head = ParallelLMHead(config.vocab_size, W, params_dtype=dtype)
        self.logits_processor = LogitsProcessor(config.vocab_size, final_logit_softcapping=config.logit_softcap or None)
        self.logits_processor.softcap_fused = True
        self.layer_probe = None      # tests: a callable (layer index, fp32 stream) run after every layer
        for p in self.parameters():
            p.requires_grad_(False)

    def post_load_weights(self):
        for layer in self.layers:
            if layer.mlp is not None:
                layer.mlp.post_load_weights()
            if isinstance(layer.mix, PenozenLatentAttention):
                layer.mix.post_load_weights()

    @property
    def kv_geometry(self):
        """One key/value head per latent-attention layer: the row [latent | shared rotated key part], whose first kv_rank
        elements are the values (a model without such a layer keeps one token-sized dummy region)."""
        ms = self._regions
        if not ms:
            return dict(kind="mha", num_kv_heads=[1], head_dim=[8], v_head_dim=[8], num_heads=[1], num_layers=1, values_in_keys=True)
        return dict(kind="mha", num_kv_heads=[1] * len(ms), head_dim=[m.kv_rank + m.rot_dim for m in ms],
                    v_head_dim=[m.kv_rank for m in ms], num_heads=[m.heads for m in ms], num_layers=len(ms), values_in_keys=True)

    @property
    def state_geometry(self) -> List[int]:
        """Columns of a request's state row: the previous token (one int32 in an fp32 slot), then per delta layer the matrices
        S and the convolutions' last inputs."""
        return list(self._state_widths)

    @torch.no_grad()
    def forward(self, input_ids, positions, forward_batch):
        prev = forward_batch.state_pool.get_state_buffer(0).view(torch.int32)
        x = self.embed(input_ids, prev, forward_batch)
        h = self.layers[0].norm1.read_stream(x)
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            h = layer(x, h, forward_batch, self.layers[i + 1].norm1 if i + 1 < n else self.final_norm)
            if self.layer_probe is not None:
                self.layer_probe(i, x)
        return self.logits_processor(input_ids, h, self.head, forward_batch)
