"""`python bench.py --arch-compare`: Kudirax next to the Llama-family model of equal size (random weights, one GPU);
with `--arch-design tigotar`: Tigotar next to Kudirax, the closest model of the framework (fp32 stream, norms on the
sublayers' outputs, attention over a bounded range of keys through the same kernel family), at equal layer sizes;
with `--arch-design penozen`: Penozen next to Tigotar (fp32 stream, attention and a recurrence over pooled state rows,
a mixture of experts behind them);
with `--arch-design tibenex`: Tibenex next to Penozen (fp32 stream, latent attention, a recurrence with a matrix state and a
short convolution over pooled state rows).

Two parts, printed as one JSON object:
  * "models": prefill and decode throughput of a few-layer model of each design at layer sizes of real models, both driven
    through the same replay scheduler (extend batches of whole prompts; decode batches through the captured graphs).
  * "kernels": every kernel the design adds, alone, next to the kernel that does the like job for Llama, at the same
    shape: time, achieved bytes/s or flop/s of the ALGORITHMIC work, the fraction of the roofline (8 TB/s, 2.5 PFLOP/s
    dense bf16) and the ratio of the two fractions.
"""
from __future__ import annotations

import json
import math
import time

import torch

HBM = 8.0e12
MFMA = 2.5e15

SIZES = {
    # name: hidden, heads, kv heads, head size, ff, layers, vocab
    "8b-layer": dict(hidden=4096, heads=32, kv=8, dim=128, ff=14336, layers=4, vocab=32000),
    "3b-layer": dict(hidden=3072, heads=24, kv=8, dim=128, ff=8192, layers=4, vocab=32000),
    "1b-layer": dict(hidden=2048, heads=32, kv=8, dim=64, ff=8192, layers=4, vocab=32000),
}


def _timed(fn, iters=20, warm=3):
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) / iters * 1e-3


def _configs(s, chunk):
    from semi_pd_amd.models.kudirax import kudirax_uniform
    from semi_pd_amd.models.llama import LlamaConfig
    k = kudirax_uniform(s["vocab"], s["hidden"], s["layers"], s["heads"], s["kv"], s["dim"], s["dim"], s["ff"], chunk)
    l = LlamaConfig(vocab_size=s["vocab"], hidden_size=s["hidden"], intermediate_size=s["ff"], num_hidden_layers=s["layers"],
                    num_attention_heads=s["heads"], num_key_value_heads=s["kv"], head_dim=s["dim"],
                    max_position_embeddings=16384)
    return k, l


def _model_throughput(cfg, prompt_len, prompts, decode_batch, decode_ctx, decode_steps):
    from semi_pd_amd.managers.replay_scheduler import ReplayScheduler
    from semi_pd_amd.model_executor.model_runner import ModelRunner
    from semi_pd_amd.server_args import ServerArgs
    ctx = max(prompt_len, decode_ctx + decode_steps + 8) + 8
    total = max(prompt_len * prompts, decode_batch * (decode_ctx + decode_steps + 8)) + 64
    sa = ServerArgs(model_config=cfg, load_format="dummy", context_length=ctx, max_total_tokens=total,
                    max_running_requests=decode_batch, cuda_graph_max_bs=decode_batch, skip_tokenizer_init=True)
    mr = ModelRunner(cfg, context_length=ctx, max_running_requests=decode_batch, max_total_tokens=total,
                     cuda_graph_max_bs=decode_batch, mem_fraction_static=0.8)
    mr.init_attention_backend()
    mr.init_cuda_graphs()
    sched = ReplayScheduler(sa, mr)
    g = torch.Generator().manual_seed(0)

    def toks(n):
        return torch.randint(0, cfg.vocab_size, (n,), generator=g).tolist()

    def prefill_once(tag):
        ids = [f"{tag}{i}" for i in range(prompts)]
        sched.replay_step([{"id": i, "tokens": toks(prompt_len), "want": [prompt_len - 1]} for i in ids], ids)

    prefill_once("w")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reps = 3
    for r in range(reps):
        prefill_once(f"p{r}")
    torch.cuda.synchronize()
    prefill_tps = reps * prompts * prompt_len / (time.perf_counter() - t0)
    # decode: requests of decode_ctx tokens (admitted four at a time), then single-token steps through the graphs
    ids = [f"d{i}" for i in range(decode_batch)]
    for a in range(0, decode_batch, 4):
        sched.replay_step([{"id": i, "tokens": toks(decode_ctx), "want": []} for i in ids[a:a + 4]], [])
    step = [{"id": i, "tokens": [1], "want": [0]} for i in ids]
    for _ in range(3):
        sched.replay_step(step, [])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(decode_steps):
        sched.replay_step(step, [])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    sched.replay_step([], ids)
    out = {"prefill_tokens_per_s": round(prefill_tps), "decode_tokens_per_s": round(decode_steps * decode_batch / dt),
           "decode_step_ms": round(dt / decode_steps * 1e3, 3)}
    del sched, mr
    torch.cuda.empty_cache()
    return out


def _kernel_pairs(s, chunk, dev):
    """[(what, new kernel's record, like kernel's record)] at the layer shape `s`."""
    from semi_pd_amd import ops
    dt = torch.bfloat16
    H, G, D, W, FF = s["heads"], s["kv"], s["dim"], s["hidden"], s["ff"]
    E = D
    out = []

    def rec(t, nbytes=0.0, flops=0.0):
        frac = max(nbytes / t / HBM, flops / t / MFMA)
        return {"us": round(t * 1e6, 1), "TB_per_s": round(nbytes / t / 1e12, 2), "TFLOP_per_s": round(flops / t / 1e12, 1),
                "of_roofline": round(frac, 3)}

    # ---- prompt attention: 4 requests x 2048 new tokens ------------------------------------------------------------
    B, L = 4, 2048
    T = B * L
    n_slots = T + 1
    kp = torch.randn(n_slots, G, D, device=dev, dtype=dt)
    vp = torch.randn(n_slots, G, E, device=dev, dtype=dt)
    r2t = (torch.arange(T, device=dev, dtype=torch.int32) + 1).view(B, L).contiguous()
    q = torch.randn(T, H * D, device=dev, dtype=dt)
    o = torch.empty(T, H * E, device=dev, dtype=dt)
    gate = torch.randn(T, H * E, device=dev, dtype=dt)
    sink = torch.zeros(H, device=dev)
    rows = torch.arange(B, device=dev)
    lens = torch.full((B,), L, device=dev, dtype=torch.int64)
    q_start = (torch.arange(B, device=dev, dtype=torch.int32) * L)
    q_len = torch.full((B,), L, device=dev, dtype=torch.int32)
    t_new = _timed(lambda: ops.local_attention_fwd(q, o, kp, vp, r2t, rows, lens, q_start, q_len, L, D ** -0.5, 30.0, chunk, sink, gate))
    pairs_new = B * sum((p % chunk) + 1 for p in range(L)) if chunk else B * L * (L + 1) / 2
    k_ext = torch.randn(T, G, D, device=dev, dtype=dt)
    v_ext = torch.randn(T, G, D, device=dev, dtype=dt)
    qo = (torch.arange(B + 1, device=dev, dtype=torch.int32) * L)
    kvi = torch.zeros(B + 1, device=dev, dtype=torch.int32)
    idx = torch.zeros(1, device=dev, dtype=torch.int32)
    o3 = o.view(T, H, E)
    t_old = _timed(lambda: ops.extend_attention_fwd(q.view(T, H, D), k_ext, v_ext, o3, kp, vp, qo, kvi, idx, None, None, L))
    pairs_old = B * L * (L + 1) / 2
    out.append((f"prompt attention, {B} x {L} tokens (new: blocks of {chunk})", rec(t_new, flops=2.0 * H * (D + E) * pairs_new),
                rec(t_old, flops=2.0 * H * 2 * D * pairs_old)))
    # ---- decode attention: 32 requests at 1100 tokens ----------------------------------------------------------------
    B2, C = 32, 1000
    n2 = B2 * C + 1
    kp2 = torch.randn(n2, G, D, device=dev, dtype=dt)
    vp2 = torch.randn(n2, G, E, device=dev, dtype=dt)
    r2t2 = (torch.arange(B2 * C, device=dev, dtype=torch.int32) + 1).view(B2, C).contiguous()
    q2 = torch.randn(B2, H * D, device=dev, dtype=dt)
    o2 = torch.empty(B2, H * E, device=dev, dtype=dt)
    g2 = torch.randn(B2, H * E, device=dev, dtype=dt)
    rows2 = torch.arange(B2, device=dev)
    lens2 = torch.full((B2,), C, device=dev, dtype=torch.int64)
    t_new = _timed(lambda: ops.local_attention_fwd(q2, o2, kp2, vp2, r2t2, rows2, lens2, None, None, 1, D ** -0.5, 30.0, chunk, sink, g2))
    keys_new = ((C - 1) % chunk) + 1 if chunk else C
    from semi_pd_amd.layers.attention_backend import choose_kv_splits
    splits = choose_kv_splits(B2, G, C, torch.cuda.get_device_properties(dev).multi_processor_count, 32)
    logits = torch.empty(B2, H, splits, E + 1, device=dev, dtype=torch.float32)
    indptr = (torch.arange(B2 + 1, device=dev, dtype=torch.int32) * C)
    indices = r2t2.view(-1)
    t_old = _timed(lambda: ops.decode_attention_fwd(q2.view(B2, H, D), kp2, vp2, o2.view(B2, H, E), indptr, indices, logits, splits, D ** -0.5))
    out.append((f"decode attention, {B2} requests at {C} tokens (new: {keys_new} visible keys)",
                rec(t_new, nbytes=B2 * G * (D + E) * 2.0 * keys_new), rec(t_old, nbytes=B2 * G * 2 * D * 2.0 * C)))
    # ---- norm + residual -------------------------------------------------------------------------------------------
    for Tn in (8192, 32):
        y = torch.randn(Tn, W, device=dev, dtype=dt)
        res = torch.randn(Tn, W, device=dev, dtype=torch.float32)
        w = torch.ones(W, device=dev, dtype=dt)
        b = torch.zeros(W, device=dev, dtype=dt)
        t_new = _timed(lambda: ops.layernorm(y, w, b, 1e-5, residual=res, in_bias=b))
        r16 = torch.randn(Tn, W, device=dev, dtype=dt)
        t_old = _timed(lambda: ops.fused_add_rmsnorm(y, r16, w, 1e-5))
        out.append((f"norm + residual add, {Tn} rows of {W}", rec(t_new, nbytes=Tn * W * (2 + 4 + 4 + 2.0)),
                    rec(t_old, nbytes=Tn * W * 4 * 2.0)))
    # ---- the step between the projection and the attention ---------------------------------------------------------------
    Tn = 8192
    cols = H * D + 2 * G * D + H * E
    p = torch.randn(Tn, cols, device=dev, dtype=dt)
    kp3 = torch.zeros(Tn + 1, G, D, device=dev, dtype=dt)
    vp3 = torch.zeros(Tn + 1, G, E, device=dev, dtype=dt)
    loc = torch.arange(1, Tn + 1, device=dev)
    v0 = torch.randn(Tn, G * E, device=dev, dtype=dt)
    mix = torch.tensor(0.5, device=dev, dtype=dt)
    t_new = _timed(lambda: ops.unit_norm_and_store_kv(p, H, G, D, E, H * D, H * D + G * D, 1e-5, kp3, vp3, loc, v_first=v0, mix=mix))
    from oracle import ops as O
    cache = O.cos_sin_cache_from_inv_freq(O.rope_inv_freq(D, 10000.0), Tn + 1).to(dev)
    qq = torch.randn(Tn, H * D, device=dev, dtype=dt)
    kk = torch.randn(Tn, G * D, device=dev, dtype=dt)
    vv = torch.randn(Tn, G * D, device=dev, dtype=dt)
    pos = torch.arange(Tn, device=dev)
    t_old = _timed(lambda: ops.rope_and_store_kv(pos, qq, kk, vv, D, cache, True, kp3, vp3, loc))
    out.append((f"q / k preparation + KV-pool store, {Tn} tokens (new: unit norm + blend; like: rotation)",
                rec(t_new, nbytes=Tn * 2.0 * (2 * H * D + 2 * G * D + 3 * G * E)), rec(t_old, nbytes=Tn * 2.0 * (2 * H * D + 4 * G * D))))
    # ---- activation --------------------------------------------------------------------------------------------------
    u = torch.randn(Tn, FF, device=dev, dtype=dt)
    bb = torch.zeros(FF, device=dev, dtype=dt)
    t_new = _timed(lambda: ops.bias_relu_square_(u, bb))
    gu = torch.randn(Tn, 2 * FF, device=dev, dtype=dt)
    t_old = _timed(lambda: ops.silu_and_mul(gu))
    out.append((f"activation, {Tn} rows of {FF} (new: bias + squared ReLU in place; like: SiLU * mul)",
                rec(t_new, nbytes=Tn * FF * 2 * 2.0), rec(t_old, nbytes=Tn * FF * 3 * 2.0)))
    return out


TIGOTAR_SIZES = {
    # experts x ff: `top` experts of ff = the dense feed-forward of the model next to it; the recurrence is as wide as the model
    "8b-layer": dict(hidden=4096, heads=32, kv=8, dim=128, ff=14336, experts=8, top=2, layers=4, loop=(1, 3, 2), vocab=32000),
    "3b-layer": dict(hidden=3072, heads=24, kv=8, dim=128, ff=8192, experts=8, top=2, layers=4, loop=(1, 3, 2), vocab=32000),
    "1b-layer": dict(hidden=2048, heads=32, kv=8, dim=64, ff=8192, experts=16, top=4, layers=4, loop=(1, 3, 2), vocab=32000),
}


def _tigotar_kernel_pairs(s, window, keep, dev):
    """[(what, Tigotar kernel's record, like kernel's record)] at the layer shape `s`."""
    from semi_pd_amd import ops
    from semi_pd_amd.layers.moe import fused_experts, fused_experts_ungated
    dt = torch.bfloat16
    H, G, D, W = s["heads"], s["kv"], s["dim"], s["hidden"]
    X, K, F = s["experts"], s["top"], s["ff"] // s["top"]
    E, R = D, W
    out = []

    def rec(t, nbytes=0.0, flops=0.0):
        frac = max(nbytes / t / HBM, flops / t / MFMA)
        return {"us": round(t * 1e6, 1), "TB_per_s": round(nbytes / t / 1e12, 2), "TFLOP_per_s": round(flops / t / 1e12, 1),
                "of_roofline": round(frac, 3)}

    # ---- prompt attention: 4 requests x 2048 new tokens; window of `window` + `keep` kept against blocks of `window` ----------
    B, L = 4, 2048
    T = B * L
    kp = torch.randn(T + 1, G, D, device=dev, dtype=dt)
    vp = torch.randn(T + 1, G, E, device=dev, dtype=dt)
    r2t = (torch.arange(T, device=dev, dtype=torch.int32) + 1).view(B, L).contiguous()
    q = torch.randn(T, H * D, device=dev, dtype=dt)
    o = torch.empty(T, H * E, device=dev, dtype=dt)
    hb = torch.full((H,), -3.0, device=dev)
    sink = torch.zeros(H, device=dev)
    rows = torch.arange(B, device=dev)
    lens = torch.full((B,), L, device=dev, dtype=torch.int64)
    q_start = (torch.arange(B, device=dev, dtype=torch.int32) * L)
    q_len = torch.full((B,), L, device=dev, dtype=torch.int32)
    t_new = _timed(lambda: ops.window_attention_fwd(q, o, kp, vp, r2t, rows, lens, q_start, q_len, L, D ** -0.5, window, keep, hb,
                                                    True, None, 1.2))
    pairs_new = B * sum(min(p + 1, window) + max(0, min(keep, p + 1 - window)) for p in range(L))
    t_old = _timed(lambda: ops.local_attention_fwd(q, o, kp, vp, r2t, rows, lens, q_start, q_len, L, D ** -0.5, 30.0, window, sink, None))
    pairs_old = B * sum((p % window) + 1 for p in range(L))
    out.append((f"prompt attention, {B} x {L} tokens (window {window} + {keep} kept, sigmoid weights; like: blocks of {window}, softmax)",
                rec(t_new, flops=2.0 * H * (D + E) * pairs_new), rec(t_old, flops=2.0 * H * (D + E) * pairs_old)))
    # ---- decode attention: 32 requests at 2000 tokens ----------------------------------------------------------------
    B2, C = 32, 2000
    kp2 = torch.randn(B2 * C + 1, G, D, device=dev, dtype=dt)
    vp2 = torch.randn(B2 * C + 1, G, E, device=dev, dtype=dt)
    r2t2 = (torch.arange(B2 * C, device=dev, dtype=torch.int32) + 1).view(B2, C).contiguous()
    q2 = torch.randn(B2, H * D, device=dev, dtype=dt)
    o2 = torch.empty(B2, H * E, device=dev, dtype=dt)
    rows2 = torch.arange(B2, device=dev)
    lens2 = torch.full((B2,), C, device=dev, dtype=torch.int64)
    t_new = _timed(lambda: ops.window_attention_fwd(q2, o2, kp2, vp2, r2t2, rows2, lens2, None, None, 1, D ** -0.5, window, keep, hb,
                                                    True, None, 1.2))
    keys_new = min(C, window) + max(0, min(keep, C - window))
    t_old = _timed(lambda: ops.local_attention_fwd(q2, o2, kp2, vp2, r2t2, rows2, lens2, None, None, 1, D ** -0.5, 30.0, window, sink, None))
    keys_old = ((C - 1) % window) + 1
    out.append((f"decode attention, {B2} requests at {C} tokens ({keys_new} visible keys; like: {keys_old})",
                rec(t_new, nbytes=B2 * G * (D + E) * 2.0 * keys_new), rec(t_old, nbytes=B2 * G * (D + E) * 2.0 * keys_old)))
    # ---- the seam between two sublayers ----------------------------------------------------------------------------------
    for Tn in (8192, 32):
        y = torch.randn(Tn, W, device=dev, dtype=dt)
        res = torch.randn(Tn, W, device=dev, dtype=torch.float32)
        w = torch.ones(W, device=dev, dtype=dt)
        b = torch.zeros(W, device=dev, dtype=dt)
        al = torch.tensor(0.5, device=dev, dtype=dt)
        t_new = _timed(lambda: ops.dyn_tanh(y, (w, b, al), residual=res, params_out=(w, b, al)))
        t_old = _timed(lambda: ops.layernorm(y, w, b, 1e-5, residual=res, in_bias=b))
        nb = Tn * W * (2 + 4 + 4 + 2.0)
        out.append((f"stream += squash(y), next input = squash(stream), {Tn} rows of {W} (like: LayerNorm + residual add)",
                    rec(t_new, nbytes=nb), rec(t_old, nbytes=nb)))
    # ---- the step between the projection and the attention ---------------------------------------------------------------
    Tn = 8192
    cols = H * D + G * D + G * E + 3 * R
    p = torch.randn(Tn, cols, device=dev, dtype=dt)
    kp3 = torch.zeros(Tn + 1, G, D, device=dev, dtype=dt)
    vp3 = torch.zeros(Tn + 1, G, E, device=dev, dtype=dt)
    loc = torch.arange(1, Tn + 1, device=dev)
    pos = torch.arange(Tn, device=dev)
    bq, bk, bv = (torch.zeros(n, device=dev, dtype=dt) for n in (H * D, G * D, G * E))
    inv_freq = 10000.0 ** (-2.0 * torch.arange(D // 2, dtype=torch.float32, device=dev) / D)
    t_new = _timed(lambda: ops.bias_rope_vnorm_kv_store(p, H, G, D, E, H * D, H * D + G * D, bq, bk, bv, pos, inv_freq, D, 1e-6, kp3, vp3, loc))
    pk = torch.randn(Tn, H * D + G * D + G * E + H * E, device=dev, dtype=dt)
    t_old = _timed(lambda: ops.unit_norm_and_store_kv(pk, H, G, D, E, H * D, H * D + G * D, 1e-5, kp3, vp3, loc))
    nb = Tn * 2.0 * (2 * H * D + 2 * G * D + 2 * G * E)
    out.append((f"q / k / v preparation + KV-pool store, {Tn} tokens (biases, pair rotation, value norm; like: unit norm of q and k)",
                rec(t_new, nbytes=nb), rec(t_old, nbytes=nb)))
    # ---- the recurrence: a prompt batch (chunked form) and a decode batch ---------------------------------------------------
    state = torch.zeros(B2 + 1, R, device=dev)
    yb = torch.empty(Tn, R, device=dev, dtype=dt)
    u = torch.randn(Tn, R, device=dev, dtype=dt)
    bb = torch.zeros(R, device=dev, dtype=dt)
    st4 = torch.arange(1, B + 1, device=dev)
    t_new = _timed(lambda: ops.min_gru(p, H * D + G * D + G * E, H * D + G * D + G * E + R, H * D + G * D + G * E + 2 * R, R, bb, bb, yb,
                                       state, st4, lens, q_start, q_len, L))
    t_old = _timed(lambda: ops.bias_relu_square_(u, bb))
    out.append((f"minGRU over {B} x {L} tokens, {R} channels (three passes over chunks of 32; like: an in-place element-wise kernel over as many rows)",
                rec(t_new, nbytes=Tn * R * 2.0 * (3 + 2 + 1)), rec(t_old, nbytes=Tn * R * 2.0 * 2)))
    pd = torch.randn(B2, cols, device=dev, dtype=dt)
    yd = torch.empty(B2, R, device=dev, dtype=dt)
    ud = torch.randn(B2, R, device=dev, dtype=dt)
    st32 = torch.arange(1, B2 + 1, device=dev)
    t_new = _timed(lambda: ops.min_gru(pd, H * D + G * D + G * E, H * D + G * D + G * E + R, H * D + G * D + G * E + 2 * R, R, bb, bb, yd,
                                       state, st32, lens2, None, None, 1))
    t_old = _timed(lambda: ops.bias_relu_square_(ud, bb))
    out.append((f"minGRU decode step, {B2} requests, {R} channels (like: an in-place element-wise kernel over as many rows; both are launch-bound)",
                rec(t_new, nbytes=B2 * R * (2.0 * 4 + 8)), rec(t_old, nbytes=B2 * R * 2.0 * 2)))
    # ---- experts: ungated (two GEMMs per expert) against gated SiLU (three), same sizes ----------------------------------------
    w_up = torch.randn(X, F, W, device=dev, dtype=dt) * 0.02
    w_down = torch.randn(X, W, F, device=dev, dtype=dt) * 0.02
    w13 = torch.randn(X, 2 * F, W, device=dev, dtype=dt) * 0.02
    for Tn in (8192, 32):
        h = torch.randn(Tn, W, device=dev, dtype=dt)
        tw, ti = ops.topk_softmax(torch.randn(Tn, X, device=dev), K, True)
        t_new = _timed(lambda: fused_experts_ungated(h, w_up, w_down, tw, ti))
        t_old = _timed(lambda: fused_experts(h, w13, w_down, tw, ti))
        if Tn > 1024:
            new, old = rec(t_new, flops=2.0 * Tn * K * 2 * W * F), rec(t_old, flops=2.0 * Tn * K * 3 * W * F)
        else:   # every expert is touched: the call streams all weights once
            new, old = rec(t_new, nbytes=X * 2.0 * W * F * 2), rec(t_old, nbytes=X * 3.0 * W * F * 2)
        out.append((f"experts, {Tn} tokens, top {K} of {X} x {F} (up, squared ReLU, down; like: gate | up, SiLU * mul, down)", new, old))
    return out


def main_tigotar(args) -> dict:
    from semi_pd_amd.models.kudirax import kudirax_uniform
    from semi_pd_amd.models.tigotar import tigotar_uniform
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    window, keep = int(getattr(args, "arch_chunk", 1024) or 1024), 4
    names = [n for n in (getattr(args, "arch_sizes", "") or ",".join(TIGOTAR_SIZES)).split(",") if n]
    result = {"what": "Tigotar next to Kudirax at equal layer sizes", "dtype": "bf16", "data": "synthetic", "window": window,
              "kept_first": keep, "models": {}, "kernels": {}}
    for name in names:
        s = TIGOTAR_SIZES[name]
        result["kernels"][name] = [
            {"kernel": what, "tigotar": new, "like": old,
             "roofline_fraction_ratio": round(new["of_roofline"] / max(old["of_roofline"], 1e-9), 2)}
            for what, new, old in _tigotar_kernel_pairs(s, window, keep, dev)]
        tcfg = tigotar_uniform(s["vocab"], s["hidden"], s["layers"], s["heads"], s["kv"], s["dim"], s["dim"], s["hidden"],
                               s["experts"], s["top"], s["ff"] // s["top"], window, keep, loop=s["loop"])
        runs = len(tcfg.runs())
        kcfg = kudirax_uniform(s["vocab"], s["hidden"], runs, s["heads"], s["kv"], s["dim"], s["dim"], s["ff"], window)
        result["models"][name] = {
            "layer_runs": runs,
            "tigotar": _model_throughput(tcfg, 2048, 4, 32, 1100, 20),
            "kudirax": _model_throughput(kcfg, 2048, 4, 32, 1100, 20)}
    print(json.dumps(result), flush=True)
    return result


PENOZEN_SIZES = {
    # latent attention: `heads` queries of [dim unrotated | rot rotated] over rows [rank | rot]; delta rule: `heads` value heads of
    # vdim over `kv` query/key heads of `kdim`; experts as in TIGOTAR_SIZES; two layers of each mixer, in turn
    "8b-layer": dict(hidden=4096, heads=32, dim=64, rot=64, vdim=128, rank=192, dheads=32, kv=8, kdim=128, dvdim=128, ff=14336,
                     experts=8, top=2, vocab=32000),
    "3b-layer": dict(hidden=3072, heads=24, dim=64, rot=64, vdim=128, rank=192, dheads=24, kv=8, kdim=128, dvdim=128, ff=8192,
                     experts=8, top=2, vocab=32000),
    "1b-layer": dict(hidden=2048, heads=32, dim=32, rot=32, vdim=64, rank=96, dheads=32, kv=8, kdim=64, dvdim=64, ff=8192,
                     experts=16, top=4, vocab=32000),
}
VALU = 157.3e12      # fp32 vector rate: what a recurrence that is a chain of small matrix-vector steps runs on


def _penozen_kernel_pairs(s, t, window, keep, dev):
    """[(what, Penozen kernel's record, like kernel's record)]: `s` Penozen's layer shape, `t` Tigotar's at the same size."""
    from semi_pd_amd import ops
    from semi_pd_amd.layers.moe import fused_experts_clamped, fused_experts_ungated
    dt = torch.bfloat16
    W = s["hidden"]
    H, D, Pr, E, R = s["heads"], s["dim"], s["rot"], s["vdim"], s["rank"]
    tH, tG, tD = t["heads"], t["kv"], t["dim"]
    X, K, F = s["experts"], s["top"], s["ff"] // s["top"]
    out = []

    def rec(tm, nbytes=0.0, flops=0.0, vflops=0.0):
        frac = max(nbytes / tm / HBM, flops / tm / MFMA, vflops / tm / VALU)
        return {"us": round(tm * 1e6, 1), "TB_per_s": round(nbytes / tm / 1e12, 2),
                "TFLOP_per_s": round(max(flops, vflops) / tm / 1e12, 1), "of_roofline": round(frac, 3)}

    # ---- prompt attention: 4 requests x 2048 new tokens ------------------------------------------------------------------
    B, L = 4, 2048
    T = B * L
    pool = torch.randn(T + 1, R + Pr, device=dev, dtype=dt)
    r2t = (torch.arange(T, device=dev, dtype=torch.int32) + 1).view(B, L).contiguous()
    q = torch.randn(T, H * (R + Pr), device=dev, dtype=dt)
    o = torch.empty(T, H * R, device=dev, dtype=dt)
    sink = torch.zeros(H, device=dev)
    rows = torch.arange(B, device=dev)
    lens = torch.full((B,), L, device=dev, dtype=torch.int64)
    q_start = (torch.arange(B, device=dev, dtype=torch.int32) * L)
    q_len = torch.full((B,), L, device=dev, dtype=torch.int32)
    # a prompt batch expands keys and values of all heads from the latent rows and attends head by head (the model's path for
    # batches from 256 new tokens up); the same batch over the latent rows themselves (the path of short portions) for reference
    from semi_pd_amd.layers.basic import dense_linear
    w_key = torch.randn(H * (D + Pr), R + Pr, device=dev, dtype=dt) * 0.05
    w_val = torch.randn(H * E, R + Pr, device=dev, dtype=dt) * 0.05
    slots = torch.arange(1, T + 1, device=dev)
    tab = torch.arange(T, device=dev, dtype=torch.int32).view(B, L).contiguous()
    qh = torch.randn(T, H * (D + Pr), device=dev, dtype=dt)
    oh = torch.empty(T, H * E, device=dev, dtype=dt)
    gate = torch.randn(T, H * E, device=dev, dtype=dt)

    def expanded():
        ctx = ops.gather_rows(pool, slots)
        keys, vals = dense_linear(ctx, w_key), dense_linear(ctx, w_val)
        ops.local_attention_fwd(qh, oh, keys.view(-1, H, D + Pr), vals.view(-1, H, E), tab, rows, lens, q_start, q_len, L, 0.1, 0.0, 0,
                                sink, gate)

    t_new = _timed(expanded)
    t_lat = _timed(lambda: ops.latent_attention_fwd(q, o, pool, R, r2t, rows, lens, q_start, q_len, L, 0.1, sink))
    pairs_new = B * L * (L + 1) / 2
    kp = torch.randn(T + 1, tG, tD, device=dev, dtype=dt)
    vp = torch.randn(T + 1, tG, tD, device=dev, dtype=dt)
    tq = torch.randn(T, tH * tD, device=dev, dtype=dt)
    to = torch.empty(T, tH * tD, device=dev, dtype=dt)
    hb = torch.full((tH,), -3.0, device=dev)
    t_old = _timed(lambda: ops.window_attention_fwd(tq, to, kp, vp, r2t, rows, lens, q_start, q_len, L, tD ** -0.5, window, keep, hb,
                                                    True, None, 1.2))
    pairs_old = B * sum(min(p + 1, window) + max(0, min(keep, p + 1 - window)) for p in range(L))
    out.append((f"prompt attention, {B} x {L} tokens ({H} heads of {D} + {Pr} / {E} expanded from latent rows of {R} + {Pr}: gather, two "
                f"GEMMs, causal softmax with a sink and the output gate; like: window {window} + {keep} kept, sigmoid weights, {tH} heads "
                f"of {tD})",
                rec(t_new, flops=2.0 * H * (D + Pr + E) * pairs_new + 2.0 * T * (R + Pr) * H * (D + Pr + E)),
                rec(t_old, flops=2.0 * tH * 2 * tD * pairs_old)))
    out.append((f"the same batch over the latent rows themselves ({H} heads x [{R} + {Pr}] queries, one shared key/value row per token: the "
                "path of portions below 256 tokens; like: the same kernel as above)",
                rec(t_lat, flops=2.0 * H * (2 * R + Pr) * pairs_new), rec(t_old, flops=2.0 * tH * 2 * tD * pairs_old)))
    # ---- decode attention: 32 requests at 2000 tokens --------------------------------------------------------------------
    B2, C = 32, 2000
    pool2 = torch.randn(B2 * C + 1, R + Pr, device=dev, dtype=dt)
    r2t2 = (torch.arange(B2 * C, device=dev, dtype=torch.int32) + 1).view(B2, C).contiguous()
    q2 = torch.randn(B2, H * (R + Pr), device=dev, dtype=dt)
    o2 = torch.empty(B2, H * R, device=dev, dtype=dt)
    rows2 = torch.arange(B2, device=dev)
    lens2 = torch.full((B2,), C, device=dev, dtype=torch.int64)
    splits = max(1, min(16, 512 // (B2 * ((H + 15) // 16)), C // 128))       # HipAttnBackend.forward_latent's rule on 256 CUs
    t_new = _timed(lambda: ops.latent_attention_fwd(q2, o2, pool2, R, r2t2, rows2, lens2, None, None, 1, 0.1, sink, n_splits=splits))
    kp2 = torch.randn(B2 * C + 1, tG, tD, device=dev, dtype=dt)
    vp2 = torch.randn(B2 * C + 1, tG, tD, device=dev, dtype=dt)
    tq2 = torch.randn(B2, tH * tD, device=dev, dtype=dt)
    to2 = torch.empty(B2, tH * tD, device=dev, dtype=dt)
    t_old = _timed(lambda: ops.window_attention_fwd(tq2, to2, kp2, vp2, r2t2, rows2, lens2, None, None, 1, tD ** -0.5, window, keep, hb,
                                                    True, None, 1.2))
    keys_old = min(C, window) + max(0, min(keep, C - window))
    out.append((f"decode attention, {B2} requests at {C} tokens (every latent row once for all {H} heads, {splits} workgroups share a "
                f"request's keys, + merge; like: {keys_old} visible keys, {tG} key/value heads)",
                rec(t_new, nbytes=B2 * (R + Pr) * 2.0 * C, flops=2.0 * B2 * H * (2 * R + Pr) * C),
                rec(t_old, nbytes=B2 * tG * 2 * tD * 2.0 * keys_old)))
    # ---- the seam between two sublayers ----------------------------------------------------------------------------------
    for Tn in (8192, 32):
        y = torch.randn(Tn, W, device=dev, dtype=dt)
        res = torch.randn(Tn, W, device=dev, dtype=torch.float32)
        w = torch.ones(W, device=dev, dtype=dt)
        b = torch.zeros(W, device=dev, dtype=dt)
        al = torch.tensor(0.5, device=dev, dtype=dt)
        t_new = _timed(lambda: ops.rms_stream(y, res, w, 1e-5, 1.0))
        t_old = _timed(lambda: ops.dyn_tanh(y, (w, b, al), residual=res, params_out=(w, b, al)))
        nb = Tn * W * (2 + 4 + 4 + 2.0)
        out.append((f"stream += y, next input = RMS norm(stream), {Tn} rows of {W} (like: stream += squash(y), next = squash(stream))",
                    rec(t_new, nbytes=nb), rec(t_old, nbytes=nb)))
    # ---- the step between the projection and the attention ---------------------------------------------------------------
    Tn = 8192
    p = torch.randn(Tn, H * (D + Pr) + R + Pr + H * E, device=dev, dtype=dt)
    pool3 = torch.zeros(Tn + 1, R + Pr, device=dev, dtype=dt)
    q3 = torch.empty(Tn, H * (R + Pr), device=dev, dtype=dt)
    loc = torch.arange(1, Tn + 1, device=dev)
    pos = torch.arange(Tn, device=dev)
    nw = torch.ones(R, device=dev, dtype=dt)
    freq = 10000.0 ** (-2.0 * torch.arange(Pr // 2, dtype=torch.float32, device=dev) / Pr)
    t_new = _timed(lambda: ops.latent_prep(p, p[:, H * (D + Pr): H * (D + Pr) + R + Pr], H, D, Pr, R, nw, 1e-5, pos, freq, Pr, 1.07, pool3, loc, q3))
    cols = tH * tD + 2 * tG * tD + 3 * W
    tp = torch.randn(Tn, cols, device=dev, dtype=dt)
    kp3 = torch.zeros(Tn + 1, tG, tD, device=dev, dtype=dt)
    vp3 = torch.zeros(Tn + 1, tG, tD, device=dev, dtype=dt)
    bq, bk, bv = (torch.zeros(n, device=dev, dtype=dt) for n in (tH * tD, tG * tD, tG * tD))
    inv_freq = 10000.0 ** (-2.0 * torch.arange(tD // 2, dtype=torch.float32, device=dev) / tD)
    t_old = _timed(lambda: ops.bias_rope_vnorm_kv_store(tp, tH, tG, tD, tD, tH * tD, tH * tD + tG * tD, bq, bk, bv, pos, inv_freq, tD, 1e-6,
                                                        kp3, vp3, loc))
    out.append((f"latent norm + rotation of the shared key part and of every head's rotated query part + pool store, {Tn} tokens "
                "(like: biases, pair rotation of q and k, value norm, KV store)",
                rec(t_new, nbytes=Tn * 2.0 * (2 * (R + Pr) + 2 * H * Pr)), rec(t_old, nbytes=Tn * 2.0 * (2 * tH * tD + 4 * tG * tD))))
    # ---- the recurrences: a prompt batch and a decode batch --------------------------------------------------------------
    DH, G, KD, VD, taps = s["dheads"], s["kv"], s["kdim"], s["dvdim"], 4
    gd, hv = G * KD, DH * VD
    width = 2 * gd + 2 * hv + 2 * DH
    offs = [0, gd, 2 * gd, 2 * gd + hv, 2 * gd + 2 * hv, 2 * gd + 2 * hv + DH]
    cw = [torch.randn(n, taps, device=dev, dtype=dt) * 0.5 for n in (gd, gd, hv)]
    a_log, dt_bias = torch.zeros(DH, device=dev) - 1.0, torch.zeros(DH, device=dev)
    onw = torch.ones(VD, device=dev, dtype=dt)
    S = torch.zeros(B2 + 1, DH * KD * VD, device=dev)
    cs = torch.zeros(B2 + 1, (taps - 1) * (2 * gd + hv), device=dev)
    dp = torch.randn(T, width, device=dev, dtype=dt)
    st4 = torch.arange(1, B + 1, device=dev)
    t_new = _timed(lambda: ops.delta_rule(dp, offs, cw[0], cw[1], cw[2], a_log, dt_bias, onw, 1e-5, S, cs, st4, lens, q_start, q_len, DH, G,
                                          KD, VD), iters=5, warm=1)
    Rw = W
    gp = torch.randn(T, 3 * Rw, device=dev, dtype=dt)
    gstate = torch.zeros(B2 + 1, Rw, device=dev)
    yb = torch.empty(T, Rw, device=dev, dtype=dt)
    bb = torch.zeros(Rw, device=dev, dtype=dt)
    t_old = _timed(lambda: ops.min_gru(gp, 0, Rw, 2 * Rw, Rw, bb, bb, yb, gstate, st4, lens, q_start, q_len, L))
    out.append((f"gated delta rule over {B} x {L} tokens, {DH} heads of {KD} x {VD} over {G} key heads (convolutions, unit norms, the "
                f"recurrence, output norm and gate; 8 flop per element of S and token on the vector units; like: minGRU, {Rw} channels, "
                "one multiply-add per channel and token, bound by its reads)",
                rec(t_new, nbytes=T * 2.0 * (width + hv), vflops=8.0 * T * DH * KD * VD), rec(t_old, nbytes=T * Rw * 2.0 * (3 + 1))))
    dpd = torch.randn(B2, width, device=dev, dtype=dt)
    st32 = torch.arange(1, B2 + 1, device=dev)
    t_new = _timed(lambda: ops.delta_rule(dpd, offs, cw[0], cw[1], cw[2], a_log, dt_bias, onw, 1e-5, S, cs, st32, lens2, None, None, DH, G,
                                          KD, VD))
    gpd = torch.randn(B2, 3 * Rw, device=dev, dtype=dt)
    yd = torch.empty(B2, Rw, device=dev, dtype=dt)
    t_old = _timed(lambda: ops.min_gru(gpd, 0, Rw, 2 * Rw, Rw, bb, bb, yd, gstate, st32, lens2, None, None, 1))
    out.append((f"gated delta rule decode step, {B2} requests (reads and writes {DH * KD * VD * 4 / 1e6:.1f} MB of state per request; "
                f"like: minGRU decode step, {Rw * 4 / 1e3:.0f} KB per request, launch-bound)",
                rec(t_new, nbytes=B2 * DH * KD * VD * 4.0 * 2), rec(t_old, nbytes=B2 * Rw * (2.0 * 4 + 8))))
    # ---- experts: gated with clamps (three matrices per expert) against ungated (two), same sizes -------------------------------
    w_up = torch.randn(X, F, W, device=dev, dtype=dt) * 0.02
    w_down = torch.randn(X, W, F, device=dev, dtype=dt) * 0.02
    w13 = torch.randn(X, 2 * F, W, device=dev, dtype=dt) * 0.02
    for Tn in (8192, 32):
        h = torch.randn(Tn, W, device=dev, dtype=dt)
        tw, ti = ops.topk_sigmoid(torch.randn(Tn, X, device=dev), K, True, 1e-20)
        t_new = _timed(lambda: fused_experts_clamped(h, w13, w_down, tw, ti, 7.0, 1.702))
        t_old = _timed(lambda: fused_experts_ungated(h, w_up, w_down, tw, ti))
        if Tn > 1024:
            new, old = rec(t_new, flops=2.0 * Tn * K * 3 * W * F), rec(t_old, flops=2.0 * Tn * K * 2 * W * F)
        else:   # every expert is touched: the call streams all weights once
            new, old = rec(t_new, nbytes=X * 3.0 * W * F * 2), rec(t_old, nbytes=X * 2.0 * W * F * 2)
        out.append((f"experts, {Tn} tokens, top {K} of {X} x {F} (gate | up, clamped gated activation, down; like: up, squared ReLU, down)",
                    new, old))
    return out


def main_penozen(args) -> dict:
    from semi_pd_amd.models.penozen import penozen_uniform
    from semi_pd_amd.models.tigotar import tigotar_uniform
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    window, keep = int(getattr(args, "arch_chunk", 1024) or 1024), 4
    names = [n for n in (getattr(args, "arch_sizes", "") or ",".join(PENOZEN_SIZES)).split(",") if n]
    result = {"what": "Penozen next to Tigotar at equal layer sizes", "dtype": "bf16", "data": "synthetic", "models": {}, "kernels": {}}
    for name in names:
        s, t = PENOZEN_SIZES[name], TIGOTAR_SIZES[name]
        result["kernels"][name] = [
            {"kernel": what, "penozen": new, "like": old,
             "roofline_fraction_ratio": round(new["of_roofline"] / max(old["of_roofline"], 1e-9), 2)}
            for what, new, old in _penozen_kernel_pairs(s, t, window, keep, dev)]
        pcfg = penozen_uniform(s["vocab"], s["hidden"], "adad", s["heads"], s["dim"], s["rot"], s["vdim"], s["rank"], s["dheads"], s["kv"],
                               s["kdim"], s["dvdim"], s["experts"], s["top"], s["ff"] // s["top"])
        tcfg = tigotar_uniform(t["vocab"], t["hidden"], 4, t["heads"], t["kv"], t["dim"], t["dim"], t["hidden"], t["experts"], t["top"],
                               t["ff"] // t["top"], window, keep, loop=None)
        result["models"][name] = {
            "layers": 4,
            "penozen": _model_throughput(pcfg, 2048, 4, 32, 1100, 20),
            "tigotar": _model_throughput(tcfg, 2048, 4, 32, 1100, 20)}
    print(json.dumps(result), flush=True)
    return result


TIBENEX_SIZES = {
    # latent attention as in PENOZEN_SIZES (+ a query latent of `qrank`); attention whose heads talk: `theads` queries over `tkv`
    # key/value heads of `tdim` / `tvdim` (value row = tkv * tvdim elements); state space: `sheads` heads of `svdim` values,
    # `state` rows per head, `groups` groups; a dense gated feed-forward of `ff`
    "8b-layer": dict(hidden=4096, heads=32, dim=64, rot=64, vdim=128, rank=192, qrank=1536, theads=32, tkv=2, tdim=128, tvdim=128,
                     sheads=128, svdim=64, state=128, groups=8, ff=14336, vocab=32000),
    "3b-layer": dict(hidden=3072, heads=24, dim=64, rot=64, vdim=128, rank=192, qrank=1024, theads=24, tkv=2, tdim=128, tvdim=128,
                     sheads=96, svdim=64, state=128, groups=8, ff=8192, vocab=32000),
    "1b-layer": dict(hidden=2048, heads=32, dim=32, rot=32, vdim=64, rank=96, qrank=768, theads=32, tkv=2, tdim=64, tvdim=64,
                     sheads=64, svdim=64, state=64, groups=8, ff=8192, vocab=32000),
}


def _tibenex_kernel_pairs(s, pz, dev):
    """[(what, Tibenex kernel's record, like kernel's record)]: `s` Tibenex's layer shape, `pz` Penozen's at the same size."""
    from semi_pd_amd import ops
    dt = torch.bfloat16
    W = s["hidden"]
    out = []

    def rec(tm, nbytes=0.0, flops=0.0, vflops=0.0):
        frac = max(nbytes / tm / HBM, flops / tm / MFMA, vflops / tm / VALU)
        return {"us": round(tm * 1e6, 1), "TB_per_s": round(nbytes / tm / 1e12, 2),
                "TFLOP_per_s": round(max(flops, vflops) / tm / 1e12, 1), "of_roofline": round(frac, 3)}

    B, L = 4, 2048
    T = B * L
    B2, C = 32, 2000
    rows, lens = torch.arange(B, device=dev), torch.full((B,), L, device=dev, dtype=torch.int64)
    q_start = torch.arange(B, device=dev, dtype=torch.int32) * L
    q_len = torch.full((B,), L, device=dev, dtype=torch.int32)
    rows2, lens2 = torch.arange(B2, device=dev), torch.full((B2,), C, device=dev, dtype=torch.int64)
    r2t = (torch.arange(T, device=dev, dtype=torch.int32) + 1).view(B, L).contiguous()
    r2t2 = (torch.arange(B2 * C, device=dev, dtype=torch.int32) + 1).view(B2, C).contiguous()
    # ---- the seam: norm after the sum (+ the shift for the next mixer in decode batches) against stream += y, norm -----------
    st_slab = torch.zeros(B2 + 1, W, device=dev)
    st32 = torch.arange(1, B2 + 1, device=dev)
    for Tn in (8192, 32):
        y = torch.randn(Tn, W, device=dev, dtype=dt)
        res = torch.randn(Tn, W, device=dev, dtype=torch.float32)
        w = torch.ones(W, device=dev, dtype=dt)
        if Tn > 32:
            t_new = _timed(lambda: ops.postnorm_stream(y, w, res, 2.0, w, 1e-6))
            nb_new = Tn * W * (2 + 4 + 4 + 2.0)
            what = "stream = norm(alpha stream + scale * y), copy for the next sublayer"
        else:
            t_new = _timed(lambda: ops.postnorm_stream(y, w, res, 2.0, w, 1e-6, shift_mu=w, prev=st_slab, state_indices=st32, seq_lens=lens2))
            nb_new = Tn * W * (2 + 4 + 4 + 2.0 + 8)
            what = "stream = norm(alpha stream + scale * y), the next mixer's shifted input, the previous row in the state"
        t_old = _timed(lambda: ops.rms_stream(y, res, w, 1e-5, 1.0))
        out.append((f"{what}, {Tn} rows of {W} (like: stream += y, next input = RMS norm(stream))",
                    rec(t_new, nbytes=nb_new), rec(t_old, nbytes=Tn * W * (2 + 4 + 4 + 2.0))))
    res = torch.randn(T, W, device=dev, dtype=torch.float32)
    mu = torch.rand(W, device=dev).to(dt)
    st4 = torch.arange(1, B + 1, device=dev)
    t_new = _timed(lambda: ops.token_shift(res, mu, st_slab, st4, lens, q_start, q_len))
    t_old = _timed(lambda: ops.rms_stream(None, res, mu, 1e-5, 1.0))
    out.append((f"token shift of a prompt batch, {T} rows of {W} (reads two fp32 rows per row; like: RMS norm of the stream into the "
                "activation type, one row per row)", rec(t_new, nbytes=T * W * (4 + 4 + 2.0)), rec(t_old, nbytes=T * W * (4 + 2.0))))
    # ---- attention whose heads talk ----------------------------------------------------------------------------------------
    H, G, D, E = s["theads"], s["tkv"], s["tdim"], s["tvdim"]
    pH, pD, pP, pE, pR = pz["heads"], pz["dim"], pz["rot"], pz["vdim"], pz["rank"]
    Tn = 8192
    p = torch.randn(Tn, (H + G) * D + G * E, device=dev, dtype=dt)
    kp = torch.zeros(max(Tn, B2 * C) + 1, G, D, device=dev, dtype=dt)
    vp = torch.zeros(max(Tn, B2 * C) + 1, G, E, device=dev, dtype=dt)
    loc, pos = torch.arange(1, Tn + 1, device=dev), torch.arange(Tn, device=dev)
    qw, kw = torch.ones(H * D, device=dev, dtype=dt), torch.ones(G * D, device=dev, dtype=dt)
    temp = torch.ones(H, device=dev)
    freq = 10000.0 ** (-2.0 * torch.arange(D // 2, dtype=torch.float32, device=dev) / D)
    t_new = _timed(lambda: ops.qk_norm_rope_kv_store(p, H, G, D, E, H * D, (H + G) * D, qw, kw, 1e-6, pos, freq, D, False, 1.0, temp, kp, vp, loc))
    pp = torch.randn(Tn, pH * (pD + pP) + pR + pP + pH * pE, device=dev, dtype=dt)
    pool3 = torch.zeros(Tn + 1, pR + pP, device=dev, dtype=dt)
    q3 = torch.empty(Tn, pH * (pR + pP), device=dev, dtype=dt)
    nw = torch.ones(pR, device=dev, dtype=dt)
    pfreq = 10000.0 ** (-2.0 * torch.arange(pP // 2, dtype=torch.float32, device=dev) / pP)
    t_old = _timed(lambda: ops.latent_prep(pp, pp[:, pH * (pD + pP): pH * (pD + pP) + pR + pP], pH, pD, pP, pR, nw, 1e-5, pos, pfreq, pP, 1.07,
                                           pool3, loc, q3))
    out.append((f"norm of q and k over the whole projection + rotation + temperature + KV store, {Tn} tokens, {H} / {G} heads of {D} / {E} "
                "(like: latent norm, rotation of the shared key part and the heads' rotated query parts, pool store)",
                rec(t_new, nbytes=Tn * 2.0 * (2 * H * D + 2 * G * D + 2 * G * E)), rec(t_old, nbytes=Tn * 2.0 * (2 * (pR + pP) + 2 * pH * pP))))
    kp.normal_()
    vp.normal_()
    q = torch.randn(T, H * D, device=dev, dtype=dt)
    parts = torch.empty(T, H * G * E, device=dev, dtype=dt)
    talk = torch.eye(H, device=dev) + 0.1
    o = torch.empty(T, H * E, device=dev, dtype=dt)

    def talking():
        ops.shared_value_attention_fwd(q, parts, kp, vp, r2t, rows, lens, q_start, q_len, L, D ** -0.5)
        ops.talk_mix(parts, talk, G, out=o)

    t_new = _timed(talking)
    pairs = B * L * (L + 1) / 2
    # the like kernel: Penozen's prompt attention head by head over expanded keys and values, with the sink and the gate
    keys = torch.randn(T, pH, pD + pP, device=dev, dtype=dt)
    vals = torch.randn(T, pH, pE, device=dev, dtype=dt)
    tab = torch.arange(T, device=dev, dtype=torch.int32).view(B, L).contiguous()
    qh = torch.randn(T, pH * (pD + pP), device=dev, dtype=dt)
    oh = torch.empty(T, pH * pE, device=dev, dtype=dt)
    gate = torch.randn(T, pH * pE, device=dev, dtype=dt)
    sink = torch.zeros(pH, device=dev)
    t_old = _timed(lambda: ops.local_attention_fwd(qh, oh, keys, vals, tab, rows, lens, q_start, q_len, L, 0.1, 0.0, 0, sink, gate))
    out.append((f"prompt attention, {B} x {L} tokens, {H} heads of {D} whose weights meet the values of all {G} key/value heads of {E}, + the "
                f"mix of the heads ({H} x {H}) (like: {pH} heads of {pD + pP} / {pE}, causal softmax with a sink and the output gate)",
                rec(t_new, flops=2.0 * H * (D + G * E) * pairs + 2.0 * T * H * H * E), rec(t_old, flops=2.0 * pH * (pD + pP + pE) * pairs)))
    q2 = torch.randn(B2, H * D, device=dev, dtype=dt)
    parts2 = torch.empty(B2, H * G * E, device=dev, dtype=dt)
    o2 = torch.empty(B2, H * E, device=dev, dtype=dt)

    tsplits = max(1, min(16, 512 // (B2 * G * ((H // G + 15) // 16)), C // 128))     # HipAttnBackend.forward_shared_values' rule on 256 CUs

    def talking_decode():
        ops.shared_value_attention_fwd(q2, parts2, kp, vp, r2t2, rows2, lens2, None, None, 1, D ** -0.5, n_splits=tsplits)
        ops.talk_mix(parts2, talk, G, out=o2)

    t_new = _timed(talking_decode)
    pool2 = torch.randn(B2 * C + 1, pR + pP, device=dev, dtype=dt)
    ql = torch.randn(B2, pH * (pR + pP), device=dev, dtype=dt)
    ol = torch.empty(B2, pH * pR, device=dev, dtype=dt)
    splits = max(1, min(16, 512 // (B2 * ((pH + 15) // 16)), C // 128))
    t_old = _timed(lambda: ops.latent_attention_fwd(ql, ol, pool2, pR, r2t2, rows2, lens2, None, None, 1, 0.1, sink, n_splits=splits))
    out.append((f"decode attention, {B2} requests at {C} tokens, {G} key/value heads of {D} / {E}, {tsplits} workgroups share a request's keys, + merge, + the mix of the heads (like: every latent "
                f"row of {pR} + {pP} once for all {pH} heads, {splits} workgroups share a request's keys, + merge)",
                rec(t_new, nbytes=B2 * G * (D + E) * 2.0 * C), rec(t_old, nbytes=B2 * (pR + pP) * 2.0 * C)))
    # ---- the recurrences: a prompt batch and a decode batch ----------------------------------------------------------------
    SH, SE, N, SG, taps = s["sheads"], s["svdim"], s["state"], s["groups"], 4
    inner, Cc = SH * SE, SH * SE + 2 * SG * N
    width = 2 * inner + 2 * SG * N + SH
    conv_w = torch.randn(Cc, taps, device=dev, dtype=dt) * 0.5
    conv_b = torch.zeros(Cc, device=dev, dtype=dt)
    a_log, dt_bias, dsk = torch.zeros(SH, device=dev) - 1.0, torch.zeros(SH, device=dev), torch.ones(SH, device=dev)
    onw = torch.ones(inner, device=dev, dtype=dt)
    S = torch.zeros(B2 + 1, inner * N, device=dev)
    cs = torch.zeros(B2 + 1, (taps - 1) * Cc, device=dev)
    sp = torch.randn(T, width, device=dev, dtype=dt)
    t_new = _timed(lambda: ops.state_space(sp, 0, inner, inner + Cc, conv_w, conv_b, dt_bias, a_log, dsk, onw, 1, 1e-5, S, cs, st4, lens,
                                           q_start, q_len, SH, SG, N, SE), iters=5, warm=1)
    DH, DG, KD, VD = pz["dheads"], pz["kv"], pz["kdim"], pz["dvdim"]
    gd, hv = DG * KD, DH * VD
    dwidth = 2 * gd + 2 * hv + 2 * DH
    offs = [0, gd, 2 * gd, 2 * gd + hv, 2 * gd + 2 * hv, 2 * gd + 2 * hv + DH]
    cw = [torch.randn(n, taps, device=dev, dtype=dt) * 0.5 for n in (gd, gd, hv)]
    da_log, ddt = torch.zeros(DH, device=dev) - 1.0, torch.zeros(DH, device=dev)
    dnw = torch.ones(VD, device=dev, dtype=dt)
    dS = torch.zeros(B2 + 1, DH * KD * VD, device=dev)
    dcs = torch.zeros(B2 + 1, (taps - 1) * (2 * gd + hv), device=dev)
    dp = torch.randn(T, dwidth, device=dev, dtype=dt)
    t_old = _timed(lambda: ops.delta_rule(dp, offs, cw[0], cw[1], cw[2], da_log, ddt, dnw, 1e-5, dS, dcs, st4, lens, q_start, q_len, DH, DG,
                                          KD, VD), iters=5, warm=1)
    out.append((f"state-space recurrence over {B} x {L} tokens, {SH} heads of {N} x {SE} in {SG} groups (convolution, step sizes, the "
                f"recurrence, gate and grouped norm; 4 flop per element of S and token on the vector units; like: gated delta rule, {DH} "
                f"heads of {KD} x {VD}, 8 flop per element)",
                rec(t_new, nbytes=T * 2.0 * (width + inner), vflops=4.0 * T * inner * N),
                rec(t_old, nbytes=T * 2.0 * (dwidth + hv), vflops=8.0 * T * DH * KD * VD)))
    spd = torch.randn(B2, width, device=dev, dtype=dt)
    t_new = _timed(lambda: ops.state_space(spd, 0, inner, inner + Cc, conv_w, conv_b, dt_bias, a_log, dsk, onw, 1, 1e-5, S, cs, st32, lens2,
                                           None, None, SH, SG, N, SE))
    dpd = torch.randn(B2, dwidth, device=dev, dtype=dt)
    t_old = _timed(lambda: ops.delta_rule(dpd, offs, cw[0], cw[1], cw[2], da_log, ddt, dnw, 1e-5, dS, dcs, st32, lens2, None, None, DH, DG,
                                          KD, VD))
    out.append((f"state-space decode step, {B2} requests (reads and writes {inner * N * 4 / 1e6:.1f} MB of state per request; like: gated "
                f"delta rule decode step, {DH * KD * VD * 4 / 1e6:.1f} MB per request)",
                rec(t_new, nbytes=B2 * inner * N * 4.0 * 2), rec(t_old, nbytes=B2 * DH * KD * VD * 4.0 * 2)))
    return out


def main_tibenex(args) -> dict:
    from semi_pd_amd.models.penozen import penozen_uniform
    from semi_pd_amd.models.tibenex import tibenex_uniform
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    names = [n for n in (getattr(args, "arch_sizes", "") or ",".join(TIBENEX_SIZES)).split(",") if n]
    result = {"what": "Tibenex next to Penozen at equal layer sizes", "dtype": "bf16", "data": "synthetic", "models": {}, "kernels": {}}
    for name in names:
        s, pz = TIBENEX_SIZES[name], PENOZEN_SIZES[name]
        result["kernels"][name] = [
            {"kernel": what, "tibenex": new, "like": old,
             "roofline_fraction_ratio": round(new["of_roofline"] / max(old["of_roofline"], 1e-9), 2)}
            for what, new, old in _tibenex_kernel_pairs(s, pz, dev)]
        tcfg = tibenex_uniform(s["vocab"], s["hidden"], "lmam", s["ff"], s["theads"], s["tkv"], s["tdim"], s["tvdim"], s["rot"], s["rank"],
                               s["qrank"], s["sheads"], s["svdim"], s["state"], s["groups"], latent_heads=s["heads"], latent_dim=s["dim"],
                               latent_vdim=s["vdim"])
        pcfg = penozen_uniform(pz["vocab"], pz["hidden"], "adad", pz["heads"], pz["dim"], pz["rot"], pz["vdim"], pz["rank"], pz["dheads"],
                               pz["kv"], pz["kdim"], pz["dvdim"], pz["experts"], pz["top"], pz["ff"] // pz["top"])
        result["models"][name] = {
            "layers": 4,
            "tibenex": _model_throughput(tcfg, 2048, 4, 32, 1100, 20),
            "penozen": _model_throughput(pcfg, 2048, 4, 32, 1100, 20)}
    print(json.dumps(result), flush=True)
    return result


def main(args) -> dict:
    if getattr(args, "arch_design", "kudirax") == "tibenex":
        return main_tibenex(args)
    if getattr(args, "arch_design", "kudirax") == "tigotar":
        return main_tigotar(args)
    if getattr(args, "arch_design", "kudirax") == "penozen":
        return main_penozen(args)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    chunk = int(getattr(args, "arch_chunk", 1024) or 0)
    names = [n for n in (getattr(args, "arch_sizes", "") or ",".join(SIZES)).split(",") if n]
    result = {"what": "Kudirax next to Llama at equal layer sizes", "dtype": "bf16", "data": "synthetic", "block": chunk,
              "models": {}, "kernels": {}}
    for name in names:
        s = SIZES[name]
        result["kernels"][name] = [
            {"kernel": what, "kudirax": new, "llama": old,
             "roofline_fraction_ratio": round(new["of_roofline"] / max(old["of_roofline"], 1e-9), 2)}
            for what, new, old in _kernel_pairs(s, chunk, dev)]
        kcfg, lcfg = _configs(s, chunk)
        result["models"][name] = {
            "layers": s["layers"],
            "kudirax": _model_throughput(kcfg, 2048, 4, 32, 1100, 20),
            "llama": _model_throughput(lcfg, 2048, 4, 32, 1100, 20)}
    print(json.dumps(result), flush=True)
    return result
