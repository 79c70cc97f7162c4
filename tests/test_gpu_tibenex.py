"""Tibenex on the GPU against the plain host statement (oracle/tibenex.py): every mechanism alone, then whole models through
the replay scheduler (whole prompts, token-by-token decoding, portions down to two tokens, unequal requests side by side,
slots and state rows that change hands) and greedy generation through the Engine."""
import json
import os

import pytest
import torch

from oracle import tibenex as O

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = {torch.float32: dict(rtol=3e-5, atol=3e-5), torch.bfloat16: dict(rtol=3e-2, atol=3e-2)}


def _batch(parts):
    """parts: [(slot, lo, hi)] -> (slots, lengths after the step, q_start, q_len) on the device."""
    slots = torch.tensor([s for s, _, _ in parts], device=DEV)
    lens = torch.tensor([hi for _, _, hi in parts], device=DEV)
    n = torch.tensor([hi - lo for _, lo, hi in parts], dtype=torch.int32, device=DEV)
    return slots, lens, (torch.cumsum(n, 0) - n).int(), n


# ----------------------------------------------------------------------------------------------- the seam: norm after the sum
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width", [(1, 8), (5, 100), (37, 256), (3, 4104)])
def test_postnorm_seam(dtype, rows, width):
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(width)
    w = (1 + 0.2 * torch.randn(width, generator=g)).to(dtype)
    ls = (0.5 * torch.randn(width, generator=g)).to(dtype)
    y = (2 * torch.randn(rows, width, generator=g)).to(dtype)
    x = 3 * torch.randn(rows, width, generator=g)
    eps, alpha = 1e-5, 1.7
    want = O.rms_norm(alpha * x + y.float() * ls.float(), w, eps)
    stream = x.to(DEV)
    out = ops.postnorm_stream(y.to(DEV), ls.to(DEV), stream, alpha, w.to(DEV), eps)
    torch.testing.assert_close(stream.cpu(), want, rtol=1e-5, atol=1e-5)                  # the stream keeps fp32
    torch.testing.assert_close(out.float().cpu(), want, **TOL[dtype])
    stream = x.to(DEV)                                                                    # no layer scale, no copy wanted
    assert ops.postnorm_stream(y.to(DEV), None, stream, alpha, w.to(DEV), eps, want_out=False) is None
    torch.testing.assert_close(stream.cpu(), O.rms_norm(alpha * x + y.float(), w, eps), rtol=1e-5, atol=1e-5)
    tiny = torch.full((2, width), 1e-4)                                                   # eps inside the root matters here
    stream = tiny.to(DEV)
    ops.postnorm_stream(None, None, stream, 1.0, w.to(DEV), 1e-3, want_out=False)
    torch.testing.assert_close(stream.cpu(), O.rms_norm(tiny, w, 1e-3), rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_token_shift_with_the_previous_row_in_the_state(dtype):
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(3)
    W = 72
    mu = torch.rand(W, generator=g).to(dtype)
    seqs = {1: torch.randn(40, W, generator=g), 3: torch.randn(9, W, generator=g), 2: torch.randn(1, W, generator=g)}
    want = {s: O.token_shift(x, mu) for s, x in seqs.items()}
    slab = torch.full((5, W + 6), 123.0, device=DEV)            # state rows full of something else; columns 2 .. 2 + W are ours
    prev = slab[:, 2: 2 + W]

    def run(parts, decode=False, fused=False):
        x = torch.cat([seqs[s][lo:hi] for s, lo, hi in parts]).to(DEV)
        slots, lens, start, n = _batch(parts)
        if fused:          # the seam's own form for one row per request: the stream is normed first (weight 1, nothing added)
            out = ops.postnorm_stream(None, None, x.clone(), 1.0, torch.ones(W, dtype=dtype, device=DEV), 1e-6, shift_mu=mu.to(DEV),
                                      prev=prev, state_indices=slots, seq_lens=lens)
            for at, (s, lo, hi) in enumerate(parts):
                normed = O.rms_norm(seqs[s], None, 1e-6)
                torch.testing.assert_close(out[at: at + 1].float().cpu(), O.token_shift(normed[:hi], mu)[lo:hi], **TOL[dtype])
                torch.testing.assert_close(prev[s].cpu(), normed[lo], rtol=1e-5, atol=1e-5)
            return
        out = ops.token_shift(x, mu.to(DEV), prev, slots, lens, None if decode else start, None if decode else n)
        at = 0
        for s, lo, hi in parts:
            torch.testing.assert_close(out[at: at + hi - lo].float().cpu(), want[s][lo:hi], **TOL[dtype])
            at += hi - lo

    run([(1, 0, 17), (3, 0, 2), (2, 0, 1)])                      # first portions: zeros in front of position 0
    run([(3, 2, 4), (1, 17, 18)])                                # the row in front comes from the state row
    run([(1, 18, 19), (3, 4, 5)], decode=True)
    run([(3, 5, 9), (1, 19, 40)])
    seqs[2], want[2] = seqs[3], want[3]                          # slot 2 changes hands: what the row held is not looked at
    run([(2, 0, 1)])
    run([(2, 1, 2)], decode=True)
    assert torch.equal(slab[:, :2].cpu(), torch.full((5, 2), 123.0)) and torch.equal(slab[:, 2 + W:].cpu(), torch.full((5, 4), 123.0))
    # the seam that shifts for the next mixer (decode batches); the state rows hold normed streams there
    for s in (1, 3):
        prev[s] = 55.0                                           # position 0 ignores what the row holds
        for t in range(4):
            run([(s, t, t + 1)], fused=True)


def test_embedding_and_head_gates():
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(9)
    for dtype in (torch.float32, torch.bfloat16):
        emb = torch.randn(300, 40, generator=g).to(dtype)
        ids = torch.randint(0, 300, (23,), generator=g)
        out = ops.embed_stream(ids.to(DEV), emb.to(DEV), 2.5)
        assert out.dtype == torch.float32
        torch.testing.assert_close(out.cpu(), emb[ids].float() * 2.5, rtol=1e-6, atol=1e-6)
        x = torch.randn(7, 3 * 20 + 4, generator=g).to(dtype)
        gate = torch.randn(7, 3 + 5, generator=g).to(dtype)
        xd = x.to(DEV)
        ops.sigmoid_gate_heads_(xd[:, 4:], gate.to(DEV)[:, 5:])
        want = x.float().clone()
        want[:, 4:] = (x[:, 4:].float().view(7, 3, 20) * torch.sigmoid(gate[:, 5:].float()).view(7, 3, 1)).view(7, 60)
        torch.testing.assert_close(xd.float().cpu(), want, **TOL[dtype])


# ----------------------------------------------------------------------------------------------- preparation steps
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,D,Pr,R,rot,scaling", [(4, 48, 16, 96, 16, True), (3, 20, 12, 36, 8, False), (1, 8, 8, 16, 8, True), (2, 16, 4, 24, 0, False)])
def test_latent_preparation_in_halves(dtype, H, D, Pr, R, rot, scaling):
    from semi_pd_amd import ops
    from semi_pd_amd.models.penozen import stretched_frequencies
    g = torch.Generator().manual_seed(R + rot)
    T, N, eps = 11, 40, 1e-5
    rotd = {"base": 5000.0, "dims": rot}
    if scaling:
        rotd["scaling"] = {"factor": 4.0, "original": 256, "fast": 16.0, "slow": 2.0}
    q = torch.randn(T, H * (D + Pr), generator=g).to(dtype)
    lat = torch.randn(T, 5 + R + Pr, generator=g).to(dtype)       # the latent is a column range of another projection
    nw = (1 + 0.2 * torch.randn(R, generator=g)).to(dtype)
    pos = torch.tensor([0, 1, 2, 3, 500, 501, 77, 4000, 4001, 9, 10])
    loc = (torch.randperm(N - 1, generator=g) + 1)[:T]
    freq, mscale = stretched_frequencies(rot, rotd["base"], rotd.get("scaling")) if rot else (None, 1.0)
    pool = torch.zeros(N, R + Pr, dtype=dtype, device=DEV)
    q_out = torch.zeros(T, H * (R + Pr), dtype=dtype, device=DEV)
    ops.latent_prep(q.to(DEV), lat.to(DEV)[:, 5:], H, D, Pr, R, nw.to(DEV), eps, pos.to(DEV), freq.to(DEV) if rot else None, rot, mscale,
                    pool, loc.to(DEV), q_out, halves=True)

    def rotated(x, n):          # the oracle turns positions 0 .. T-1 of one sequence: one call per token at its own position
        x = x.view(T, n, Pr)
        return torch.stack([O.rotate(x[t: t + 1].expand(int(pos[t]) + 1, n, Pr), rotd, halves=True)[-1] if rot else x[t].float()
                            for t in range(T)])

    want_pool = torch.cat([O.rms_norm(lat[:, 5: 5 + R], nw, eps), rotated(lat[:, 5 + R:].contiguous(), 1).view(T, Pr)], 1)
    tol = TOL[dtype] if dtype == torch.float32 else dict(rtol=2e-2, atol=3e-2)
    # fp32 sines of angles in the thousands: the two computations of the angle part by ~1e-4 there
    if dtype == torch.float32:
        tol = dict(rtol=1e-3, atol=1e-3)
    torch.testing.assert_close(pool[loc.to(DEV)].float().cpu(), want_pool, **tol)
    want_q = rotated(q.view(T, H, D + Pr)[..., D:].contiguous(), H)
    torch.testing.assert_close(q_out.view(T, H, R + Pr)[..., R:].float().cpu(), want_q, **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,D,E,rot", [(8, 4, 64, 32, 32), (3, 3, 20, 12, 20), (4, 1, 32, 16, 0), (1, 1, 8, 8, 2), (6, 2, 24, 40, 10)])
def test_whole_projection_norm_rotation_and_store(dtype, H, G, D, E, rot):
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(H * D + rot)
    T, N, eps = 9, 30, 1e-5
    rotd = {"base": 300.0, "dims": rot}
    extra = 8
    row = torch.randn(T, H * D + G * D + G * E + extra, generator=g).to(dtype)
    qw, kw = (1 + 0.3 * torch.randn(H * D, generator=g)).to(dtype), (1 + 0.3 * torch.randn(G * D, generator=g)).to(dtype)
    temp = 0.5 + torch.rand(H, generator=g)
    pos = torch.tensor([0, 1, 2, 40, 41, 7, 300, 301, 5])
    loc = (torch.randperm(N - 1, generator=g) + 1)[:T]
    kp, vp = torch.zeros(N, G, D, dtype=dtype, device=DEV), torch.zeros(N, G, E, dtype=dtype, device=DEV)
    freq = torch.tensor([rotd["base"] ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32) if rot else None
    rd = row.to(DEV)
    ops.qk_norm_rope_kv_store(rd, H, G, D, E, H * D, (H + G) * D, qw.to(DEV), kw.to(DEV), eps, pos.to(DEV), freq.to(DEV) if rot else None,
                              rot, False, 1.0, temp.to(DEV), kp, vp, loc.to(DEV))

    def rotated(x, n):
        x = x.view(T, n, D)
        return torch.stack([O.rotate(x[t: t + 1].expand(int(pos[t]) + 1, n, D), rotd, halves=False)[-1] if rot else x[t].float()
                            for t in range(T)])

    q_want = rotated(O.rms_norm(row[:, : H * D], qw, eps), H) * temp.view(1, H, 1)
    k_want = rotated(O.rms_norm(row[:, H * D: (H + G) * D], kw, eps), G)
    tol = dict(rtol=1e-4, atol=1e-4) if dtype == torch.float32 else dict(rtol=2e-2, atol=4e-2)
    torch.testing.assert_close(rd[:, : H * D].float().cpu().view(T, H, D), q_want, **tol)
    torch.testing.assert_close(kp[loc.to(DEV)].float().cpu(), k_want, **tol)
    assert torch.equal(vp[loc.to(DEV)].cpu().view(T, G * E), row[:, (H + G) * D: (H + G) * D + G * E])
    assert torch.equal(rd[:, (H + G) * D:].cpu(), row[:, (H + G) * D:])                    # v and what lies behind it are left alone


# ----------------------------------------------------------------------------------------------- attention whose heads talk
def _talking_truth(q, k, v, talk, scale):
    """q [T, H, D] (the last T positions), k [S, G, D], v [S, G, E] -> [T, H, E]; weights mixed after the softmax."""
    T, H, _ = q.shape
    S, G, E = v.shape
    of = torch.arange(H) // (H // G)
    s = torch.einsum("ihd,jhd->hij", q.float(), k.float()[:, of]) * scale
    hidden = torch.arange(S).view(1, 1, S) > torch.arange(S - T, S).view(1, T, 1)
    p = torch.softmax(s.masked_fill(hidden, float("-inf")), -1)
    p = torch.einsum("hg,gij->hij", talk.float(), p)
    return (p @ v.float()[:, of].transpose(0, 1)).transpose(0, 1)


@pytest.mark.parametrize("dtype,form", [(torch.float32, 0), (torch.bfloat16, 0), (torch.bfloat16, 1)])
@pytest.mark.parametrize("H,G,D,E", [(8, 4, 64, 32), (8, 8, 32, 16), (4, 1, 32, 48), (3, 1, 20, 12), (6, 3, 40, 24)])
def test_attention_over_shared_values_with_mixed_heads(dtype, form, H, G, D, E):
    """Prompt portions behind cached prefixes, single tokens beside them and a decode batch, slots scattered over the pool;
    a far key that one head's query is lined up with has to carry that head's weights into every head it talks to."""
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(H * 100 + D)
    lens = [700, 65, 1, 130]                                       # tokens each request holds after the prompt step
    news = [40, 65, 1, 2]
    N = sum(lens) + 40
    scale = D ** -0.5
    talk = torch.eye(H) + 0.5 * torch.randn(H, H, generator=g)
    ks = [torch.randn(n + 1, G, D, generator=g) for n in lens]     # one more for the decode step
    vs = [torch.randn(n + 1, G, E, generator=g) for n in lens]
    qs = [torch.randn(n + 1, H, D, generator=g) for n in lens]
    # request 0: the last query of head 1 lines up with key 3 (far back) of its key head
    if H > 1:
        qs[0][lens[0] - 1, 1] = 12.0 * ks[0][3, 1 // (H // G)]
    ks, vs, qs = [[t.to(dtype) for t in x] for x in (ks, vs, qs)]
    perm = torch.randperm(N - 1, generator=g) + 1
    kp, vp = torch.zeros(N, G, D, dtype=dtype), torch.zeros(N, G, E, dtype=dtype)
    r2t = torch.zeros(6, max(lens) + 8, dtype=torch.int32)
    rows = [4, 1, 3, 2]
    at = 0
    for b, n in enumerate(lens):
        slots = perm[at: at + n + 1]
        at += n + 1
        kp[slots], vp[slots] = ks[b], vs[b]
        r2t[rows[b], : n + 1] = slots.int()
    kp, vp, r2t = kp.to(DEV), vp.to(DEV), r2t.to(DEV)
    rp = torch.tensor(rows, device=DEV)
    q = torch.cat([qs[b][lens[b] - news[b]: lens[b]] for b in range(4)]).view(-1, H * D).to(DEV)
    n_new = torch.tensor(news, dtype=torch.int32, device=DEV)
    parts = torch.empty(q.shape[0], H * G * E, dtype=dtype, device=DEV)
    ops.shared_value_attention_fwd(q, parts, kp, vp, r2t, rp, torch.tensor(lens, device=DEV), (torch.cumsum(n_new, 0) - n_new).int(),
                                   n_new, max(news), scale, form=form)
    out = ops.talk_mix(parts, talk.to(DEV), G).float().cpu().view(-1, H, E)
    tol = dict(rtol=2e-4, atol=2e-4) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)
    at = 0
    for b in range(4):
        want = _talking_truth(qs[b][lens[b] - news[b]: lens[b]], ks[b][: lens[b]], vs[b][: lens[b]], talk, scale)
        torch.testing.assert_close(out[at: at + news[b]], want, **tol)
        at += news[b]
    # the far key: head 1's own weights sit on key 3 of 700, so its block of `parts` holds the values of that one token
    if H > 1:
        own = parts.view(-1, H, G, E)[news[0] - 1, 1].float().cpu()
        torch.testing.assert_close(own, vs[0][3].float(), rtol=2e-2, atol=2e-2)
    # a decode batch: one more token each
    lens1 = [n + 1 for n in lens]
    q1 = torch.stack([qs[b][lens[b]] for b in range(4)]).view(4, H * D).to(DEV)
    for n_splits in (1, 3):                                    # (the keys of a request shared out over three workgroups)
        parts = torch.empty(4, H * G * E, dtype=dtype, device=DEV)
        ops.shared_value_attention_fwd(q1, parts, kp, vp, r2t, rp, torch.tensor(lens1, device=DEV), None, None, 1, scale, form=form,
                                       n_splits=n_splits)
        out = ops.talk_mix(parts, talk.to(DEV), G).float().cpu().view(4, H, E)
        for b in range(4):
            want = _talking_truth(qs[b][lens[b]: lens[b] + 1], ks[b], vs[b], talk, scale)
            torch.testing.assert_close(out[b: b + 1], want, **tol)


# ----------------------------------------------------------------------------------------------- state-space recurrence
def _ssm_truth(p, w, m, eps):
    """The mixer of the plain statement behind its input projection: p [T, z | x | B | C | dt] -> [T, H E]."""
    H, E, N, G, parts = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    T, inner = p.shape[0], H * E
    p = p.float()
    z, xbc, dt = p[:, :inner], p[:, inner: 2 * inner + 2 * G * N], p[:, 2 * inner + 2 * G * N:]
    xbc = O.causal_conv_silu(xbc, w["conv"], w["conv.b"])
    of = torch.arange(H) // (H // G)
    B = xbc[:, inner: inner + G * N].view(T, G, N)[:, of]
    C = xbc[:, inner + G * N:].view(T, G, N)[:, of]
    dt = torch.nn.functional.softplus(dt + w["dt_bias"].float())
    y = O.state_space_scan(xbc[:, :inner].view(T, H, E), dt, torch.exp(w["A_log"].float()), B, C, w["D"].float()).reshape(T, inner)
    y = y * torch.nn.functional.silu(z)
    return O.rms_norm(y.view(T, parts, inner // parts), None, eps).reshape(T, inner) * w["norm"].float()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,E,N,G,parts,taps", [(6, 40, 32, 3, 2, 4), (3, 20, 8, 1, 1, 1), (4, 70, 48, 4, 4, 2), (2, 16, 128, 2, 1, 4),
                                                (2, 8, 200, 1, 2, 3), (64, 64, 16, 8, 8, 4)])
def test_state_space_over_portions_and_decode_steps(dtype, H, E, N, G, parts, taps):
    """Whole sequences, portions down to one token, decode batches (the one-launch form where the state is small, the four
    launches where it is not), rows that change hands; long sequences for the decay to matter."""
    from semi_pd_amd import ops
    g = torch.Generator().manual_seed(H * E + N)
    m = {"heads": H, "vdim": E, "state": N, "groups": G, "norm_groups": parts}
    inner, C = H * E, H * E + 2 * G * N
    eps = 1e-5
    w = {"conv": (torch.randn(C, taps, generator=g) * 0.5).to(dtype), "conv.b": (0.2 * torch.randn(C, generator=g)).to(dtype),
         "dt_bias": torch.randn(H, generator=g) * 0.5 - 1, "A_log": torch.randn(H, generator=g) * 0.5 - 1,
         "D": torch.randn(H, generator=g), "norm": (1 + 0.1 * torch.randn(inner, generator=g)).to(dtype)}
    cols = 2 * inner + 2 * G * N + H
    seqs = {1: torch.randn(150, cols, generator=g).to(dtype), 2: torch.randn(37, cols, generator=g).to(dtype),
            3: torch.randn(3, cols, generator=g).to(dtype)}
    want = {s: _ssm_truth(p, w, m, eps) for s, p in seqs.items()}
    sw, cw = inner * N, max((taps - 1) * C, 1)
    slab = torch.full((5, 3 + sw + cw + 2), 7.0, device=DEV)     # rows full of something else
    state, conv_state = slab[:, 3: 3 + sw], slab[:, 3 + sw: 3 + sw + cw]
    wd = {k: v.to(DEV) for k, v in w.items()}
    tol = dict(rtol=2e-4, atol=2e-4) if dtype == torch.float32 else dict(rtol=3e-2, atol=3e-2)

    def run(partsl, decode=False):
        p = torch.cat([seqs[s][lo:hi] for s, lo, hi in partsl]).to(DEV)
        slots, lens, start, n = _batch(partsl)
        out = ops.state_space(p, 0, inner, inner + C, wd["conv"], wd["conv.b"], wd["dt_bias"], wd["A_log"], wd["D"], wd["norm"], parts,
                              eps, state, conv_state if taps > 1 else None, slots, lens, None if decode else start,
                              None if decode else n, H, G, N, E)
        at = 0
        for s, lo, hi in partsl:
            torch.testing.assert_close(out[at: at + hi - lo].float().cpu(), want[s][lo:hi], **tol)
            at += hi - lo

    run([(1, 0, 100), (2, 0, 2), (3, 0, 1)])
    run([(1, 100, 101), (2, 2, 3), (3, 1, 2)], decode=True)
    run([(2, 3, 20), (1, 101, 103), (3, 2, 3)])
    run([(1, 103, 104)], decode=True)
    run([(1, 104, 150), (2, 20, 37)])
    seqs[3], want[3] = seqs[2], want[2]                          # row 3 changes hands: what it held is not looked at
    run([(3, 0, 1)])
    run([(3, 1, 2)], decode=True)
    run([(3, 2, 37)])
    assert torch.equal(slab[:, :3].cpu(), torch.full((5, 3), 7.0)) and torch.equal(slab[:, -2:].cpu(), torch.full((5, 2), 7.0))
    assert torch.equal(slab[0].cpu(), torch.full((slab.shape[1],), 7.0)) and torch.equal(slab[4].cpu(), torch.full((slab.shape[1],), 7.0))


# ----------------------------------------------------------------------------------------------- whole models
def _latent(heads, dim, rot_dim, vdim, kv_rank, q_rank, dims=None, scaling=None, base=5000.0):
    rot = {"base": base, "dims": rot_dim if dims is None else dims}
    if scaling:
        rot["scaling"] = {"factor": scaling, "original": 64, "fast": 16.0, "slow": 2.0}
    return "latent_attention", {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
                                "scale": (dim + rot_dim) ** -0.5, "rot": rot}


def _attn(heads, kv_heads, dim, vdim, dims, base=300.0):
    return "attention", {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "rot": {"base": base, "dims": dims}}


def _ssm(heads, vdim, state, groups, norm_groups, conv):
    return "mamba2", {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups, "conv": conv}


def _layer(mixer, ff):
    return {"type": mixer[0], "mixer": mixer[1], "mlp": {"kind": "dense", "ff": ff} if ff else None}


def _config(vocab, width, layers, eps=1e-5, scale=2.0, alpha=2.0):
    return {"architecture": "Tibenex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "postln_alpha": alpha,
            "embedding": {"scale": scale}, "layers": layers}


CONFIGS = {
    # the recurrence first, layers of different geometry, one without feed-forward, a partial rotation, with and without
    # stretching, as many key/value heads as heads and fewer
    "mixed": _config(200, 64, [_layer(_ssm(4, 24, 16, 2, 2, 4), 96),
                               _layer(_attn(4, 2, 32, 32, 8), None),
                               _layer(_latent(4, 16, 16, 24, 48, 40, scaling=4.0), 64),
                               _layer(_attn(2, 2, 64, 16, 64), 128),
                               _layer(_ssm(2, 32, 64, 1, 1, 2), 64),
                               _layer(_latent(2, 32, 32, 16, 32, 24, dims=16), None)]),
    # sizes of one; a convolution of one tap; alpha and the embedding scale 1
    "minimal": _config(64, 32, [_layer(_ssm(1, 8, 8, 1, 1, 1), 16), _layer(_attn(1, 1, 8, 8, 2), 16), _layer(_latent(1, 8, 8, 8, 16, 8), 16)],
                       eps=1e-6, scale=1.0, alpha=1.0),
    # sizes no vector path takes
    "awkward": _config(301, 100, [_layer(_attn(3, 1, 20, 12, 6), 28), _layer(_ssm(3, 20, 12, 3, 3, 3), None),
                                  _layer(_latent(3, 20, 10, 12, 36, 28, dims=6, scaling=2.0), 30), _layer(_ssm(5, 12, 40, 1, 5, 5), 36)],
                       alpha=3.5),
    "attention_only": _config(128, 64, [_layer(_attn(8, 2, 32, 16, 32), 64), _layer(_latent(8, 16, 16, 16, 32, 48, scaling=2.0), None),
                                        _layer(_attn(2, 1, 64, 64, 16), 64)]),
    "recurrence_only": _config(128, 64, [_layer(_ssm(2, 64, 64, 1, 2, 4), None), _layer(_ssm(8, 16, 16, 4, 1, 4), 64)]),
}


def _write_checkpoint(path, cfg, seed):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    w = O.random_weights(cfg, seed)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(path, "model.safetensors"))
    return w


def _scheduler(path, dtype, max_tokens, max_requests=4, graphs=True):
    from semi_pd_amd.entrypoints.engine import _build_runner
    from semi_pd_amd.managers.replay_scheduler import ReplayScheduler
    from semi_pd_amd.semi_pd.utils import InstanceRole
    from semi_pd_amd.server_args import ServerArgs
    sa = ServerArgs(model_path=path, load_format="auto", dtype=dtype, context_length=max_tokens, max_total_tokens=max_tokens,
                    max_running_requests=max_requests, cuda_graph_max_bs=max_requests, disable_cuda_graph=not graphs,
                    skip_tokenizer_init=True)
    mr = _build_runner(sa, 0, 0, InstanceRole.OTHER, 29653, max_total_tokens=max_tokens)
    mr.init_attention_backend()
    mr.init_cuda_graphs()
    return ReplayScheduler(sa, mr)


def _tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def _run_schedule(sched, prompts, schedule):
    """schedule: steps of [(request name, token count)]; every position's logits are asked for.  Returns name -> [T, vocab]."""
    at = {n: 0 for n in prompts}
    got = {n: [] for n in prompts}
    for step in schedule:
        entries, end = [], []
        for name, count in step:
            lo, hi = at[name], at[name] + count
            entries.append({"id": name, "tokens": prompts[name][lo:hi], "want": list(range(count))})
            at[name] = hi
            if hi == len(prompts[name]):
                end.append(name)
        logits = sched.replay_step(entries, end).cpu()
        k = 0
        for name, count in step:
            got[name].append(logits[k: k + count])
            k += count
    assert all(at[n] == len(prompts[n]) for n in prompts)
    return {n: torch.cat(v) for n, v in got.items()}


def _rel_err(got, want, outliers=False):
    """Error of the positions (mean taken off, relative to the spread of the position's logits): the largest one; with
    `outliers` (16-bit runs) an outlier counts half as long as 97 of 100 positions stay below the figure returned (a norm
    behind a sum that nearly cancels passes 16-bit rounding on enlarged)."""
    d = (got - want) - (got - want).mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / want.std(-1)
    if not outliers:
        return e.max().item()
    return max(e.max().item() / 2, torch.quantile(e, 0.97).item())


LIMIT = {"float32": 3e-5, "bfloat16": 4e-2}


@pytest.fixture(scope="module", params=["float32", "bfloat16"])
def mixed_model(request, tmp_path_factory):
    path = str(tmp_path_factory.mktemp("tibenex_mixed"))
    cfg = CONFIGS["mixed"]
    w = _write_checkpoint(path, cfg, seed=11)
    # a pool far smaller than the tokens that pass through it: slots, rows and state rows come back and are used again
    sched = _scheduler(path, request.param, max_tokens=448)
    lens = {"a": 150, "b": 1, "c": 97, "d": 2, "e": 64, "f": 131}
    prompts = {n: _tokens(k, cfg["vocab"], seed=ord(n)) for n, k in lens.items()}
    truth = {n: O.forward(cfg, w, t) for n, t in prompts.items()}
    return request.param, sched, prompts, truth, (cfg, w)


def _pools_are_whole(sched):
    assert sched.token_to_kv_pool_allocator.available_size() == 448 and sched.req_to_token_pool.available_size() == 5
    assert sched.model_runner.state_pool.available_size() == 4 and not sched.live


def test_every_layer_matches_the_plain_model(mixed_model):
    dtype, sched, prompts, truth, (cfg, w) = mixed_model
    t = prompts["c"]
    _, layers = O.forward_layers(cfg, w, t)
    seen = []
    sched.model_runner.model.layer_probe = lambda i, x: seen.append(x.detach().float().cpu().clone())
    try:
        sched.replay_step([{"id": "p", "tokens": t, "want": [0]}], ["p"])
    finally:
        sched.model_runner.model.layer_probe = None
    assert len(seen) == len(layers)
    for got, want in zip(seen, layers):
        err = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt()
        if dtype == "float32":
            assert err.max().item() < 2e-5
        else:
            assert torch.quantile(err, 0.97).item() < 3e-2 and err.max().item() < 8e-2
    _pools_are_whole(sched)


def test_whole_prompts_match_the_plain_model(mixed_model):
    dtype, sched, prompts, truth, _ = mixed_model
    for n in prompts:
        got = _run_schedule(sched, {n: prompts[n]}, [[(n, len(prompts[n]))]])
        assert _rel_err(got[n], truth[n], dtype != "float32") < LIMIT[dtype], n
    _pools_are_whole(sched)


def test_decoding_token_by_token_matches_the_prompt_pass(mixed_model):
    dtype, sched, prompts, truth, _ = mixed_model
    # from the very first token on (zeros in front of it, an empty state), and behind a prompt
    got = _run_schedule(sched, {"a": prompts["a"]}, [[("a", 1)]] * 150)
    assert _rel_err(got["a"], truth["a"], dtype != "float32") < LIMIT[dtype]
    got = _run_schedule(sched, {"f": prompts["f"]}, [[("f", 90)]] + [[("f", 1)]] * 41)
    assert _rel_err(got["f"], truth["f"], dtype != "float32") < LIMIT[dtype]
    _pools_are_whole(sched)


def test_portions_of_every_size_down_to_two(mixed_model):
    dtype, sched, prompts, truth, _ = mixed_model
    for cuts in ([2] * 75, [64, 2, 3, 17, 64], [1, 2, 1, 146], [149, 1], [33, 31, 32, 54]):
        assert sum(cuts) == 150
        got = _run_schedule(sched, {"a": prompts["a"]}, [[("a", c)] for c in cuts])
        assert _rel_err(got["a"], truth["a"], dtype != "float32") < LIMIT[dtype], cuts
    _pools_are_whole(sched)


def test_unequal_requests_side_by_side_with_reuse(mixed_model):
    dtype, sched, prompts, truth, _ = mixed_model
    schedule = [[("a", 100), ("b", 1), ("c", 2)],
                [("a", 1), ("c", 60), ("d", 2)],             # b and d end: their rows, slots and state rows go back
                [("a", 1), ("c", 1), ("e", 33), ("f", 2)],   # e and f take them over
                [("c", 34), ("e", 1), ("f", 100)],           # a sits out a step
                [("a", 48), ("e", 30), ("f", 29)]]
    got = _run_schedule(sched, prompts, schedule)
    for n in prompts:
        assert _rel_err(got[n], truth[n], dtype != "float32") < LIMIT[dtype], n
    _pools_are_whole(sched)
    # all four live requests decode side by side through one captured graph
    four = {n: prompts[n][:64] for n in ("a", "c", "e", "f")}
    got = _run_schedule(sched, four, [[(n, 40) for n in four]] + [[(n, 1) for n in four]] * 24)
    for n in four:
        assert _rel_err(got[n], truth[n][:64], dtype != "float32") < LIMIT[dtype], n
    _pools_are_whole(sched)


def test_logits_do_not_depend_on_the_cut_or_the_neighbours(mixed_model):
    dtype, sched, prompts, truth, _ = mixed_model
    alone = _run_schedule(sched, {"c": prompts["c"]}, [[("c", 97)]])["c"]
    cut = _run_schedule(sched, {"c": prompts["c"], "e": prompts["e"]}, [[("c", 50), ("e", 64)], [("c", 47)]])["c"]
    assert _rel_err(cut, alone, dtype != "float32") < (5e-5 if dtype == "float32" else 4e-2)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["minimal", "awkward", "attention_only", "recurrence_only"])
def test_other_sizes_and_orders(name, dtype, tmp_path):
    cfg = CONFIGS[name]
    w = _write_checkpoint(str(tmp_path), cfg, seed=5)
    sched = _scheduler(str(tmp_path), dtype, max_tokens=256)
    prompts = {"x": _tokens(90, cfg["vocab"], 1), "y": _tokens(37, cfg["vocab"], 2)}
    truth = {n: O.forward(cfg, w, t) for n, t in prompts.items()}
    got = _run_schedule(sched, prompts, [[("x", 60), ("y", 2)], [("x", 1), ("y", 30)], [("x", 1), ("y", 1)], [("x", 28), ("y", 4)]])
    for n in prompts:
        assert _rel_err(got[n], truth[n], dtype != "float32") < LIMIT[dtype], n
    got = _run_schedule(sched, {"x": prompts["x"]}, [[("x", 70)]] + [[("x", 1)]] * 20)
    assert _rel_err(got["x"], truth["x"], dtype != "float32") < LIMIT[dtype]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_eager_decode_steps_with_the_separate_shift_launch(dtype, tmp_path, monkeypatch):
    """Without captured graphs, and with the token shift of decode batches as a launch of its own instead of inside the seam."""
    monkeypatch.setenv("SEMIPD_TIBENEX_FUSED_SHIFT", "0")
    cfg = CONFIGS["mixed"]
    w = _write_checkpoint(str(tmp_path), cfg, seed=8)
    sched = _scheduler(str(tmp_path), dtype, max_tokens=256, graphs=False)
    assert not sched.model_runner.model.fused_shift
    prompts = {"x": _tokens(80, cfg["vocab"], 1), "y": _tokens(50, cfg["vocab"], 2)}
    got = _run_schedule(sched, prompts, [[("x", 40), ("y", 10)]] + [[("x", 1), ("y", 1)]] * 40)
    for n in prompts:
        assert _rel_err(got[n], O.forward(cfg, w, prompts[n]), dtype != "float32") < LIMIT[dtype], n


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["mixed", "awkward", "attention_only"])
def test_prompt_batches_that_expand_keys_from_the_latent_rows(name, dtype, tmp_path, monkeypatch):
    """Every extend batch takes the form that large prompt batches take by themselves: keys and values of all heads expanded
    from the requests' latent rows (those of earlier portions included), attention head by head, the heads' gates behind
    it.  Decode steps between the portions attend over the latent rows; both forms have to agree with the plain model."""
    monkeypatch.setenv("SEMIPD_LATENT_EXPAND", "2")
    cfg = CONFIGS[name]
    w = _write_checkpoint(str(tmp_path), cfg, seed=7)
    sched = _scheduler(str(tmp_path), dtype, max_tokens=336)
    prompts = {"x": _tokens(120, cfg["vocab"], 3), "y": _tokens(45, cfg["vocab"], 4), "z": _tokens(70, cfg["vocab"], 5)}
    got = _run_schedule(sched, prompts, [[("x", 64), ("y", 2)], [("x", 1), ("y", 1)], [("x", 2), ("y", 40), ("z", 33)], [("x", 1), ("z", 1)],
                                         [("x", 52), ("y", 2), ("z", 36)]])
    for n in prompts:
        assert _rel_err(got[n], O.forward(cfg, w, prompts[n]), dtype != "float32") < LIMIT[dtype], n


def test_a_far_token_decides_the_logits(tmp_path):
    """Weights made so that attention's first head looks far back: the temperature of one head of the talking attention is
    large, so its softmax is nearly one-hot on some key hundreds of tokens back; replacing that far token has to change the
    last position's logits in the engine exactly as in the plain model, in the prompt pass and when decoding."""
    cfg = _config(96, 64, [_layer(_attn(4, 2, 32, 32, 8), 64), _layer(_latent(2, 16, 16, 16, 32, 24), None)])
    w = _write_checkpoint(str(tmp_path), cfg, seed=3)
    w["l0.mix.temp"][0] = 24.0
    from safetensors.torch import save_file
    save_file({k: v.contiguous() for k, v in w.items()}, os.path.join(str(tmp_path), "model.safetensors"))
    sched = _scheduler(str(tmp_path), "float32", max_tokens=1408, max_requests=2)
    t = _tokens(700, 96, 9)
    want = O.forward(cfg, w, t)
    # which far token matters most to the last position?  (found with the plain model, then checked in the engine)
    base = want[-1]
    moved = []
    for j in (5, 60, 200, 333):
        t2 = list(t)
        t2[j] = (t2[j] + 17) % 96
        moved.append(((O.forward(cfg, w, t2)[-1] - base).abs().max().item(), j, t2))
    change, j, t2 = max(moved)
    assert change > 1e-3
    want2 = O.forward(cfg, w, t2)
    for seq, truth in ((t, want), (t2, want2)):
        got = _run_schedule(sched, {"p": seq}, [[("p", 640)], [("p", 2)]] + [[("p", 1)]] * 58)
        assert _rel_err(got["p"], truth) < LIMIT["float32"]
        got = _run_schedule(sched, {"p": seq}, [[("p", 700)]])
        assert _rel_err(got["p"], truth) < LIMIT["float32"]


def test_long_prompt_and_long_decoding(tmp_path):
    """600 tokens in one portion (many tiles of the prompt attention, many stages of the recurrence), then 200 decode steps,
    in fp32 against the plain model."""
    cfg = CONFIGS["mixed"]
    w = _write_checkpoint(str(tmp_path), cfg, seed=31)
    sched = _scheduler(str(tmp_path), "float32", max_tokens=832, max_requests=2)
    t = _tokens(800, cfg["vocab"], 77)
    got = _run_schedule(sched, {"p": t}, [[("p", 600)]] + [[("p", 1)]] * 200)
    assert _rel_err(got["p"], O.forward(cfg, w, t)) < LIMIT["float32"]


def _check_generation(cfg, w, prompts, outs, steps):
    exact = total = 0
    for p, o in zip(prompts, outs):
        assert len(o) == steps
        logits = O.forward(cfg, w, p + o)
        for i, tok in enumerate(o):
            row = logits[len(p) + i - 1]
            assert row[tok] >= row.max() - 0.08 * row.std(), (len(p), i)
            exact += int(row.argmax().item() == tok)
            total += 1
    assert exact >= 0.9 * total


def test_greedy_generation_through_the_engine(tmp_path):
    """Prompts of unequal length through Engine.generate (the unified scheduler: chunked prefill, decode graphs, sampler):
    every generated token is the plain model's argmax given the tokens before it, or within a small margin of it."""
    from semi_pd_amd.entrypoints.engine import Engine
    from semi_pd_amd.managers.io_struct import SamplingParams
    from semi_pd_amd.server_args import ServerArgs
    cfg = CONFIGS["mixed"]
    w = _write_checkpoint(str(tmp_path), cfg, seed=21)
    prompts = [_tokens(n, cfg["vocab"], seed=n) for n in (3, 70, 33, 1, 120)]
    sa = ServerArgs(model_path=str(tmp_path), load_format="auto", dtype="bfloat16", context_length=256, max_total_tokens=1024,
                    max_running_requests=8, cuda_graph_max_bs=8, chunked_prefill_size=64, skip_tokenizer_init=True)
    eng = Engine(sa)
    try:
        outs = eng.generate(prompts, SamplingParams(max_new_tokens=24, ignore_eos=True), timeout=300)
    finally:
        eng.shutdown()
    _check_generation(cfg, w, prompts, outs, 24)


def test_greedy_generation_through_the_semi_pd_engine(tmp_path):
    """The same through a prefill and a decode process on one GPU: the rows of every attention layer of either kind, the slab
    of state rows (the previous token's stream of every layer, the recurrence's matrices, the convolutions' inputs) and
    every parameter reach the prefill process through IPC handles; prompts are cut into 48-token portions in the prefill
    process and decoded in the other."""
    from semi_pd_amd.entrypoints.engine import Engine
    from semi_pd_amd.managers.io_struct import SamplingParams
    from semi_pd_amd.server_args import ServerArgs
    cfg = CONFIGS["mixed"]
    w = _write_checkpoint(str(tmp_path), cfg, seed=22)
    prompts = [_tokens(n, cfg["vocab"], seed=100 + n) for n in (5, 90, 47, 130)]
    sa = ServerArgs(model_path=str(tmp_path), load_format="auto", dtype="bfloat16", context_length=256, max_total_tokens=2048,
                    max_running_requests=8, cuda_graph_max_bs=8, chunked_prefill_size=48, skip_tokenizer_init=True,
                    enable_semi_pd=True, cu_mask_mode="env", prefill_cu_percent=50, decode_cu_percent=50, tune_prefill_gemm=False,
                    watchdog_timeout=120.0)
    eng = Engine(sa)
    try:
        outs = eng.generate(prompts, SamplingParams(max_new_tokens=16, ignore_eos=True), timeout=300)
    finally:
        eng.shutdown()
    _check_generation(cfg, w, prompts, outs, 16)
