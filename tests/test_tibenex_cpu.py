"""Host-side pieces of the Tibenex integration: configuration reader, checkpoint name mapping, the pool that holds latent rows
(values a prefix of the keys) next to regions with values of their own, the columns of the state rows, and the plain
model's own invariants (tests/test_gpu_tibenex.py compares the engine with it)."""
import json

import pytest
import torch

from oracle import tibenex as O


def _latent(heads, dim, rot_dim, vdim, rank, q_rank, dims=None, scaling=None):
    rot = {"base": 3000.0, "dims": rot_dim if dims is None else dims}
    if scaling:
        rot["scaling"] = {"factor": scaling, "original": 64, "fast": 8.0, "slow": 1.0}
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
                                                  "q_rank": q_rank, "scale": 0.2, "rot": rot}}


def _attn(heads, kv_heads, dim, vdim, dims):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.3,
                                           "rot": {"base": 700.0, "dims": dims}}}


def _ssm(heads, vdim, state, groups, norm_groups, conv):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "norm_groups": norm_groups,
                                        "conv": conv}}


def _with(layer, ff):
    layer = dict(layer)
    layer["mlp"] = None if ff is None else {"kind": "dense", "ff": ff}
    return layer


CFG = {"architecture": "Tibenex", "vocab": 90, "width": 48, "norm": {"eps": 1e-5}, "postln_alpha": 1.75, "embedding": {"scale": 6.5},
       "layers": [_with(_ssm(4, 6, 8, 2, 3, 3), 20), _with(_latent(3, 16, 8, 12, 24, 20, dims=4, scaling=4.0), None),
                  _with(_attn(4, 2, 8, 6, 4), 12), _with(_ssm(2, 16, 16, 1, 1, 1), None), _with(_latent(2, 8, 16, 8, 40, 12), 8)]}


def test_config_reader_takes_every_size_from_the_file():
    from semi_pd_amd.model_loader import config_from_hf_dict
    c = config_from_hf_dict(CFG)
    assert type(c).__name__ == "TibenexConfig" and c.architectures == ("Tibenex",)
    assert (c.vocab_size, c.hidden_size, c.norm_eps, c.postln_alpha, c.embedding_scale, c.num_hidden_layers) == (90, 48, 1e-5, 1.75, 6.5, 5)
    assert [l.kind for l in c.layers] == ["mamba2", "latent_attention", "attention", "mamba2", "latent_attention"]
    assert [l.ff for l in c.layers] == [20, 0, 12, 0, 8]
    a = c.layers[1].mixer
    assert (a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank, a.q_rank, a.scale, a.rot.dims, a.rot.base) == (3, 16, 8, 12, 24, 20, 0.2, 4, 3000.0)
    assert a.rot.scaling == {"factor": 4.0, "original": 64.0, "fast": 8.0, "slow": 1.0} and c.layers[4].mixer.rot.scaling is None
    t = c.layers[2].mixer
    assert (t.heads, t.kv_heads, t.dim, t.vdim, t.scale, t.rot.dims, t.rot.base) == (4, 2, 8, 6, 0.3, 4, 700.0)
    s = c.layers[0].mixer
    assert (s.heads, s.vdim, s.state, s.groups, s.norm_groups, s.conv) == (4, 6, 8, 2, 3, 3)
    for path, value in ((("layers", 0, "type"), "delta"), (("layers", 2, "mlp", "kind"), "moe"),
                        (("layers", 2, "mixer", "kv_heads"), 3), (("layers", 1, "mixer", "rot", "dims"), 7),
                        (("layers", 1, "mixer", "rot", "dims"), 10), (("layers", 2, "mixer", "rot", "dims"), 12),
                        (("layers", 0, "mixer", "groups"), 3), (("layers", 0, "mixer", "norm_groups"), 5),
                        (("layers", 0, "mixer", "conv"), 0), (("layers", 1, "mixer", "rot", "kind"), "ntk")):
        bad = json.loads(json.dumps(CFG))
        node = bad
        for k in path[:-1]:
            node = node[k]
        node[path[-1]] = value
        with pytest.raises(ValueError):
            config_from_hf_dict(bad)
    bad = json.loads(json.dumps(CFG))
    del bad["layers"][1]["mixer"]["rot"]["scaling"]["slow"]
    with pytest.raises(ValueError):
        config_from_hf_dict(bad)


def test_checkpoint_names_reach_every_parameter_and_merge_the_projections():
    from semi_pd_amd.model_executor.model_runner import build_model
    from semi_pd_amd.model_loader import config_from_hf_dict, load_weights
    c = config_from_hf_dict(CFG)
    w = O.random_weights(CFG, seed=2)
    with torch.device("cpu"):
        model = build_model(c, torch.float32)
    loaded = load_weights(model, c, w.items())
    params = dict(model.named_parameters())
    assert set(loaded) == set(params)
    pre = "layers.1.mix."
    assert torch.equal(params[pre + "in_proj.weight"], torch.cat([w["l1.mix.dq"], w["l1.mix.dkv"], w["l1.mix.g"]]).float())
    assert torch.equal(params[pre + "q_up"], w["l1.mix.uq"].float()) and torch.equal(params[pre + "q_norm"], w["l1.mix.dq.norm"].float())
    assert torch.equal(params[pre + "w_uk"], w["l1.mix.uk"].float().view(3, 16, 24))
    assert torch.equal(params[pre + "w_uv"][2], w["l1.mix.uv"].float()[24:36])
    assert torch.equal(params[pre + "latent_norm"], w["l1.mix.dkv.norm"].float())
    pre = "layers.2.mix."
    assert torch.equal(params[pre + "in_proj.weight"], torch.cat([w["l2.mix." + n] for n in "qkv"]).float())
    assert torch.equal(params[pre + "talk"], w["l2.mix.talk"].float()) and params[pre + "talk"].dtype == torch.float32
    assert torch.equal(params[pre + "temp"], w["l2.mix.temp"].float()) and params[pre + "q_norm"].shape == (32,)
    pre = "layers.0.mix."
    assert torch.equal(params[pre + "in_proj.weight"], w["l0.mix.in"].float()) and params[pre + "in_proj.weight"].shape == (2 * 24 + 2 * 16 + 4, 48)
    assert torch.equal(params[pre + "conv"], w["l0.mix.conv"].float()) and params[pre + "conv"].shape == (24 + 32, 3)
    assert torch.equal(params[pre + "conv_bias"], w["l0.mix.conv.b"].float())
    assert torch.equal(params[pre + "a_log"], w["l0.mix.A_log"].float()) and params[pre + "dt_bias"].dtype == torch.float32
    assert torch.equal(params[pre + "d_skip"], w["l0.mix.D"].float()) and torch.equal(params[pre + "out_norm"], w["l0.mix.norm"].float())
    assert torch.equal(params["layers.0.mlp.gate_up_proj.weight"], torch.cat([w["l0.mlp.gate"], w["l0.mlp.up"]]).float())
    assert torch.equal(params["layers.0.mlp.down_proj.weight"], w["l0.mlp.down"].float())
    assert torch.equal(params["layers.0.norm1.layer_scale"], w["l0.ls1"].float()) and torch.equal(params["layers.0.norm2.weight"], w["l0.norm2"].float())
    assert torch.equal(params["layers.3.shift.mu"], w["l3.shift"].float())
    assert torch.equal(params["final_norm_weight"], w["final.norm"].float())
    assert not any(n.startswith("layers.1.norm2") or n.startswith("layers.1.mlp") for n in params)   # no feed-forward, no second norm
    # one pool region per attention layer of either kind; latent rows are keys and values at once
    geo = model.kv_geometry
    assert geo["num_kv_heads"] == [1, 2, 1] and geo["head_dim"] == [32, 8, 56] and geo["v_head_dim"] == [24, 6, 40]
    assert geo["values_in_keys"] == [True, False, True] and geo["num_heads"] == [3, 4, 2]
    # state columns: per layer the previous token's stream, and S and the convolution's inputs of a state-space layer
    assert model.state_geometry == [48, 4 * 8 * 6, 2 * (24 + 32), 48, 48, 48, 2 * 16 * 16, 1, 48]
    with pytest.raises(KeyError):
        load_weights(model, c, list(w.items()) + [("l1.mix.talk", torch.zeros(1))])
    with pytest.raises(KeyError):
        load_weights(model, c, list(w.items()) + [("l1.mlp.gate", torch.zeros(1))])
    short = dict(w)
    del short["l0.mlp.up"]
    with pytest.raises(RuntimeError):
        load_weights(model, c, short.items())


def test_pool_with_latent_rows_next_to_regions_with_values_of_their_own():
    from semi_pd_amd.mem_cache.memory_pool import MHATokenToKVPool
    pool = MHATokenToKVPool(10, 1, torch.float32, [1, 2, 1], [32, 8, 56], 3, "cpu", v_head_dim=[24, 6, 40],
                            values_in_keys=[True, False, True])
    assert [tuple(k.shape) for k in pool.k_buffer] == [(11, 1, 32), (11, 2, 8), (11, 1, 56)]
    assert [tuple(v.shape) for v in pool.v_buffer] == [(11, 1, 24), (11, 2, 6), (11, 1, 40)]
    pool.k_buffer[2][3, 0, :] = torch.arange(56.0)
    assert torch.equal(pool.get_value_buffer(2)[3, 0], torch.arange(40.0))          # the same memory
    assert pool.v_buffer[0].data_ptr() == pool.k_buffer[0].data_ptr()
    assert pool.v_buffer[1].data_ptr() != pool.k_buffer[1].data_ptr() and pool.v_buffer[1].is_contiguous()
    k_bytes, v_bytes = pool.get_kv_size_bytes()
    assert k_bytes == 11 * (32 + 16 + 56) * 4 and v_bytes == 11 * 12 * 4
    # every region lies in the one slab and none overlaps another
    spans = sorted((t.data_ptr(), t.data_ptr() + t.numel() * 4) for t in pool.k_buffer + [pool.v_buffer[1]])
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
    assert spans[0][0] >= pool.slab.data_ptr() and spans[-1][1] <= pool.slab.data_ptr() + pool.slab.numel()
    with pytest.raises(ValueError):
        MHATokenToKVPool(10, 1, torch.float32, [1, 2], [32, 8], 2, "cpu", v_head_dim=[24, 6], values_in_keys=[True, True])


def test_plain_model_invariants():
    w = O.random_weights(CFG, seed=3)
    g = torch.Generator().manual_seed(0)
    toks = torch.randint(0, CFG["vocab"], (40,), generator=g).tolist()
    full, layers = O.forward_layers(CFG, w, toks)
    assert full.shape == (40, 90) and len(layers) == 5
    torch.testing.assert_close(O.forward(CFG, w, toks[:17]), full[:17], rtol=1e-4, atol=1e-4)      # causal
    # the norm comes after the sum: every layer leaves rows whose mean square is that of the norm's weight pattern
    for i, x in enumerate(layers):
        last = "norm2" if CFG["layers"][i]["mlp"] is not None else "norm1"
        unit = x / w[f"l{i}.{last}"].float()
        torch.testing.assert_close((unit * unit).mean(-1), torch.ones(40), rtol=1e-3, atol=1e-3)
    # the shift reads zeros in front of the first token
    h = torch.randn(3, 48, generator=g)
    mu = torch.rand(48, generator=g)
    s = O.token_shift(h, mu)
    torch.testing.assert_close(s[0], h[0] * (1 - mu))
    torch.testing.assert_close(s[2], h[2] + (h[1] - h[2]) * mu)
    # rotation: both pairings turn by the same angles and keep lengths; elements behind `dims` pass
    x = torch.randn(6, 2, 12, generator=g)
    rot = {"base": 50.0, "dims": 8}
    a, b = O.rotate(x, rot, halves=True), O.rotate(x, rot, halves=False)
    torch.testing.assert_close(a.norm(dim=-1), x.norm(dim=-1))
    torch.testing.assert_close(b.norm(dim=-1), x.norm(dim=-1))
    assert torch.equal(a[..., 8:], x[..., 8:]) and torch.equal(b[..., 8:], x[..., 8:]) and torch.equal(a[0], x[0])
    perm = [0, 4, 1, 5, 2, 6, 3, 7]          # the interleaved order of a vector laid out in halves
    torch.testing.assert_close(O.rotate(x[..., perm + list(range(8, 12))], rot, halves=False)[..., :8],
                               a[..., perm], rtol=1e-5, atol=1e-5)
    # the heads' weights mixed by the identity leave ordinary grouped attention; rows of the mix still sum like the talk rows
    m = CFG["layers"][2]["mixer"]
    w2 = dict(w)
    w2["l2.mix.talk"] = torch.eye(4)
    hh = torch.randn(9, 48, generator=g)
    plain = O.attention_mixer(hh, w2, "l2.mix.", m, 1e-5)
    w2["l2.mix.talk"] = torch.eye(4)[[1, 0, 3, 2]]       # heads swapped inside their key/value head: the outputs swap too
    swapped = O.attention_mixer(hh, w2, "l2.mix.", m, 1e-5)
    wo = w["l2.mix.o"].float()
    wo_sw = wo.view(48, 4, 6)[:, [1, 0, 3, 2]].reshape(48, 24)
    w3 = dict(w2)
    w3["l2.mix.o"] = wo_sw
    torch.testing.assert_close(O.attention_mixer(hh, w3, "l2.mix.", m, 1e-5), plain, rtol=1e-4, atol=1e-4)
    assert not torch.allclose(swapped, plain)
    # the convolution looks back over zeros in front of the sequence; its last column is the current token's
    x = torch.randn(5, 3, generator=g)
    taps, bias = torch.randn(3, 2, generator=g), torch.randn(3, generator=g)
    y = O.causal_conv_silu(x, taps, bias)
    torch.testing.assert_close(y[0], torch.nn.functional.silu(bias + taps[:, 1] * x[0]))
    torch.testing.assert_close(y[3], torch.nn.functional.silu(bias + taps[:, 1] * x[3] + taps[:, 0] * x[2]))
    # the recurrence with no decay (dt -> 0 keeps, here decay_rate 0) sums dt B x^T; C reads it back
    xs, dt = torch.randn(4, 1, 3, generator=g), torch.rand(4, 1, generator=g)
    B = torch.zeros(4, 1, 2)
    B[:, 0, 0] = 1.0
    C = B.clone()
    out = O.state_space_scan(xs, dt, torch.zeros(1), B, C, torch.zeros(1))
    torch.testing.assert_close(out[:, 0], torch.cumsum(dt.view(4, 1) * xs[:, 0], 0))


def test_command_line_of_a_model_folder(tmp_path):
    """A Tibenex folder on the command line: the class comes from config.json; float32 is accepted (every kernel of the path
    takes it); the trace runner wants a device; a checkout without a library builds the sources this model calls."""
    import argparse
    from semi_pd_amd import _lib
    from semi_pd_amd.entrypoints import trace_replay
    from semi_pd_amd.server_args import add_cli_args, from_cli_args
    with open(tmp_path / "config.json", "w") as f:
        json.dump(CFG, f)
    ap = argparse.ArgumentParser()
    add_cli_args(ap)
    sa = from_cli_args(ap.parse_args(["--model-path", str(tmp_path), "--dtype", "float32", "--skip-tokenizer-init"]))
    assert type(sa.model_config).__name__ == "TibenexConfig" and sa.torch_dtype == torch.float32
    assert "state_space.hip" in _lib.MODEL_SOURCES["Tibenex"] and "local_attention.hip" in _lib.MODEL_SOURCES["Tibenex"]
    if not torch.cuda.is_available():
        assert trace_replay.main(["--model", str(tmp_path), "--dtype", "bfloat16", "--out", str(tmp_path / "o"),
                                  "--max-tokens", "64"]) == 2
