"""Host-side pieces of the Penozen integration: configuration reader, checkpoint name mapping, the pool of latent rows whose
values are a prefix of the keys, the columns of the state rows, the stretched rotation frequencies, and the plain model's
own invariants (tests/test_gpu_penozen.py compares the engine with it)."""
import json
import math

import pytest
import torch

from oracle import penozen as P


def _attn(heads, dim, rot_dim, vdim, rank, dims=None, scaling=None):
    rot = {"base": 3000.0, "dims": rot_dim if dims is None else dims}
    if scaling:
        rot["scaling"] = {"factor": scaling, "original": 64, "fast": 8.0, "slow": 1.0}
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
                                                  "scale": 0.2, "rot": rot}}


def _delta(heads, kv_heads, dim, vdim, conv):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}}


def _with(layer, moe):
    layer = dict(layer)
    layer["mlp"] = None if moe is None else {"kind": "moe", "expert": {"ff": moe[2], "limit": moe[3]},
                                             "router": {"experts": moe[0], "top": moe[1]}}
    return layer


CFG = {"architecture": "Penozen", "vocab": 90, "width": 48, "norm": {"eps": 1e-5}, "logit_softcap": 12.0,
       "embedding": {"scale": 6.5, "bigram": {"buckets": 53, "mul_prev": 1009, "mul_cur": 7}},
       "layers": [_with(_attn(3, 16, 8, 12, 24, dims=4, scaling=4.0), (3, 2, 20, 1.5)), _with(_delta(4, 2, 8, 6, 3), None),
                  _with(_delta(2, 2, 16, 16, 1), (5, 5, 12, 0.5)), _with(_attn(2, 8, 16, 8, 40), (2, 1, 8, 2.0))]}


def test_config_reader_takes_every_size_from_the_file():
    from semi_pd_amd.model_loader import config_from_hf_dict
    c = config_from_hf_dict(CFG)
    assert type(c).__name__ == "PenozenConfig" and c.architectures == ("Penozen",)
    assert (c.vocab_size, c.hidden_size, c.norm_eps, c.logit_softcap, c.num_hidden_layers) == (90, 48, 1e-5, 12.0, 4)
    assert (c.embedding_scale, c.bigram_buckets, c.bigram_mul_prev, c.bigram_mul_cur) == (6.5, 53, 1009, 7)
    assert [l.kind for l in c.layers] == ["latent_attention", "delta", "delta", "latent_attention"]
    a = c.layers[0].mixer
    assert (a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank, a.scale, a.rot_dims, a.rot_base) == (3, 16, 8, 12, 24, 0.2, 4, 3000.0)
    assert a.rot_scaling == {"factor": 4.0, "original": 64.0, "fast": 8.0, "slow": 1.0} and c.layers[3].mixer.rot_scaling is None
    d = c.layers[1].mixer
    assert (d.heads, d.kv_heads, d.dim, d.vdim, d.conv) == (4, 2, 8, 6, 3)
    assert [(l.experts, l.top, l.ff, l.limit) for l in c.layers] == [(3, 2, 20, 1.5), (0, 0, 0, 0.0), (5, 5, 12, 0.5), (2, 1, 8, 2.0)]
    for path, value in ((("layers", 0, "type"), "attention"), (("layers", 2, "mlp", "kind"), "dense"),
                        (("layers", 1, "mixer", "kv_heads"), 3), (("layers", 0, "mixer", "rot", "dims"), 7),
                        (("layers", 0, "mixer", "rot", "dims"), 10), (("layers", 3, "mlp", "router", "top"), 3),
                        (("layers", 1, "mixer", "conv"), 0), (("layers", 0, "mixer", "rot", "kind"), "ntk")):
        bad = json.loads(json.dumps(CFG))
        node = bad
        for k in path[:-1]:
            node = node[k]
        node[path[-1]] = value
        with pytest.raises(ValueError):
            config_from_hf_dict(bad)
    bad = json.loads(json.dumps(CFG))
    del bad["layers"][0]["mixer"]["rot"]["scaling"]["slow"]
    with pytest.raises(ValueError):
        config_from_hf_dict(bad)


def test_checkpoint_names_reach_every_parameter_and_merge_the_projections():
    from semi_pd_amd.model_executor.model_runner import build_model
    from semi_pd_amd.model_loader import config_from_hf_dict, load_weights
    c = config_from_hf_dict(CFG)
    w = P.random_weights(CFG, seed=2)
    with torch.device("cpu"):
        model = build_model(c, torch.float32)
    loaded = load_weights(model, c, w.items())
    params = dict(model.named_parameters())
    assert set(loaded) == set(params)
    pre = "layers.0.mix."
    assert torch.equal(params[pre + "in_proj.weight"], torch.cat([w["l0.mix.q"], w["l0.mix.dkv"], w["l0.mix.g"]]).float())
    assert torch.equal(params[pre + "w_uk"], w["l0.mix.uk"].float().view(3, 16, 24))
    assert torch.equal(params[pre + "w_uv"][2], w["l0.mix.uv"].float()[24:36])
    assert torch.equal(params[pre + "latent_norm"], w["l0.mix.dkv.norm"].float())
    assert torch.equal(params[pre + "sink"], w["l0.mix.sink"].float()) and params[pre + "sink"].dtype == torch.float32
    pre = "layers.1.mix."
    assert torch.equal(params[pre + "in_proj.weight"], torch.cat([w["l1.mix." + n] for n in "qkvgab"]).float())
    assert torch.equal(params[pre + "conv_k"], w["l1.mix.k.conv"].float()) and params[pre + "conv_v"].shape == (24, 3)
    assert torch.equal(params[pre + "a_log"], w["l1.mix.A_log"].float()) and params[pre + "dt_bias"].dtype == torch.float32
    assert torch.equal(params[pre + "out_norm"], w["l1.mix.norm"].float())
    assert torch.equal(params[pre + "out_proj.weight"], w["l1.mix.o"].float())
    w13 = params["layers.2.mlp.w13"]
    assert w13.shape == (5, 24, 48)
    assert torch.equal(w13[3, :12], w["l2.mlp.e3.gate"].float()) and torch.equal(w13[3, 12:], w["l2.mlp.e3.up"].float())
    assert torch.equal(params["layers.2.mlp.w_down"][4], w["l2.mlp.e4.down"].float())
    assert torch.equal(params["layers.0.mlp.router"], w["l0.mlp.router"].float())
    assert torch.equal(params["embed.bigram"], w["bigram"].float()) and params["embed.bigram"].shape == (54, 48)
    assert torch.equal(params["final_norm.weight"], w["final.norm"].float())
    assert not any(n.startswith("layers.1.norm2") or n.startswith("layers.1.mlp") for n in params)   # no experts, no second norm
    # one pool region per latent-attention layer: a row [latent | rotated key part] whose first kv_rank elements are the values
    geo = model.kv_geometry
    assert geo["num_kv_heads"] == [1, 1] and geo["head_dim"] == [32, 56] and geo["v_head_dim"] == [24, 40] and geo["values_in_keys"]
    # state columns: the previous token, then S and the convolutions' inputs of every delta layer
    assert model.state_geometry == [1, 4 * 8 * 6, 2 * (2 * 2 * 8 + 4 * 6), 2 * 16 * 16, 1]
    with pytest.raises(KeyError):
        load_weights(model, c, list(w.items()) + [("l1.mix.sink", torch.zeros(1))])
    with pytest.raises(KeyError):
        load_weights(model, c, list(w.items()) + [("l1.mlp.router", torch.zeros(1))])
    short = dict(w)
    del short["l2.mlp.e4.up"]
    with pytest.raises(RuntimeError):
        load_weights(model, c, short.items())


def test_latent_rows_are_keys_and_values_at_once():
    from semi_pd_amd.mem_cache.memory_pool import MHATokenToKVPool
    pool = MHATokenToKVPool(10, 1, torch.float32, [1, 1], [32, 56], 2, "cpu", v_head_dim=[24, 40], values_in_keys=True)
    assert [tuple(k.shape) for k in pool.k_buffer] == [(11, 1, 32), (11, 1, 56)]
    assert [tuple(v.shape) for v in pool.v_buffer] == [(11, 1, 24), (11, 1, 40)]
    pool.k_buffer[1][3, 0, :] = torch.arange(56.0)
    assert torch.equal(pool.get_value_buffer(1)[3, 0], torch.arange(40.0))          # the same memory
    assert pool.v_buffer[1].data_ptr() == pool.k_buffer[1].data_ptr()
    k_bytes, v_bytes = pool.get_kv_size_bytes()
    assert k_bytes == 11 * (32 + 56) * 4 and v_bytes == 0
    assert pool.slab.numel() < 11 * (32 + 56) * 4 + 2 * 256                          # no room is set aside for values
    with pytest.raises(ValueError):
        MHATokenToKVPool(10, 1, torch.float32, [2], [32], 1, "cpu", v_head_dim=[24], values_in_keys=True)
    with pytest.raises(ValueError):
        MHATokenToKVPool(10, 1, torch.float32, [1], [32], 1, "cpu", v_head_dim=[40], values_in_keys=True)


def test_stretched_frequencies():
    from semi_pd_amd.models.penozen import stretched_frequencies
    f, m = stretched_frequencies(16, 10000.0, None)
    assert m == 1.0 and torch.allclose(f, torch.tensor([10000.0 ** (-2 * i / 16) for i in range(8)]))
    sc = {"factor": 8.0, "original": 128.0, "fast": 16.0, "slow": 1.0}
    f2, m2 = stretched_frequencies(16, 10000.0, sc)
    assert abs(m2 - (0.1 * math.log(8.0) + 1)) < 1e-12
    # pairs that turn often keep their frequency, pairs that turn less than once over the original length are slowed by the
    # factor, the ramp between them falls monotonically
    ratio = f2 / f
    assert ratio[0] == 1.0 and abs(ratio[-1] - 1 / 8.0) < 1e-6 and (ratio[1:] <= ratio[:-1] + 1e-7).all()
    ref, mref = P.yarn_frequencies({"dims": 16, "base": 10000.0, "scaling": sc})
    assert torch.allclose(f2, ref.float(), rtol=1e-6, atol=0) and abs(m2 - mref) < 1e-12
    # bounds that coincide: the ramp's width is 0.001, a step
    f3, _ = stretched_frequencies(8, 100.0, {"factor": 2.0, "original": 50.0, "fast": 3.0, "slow": 3.0})
    ref3, _ = P.yarn_frequencies({"dims": 8, "base": 100.0, "scaling": {"factor": 2.0, "original": 50.0, "fast": 3.0, "slow": 3.0}})
    assert torch.allclose(f3, ref3.float(), rtol=1e-6, atol=0)


def test_plain_model_invariants():
    w = P.random_weights(CFG, seed=3)
    g = torch.Generator().manual_seed(0)
    toks = torch.randint(0, CFG["vocab"], (40,), generator=g).tolist()
    full = P.forward(CFG, w, toks)
    assert full.shape == (40, 90) and full.abs().max() <= 12.0                       # the cap
    torch.testing.assert_close(P.forward(CFG, w, toks[:17]), full[:17], rtol=1e-4, atol=1e-4)      # causal
    # the first token takes the bigram table's last row, every other one the hashed row
    e = P.embed_tokens(CFG, w, [5, 9])
    torch.testing.assert_close(e[0], w["embed"][5].float() * 6.5 + w["bigram"][53].float())
    torch.testing.assert_close(e[1], w["embed"][9].float() * 6.5 + w["bigram"][(5 * 1009 + 9 * 7) % 53].float())
    # the sink only takes weight away: rows sum to less than one, and to one as the sink goes to minus infinity
    s = torch.randn(2, 5, 5, generator=g)
    p = P.sink_softmax(s, torch.tensor([0.5, -40.0]))
    assert (p[0].sum(-1) < 1).all() and torch.allclose(p[1].sum(-1), torch.ones(5)) and p[0, 0, 1:].abs().max() == 0
    # the delta rule with beta = 1 and no decay stores k -> v exactly: reading with q = k gives v back
    k = torch.nn.functional.normalize(torch.randn(1, 1, 6, generator=g), dim=-1)
    v = torch.randn(1, 1, 4, generator=g)
    o = P.delta_rule(k, k, v, torch.ones(1, 1), torch.ones(1, 1))
    torch.testing.assert_close(o, v)
    # the convolution looks back over zeros in front of the sequence; its last column is the current token's
    x = torch.randn(5, 3, generator=g)
    taps = torch.randn(3, 2, generator=g)
    y = P.short_conv_silu(x, taps)
    torch.testing.assert_close(y[0], torch.nn.functional.silu(taps[:, 1] * x[0]))
    torch.testing.assert_close(y[3], torch.nn.functional.silu(taps[:, 1] * x[3] + taps[:, 0] * x[2]))
    # experts: clamps bound the activation; with every expert chosen the weights sum to one
    h = torch.randn(4, 48, generator=g) * 10
    out = P.expert_mixture(h, w, "l2.mlp.", CFG["layers"][2]["mlp"])
    assert torch.isfinite(out).all()
    assert torch.isinf(P.router_margin(h, w, "l2.mlp.", CFG["layers"][2]["mlp"])).all()


def test_command_line_of_a_model_folder(tmp_path):
    """A Penozen folder on the command line: the class comes from config.json; float32 is accepted (every kernel of the path
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
    assert type(sa.model_config).__name__ == "PenozenConfig" and sa.torch_dtype == torch.float32
    assert "delta_rule.hip" in _lib.MODEL_SOURCES["Penozen"] and "local_attention.hip" in _lib.MODEL_SOURCES["Penozen"]
    if not torch.cuda.is_available():
        assert trace_replay.main(["--model", str(tmp_path), "--dtype", "bfloat16", "--out", str(tmp_path / "o"),
                                  "--max-tokens", "64"]) == 2
