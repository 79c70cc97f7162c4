"""Checkpoint loading for `--load-format auto`: HF config.json -> model config, *.safetensors shards ->
the product's (stacked, tensor-parallel) parameters.

Reference: model_loader/loader.py (DefaultModelLoader: config + safetensors iterator) and the
per-model `load_weights` stacked-parameter mappings: models/llama.py:370-420 (q/k/v -> qkv_proj,
gate/up -> gate_up_proj), models/deepseek_v2.py:1150-1227 (experts.{e}.{gate,up,down}_proj ->
w13_weight / w2_weight), OPT per HF naming.  The pieces of a stacked parameter are collected on the
host until complete, then the rank's shard is cut with the same `tp_shard` the dummy initialiser
uses, so a loaded model and a dummy one are laid out identically (and exported through IPC the same
way)."""
from __future__ import annotations

import dataclasses
import glob
import json
import os
import re
from typing import Dict, Iterable, Iterator, List, Optional, Tuple

import torch
from torch import nn


# ----------------------------------------------------------------------------------- config
def _config_classes():
    from semi_pd_amd.models.deepseek_v2 import DeepseekV2Config
    from semi_pd_amd.models.llama import LlamaConfig
    from semi_pd_amd.models.kudirax import KudiraxConfig
    from semi_pd_amd.models.opt import OPTConfig
    from semi_pd_amd.models.penozen import PenozenConfig
    from semi_pd_amd.models.tibenex import TibenexConfig
    from semi_pd_amd.models.tigotar import TigotarConfig
    return {"Tibenex": TibenexConfig, "Tigotar": TigotarConfig, "Penozen": PenozenConfig, "LlamaForCausalLM": LlamaConfig, "OPTForCausalLM": OPTConfig,
            "DeepseekV2ForCausalLM": DeepseekV2Config, "DeepseekV3ForCausalLM": DeepseekV2Config,
            "Kudirax": KudiraxConfig}


def config_from_hf_dict(d: dict):
    # HF checkpoints list "architectures"; a config.json of this project's own designs names one "architecture"
    archs = d.get("architectures") or ([d["architecture"]] if d.get("architecture") else [])
    classes = _config_classes()
    arch = next((a for a in archs if a in classes), None)
    if arch is None:
        raise ValueError(f"unsupported architectures {archs}; supported: {sorted(classes)}")
    cls = classes[arch]
    if hasattr(cls, "from_dict"):
        return cls.from_dict(d)      # nested per-layer configuration: the class reads its own keys
    if arch == "OPTForCausalLM" and d.get("word_embed_proj_dim", d.get("hidden_size")) != d.get("hidden_size"):
        raise ValueError("OPT checkpoints with word_embed_proj_dim != hidden_size are not supported")
    names = {f.name for f in dataclasses.fields(cls)}
    if d.get("quantization_config") and "quantization_config" not in names:
        raise ValueError(f"{arch}: quantised checkpoints are supported for the DeepSeek family only")
    # config keys that change the computation and have no implementation here must not be dropped silently:
    # the checkpoint would load (unmatched bias tensors) and produce wrong logits
    if arch == "LlamaForCausalLM":
        for key in ("attention_bias", "mlp_bias"):
            if d.get(key):
                raise ValueError(f"{arch}: {key}=true checkpoints are not supported (linears run without bias)")
        if d.get("hidden_act", "silu") != "silu":
            raise ValueError(f"{arch}: hidden_act={d['hidden_act']!r} is not supported (SiLU * mul only)")
    if arch in ("DeepseekV2ForCausalLM", "DeepseekV3ForCausalLM") and d.get("attention_bias"):
        raise ValueError(f"{arch}: attention_bias=true checkpoints are not supported")
    kw = {k: v for k, v in d.items() if k in names and k != "architectures"}
    return cls(architectures=(arch,), **kw)


def load_hf_config(model_path: str):
    with open(os.path.join(model_path, "config.json")) as f:
        return config_from_hf_dict(json.load(f))


# ----------------------------------------------------------------------------------- weights
def safetensors_weights_iterator(model_path: str) -> Iterator[Tuple[str, torch.Tensor]]:
    """loader.py _get_weights_iterator: every tensor of every *.safetensors shard (host memory)."""
    from safetensors import safe_open
    files = sorted(glob.glob(os.path.join(model_path, "*.safetensors")))
    if not files:
        bins = sorted(glob.glob(os.path.join(model_path, "pytorch_model*.bin")))
        if not bins:
            raise FileNotFoundError(f"no *.safetensors or pytorch_model*.bin under {model_path}")
        for b in bins:
            for k, v in torch.load(b, map_location="cpu", weights_only=True).items():
                yield k, v
        return
    for fpath in files:
        with safe_open(fpath, framework="pt", device="cpu") as f:
            for k in f.keys():
                yield k, f.get_tensor(k)


class _Stacker:
    """Collects the parts of stacked parameters; `add` returns the finished (name, tensor) pairs."""

    def __init__(self):
        self.pending: Dict[str, Dict[int, torch.Tensor]] = {}

    def add(self, name: str, index: int, count: int, t: torch.Tensor, dim: Optional[int] = 0):
        parts = self.pending.setdefault(name, {})
        parts[index] = t
        if len(parts) < count:
            return []
        del self.pending[name]
        ordered = [parts[i] for i in range(count)]
        return [(name, torch.cat(ordered, dim) if dim is not None else torch.stack(ordered, 0))]


_QKV = {"q_proj": 0, "k_proj": 1, "v_proj": 2}
_GATE_UP = {"gate_proj": 0, "up_proj": 1}
_KUDIRAX_RE = re.compile(r"^l(\d+)\.(mix|mlp|norm1|norm2)(?:\.(.+))?$")
_KUDIRAX_MERGED = {"q": 0, "k": 1, "v": 2, "g": 3}


def _kudirax_items(config, weights):
    """Kudirax checkpoint names (embed, l<i>.mix.q ..., l<i>.norm1[.b], l<i>.mlp.up[.b] ..., final.norm[.b], head) ->
    product parameters; q | k | v | g stack into the mixer's merged projection."""
    st = _Stacker()
    top = {"embed": "embed.weight", "head": "head.weight", "final.norm": "final_norm.weight", "final.norm.b": "final_norm.bias"}
    for name, t in weights:
        if name in top:
            yield top[name], t
            continue
        m = _KUDIRAX_RE.match(name)
        if not m:
            raise KeyError(f"checkpoint tensor {name} has no counterpart in a Kudirax model")
        i, part, leaf = int(m.group(1)), m.group(2), m.group(3)
        base = f"layers.{i}."
        if part in ("norm1", "norm2"):
            if part == "norm2" and not config.layers[i].ff:
                continue                      # a layer without feed-forward has no second norm to apply
            yield base + part + (".bias" if leaf == "b" else ".weight"), t
        elif part == "mix":
            if leaf in _KUDIRAX_MERGED:
                yield from st.add(base + "mix.qkvg_proj.weight", _KUDIRAX_MERGED[leaf], 4, t)
            elif leaf == "o":
                yield base + "mix.o_proj.weight", t
            elif leaf in ("sink", "vmix"):
                yield base + "mix." + leaf, t
            else:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a Kudirax model")
        else:
            which, _, b = leaf.partition(".")
            if which not in ("up", "down") or b not in ("", "b"):
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a Kudirax model")
            yield base + f"mlp.{which}." + ("bias" if b else "weight"), t
    if st.pending:
        raise RuntimeError(f"checkpoint ended with incomplete stacked parameters: {list(st.pending)[:4]}")


_TIGOTAR_RE = re.compile(r"^l(\d+)\.(mix|mlp|norm1b|norm2b|norm1|norm2)(?:\.(.+))?$")
_TIGOTAR_IN = {"left.q": 0, "left.k": 1, "left.v": 2, "right.z": 3, "right.x": 4, "right.g": 5}
_TIGOTAR_OUT = {"left.o": 0, "right.o": 1}
_TIGOTAR_BIAS = {"left.q.b": "bias_q", "left.k.b": "bias_k", "left.v.b": "bias_v", "right.z.b": "bias_z", "right.x.b": "bias_x",
                 "left.pb": "head_bias"}
_DYN_TANH_LEAF = {None: "weight", "b": "bias", "alpha": "alpha"}


def _tigotar_items(config, weights):
    """Tigotar checkpoint names (embed, embed.norm[.b|.alpha], loop.in, loop.step, l<i>.norm1[b][.b|.alpha], l<i>.mix.left.q[.b]
    ..., l<i>.mix.right.z[.b] ..., l<i>.mlp.router, l<i>.mlp.e<j>.up|down, final.norm..., head) -> product parameters:
    q | k | v | z | x | g stack into the mixer's merged input projection, left.o | right.o side by side into its output
    projection, the experts' matrices into [E, ...] stacks."""
    st = _Stacker()
    top = {"embed": "embed.weight", "head": "head.weight", "loop.in": "loop_in.weight", "loop.step": "loop_step"}
    for name, t in weights:
        if name in top:
            if name.startswith("loop.") and not config.has_loop:
                continue                      # nothing is repeated: the pass entry does not exist
            yield top[name], t
            continue
        m = re.match(r"^(embed|final)\.norm(?:\.(b|alpha))?$", name)
        if m:
            yield f"{m.group(1)}_norm." + _DYN_TANH_LEAF[m.group(2)], t
            continue
        m = _TIGOTAR_RE.match(name)
        if not m or int(m.group(1)) >= len(config.layers):
            raise KeyError(f"checkpoint tensor {name} has no counterpart in a Tigotar model")
        i, part, leaf = int(m.group(1)), m.group(2), m.group(3)
        base = f"layers.{i}."
        lc = config.layers[i]
        if part.startswith("norm"):
            if part in ("norm2", "norm2b") and not lc.experts:
                continue                      # a layer without feed-forward has no second pair of squashings to apply
            if leaf not in _DYN_TANH_LEAF:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a Tigotar model")
            yield base + part + "." + _DYN_TANH_LEAF[leaf], t
        elif part == "mix":
            if leaf in _TIGOTAR_IN:
                yield from st.add(base + "mix.in_proj.weight", _TIGOTAR_IN[leaf], 6, t)
            elif leaf in _TIGOTAR_OUT:
                yield from st.add(base + "mix.out_proj.weight", _TIGOTAR_OUT[leaf], 2, t, dim=1)
            elif leaf in _TIGOTAR_BIAS:
                yield base + "mix." + _TIGOTAR_BIAS[leaf], t
            else:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a Tigotar model")
        else:
            if not lc.experts:
                raise KeyError(f"checkpoint tensor {name}: layer {i} has no feed-forward")
            if leaf == "router":
                yield base + "mlp.router", t
                continue
            em = re.match(r"^e(\d+)\.(up|down)$", leaf or "")
            if not em or int(em.group(1)) >= lc.experts:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a Tigotar model")
            yield from st.add(base + "mlp.w_" + em.group(2), int(em.group(1)), lc.experts, t, dim=None)
    if st.pending:
        raise RuntimeError(f"checkpoint ended with incomplete stacked parameters: {list(st.pending)[:4]}")


_PENOZEN_RE = re.compile(r"^l(\d+)\.(mix|mlp|norm1|norm2)(?:\.(.+))?$")
_PENOZEN_LATENT_IN = {"q": 0, "dkv": 1, "g": 2}
_PENOZEN_DELTA_IN = {"q": 0, "k": 1, "v": 2, "g": 3, "a": 4, "b": 5}
_PENOZEN_DELTA_LEAF = {"q.conv": "conv_q", "k.conv": "conv_k", "v.conv": "conv_v", "A_log": "a_log", "dt_bias": "dt_bias",
                       "norm": "out_norm"}


def _penozen_items(config, weights):
    """Penozen checkpoint names (embed, bigram, l<i>.norm1|norm2, l<i>.mix.q|dkv|dkv.norm|uk|uv|sink|g|o of a latent-attention
    layer, l<i>.mix.q|k|v[.conv]|b|a|A_log|dt_bias|norm|g|o of a delta layer, l<i>.mlp.router, l<i>.mlp.e<j>.gate|up|down,
    final.norm, head) -> product parameters: q | dkv | g (q | k | v | g | a | b) stack into the mixer's merged input
    projection, the up-projections of keys and values are cut by head, every expert's gate and up rows stack into [E, 2F, W]."""
    st = _Stacker()
    top = {"embed": "embed.weight", "bigram": "embed.bigram", "head": "head.weight", "final.norm": "final_norm.weight"}
    for name, t in weights:
        if name in top:
            yield top[name], t
            continue
        m = _PENOZEN_RE.match(name)
        if not m or int(m.group(1)) >= len(config.layers):
            raise KeyError(f"checkpoint tensor {name} has no counterpart in a Penozen model")
        i, part, leaf = int(m.group(1)), m.group(2), m.group(3)
        base = f"layers.{i}."
        lc = config.layers[i]
        if part in ("norm1", "norm2"):
            if leaf is not None:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a Penozen model")
            if part == "norm2" and not lc.experts:
                continue                      # a layer without feed-forward has no second norm to apply
            yield base + part + ".weight", t
        elif part == "mix" and lc.kind == "latent_attention":
            mc = lc.mixer
            if leaf in _PENOZEN_LATENT_IN:
                yield from st.add(base + "mix.in_proj.weight", _PENOZEN_LATENT_IN[leaf], 3, t)
            elif leaf == "o":
                yield base + "mix.out_proj.weight", t
            elif leaf == "dkv.norm":
                yield base + "mix.latent_norm", t
            elif leaf == "uk":
                yield base + "mix.w_uk", t.reshape(mc.heads, mc.dim, mc.kv_rank)
            elif leaf == "uv":
                yield base + "mix.w_uv", t.reshape(mc.heads, mc.vdim, mc.kv_rank)
            elif leaf == "sink":
                yield base + "mix.sink", t
            else:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a latent-attention layer")
        elif part == "mix":
            if leaf in _PENOZEN_DELTA_IN:
                yield from st.add(base + "mix.in_proj.weight", _PENOZEN_DELTA_IN[leaf], 6, t)
            elif leaf == "o":
                yield base + "mix.out_proj.weight", t
            elif leaf in _PENOZEN_DELTA_LEAF:
                yield base + "mix." + _PENOZEN_DELTA_LEAF[leaf], t
            else:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a delta layer")
        else:
            if not lc.experts:
                raise KeyError(f"checkpoint tensor {name}: layer {i} has no feed-forward")
            if leaf == "router":
                yield base + "mlp.router", t
                continue
            em = re.match(r"^e(\d+)\.(gate|up|down)$", leaf or "")
            if not em or int(em.group(1)) >= lc.experts:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a Penozen model")
            e, which = int(em.group(1)), em.group(2)
            if which == "down":
                yield from st.add(base + "mlp.w_down", e, lc.experts, t, dim=None)
            else:
                # (gate rows of expert e, then its up rows; the experts' blocks follow each other)
                for done_name, full in st.add(base + "mlp.w13", 2 * e + (which == "up"), 2 * lc.experts, t):
                    yield done_name, full.reshape(lc.experts, 2 * lc.ff, full.shape[1])
    if st.pending:
        raise RuntimeError(f"checkpoint ended with incomplete stacked parameters: {list(st.pending)[:4]}")


_TIBENEX_RE = re.compile(r"^l(\d+)\.(mix|mlp|norm1|norm2|ls1|ls2|shift)(?:\.(.+))?$")
_TIBENEX_LATENT_IN = {"dq": 0, "dkv": 1, "g": 2}
_TIBENEX_LATENT_LEAF = {"dq.norm": "q_norm", "uq": "q_up", "dkv.norm": "latent_norm", "o": "out_proj.weight"}
_TIBENEX_ATTN_IN = {"q": 0, "k": 1, "v": 2}
_TIBENEX_ATTN_LEAF = {"q.norm": "q_norm", "k.norm": "k_norm", "talk": "talk", "temp": "temp", "o": "out_proj.weight"}
_TIBENEX_SSM_LEAF = {"in": "in_proj.weight", "conv": "conv", "conv.b": "conv_bias", "dt_bias": "dt_bias", "A_log": "a_log", "D": "d_skip",
                     "norm": "out_norm", "o": "out_proj.weight"}
_TIBENEX_SEAM = {"norm1": "norm1.weight", "norm2": "norm2.weight", "ls1": "norm1.layer_scale", "ls2": "norm2.layer_scale",
                 "shift": "shift.mu"}


def _tibenex_items(config, weights):
    """Tibenex checkpoint names (embed, l<i>.norm1|norm2|ls1|ls2|shift, l<i>.mix.dq|dq.norm|uq|dkv|dkv.norm|uk|uv|g|o of a
    latent-attention layer, l<i>.mix.q|k|v|q.norm|k.norm|talk|temp|o of an attention layer, l<i>.mix.in|conv|conv.b|dt_bias|
    A_log|D|norm|o of a state-space layer, l<i>.mlp.gate|up|down, final.norm, head) -> product parameters: dq | dkv | g
    (q | k | v) stack into the mixer's merged input projection, the up-projections of keys and values are cut by head, gate
    and up stack into the feed-forward's merged projection."""
    st = _Stacker()
    top = {"embed": "embed.weight", "head": "head.weight", "final.norm": "final_norm_weight"}
    for name, t in weights:
        if name in top:
            yield top[name], t
            continue
        m = _TIBENEX_RE.match(name)
        if not m or int(m.group(1)) >= len(config.layers):
            raise KeyError(f"checkpoint tensor {name} has no counterpart in a Tibenex model")
        i, part, leaf = int(m.group(1)), m.group(2), m.group(3)
        base = f"layers.{i}."
        lc = config.layers[i]
        if part in _TIBENEX_SEAM:
            if leaf is not None:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a Tibenex model")
            if part in ("norm2", "ls2") and not lc.ff:
                continue                      # a layer without feed-forward has no second sum to norm
            yield base + _TIBENEX_SEAM[part], t
        elif part == "mix" and lc.kind == "latent_attention":
            mc = lc.mixer
            if leaf in _TIBENEX_LATENT_IN:
                yield from st.add(base + "mix.in_proj.weight", _TIBENEX_LATENT_IN[leaf], 3, t)
            elif leaf in _TIBENEX_LATENT_LEAF:
                yield base + "mix." + _TIBENEX_LATENT_LEAF[leaf], t
            elif leaf == "uk":
                yield base + "mix.w_uk", t.reshape(mc.heads, mc.dim, mc.kv_rank)
            elif leaf == "uv":
                yield base + "mix.w_uv", t.reshape(mc.heads, mc.vdim, mc.kv_rank)
            else:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a latent-attention layer")
        elif part == "mix" and lc.kind == "attention":
            if leaf in _TIBENEX_ATTN_IN:
                yield from st.add(base + "mix.in_proj.weight", _TIBENEX_ATTN_IN[leaf], 3, t)
            elif leaf in _TIBENEX_ATTN_LEAF:
                yield base + "mix." + _TIBENEX_ATTN_LEAF[leaf], t
            else:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in an attention layer")
        elif part == "mix":
            if leaf not in _TIBENEX_SSM_LEAF:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a state-space layer")
            yield base + "mix." + _TIBENEX_SSM_LEAF[leaf], t
        else:
            if not lc.ff:
                raise KeyError(f"checkpoint tensor {name}: layer {i} has no feed-forward")
            if leaf in ("gate", "up"):
                yield from st.add(base + "mlp.gate_up_proj.weight", int(leaf == "up"), 2, t)
            elif leaf == "down":
                yield base + "mlp.down_proj.weight", t
            else:
                raise KeyError(f"checkpoint tensor {name} has no counterpart in a Tibenex model")
    if st.pending:
        raise RuntimeError(f"checkpoint ended with incomplete stacked parameters: {list(st.pending)[:4]}")


_EXPERT_RE = re.compile(r"^(.*\.mlp\.experts)\.(\d+)\.(gate_proj|up_proj|down_proj)\.(weight|weight_scale_inv)$")


def product_items(config, weights: Iterable[Tuple[str, torch.Tensor]]) -> Iterator[Tuple[str, torch.Tensor]]:
    """HF tensor names -> (product parameter name, full unsharded tensor)."""
    arch = config.architectures[0]
    if arch == "Kudirax":
        yield from _kudirax_items(config, weights)
        return
    if arch == "Tigotar":
        yield from _tigotar_items(config, weights)
        return
    if arch == "Penozen":
        yield from _penozen_items(config, weights)
        return
    if arch == "Tibenex":
        yield from _tibenex_items(config, weights)
        return
    st = _Stacker()
    tie = bool(getattr(config, "tie_word_embeddings", False))
    n_exp = int(getattr(config, "n_routed_experts", 0) or 0)
    expert_parts: Dict[str, Dict[Tuple[int, str], torch.Tensor]] = {}
    for name, t in weights:
        if "rotary_emb.inv_freq" in name:
            continue
        if arch == "OPTForCausalLM":
            if name == "lm_head.weight":
                continue  # tied to embed_tokens
            name = name[len("model.decoder."):] if name.startswith("model.decoder.") else name
            name = name.replace(".self_attn.out_proj.", ".out_proj.")
            m = re.match(r"^(layers\.\d+)\.self_attn\.([qkv]_proj)\.(weight|bias)$", name)
            if m:
                yield from st.add(f"{m.group(1)}.qkv_proj.{m.group(3)}", _QKV[m.group(2)], 3, t)
            else:
                yield name, t
            continue
        if name == "lm_head.weight" and tie:
            continue
        m = _EXPERT_RE.match(name)
        if m:
            prefix, e, which, leaf = m.group(1), int(m.group(2)), m.group(3), m.group(4)
            # block-quantised checkpoints carry experts.{e}.*.weight_scale_inv next to the fp8 weights; they stack
            # like the weights (models/deepseek_v2.py:1150-1227 expert_params_mapping covers both)
            parts = expert_parts.setdefault(prefix + "|" + leaf, {})
            parts[(e, which)] = t
            if len(parts) == 3 * n_exp:
                del expert_parts[prefix + "|" + leaf]
                w13 = torch.stack([torch.cat([parts[(i, "gate_proj")], parts[(i, "up_proj")]], 0)
                                   for i in range(n_exp)], 0)
                w2 = torch.stack([parts[(i, "down_proj")] for i in range(n_exp)], 0)
                yield prefix + ".w13_" + leaf, w13
                yield prefix + ".w2_" + leaf, w2
            continue
        if name.endswith(".mlp.experts.gate_up_proj"):  # checkpoints that already store fused experts
            yield name[: -len("gate_up_proj")] + "w13_weight", t
            continue
        if name.endswith(".mlp.experts.down_proj"):
            yield name[: -len("down_proj")] + "w2_weight", t
            continue
        head, _, leaf = name.rpartition(".")
        mod = head.rsplit(".", 1)[-1]
        base = head[: -len(mod)]
        if mod in _QKV and ".self_attn." in name and arch == "LlamaForCausalLM":
            yield from st.add(f"{base}qkv_proj.{leaf}", _QKV[mod], 3, t)
        elif mod in _GATE_UP and ".experts." not in name:
            yield from st.add(f"{base}gate_up_proj.{leaf}", _GATE_UP[mod], 2, t)
        else:
            yield name, t
    if st.pending or expert_parts:
        missing = list(st.pending) + list(expert_parts)
        raise RuntimeError(f"checkpoint ended with incomplete stacked parameters: {missing[:4]}")


@torch.no_grad()
def load_weights(model: nn.Module, config, weights: Iterable[Tuple[str, torch.Tensor]]) -> List[str]:
    """Copy every checkpoint tensor into the model (this rank's shard).  Returns the loaded names and
    raises if a parameter of the model stays uninitialised."""
    params = dict(model.named_parameters(remove_duplicate=False))
    loaded = []
    for name, full in product_items(config, weights):
        if name not in params:
            if "rotary_emb" in name:
                continue  # recomputed caches (inv_freq, cos / sin); behaviour-changing extras are rejected above
            raise KeyError(f"checkpoint tensor {name} has no counterpart in {type(model).__name__}")
        p = params[name]
        if (p.dtype == torch.float8_e4m3fn) != (full.dtype == torch.float8_e4m3fn):
            raise RuntimeError(f"{name}: checkpoint dtype {full.dtype} vs parameter {p.dtype} — block-quantised models "
                               "need a block-quantised checkpoint (and the other way round)")
        src = full.to(p.device, p.dtype)
        if tuple(src.shape) != tuple(p.shape):
            if not hasattr(p, "tp_shard"):
                raise RuntimeError(f"{name}: checkpoint shape {tuple(src.shape)} vs parameter {tuple(p.shape)}")
            src = p.tp_shard(src)
        p.copy_(src)
        loaded.append(name)
    filled = {id(params[n]) for n in loaded}
    # a tied lm_head is the same Parameter object as the embedding it was loaded through
    missing = sorted(n for n, p in params.items() if id(p) not in filled)
    if missing:
        raise RuntimeError(f"parameters not found in the checkpoint: {missing[:8]}{' ...' if len(missing) > 8 else ''}")
    return loaded
