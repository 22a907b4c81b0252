"""Weight sources for the Llama-2-class adapter.

* ``make_weights_np``  -- seeded N(0, initializer_range) weights (the reference's ``_init_weights``,
  ``promptcache/model/llama2.py:686-695``) drawn with numpy's PCG64 so the same numbers can be
  produced in any process (tests, golden generation, the GPU box) and rounded to fp16.
* ``load_hf_safetensors`` -- real checkpoints (HF layout) when a directory is available.
* ``random_weights_device`` -- seeded weights drawn directly on the GPU at true shapes (bench).

Key names: ``embed``, ``l{i}.ln1|wq|wk|wv|wo|ln2|gate|up|down``, ``norm``, ``lm_head``;
linear weights are ``[out, in]`` (``nn.Linear`` layout).
"""
from __future__ import annotations

import glob
import os
from typing import Dict

import numpy as np

from .config import LlamaShape


def weight_shapes(cfg: LlamaShape) -> Dict[str, tuple]:
    hid, inter, D = cfg.hidden_size, cfg.intermediate_size, cfg.head_dim
    H, Hkv = cfg.num_attention_heads, cfg.num_key_value_heads
    shapes = {"embed": (cfg.vocab_size, hid)}
    for i in range(cfg.num_hidden_layers):
        shapes[f"l{i}.ln1"] = (hid,)
        shapes[f"l{i}.wq"] = (H * D, hid)
        shapes[f"l{i}.wk"] = (Hkv * D, hid)
        shapes[f"l{i}.wv"] = (Hkv * D, hid)
        shapes[f"l{i}.wo"] = (hid, H * D)
        shapes[f"l{i}.ln2"] = (hid,)
        shapes[f"l{i}.gate"] = (inter, hid)
        shapes[f"l{i}.up"] = (inter, hid)
        shapes[f"l{i}.down"] = (hid, inter)
    shapes["norm"] = (hid,)
    shapes["lm_head"] = (cfg.vocab_size, hid)
    return shapes


def make_weights_np(cfg: LlamaShape, seed: int = 0, scale: float = 1.0) -> Dict[str, np.ndarray]:
    """fp16 numpy weights.  Norm gains are 1 + 0.1*N(0,1) (not all-ones) so a test notices a
    dropped or misapplied gain.  ``scale`` multiplies the linear-weight std (tests use >1 to make
    the attention logits non-trivial at tiny hidden sizes)."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shp in weight_shapes(cfg).items():
        if len(shp) == 1:
            w = 1.0 + 0.1 * rng.standard_normal(shp, dtype=np.float32)
        else:
            w = (cfg.initializer_range * scale) * rng.standard_normal(shp, dtype=np.float32)
        out[name] = w.astype(np.float16)
    return out


def falcon_weight_shapes(cfg) -> Dict[str, tuple]:
    """Key names for the Falcon adapter: ``embed``, ``l{i}.ln_w|ln_b|wqkv|wo|w1|w2``, ``lnf_w``, ``lnf_b``, ``lm_head``;
    ``wqkv`` is the fused ``query_key_value`` matrix ``[(H + 2) * D, hidden]`` = H query heads, then the shared key
    head, then the shared value head (``falcon.py:393-396``)."""
    hid, D, H = cfg.hidden_size, cfg.head_dim, cfg.num_attention_heads
    shapes = {"embed": (cfg.vocab_size, hid)}
    for i in range(cfg.num_hidden_layers):
        shapes[f"l{i}.ln_w"] = (hid,)
        shapes[f"l{i}.ln_b"] = (hid,)
        shapes[f"l{i}.wqkv"] = ((H + 2) * D, hid)
        shapes[f"l{i}.wo"] = (hid, hid)
        shapes[f"l{i}.w1"] = (4 * hid, hid)
        shapes[f"l{i}.w2"] = (hid, 4 * hid)
    shapes["lnf_w"] = (hid,)
    shapes["lnf_b"] = (hid,)
    shapes["lm_head"] = (cfg.vocab_size, hid)
    return shapes


def make_falcon_weights_np(cfg, seed: int = 0, scale: float = 1.0) -> Dict[str, np.ndarray]:
    """fp16 numpy weights for a FalconShape: LayerNorm gains 1 + 0.1 N(0,1), LayerNorm biases 0.1 N(0,1)."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shp in falcon_weight_shapes(cfg).items():
        if name.endswith("_b"):
            w = 0.1 * rng.standard_normal(shp, dtype=np.float32)
        elif len(shp) == 1:
            w = 1.0 + 0.1 * rng.standard_normal(shp, dtype=np.float32)
        else:
            w = (cfg.initializer_range * scale) * rng.standard_normal(shp, dtype=np.float32)
        out[name] = w.astype(np.float16)
    if cfg.tie_word_embeddings:
        out["lm_head"] = out["embed"]
    return out


def mpt_weight_shapes(cfg) -> Dict[str, tuple]:
    """Key names for the MPT adapter: ``embed``, ``l{i}.ln1|wqkv|wo|ln2|w1|w2``, ``lnf``, ``lm_head``; ``wqkv`` is
    ``Wqkv`` [3*hid, hid] = all query heads, then all key heads, then all value heads (``mpt.py:144``)."""
    hid = cfg.hidden_size
    shapes = {"embed": (cfg.vocab_size, hid)}
    for i in range(cfg.num_hidden_layers):
        shapes[f"l{i}.ln1"] = (hid,)
        shapes[f"l{i}.wqkv"] = (3 * hid, hid)
        shapes[f"l{i}.wo"] = (hid, hid)
        shapes[f"l{i}.ln2"] = (hid,)
        shapes[f"l{i}.w1"] = (4 * hid, hid)
        shapes[f"l{i}.w2"] = (hid, 4 * hid)
    shapes["lnf"] = (hid,)
    shapes["lm_head"] = (cfg.vocab_size, hid)
    return shapes


def make_mpt_weights_np(cfg, seed: int = 0, scale: float = 1.0) -> Dict[str, np.ndarray]:
    rng = np.random.default_rng(seed)
    out = {}
    for name, shp in mpt_weight_shapes(cfg).items():
        if len(shp) == 1:
            w = 1.0 + 0.1 * rng.standard_normal(shp, dtype=np.float32)
        else:
            w = (cfg.initializer_range * scale) * rng.standard_normal(shp, dtype=np.float32)
        out[name] = w.astype(np.float16)
    if cfg.tie_word_embeddings:
        out["lm_head"] = out["embed"]
    return out


def read_checkpoint_dir(path: str):
    """Every tensor of an HF checkpoint directory, by its HF name, on the host: the ``*.safetensors`` shards when
    there are any, else the ``pytorch_model*.bin`` shards (``torch.load(weights_only=True)``) that older uploads of
    the models the reference lists ship instead."""
    files = sorted(glob.glob(os.path.join(path, "*.safetensors")))
    raw = {}
    if files:
        from safetensors import safe_open
        for fn in files:
            with safe_open(fn, framework="pt", device="cpu") as f:
                for k in f.keys():
                    raw[k] = f.get_tensor(k)
        return raw
    bins = sorted(glob.glob(os.path.join(path, "pytorch_model*.bin")))
    if not bins:
        raise FileNotFoundError(f"no *.safetensors and no pytorch_model*.bin under {path}")
    import torch
    for fn in bins:
        raw.update(torch.load(fn, map_location="cpu", weights_only=True))
    return raw


def random_mpt_weights_device(cfg, device, dtype, seed: int = 0):
    import torch

    g = torch.Generator(device=device)
    g.manual_seed(seed)
    out = {}
    for name, shp in mpt_weight_shapes(cfg).items():
        if len(shp) == 1:
            w = 1.0 + 0.1 * torch.randn(shp, generator=g, device=device, dtype=torch.float32)
        else:
            w = torch.empty(shp, device=device, dtype=torch.float32).normal_(0.0, cfg.initializer_range, generator=g)
        out[name] = w.to(dtype)
        del w
    if cfg.tie_word_embeddings:
        out["lm_head"] = out["embed"]
    return out


def load_mpt_safetensors(path: str, cfg):
    """HF mpt-7b-class checkpoint directory -> the key layout of ``mpt_weight_shapes``."""
    raw = read_checkpoint_dir(path)
    out = {"embed": raw["transformer.wte.weight"], "lnf": raw["transformer.norm_f.weight"]}
    out["lm_head"] = raw.get("lm_head.weight", out["embed"])
    names = {"ln1": "norm_1.weight", "wqkv": "attn.Wqkv.weight", "wo": "attn.out_proj.weight", "ln2": "norm_2.weight",
             "w1": "ffn.up_proj.weight", "w2": "ffn.down_proj.weight"}
    for i in range(cfg.num_hidden_layers):
        for k, hf in names.items():
            out[f"l{i}.{k}"] = raw[f"transformer.blocks.{i}.{hf}"]
    return out


_HF_MAP = {
    "ln1": "input_layernorm.weight", "wq": "self_attn.q_proj.weight", "wk": "self_attn.k_proj.weight",
    "wv": "self_attn.v_proj.weight", "wo": "self_attn.o_proj.weight",
    "ln2": "post_attention_layernorm.weight", "gate": "mlp.gate_proj.weight",
    "up": "mlp.up_proj.weight", "down": "mlp.down_proj.weight",
}


def load_hf_safetensors(path: str, cfg: LlamaShape, device, dtype):
    """Read an HF Llama checkpoint directory (``*.safetensors``) into the key layout above."""
    raw = read_checkpoint_dir(path)
    out = {"embed": raw["model.embed_tokens.weight"], "norm": raw["model.norm.weight"],
           "lm_head": raw.get("lm_head.weight", raw["model.embed_tokens.weight"])}
    for i in range(cfg.num_hidden_layers):
        for short, hf in _HF_MAP.items():
            out[f"l{i}.{short}"] = raw[f"model.layers.{i}.{hf}"]
    return {k: v.to(device=device, dtype=dtype) for k, v in out.items()}


def random_weights_device(cfg: LlamaShape, device, dtype, seed: int = 0):
    """Seeded N(0, 0.02) weights generated on ``device`` (true-shape benchmarks: 7b = 13.5 GB fp16)."""
    import torch

    g = torch.Generator(device=device)
    g.manual_seed(seed)
    out = {}
    for name, shp in weight_shapes(cfg).items():
        if len(shp) == 1:
            w = 1.0 + 0.1 * torch.randn(shp, generator=g, device=device, dtype=torch.float32)
        else:
            w = torch.empty(shp, device=device, dtype=torch.float32).normal_(0.0, cfg.initializer_range, generator=g)
        out[name] = w.to(dtype)
        del w
    return out


def random_falcon_weights_device(cfg, device, dtype, seed: int = 0):
    """Seeded weights for a FalconShape generated on ``device`` (true-shape runs: falcon-7b = 14.4 GB fp16)."""
    import torch

    g = torch.Generator(device=device)
    g.manual_seed(seed)
    out = {}
    for name, shp in falcon_weight_shapes(cfg).items():
        if name.endswith("_b"):
            w = 0.1 * torch.randn(shp, generator=g, device=device, dtype=torch.float32)
        elif len(shp) == 1:
            w = 1.0 + 0.1 * torch.randn(shp, generator=g, device=device, dtype=torch.float32)
        else:
            w = torch.empty(shp, device=device, dtype=torch.float32).normal_(0.0, cfg.initializer_range, generator=g)
        out[name] = w.to(dtype)
        del w
    if cfg.tie_word_embeddings:
        out["lm_head"] = out["embed"]
    return out


def load_falcon_safetensors(path: str, cfg):
    """Read an HF falcon-7b-class checkpoint directory (``*.safetensors``) into the key layout of
    ``falcon_weight_shapes`` (HF names: ``transformer.h.{i}.self_attention.query_key_value`` etc.)."""
    raw = read_checkpoint_dir(path)
    out = {"embed": raw["transformer.word_embeddings.weight"], "lnf_w": raw["transformer.ln_f.weight"],
           "lnf_b": raw["transformer.ln_f.bias"]}
    out["lm_head"] = raw.get("lm_head.weight", out["embed"])
    names = {"ln_w": "input_layernorm.weight", "ln_b": "input_layernorm.bias", "wqkv": "self_attention.query_key_value.weight",
             "wo": "self_attention.dense.weight", "w1": "mlp.dense_h_to_4h.weight", "w2": "mlp.dense_4h_to_h.weight"}
    for i in range(cfg.num_hidden_layers):
        for k, hf in names.items():
            out[f"l{i}.{k}"] = raw[f"transformer.h.{i}.{hf}"]
    return out


# ---- Kazolorn ------------------------------------------------------------------------------------------------------------
def kazolorn_weight_shapes(cfg) -> Dict[str, tuple]:
    """Tensor names and shapes of a Kazolorn checkpoint (``model.safetensors``): ``embed``, per layer ``l{i}.norm1|norm2``,
    ``l{i}.mix.q|k|o`` (+ ``.b`` biases) and ``l{i}.mix.talk`` [H, H], ``l{i}.mlp.up|down|act`` (dense) or
    ``l{i}.mlp.router`` and ``l{i}.mlp.e{j}.gate|up|down`` (sparse), ``l{i}.ls1|ls2`` (layer scales), ``l{i}.dwa`` [i + 2]
    (weights of the embedding output and every layer result up to this one), then ``final.norm`` and ``head``."""
    W = cfg.hidden_size
    s = {"embed": (cfg.vocab_size, W)}
    for i, l in enumerate(cfg.layers):
        p = f"l{i}."
        s[p + "norm1"] = (W,)
        s[p + "mix.q"], s[p + "mix.q.b"] = (l.heads * l.dim, W), (l.heads * l.dim,)
        s[p + "mix.k"], s[p + "mix.k.b"] = (l.kv_heads * l.dim, W), (l.kv_heads * l.dim,)
        s[p + "mix.talk"] = (l.heads, l.heads)
        s[p + "mix.o"], s[p + "mix.o.b"] = (W, l.heads * l.dim), (W,)
        s[p + "ls1"] = (W,)
        if l.mlp_kind:
            s[p + "norm2"], s[p + "ls2"] = (W,), (W,)
        if l.mlp_kind == "dense":
            s[p + "mlp.up"], s[p + "mlp.down"], s[p + "mlp.act"] = (l.ff, W), (W, l.ff), (4,)
        elif l.mlp_kind == "moe":
            s[p + "mlp.router"] = (l.experts, W)
            for e in range(l.experts):
                s[p + f"mlp.e{e}.gate"], s[p + f"mlp.e{e}.up"], s[p + f"mlp.e{e}.down"] = (l.ff, W), (l.ff, W), (W, l.ff)
        s[p + "dwa"] = (i + 2,)
    s["final.norm"] = (W,)
    s["head"] = (cfg.vocab_size, W)
    return s


def make_kazolorn_weights(cfg, seed: int = 0, device="cpu", scale: float = 1.0):
    """Seeded random weights (bfloat16 torch tensors).  Nothing is left at a value that would hide a dropped term: gains
    and layer scales scatter around 1 and 0.5, biases are non-zero, the head-mixing matrix is the identity plus noise, the
    depth weights favour the newest result without silencing the older ones, and the activation's four numbers differ."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    on_gpu = str(device) != "cpu"
    gd = torch.Generator(device=device).manual_seed(seed) if on_gpu else g

    def rnd(shape, big=False):
        if big and on_gpu:
            return torch.randn(shape, generator=gd, device=device, dtype=torch.float32)
        return torch.randn(shape, generator=g, dtype=torch.float32).to(device)

    out = {}
    for name, shp in kazolorn_weight_shapes(cfg).items():
        leaf = name.split(".", 1)[-1] if name.startswith("l") and name[1].isdigit() else name
        if leaf in ("norm1", "norm2", "final.norm"):
            w = 1.0 + 0.1 * rnd(shp)
        elif leaf in ("ls1", "ls2"):
            w = 0.5 + 0.1 * rnd(shp)
        elif leaf == "dwa":
            w = 0.15 * rnd(shp)
            w[-1] += 1.0
        elif leaf == "mix.talk":
            w = torch.eye(shp[0], device=device) + 0.2 * rnd(shp)
        elif leaf == "mlp.act":
            w = torch.tensor([0.9, 0.35, -0.25, 0.1], device=device) + 0.05 * rnd(shp)
        elif leaf.endswith(".b"):
            w = 0.1 * rnd(shp)
        elif leaf in ("embed",):
            w = rnd(shp, big=True)
        else:
            w = (scale / (shp[-1] ** 0.5)) * rnd(shp, big=True)
        out[name] = w.to(torch.bfloat16)
    return out


def load_kazolorn_safetensors(path: str, cfg):
    """The tensors of ``<path>/model.safetensors`` by their own names, on the host, checked against the shapes the
    configuration implies."""
    raw = read_checkpoint_dir(path)
    want = kazolorn_weight_shapes(cfg)
    missing = [k for k in want if k not in raw]
    if missing:
        raise KeyError(f"{path}: tensors missing for this configuration: {missing[:6]}{' ...' if len(missing) > 6 else ''}")
    for k, shp in want.items():
        if k.endswith(".dwa") and raw[k].dim() == 1 and raw[k].shape[0] >= shp[0]:
            continue                                  # (a longer table is read up to the streams the layer has)
        if tuple(raw[k].shape) != tuple(shp):
            raise ValueError(f"{path}: {k} has shape {tuple(raw[k].shape)}, the configuration implies {tuple(shp)}")
    return {k: raw[k] for k in want}


def dibizen_weight_shapes(cfg) -> Dict[str, tuple]:
    """Tensor names and shapes of a Dibizen checkpoint (``model.safetensors``): ``embed``, ``pos``; per layer ``l{i}.norm1|norm2``
    (each with ``.b`` and a scalar ``.alpha``), ``l{i}.hc1|hc2.in|out|mix`` (hyper-connection weights of the two sublayers), the
    mixer's ``l{i}.mix.*`` (lightning: ``q k v g o norm``; attention: ``q g o`` and, unless it borrows another layer's cache,
    ``k v``; mamba1: ``in conv conv.b x dt dt.b A_log D o``) and the feed-forward's ``l{i}.mlp.router|correction`` and
    ``l{i}.mlp.e{j}.up|down``; then ``final.norm`` (``.b``, ``.alpha``) and ``head``."""
    W, S = cfg.hidden_size, cfg.streams
    s = {"embed": (cfg.vocab_size, W), "pos": (cfg.max_positions, W)}

    def norm(name):
        s[name], s[name + ".b"], s[name + ".alpha"] = (W,), (W,), ()

    def hyper(name):
        s[name + ".in"], s[name + ".out"], s[name + ".mix"] = (S,), (S,), (S, S)

    for i, l in enumerate(cfg.layers):
        p = f"l{i}."
        norm(p + "norm1")
        hyper(p + "hc1")
        m = p + "mix."
        if l.kind == "lightning":
            s[m + "q"], s[m + "k"] = (l.heads * l.dim, W), (l.heads * l.dim, W)
            s[m + "v"], s[m + "g"] = (l.heads * l.vdim, W), (l.heads * l.vdim, W)
            s[m + "o"], s[m + "norm"] = (W, l.heads * l.vdim), (l.heads * l.vdim,)
        elif l.kind == "attention":
            s[m + "q"], s[m + "g"], s[m + "o"] = (l.heads * l.dim, W), (l.heads * l.vdim, W), (W, l.heads * l.vdim)
            if l.kv_from < 0:
                s[m + "k"], s[m + "v"] = (l.kv_heads * l.dim, W), (l.kv_heads * l.vdim, W)
        else:
            s[m + "in"], s[m + "conv"], s[m + "conv.b"] = (2 * l.inner, W), (l.inner, l.conv), (l.inner,)
            s[m + "x"], s[m + "dt"], s[m + "dt.b"] = (l.dt_rank + 2 * l.state, l.inner), (l.inner, l.dt_rank), (l.inner,)
            s[m + "A_log"], s[m + "D"], s[m + "o"] = (l.inner, l.state), (l.inner,), (W, l.inner)
        if l.experts + l.identity:
            norm(p + "norm2")
            hyper(p + "hc2")
            s[p + "mlp.router"], s[p + "mlp.correction"] = (l.experts + l.identity, W), (l.experts + l.identity,)
            for e in range(l.experts):
                s[p + f"mlp.e{e}.up"], s[p + f"mlp.e{e}.down"] = (l.ff, W), (W, l.ff)
    norm("final.norm")
    s["head"] = (cfg.vocab_size, W)
    return s


def make_dibizen_weights(cfg, seed: int = 0, device="cpu", scale: float = 1.0):
    """Seeded random weights (bfloat16 torch tensors) with nothing at a value that would hide a dropped term: norm gains around
    1 with non-zero biases and an alpha that keeps tanh off its flat part, stream weights that differ between streams, router
    corrections large enough to change choices, A_log / dt biases that give decays between 0 and 1."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    on_gpu = str(device) != "cpu"
    gd = torch.Generator(device=device).manual_seed(seed) if on_gpu else g

    def rnd(shape, big=False):
        if big and on_gpu:
            return torch.randn(shape, generator=gd, device=device, dtype=torch.float32)
        return torch.randn(shape, generator=g, dtype=torch.float32).to(device)

    out = {}
    S = cfg.streams
    for name, shp in dibizen_weight_shapes(cfg).items():
        leaf = name.split(".", 1)[-1] if name.startswith("l") and name[1].isdigit() else name
        if leaf.endswith(".alpha"):
            w = torch.tensor(0.6, device=device) + 0.1 * rnd(shp)
        elif leaf in ("norm1", "norm2", "final.norm", "mix.norm"):
            w = 1.0 + 0.1 * rnd(shp)
        elif leaf in ("hc1.in", "hc2.in"):
            w = 1.0 / S + 0.2 * rnd(shp)
        elif leaf in ("hc1.out", "hc2.out"):
            w = 1.0 + 0.3 * rnd(shp)
        elif leaf in ("hc1.mix", "hc2.mix"):
            w = torch.eye(S, device=device) + 0.15 * rnd(shp)
        elif leaf == "mlp.correction":
            w = 0.05 * rnd(shp)
        elif leaf == "mix.A_log":
            w = torch.log(torch.arange(1, shp[1] + 1, dtype=torch.float32, device=device)).expand(shp) + 0.1 * rnd(shp)
        elif leaf == "mix.dt.b":
            w = -2.0 + 0.5 * rnd(shp)
        elif leaf == "mix.D":
            w = 1.0 + 0.2 * rnd(shp)
        elif leaf == "mix.conv":
            w = 0.5 * rnd(shp)
        elif leaf.endswith(".b"):
            w = 0.1 * rnd(shp)
        elif leaf == "embed":
            w = rnd(shp, big=True)
        elif leaf == "pos":
            w = 0.5 * rnd(shp, big=True)
        else:
            w = (scale / (shp[-1] ** 0.5)) * rnd(shp, big=True)
        out[name] = w.to(torch.bfloat16)
    return out


def load_dibizen_safetensors(path: str, cfg):
    """The tensors of ``<path>/model.safetensors`` by their own names, on the host, checked against the shapes the
    configuration implies."""
    raw = read_checkpoint_dir(path)
    want = dibizen_weight_shapes(cfg)
    missing = [k for k in want if k not in raw]
    if missing:
        raise KeyError(f"{path}: tensors missing for this configuration: {missing[:6]}{' ...' if len(missing) > 6 else ''}")
    for k, shp in want.items():
        if k == "pos" and raw[k].dim() == 2 and raw[k].shape[1] == shp[1]:
            cfg.max_positions = int(raw[k].shape[0])  # (the table's own length says how many positions there are)
            continue
        if tuple(raw[k].shape) != tuple(shp):
            raise ValueError(f"{path}: {k} has shape {tuple(raw[k].shape)}, the configuration implies {tuple(shp)}")
    return {k: raw[k] for k in want}


def fivesun_weight_shapes(cfg) -> Dict[str, tuple]:
    """Tensor names and shapes of a Fivesun checkpoint (``model.safetensors``): ``embed``; per layer ``l{i}.norm1|norm1b`` (the
    norms before and after the mixer), ``l{i}.rg1`` (+ ``.b``: the sigmoid gate on the mixer's result), the mixer's ``l{i}.mix.*``
    (attention: ``q k v q.norm k.norm sink g o`` and ``vmix`` when it blends values; latent_attention: ``q dkv dkv.norm uk uv g
    o``; mlstm: ``q k v g o norm i i.b f f.b``) and, with a feed-forward, ``l{i}.norm2|norm2b``, ``l{i}.rg2`` (+ ``.b``) and
    ``l{i}.mlp.gate|up|down`` (each with ``.b``); then ``final.norm`` and ``head``."""
    W = cfg.hidden_size
    s = {"embed": (cfg.vocab_size, W)}
    for i, l in enumerate(cfg.layers):
        p, m = f"l{i}.", f"l{i}.mix."
        s[p + "norm1"], s[p + "norm1b"], s[p + "rg1"], s[p + "rg1.b"] = (W,), (W,), (W, W), (W,)
        if l.kind == "attention":
            s[m + "q"], s[m + "k"], s[m + "v"] = (l.heads * l.dim, W), (l.kv_heads * l.dim, W), (l.kv_heads * l.vdim, W)
            s[m + "q.norm"], s[m + "k.norm"], s[m + "sink"] = (l.dim,), (l.dim,), (l.heads,)
            s[m + "g"], s[m + "o"] = (l.heads, W), (W, l.heads * l.vdim)
            if l.v_mix:
                s[m + "vmix"] = ()
        elif l.kind == "latent_attention":
            s[m + "q"], s[m + "dkv"], s[m + "dkv.norm"] = (l.heads * (l.dim + l.rot_dim), W), (l.kv_rank + l.rot_dim, W), (l.kv_rank,)
            s[m + "uk"], s[m + "uv"] = (l.heads * l.dim, l.kv_rank), (l.heads * l.vdim, l.kv_rank)
            s[m + "g"], s[m + "o"] = (l.heads * l.vdim, W), (W, l.heads * l.vdim)
        else:
            s[m + "q"], s[m + "k"], s[m + "v"] = (l.heads * l.dim, W), (l.heads * l.dim, W), (l.heads * l.vdim, W)
            s[m + "g"], s[m + "o"], s[m + "norm"] = (l.heads * l.vdim, W), (W, l.heads * l.vdim), (l.heads * l.vdim,)
            s[m + "i"], s[m + "i.b"], s[m + "f"], s[m + "f.b"] = (l.heads, W), (l.heads,), (l.heads, W), (l.heads,)
        if l.ff:
            s[p + "norm2"], s[p + "norm2b"], s[p + "rg2"], s[p + "rg2.b"] = (W,), (W,), (W, W), (W,)
            for nm, shp in (("gate", (l.ff, W)), ("up", (l.ff, W)), ("down", (W, l.ff))):
                s[p + "mlp." + nm], s[p + "mlp." + nm + ".b"] = shp, (shp[0],)
    s["final.norm"], s["head"] = (W,), (cfg.vocab_size, W)
    return s


def make_fivesun_weights(cfg, seed: int = 0, device="cpu", scale: float = 1.0):
    """Seeded random weights (bfloat16 torch tensors) with nothing at a value that would hide a dropped term: norm gains around 1,
    non-zero biases, sinks of both signs, blend weights strictly between 0 and 1, forget-gate biases that keep the memory for tens
    of tokens."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    on_gpu = str(device) != "cpu"
    gd = torch.Generator(device=device).manual_seed(seed) if on_gpu else g

    def rnd(shape, big=False):
        if big and on_gpu:
            return torch.randn(shape, generator=gd, device=device, dtype=torch.float32)
        return torch.randn(shape, generator=g, dtype=torch.float32).to(device)

    out = {}
    for name, shp in fivesun_weight_shapes(cfg).items():
        leaf = name.split(".", 1)[-1] if name.startswith("l") and name[1].isdigit() else name
        if leaf in ("norm1", "norm2", "norm1b", "norm2b", "final.norm", "mix.norm", "mix.q.norm", "mix.k.norm", "mix.dkv.norm"):
            w = 1.0 + 0.1 * rnd(shp)
        elif leaf == "mix.vmix":
            w = torch.tensor(0.35, device=device) + 0.1 * rnd(shp)
        elif leaf == "mix.sink":
            w = 0.8 * rnd(shp)
        elif leaf == "mix.f.b":
            w = 3.0 + 0.5 * rnd(shp)
        elif leaf.endswith(".b"):
            w = 0.1 * rnd(shp)
        elif leaf == "embed":
            w = rnd(shp, big=True) / cfg.embed_scale
        else:
            w = (scale / (shp[-1] ** 0.5)) * rnd(shp, big=True)
        out[name] = w.to(torch.bfloat16)
    return out


def load_fivesun_safetensors(path: str, cfg):
    """The tensors of ``<path>/model.safetensors`` by their own names, on the host, checked against the shapes the
    configuration implies."""
    raw = read_checkpoint_dir(path)
    want = fivesun_weight_shapes(cfg)
    missing = [k for k in want if k not in raw]
    if missing:
        raise KeyError(f"{path}: tensors missing for this configuration: {missing[:6]}{' ...' if len(missing) > 6 else ''}")
    for k, shp in want.items():
        if tuple(raw[k].shape) != tuple(shp) and raw[k].numel() != 1:
            raise ValueError(f"{path}: {k} has shape {tuple(raw[k].shape)}, the configuration implies {tuple(shp)}")
    return {k: raw[k] for k in want}


def bepepel_weight_shapes(cfg) -> Dict[str, tuple]:
    """Tensor names and shapes of a Bepepel checkpoint (``model.safetensors``): ``embed``; per layer ``l{i}.norm1`` (+ ``.b``), the
    mixer's ``l{i}.mix.*`` (gla: ``q k v g o norm a1 a2 a2.b``; parallel: ``left.q|k|v`` each with ``.b`` and, with a convolution,
    ``.conv``, ``left.o``, ``right.in conv conv.b dt_bias A_log D norm o``) and, with a feed-forward, ``l{i}.norm2`` (+ ``.b``) and
    ``l{i}.mlp.gate|up|down`` (dense) or ``l{i}.mlp.router`` (+ ``.b``), ``l{i}.mlp.e{j}.gate|up|down`` and ``l{i}.mlp.shared.*``;
    then ``final.norm`` (+ ``.b``) and ``head``."""
    W = cfg.hidden_size
    s = {"embed": (cfg.vocab_size, W)}

    def unit(pre, ff):
        s[pre + "gate"], s[pre + "up"], s[pre + "down"] = (ff, W), (ff, W), (W, ff)

    for i, l in enumerate(cfg.layers):
        p, m = f"l{i}.", f"l{i}.mix."
        s[p + "norm1"], s[p + "norm1.b"] = (W,), (W,)
        if l.kind == "gla":
            HD, HV = l.heads * l.dim, l.heads * l.vdim
            s[m + "q"], s[m + "k"], s[m + "v"], s[m + "g"], s[m + "o"], s[m + "norm"] = (HD, W), (HD, W), (HV, W), (HV, W), (W, HV), (l.vdim,)
            s[m + "a1"], s[m + "a2"], s[m + "a2.b"] = (l.a_rank, W), (HD, l.a_rank), (HD,)
        else:
            a, b = l.left, l.right
            for nm, n in (("q", a.heads * a.dim), ("k", a.kv_heads * a.dim), ("v", a.kv_heads * a.vdim)):
                s[m + "left." + nm], s[m + "left." + nm + ".b"] = (n, W), (n,)
                if a.conv:
                    s[m + "left." + nm + ".conv"] = (n, a.conv)
            s[m + "left.o"] = (W, a.heads * a.vdim)
            r = m + "right."
            s[r + "in"] = (b.in_columns, W)
            if b.conv:
                s[r + "conv"], s[r + "conv.b"] = (b.conv_channels, b.conv), (b.conv_channels,)
            s[r + "dt_bias"], s[r + "A_log"], s[r + "D"], s[r + "norm"], s[r + "o"] = (b.heads,), (b.heads,), (b.heads,), (b.inner,), (W, b.inner)
        if l.ff_kind:
            s[p + "norm2"], s[p + "norm2.b"] = (W,), (W,)
            if l.ff_kind == "dense":
                unit(p + "mlp.", l.ff)
            else:
                s[p + "mlp.router"], s[p + "mlp.router.b"] = (l.experts, W), (l.experts,)
                for j in range(l.experts):
                    unit(p + f"mlp.e{j}.", l.expert_ff)
                if l.shared_ff:
                    unit(p + "mlp.shared.", l.shared_ff)
    s["final.norm"], s["final.norm.b"], s["head"] = (W,), (W,), (cfg.vocab_size, W)
    return s


def make_bepepel_weights(cfg, seed: int = 0, device="cpu", scale: float = 1.0):
    """Seeded random weights (bfloat16 torch tensors) with nothing at a value that would hide a dropped term: norm gains around 1,
    non-zero biases, decay pre-activations that keep a gla state for tens of tokens, step sizes and decay rates of the state-space
    heads spread over a decade, skip weights around 1."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(seed)
    on_gpu = str(device) != "cpu"
    gd = torch.Generator(device=device).manual_seed(seed) if on_gpu else g

    def rnd(shape, big=False):
        if big and on_gpu:
            return torch.randn(shape, generator=gd, device=device, dtype=torch.float32)
        return torch.randn(shape, generator=g, dtype=torch.float32).to(device)

    out = {}
    for name, shp in bepepel_weight_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        if name.endswith(".conv"):
            w = rnd(shp) / (shp[-1] ** 0.5)
        elif leaf in ("norm1", "norm2", "norm", "D"):
            w = 1.0 + 0.1 * rnd(shp)
        elif name.endswith("mix.a2.b"):
            w = 2.0 + 0.5 * rnd(shp)
        elif leaf == "dt_bias":
            w = -1.5 + 0.7 * rnd(shp)
        elif leaf == "A_log":
            w = 0.6 * rnd(shp)
        elif leaf == "b":
            w = 0.1 * rnd(shp)
        elif leaf == "embed":
            w = rnd(shp, big=True)
        else:
            w = (scale / (shp[-1] ** 0.5)) * rnd(shp, big=True)
        out[name] = w.to(torch.bfloat16)
    return out


def load_bepepel_safetensors(path: str, cfg):
    """The tensors of ``<path>/model.safetensors`` by their own names, on the host, checked against the shapes the
    configuration implies.  The low rank of a gla layer's decay projection is not in the configuration: it is read off
    ``l{i}.mix.a1`` and written into ``cfg``."""
    raw = read_checkpoint_dir(path)
    for i, l in enumerate(cfg.layers):
        if l.kind == "gla" and f"l{i}.mix.a1" in raw:
            l.a_rank = int(raw[f"l{i}.mix.a1"].shape[0])
    want = bepepel_weight_shapes(cfg)
    missing = [k for k in want if k not in raw]
    if missing:
        raise KeyError(f"{path}: tensors missing for this configuration: {missing[:6]}{' ...' if len(missing) > 6 else ''}")
    for k, shp in want.items():
        if tuple(raw[k].shape) != tuple(shp):
            raise ValueError(f"{path}: {k} has shape {tuple(raw[k].shape)}, the configuration implies {tuple(shp)}")
    return {k: raw[k] for k in want}
