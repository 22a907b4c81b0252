"""Model shape descriptions for the Llama-2-class adapters.

The reference reads these from HF ``config.json`` via ``LlamaConfig`` (``promptcache/model/llama2.py:262-283``);
the shape constants it quotes for its system benchmarks are at ``eval_sys.py:92-100``.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass, asdict
from typing import Optional


@dataclass
class LlamaShape:
    vocab_size: int = 32000
    hidden_size: int = 4096
    intermediate_size: int = 11008
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    num_key_value_heads: int = 32
    rms_norm_eps: float = 1e-5
    rope_theta: float = 10000.0
    max_position_embeddings: int = 4096
    initializer_range: float = 0.02
    name: str = "llama"

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def kv_bytes_per_token(self) -> int:
        """fp16 K+V bytes per token over all layers (7b = 524288)."""
        return 2 * self.num_hidden_layers * self.num_key_value_heads * self.head_dim * 2

    def to_dict(self):
        return asdict(self)

    @classmethod
    def from_hf_dir(cls, path: str) -> "LlamaShape":
        with open(os.path.join(path, "config.json")) as f:
            c = json.load(f)
        return cls(
            vocab_size=c["vocab_size"], hidden_size=c["hidden_size"],
            intermediate_size=c["intermediate_size"], num_hidden_layers=c["num_hidden_layers"],
            num_attention_heads=c["num_attention_heads"],
            num_key_value_heads=c.get("num_key_value_heads", c["num_attention_heads"]),
            rms_norm_eps=c.get("rms_norm_eps", 1e-5), rope_theta=c.get("rope_theta", 10000.0),
            max_position_embeddings=c.get("max_position_embeddings", 4096),
            name=os.path.basename(os.path.normpath(path)))


@dataclass
class FalconShape:
    """Falcon-7b-class decoder (``promptcache/model/falcon.py``: multi-query attention with ONE shared K/V head,
    parallel attention + MLP behind a single LayerNorm, GELU MLP of width 4*hidden, rotary positions, no biases in
    the linears).  The reference reads these from HF ``config.json`` via ``FalconConfig``; its cache shape is
    ``(L, 1, head_dim)`` (``promptcache/model/__init__.py:256-258``)."""
    vocab_size: int = 65024
    hidden_size: int = 4544
    num_hidden_layers: int = 32
    num_attention_heads: int = 71
    layer_norm_epsilon: float = 1e-5
    rope_theta: float = 10000.0
    initializer_range: float = 0.02
    tie_word_embeddings: bool = False
    name: str = "falcon"

    num_key_value_heads = 1            # multi_query

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def intermediate_size(self) -> int:
        return 4 * self.hidden_size

    @property
    def kv_bytes_per_token(self) -> int:
        return 2 * self.num_hidden_layers * self.head_dim * 2

    def to_dict(self):
        return asdict(self)

    @classmethod
    def from_hf_dir(cls, path: str) -> "FalconShape":
        with open(os.path.join(path, "config.json")) as f:
            c = json.load(f)
        if c.get("new_decoder_architecture") or not c.get("multi_query", True) or not c.get("parallel_attn", True) \
                or c.get("alibi") or c.get("bias"):
            raise ValueError("only the falcon-7b architecture (multi_query, parallel_attn, rotary, no bias) is supported")
        return cls(vocab_size=c["vocab_size"], hidden_size=c["hidden_size"],
                   num_hidden_layers=c.get("num_hidden_layers", c.get("n_layer")),
                   num_attention_heads=c.get("num_attention_heads", c.get("n_head")),
                   layer_norm_epsilon=c.get("layer_norm_epsilon", 1e-5), rope_theta=c.get("rope_theta", 10000.0),
                   tie_word_embeddings=c.get("tie_word_embeddings", True),
                   name=os.path.basename(os.path.normpath(path)))


FALCON_SHAPES = {
    "falcon-tiny": FalconShape(vocab_size=1024, hidden_size=128, num_hidden_layers=2, num_attention_heads=4, name="falcon-tiny"),
    # head_dim 64 like falcon-7b, an odd head count like its 71
    "falcon-mid": FalconShape(vocab_size=2048, hidden_size=448, num_hidden_layers=2, num_attention_heads=7, name="falcon-mid"),
    "falcon-7b": FalconShape(name="falcon-7b"),
}

@dataclass
class MptShape:
    """MPT-7b-class decoder (``promptcache/model/mpt.py``): multi-head attention with ALiBi position biases (no
    rotary), fused ``Wqkv`` = [q | k | v], bias-free LayerNorms, GELU MLP of width 4*d_model, lm_head tied to the
    embedding.  The reference reads these from ``MptConfig``; its cache shape is ``(n_layers, n_heads, head_dim)``
    (``promptcache/model/__init__.py:284-286``)."""
    vocab_size: int = 50432
    hidden_size: int = 4096
    num_hidden_layers: int = 32
    num_attention_heads: int = 32
    layer_norm_epsilon: float = 1e-5
    alibi_bias_max: int = 8
    initializer_range: float = 0.02
    tie_word_embeddings: bool = False
    name: str = "mpt"

    @property
    def num_key_value_heads(self) -> int:
        return self.num_attention_heads

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    @property
    def intermediate_size(self) -> int:
        return 4 * self.hidden_size

    @property
    def kv_bytes_per_token(self) -> int:
        return 2 * self.num_hidden_layers * self.num_attention_heads * self.head_dim * 2

    def to_dict(self):
        return asdict(self)

    @classmethod
    def from_hf_dir(cls, path: str) -> "MptShape":
        with open(os.path.join(path, "config.json")) as f:
            c = json.load(f)
        ac = c.get("attn_config", {})
        if not ac.get("alibi", True) or not c.get("no_bias", True) or ac.get("clip_qkv") or ac.get("qk_ln"):
            raise ValueError("only the mpt-7b architecture (alibi, no biases, no qkv clipping / qk layernorm) is supported")
        return cls(vocab_size=c["vocab_size"], hidden_size=c["d_model"], num_hidden_layers=c["n_layers"],
                   num_attention_heads=c["n_heads"], layer_norm_epsilon=c.get("layer_norm_epsilon", 1e-5),
                   alibi_bias_max=ac.get("alibi_bias_max", 8), tie_word_embeddings=True,
                   name=os.path.basename(os.path.normpath(path)))


MPT_SHAPES = {
    "mpt-tiny": MptShape(vocab_size=1024, hidden_size=128, num_hidden_layers=2, num_attention_heads=4, name="mpt-tiny"),
    # head_dim 64.  (Head counts must be powers of two: the reference's slope table raises otherwise, mpt.py:104.)
    "mpt-mid": MptShape(vocab_size=2048, hidden_size=512, num_hidden_layers=2, num_attention_heads=8, name="mpt-mid"),
    "mpt-7b": MptShape(name="mpt-7b"),
}

SHAPES = {
    # test-sized
    "tiny": LlamaShape(vocab_size=1024, hidden_size=128, intermediate_size=344, num_hidden_layers=2,
                       num_attention_heads=4, num_key_value_heads=4, rms_norm_eps=1e-6, name="tiny"),
    # D=128 like the real models (MHA: the reference's cache engine cannot stage GQA, its
    # get_cache_shape returns num_attention_heads, promptcache/model/__init__.py:110-114)
    "mid": LlamaShape(vocab_size=2048, hidden_size=512, intermediate_size=1376, num_hidden_layers=3,
                      num_attention_heads=4, num_key_value_heads=4, rms_norm_eps=1e-5, name="mid"),
    # every GEMM K a multiple of 64 (what the int8-weight images need), D = 128, MHA and GQA
    "mid64": LlamaShape(vocab_size=2048, hidden_size=512, intermediate_size=1408, num_hidden_layers=3,
                        num_attention_heads=4, num_key_value_heads=4, rms_norm_eps=1e-5, name="mid64"),
    "mid64_gqa": LlamaShape(vocab_size=2048, hidden_size=512, intermediate_size=1408, num_hidden_layers=3,
                            num_attention_heads=4, num_key_value_heads=2, rms_norm_eps=1e-5, name="mid64_gqa"),
    # GQA 2:1 so the head-broadcast index math is exercised (oracle-checked only)
    "mid_gqa": LlamaShape(vocab_size=2048, hidden_size=512, intermediate_size=1376, num_hidden_layers=3,
                          num_attention_heads=4, num_key_value_heads=2, rms_norm_eps=1e-5, name="mid_gqa"),
    # D=128, MHA, 2 layers at hidden 256 (cheap full-path checks)
    "mid_mha": LlamaShape(vocab_size=2048, hidden_size=256, intermediate_size=688, num_hidden_layers=2,
                          num_attention_heads=2, num_key_value_heads=2, rms_norm_eps=1e-5, name="mid_mha"),
    # BASELINE.json configs
    "llama2-7b": LlamaShape(name="llama2-7b"),
    "llama2-13b": LlamaShape(hidden_size=5120, intermediate_size=13824, num_hidden_layers=40,
                             num_attention_heads=40, num_key_value_heads=40, name="llama2-13b"),
    "codellama-7b": LlamaShape(vocab_size=32016, rope_theta=1e6, max_position_embeddings=16384,
                               name="codellama-7b"),
}


@dataclass
class KazolornLayer:
    """One layer of a Kazolorn stack: an attention mixer and, beside it (both read the layer's input), an optional
    feed-forward.  ``window`` 0 = every earlier key; ``mlp_kind`` None | "dense" | "moe"."""
    heads: int
    kv_heads: int
    dim: int
    scale: float
    window: int = 0
    mlp_kind: object = None
    ff: int = 0
    experts: int = 0
    top: int = 0


@dataclass
class KazolornShape:
    """Kazolorn: decoder-only, parallel layers (mixer and feed-forward of the same input, each behind its own RMS norm and a
    learned per-channel layer scale), a learned weighted sum of all earlier layer results in front of every layer, attention
    without a value projection (the keys are the values) with a linear distance bias, cross-head score mixing, a sliding
    window and a sink in the softmax denominator; dense feed-forwards use a polynomial-of-normalised-powers activation,
    sparse ones a sigmoid top-k router whose weights scale the experts' inputs.  Every size and constant comes from
    ``config.json`` (``from_config``); layers may differ from one another."""
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: list
    name: str = "kazolorn"
    initializer_range: float = 0.05

    ARCHITECTURE = "Kazolorn"

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_config(cls, c: dict, name: str = "kazolorn") -> "KazolornShape":
        if c.get("architecture") != cls.ARCHITECTURE:
            raise ValueError(f"config.json describes {c.get('architecture')!r}, not {cls.ARCHITECTURE}")
        layers = []
        for i, lc in enumerate(c["layers"]):
            if lc.get("type") != "attention":
                raise ValueError(f"layer {i}: unknown mixer type {lc.get('type')!r}")
            m = lc["mixer"]
            heads, dim = int(m["heads"]), int(m["dim"])
            kv = int(m.get("kv_heads", heads))
            if heads % kv:
                raise ValueError(f"layer {i}: {heads} query heads do not divide over {kv} key heads")
            if int(m.get("vdim", dim)) != dim:
                raise ValueError(f"layer {i}: the values are the keys, so vdim must equal dim ({m.get('vdim')} != {dim})")
            mask = m.get("mask") or {}
            lay = KazolornLayer(heads=heads, kv_heads=kv, dim=dim, scale=float(m["scale"]), window=int(mask.get("size") or 0))
            mlp = lc.get("mlp")
            if mlp:
                kind = mlp.get("kind")
                if kind == "dense":
                    lay.mlp_kind, lay.ff = "dense", int(mlp["ff"])
                elif kind == "moe":
                    lay.mlp_kind, lay.ff = "moe", int(mlp["expert"]["ff"])
                    lay.experts, lay.top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
                    if not 1 <= lay.top <= lay.experts:
                        raise ValueError(f"layer {i}: top {lay.top} of {lay.experts} experts")
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
            layers.append(lay)
        return cls(vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), norm_eps=float(c["norm"]["eps"]), layers=layers,
                   name=name)

    @classmethod
    def from_dir(cls, path: str) -> "KazolornShape":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_config(json.load(f), name=os.path.basename(os.path.normpath(path)))

    def to_config(self) -> dict:
        """The ``config.json`` form (what ``from_config`` reads)."""
        out = []
        for l in self.layers:
            mixer = {"dim": l.dim, "heads": l.heads, "kv_heads": l.kv_heads, "scale": l.scale, "vdim": l.dim}
            if l.window:
                mixer["mask"] = {"size": l.window}
            mlp = None
            if l.mlp_kind == "dense":
                mlp = {"kind": "dense", "ff": l.ff}
            elif l.mlp_kind == "moe":
                mlp = {"kind": "moe", "expert": {"ff": l.ff}, "router": {"experts": l.experts, "top": l.top}}
            out.append({"type": "attention", "mixer": mixer, "mlp": mlp})
        return {"architecture": self.ARCHITECTURE, "layers": out, "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size,
                "width": self.hidden_size}

    @classmethod
    def uniform(cls, vocab: int, width: int, n_layers: int, heads: int, kv_heads: int, dim: int, window: int, ff: int,
                experts: int = 0, top: int = 0, expert_ff: int = 0, dense_first: int = 1, eps: float = 1e-6,
                name: str = "kazolorn") -> "KazolornShape":
        """A stack of equal layers: the first ``dense_first`` with a dense feed-forward, the rest sparse (dense when
        ``experts`` is 0)."""
        layers = []
        for i in range(n_layers):
            lay = KazolornLayer(heads=heads, kv_heads=kv_heads, dim=dim, scale=dim ** -0.5, window=window)
            if experts and i >= dense_first:
                lay.mlp_kind, lay.ff, lay.experts, lay.top = "moe", expert_ff, experts, top
            else:
                lay.mlp_kind, lay.ff = "dense", ff
            layers.append(lay)
        return cls(vocab_size=vocab, hidden_size=width, norm_eps=eps, layers=layers, name=name)


@dataclass
class DibizenLayer:
    """One layer of a Dibizen stack.  ``kind``: which mixer it has --

    * ``"lightning"``: linear attention with one scalar decay per head (``decay``), ``heads`` heads of ``dim`` query/key and
      ``vdim`` value columns;
    * ``"attention"``: causal softmax attention, ``heads`` query heads over ``kv_heads`` key/value heads, scores scaled by
      ``scale``, queries scaled by a temperature that grows with the logarithm of the position (``qt_coef``, ``qt_every``;
      ``qt_every`` 0 = none), ``kv_from`` >= 0: no key/value projections of its own, it reads that layer's cache;
    * ``"mamba1"``: selective scan over ``inner`` channels with ``state`` states each, a causal convolution of ``conv`` taps in
      front, step sizes through a ``dt_rank``-wide bottleneck.

    The feed-forward (``experts`` 0 = none) is a mixture of ``experts`` squared-ReLU experts of width ``ff`` plus ``identity``
    experts that return their input; ``top`` of them are chosen per token among the best ``groups_keep`` of ``groups`` groups."""
    kind: str
    heads: int = 0
    kv_heads: int = 0
    dim: int = 0
    vdim: int = 0
    scale: float = 1.0
    decay: tuple = ()
    qt_coef: float = 0.0
    qt_every: int = 0
    kv_from: int = -1
    inner: int = 0
    state: int = 0
    conv: int = 0
    dt_rank: int = 0
    ff: int = 0
    experts: int = 0
    identity: int = 0
    top: int = 0
    groups: int = 1
    groups_keep: int = 1


@dataclass
class DibizenShape:
    """Dibizen: decoder-only, learned absolute positions, ``streams`` residual streams mixed by hyper-connections around every
    sublayer, Dynamic-Tanh norms, layers whose mixer is lightning (decayed linear) attention, gated softmax attention (which may
    borrow an earlier layer's keys and values) or a Mamba selective scan, mixture-of-experts feed-forwards with a corrected,
    group-limited softmax router and identity experts, and soft-capped logits.  Every size and constant comes from
    ``config.json`` (``from_config``); layers may differ from one another and come in any order."""
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: list
    streams: int = 1
    max_positions: int = 0
    logit_softcap: float = 0.0
    name: str = "dibizen"

    ARCHITECTURE = "Dibizen"

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_config(cls, c: dict, name: str = "dibizen") -> "DibizenShape":
        if c.get("architecture") != cls.ARCHITECTURE:
            raise ValueError(f"config.json describes {c.get('architecture')!r}, not {cls.ARCHITECTURE}")
        layers = []
        for i, lc in enumerate(c["layers"]):
            kind, m = lc.get("type"), lc.get("mixer") or {}
            if kind == "lightning":
                lay = DibizenLayer(kind, heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m.get("vdim", m["dim"])),
                                   decay=tuple(float(d) for d in m["decay"]))
                lay.kv_heads = lay.heads
                if len(lay.decay) != lay.heads:
                    raise ValueError(f"layer {i}: {len(lay.decay)} decays for {lay.heads} heads")
            elif kind == "attention":
                heads, dim = int(m["heads"]), int(m["dim"])
                kv = int(m.get("kv_heads", heads))
                if heads % kv:
                    raise ValueError(f"layer {i}: {heads} query heads do not divide over {kv} key heads")
                qt = m.get("q_temp") or {}
                lay = DibizenLayer(kind, heads=heads, kv_heads=kv, dim=dim, vdim=int(m.get("vdim", dim)),
                                   scale=float(m.get("scale", dim ** -0.5)), qt_coef=float(qt.get("coef", 0.0)),
                                   qt_every=int(qt.get("every", 0)) if qt else 0,
                                   kv_from=int(m["kv_from"]) if m.get("kv_from") is not None else -1)
                if lay.kv_from >= 0:
                    src = layers[lay.kv_from] if lay.kv_from < i else None
                    if src is None or src.kind != "attention" or src.kv_from >= 0 or \
                            (src.kv_heads, src.dim, src.vdim) != (lay.kv_heads, lay.dim, lay.vdim):
                        raise ValueError(f"layer {i}: kv_from {lay.kv_from} must name an earlier attention layer with projections "
                                         f"of its own and the same key/value heads and sizes")
            elif kind == "mamba1":
                lay = DibizenLayer(kind, inner=int(m["inner"]), state=int(m["state"]), conv=int(m["conv"]), dt_rank=int(m["dt_rank"]))
                if lay.conv < 1:
                    raise ValueError(f"layer {i}: a convolution has at least one tap")
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp = lc.get("mlp")
            if mlp:
                if mlp.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                r = mlp["router"]
                g = r.get("groups") or {}
                lay.ff, lay.experts, lay.identity = int(mlp["expert"]["ff"]), int(r["experts"]), int(r.get("identity", 0))
                lay.top, lay.groups = int(r["top"]), int(g.get("count", 1))
                lay.groups_keep = int(g.get("keep", lay.groups))
                total = lay.experts + lay.identity
                if total % lay.groups or not 1 <= lay.groups_keep <= lay.groups:
                    raise ValueError(f"layer {i}: {total} router outputs in {lay.groups} groups, {lay.groups_keep} kept")
                if not 1 <= lay.top <= total // lay.groups * lay.groups_keep:
                    raise ValueError(f"layer {i}: top {lay.top} of {total} router outputs with {lay.groups_keep} of {lay.groups} groups")
            layers.append(lay)
        return cls(vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), norm_eps=float((c.get("norm") or {}).get("eps", 1e-5)),
                   layers=layers, streams=int(c.get("streams", 1)), max_positions=int(c.get("max_positions") or 0),
                   logit_softcap=float(c.get("logit_softcap") or 0.0), name=name)

    @classmethod
    def from_dir(cls, path: str) -> "DibizenShape":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_config(json.load(f), name=os.path.basename(os.path.normpath(path)))

    def to_config(self) -> dict:
        """The ``config.json`` form (what ``from_config`` reads)."""
        out = []
        for l in self.layers:
            if l.kind == "lightning":
                mixer = {"decay": list(l.decay), "dim": l.dim, "heads": l.heads, "vdim": l.vdim}
            elif l.kind == "attention":
                mixer = {"dim": l.dim, "heads": l.heads, "kv_heads": l.kv_heads, "scale": l.scale, "vdim": l.vdim}
                if l.qt_every:
                    mixer["q_temp"] = {"coef": l.qt_coef, "every": l.qt_every}
                if l.kv_from >= 0:
                    mixer["kv_from"] = l.kv_from
            else:
                mixer = {"conv": l.conv, "dt_rank": l.dt_rank, "inner": l.inner, "state": l.state}
            mlp = None
            if l.experts + l.identity:
                mlp = {"kind": "moe", "expert": {"ff": l.ff},
                       "router": {"experts": l.experts, "groups": {"count": l.groups, "keep": l.groups_keep},
                                  "identity": l.identity, "top": l.top}}
            out.append({"type": l.kind, "mixer": mixer, "mlp": mlp})
        return {"architecture": self.ARCHITECTURE, "layers": out, "logit_softcap": self.logit_softcap,
                "max_positions": self.max_positions, "norm": {"eps": self.norm_eps}, "streams": self.streams,
                "vocab": self.vocab_size, "width": self.hidden_size}

    @classmethod
    def uniform(cls, vocab: int, width: int, pattern, heads: int, kv_heads: int, dim: int, experts: int, top: int, expert_ff: int,
                identity: int = 0, groups: int = 1, groups_keep: int = 1, streams: int = 2, inner: int = 0, state: int = 16,
                max_positions: int = 8192, name: str = "dibizen") -> "DibizenShape":
        """A stack whose layers follow ``pattern`` (a sequence of mixer kinds), all with the same sizes and feed-forward."""
        layers = []
        for kind in pattern:
            if kind == "lightning":
                lay = DibizenLayer(kind, heads=heads, kv_heads=heads, dim=dim, vdim=dim,
                                   decay=tuple(1.0 - 2.0 ** (-5.0 - 3.0 * h / max(1, heads - 1)) for h in range(heads)))
            elif kind == "attention":
                lay = DibizenLayer(kind, heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, qt_coef=0.1,
                                   qt_every=1024)
            else:
                lay = DibizenLayer("mamba1", inner=inner or 2 * width, state=state, conv=4, dt_rank=max(1, width // 16))
            lay.ff, lay.experts, lay.identity, lay.top, lay.groups, lay.groups_keep = expert_ff, experts, identity, top, groups, groups_keep
            layers.append(lay)
        return cls(vocab_size=vocab, hidden_size=width, norm_eps=1e-5, layers=layers, streams=streams, max_positions=max_positions,
                   logit_softcap=30.0, name=name)


@dataclass
class FivesunLayer:
    """One layer of a Fivesun stack.  ``kind``: which mixer it has --

    * ``"attention"``: softmax attention with ``heads`` query heads over ``kv_heads`` key/value heads (``dim`` query/key and
      ``vdim`` value columns), per-head RMS norms on queries and keys, interleaved rotary positions on the first ``rot_dims``
      columns (frequencies divided by ``rot_factor``), unit-RMS values, a learned sink per head in the softmax denominator, one
      sigmoid output gate per head, keys visible only inside the query's own block of ``mask`` positions (0: all earlier keys);
      ``v_mix``: the values are blended with those of the first such layer;
    * ``"latent_attention"``: ``heads`` heads whose keys and values are up-projections of one cached latent of ``kv_rank``
      columns per token, plus one rotated key part of ``rot_dim`` columns shared by all heads (YaRN-scaled frequencies:
      ``rot_factor``, ``yarn_original``, ``yarn_fast``, ``yarn_slow``; ``yarn_original`` 0 = plain frequencies), a sliding window
      of ``mask`` positions (0: none) and an element-wise sigmoid output gate;
    * ``"mlstm"``: the matrix memory of xLSTM -- per head a ``dim`` x ``vdim`` state with exponential input gates, sigmoid forget
      gates (pre-activations soft-capped at ``gate_cap``; 0 = not capped) and a running maximum that keeps the exponentials finite.

    ``ff`` 0: no feed-forward; else a gated dense unit of that width, ``act`` its activation (relu, silu or gelu_tanh)."""
    kind: str
    heads: int = 0
    kv_heads: int = 0
    dim: int = 0
    vdim: int = 0
    scale: float = 1.0
    mask: int = 0
    rot_base: float = 10000.0
    rot_dims: int = 0
    rot_factor: float = 1.0
    v_mix: bool = False
    kv_rank: int = 0
    rot_dim: int = 0
    yarn_original: float = 0.0
    yarn_fast: float = 32.0
    yarn_slow: float = 1.0
    gate_cap: float = 0.0
    ff: int = 0
    act: str = "relu"


@dataclass
class FivesunShape:
    """Fivesun: decoder-only, a scaled embedding, layers in any order whose mixer is chunked softmax attention with sinks,
    windowed latent attention or an mLSTM matrix memory, every sublayer between a norm before and a norm after it with a sigmoid
    gate on its result (x <- x + norm_after(gate * f(norm_before(x)))), dense gated feed-forwards with biases.  Every size and
    constant comes from ``config.json`` (``from_config``)."""
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: list
    embed_scale: float = 1.0
    name: str = "fivesun"

    ARCHITECTURE = "Fivesun"
    KINDS = ("attention", "latent_attention", "mlstm")

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @property
    def first_v_mix(self) -> int:
        """Index of the first layer whose values the later ``v_mix`` layers blend in (-1: none)."""
        for i, l in enumerate(self.layers):
            if l.kind == "attention" and l.v_mix:
                return i
        return -1

    @classmethod
    def from_config(cls, c: dict, name: str = "fivesun") -> "FivesunShape":
        if c.get("architecture") != cls.ARCHITECTURE:
            raise ValueError(f"config.json describes {c.get('architecture')!r}, not {cls.ARCHITECTURE}")
        layers = []
        for i, lc in enumerate(c["layers"]):
            kind, m = lc.get("type"), lc.get("mixer") or {}
            rot = m.get("rot") or {}
            sc = rot.get("scaling") or {}
            mask = int((m.get("mask") or {}).get("size") or 0)
            if kind == "attention":
                heads, dim = int(m["heads"]), int(m["dim"])
                kv = int(m.get("kv_heads") or heads)
                if heads % kv:
                    raise ValueError(f"layer {i}: {heads} query heads do not divide over {kv} key heads")
                lay = FivesunLayer(kind, heads=heads, kv_heads=kv, dim=dim, vdim=int(m.get("vdim") or dim),
                                   scale=float(m.get("scale", dim ** -0.5)), mask=mask, rot_base=float(rot.get("base", 10000.0)),
                                   rot_dims=int(rot.get("dims", dim if rot else 0)), rot_factor=float(sc.get("factor", 1.0)),
                                   v_mix=bool(m.get("v_mix", False)))
                if lay.rot_dims % 2 or lay.rot_dims > dim:
                    raise ValueError(f"layer {i}: {lay.rot_dims} rotated columns of {dim}")
            elif kind == "latent_attention":
                heads, dim, rd = int(m["heads"]), int(m["dim"]), int(m.get("rot_dim") or 0)
                lay = FivesunLayer(kind, heads=heads, kv_heads=1, dim=dim, vdim=int(m.get("vdim") or dim), kv_rank=int(m["kv_rank"]),
                                   rot_dim=rd, rot_dims=rd, scale=float(m.get("scale", (dim + rd) ** -0.5)), mask=mask,
                                   rot_base=float(rot.get("base", 10000.0)), rot_factor=float(sc.get("factor", 1.0)),
                                   yarn_original=float(sc.get("original", 0.0)), yarn_fast=float(sc.get("fast", 32.0)),
                                   yarn_slow=float(sc.get("slow", 1.0)))
                if rd % 2 or int(rot.get("dims", rd)) != rd:
                    raise ValueError(f"layer {i}: the rotated part has {rd} columns, the rotation {rot.get('dims')}")
            elif kind == "mlstm":
                heads, dim = int(m["heads"]), int(m["dim"])
                lay = FivesunLayer(kind, heads=heads, kv_heads=heads, dim=dim, vdim=int(m.get("vdim") or dim),
                                   gate_cap=float(m.get("gate_cap") or 0.0))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp = lc.get("mlp")
            if mlp:
                if mlp.get("kind", "dense") != "dense":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {mlp.get('kind')!r}")
                lay.ff, lay.act = int(mlp["ff"]), str(mlp.get("act", "relu"))
                if lay.act not in ("relu", "silu", "gelu_tanh"):
                    raise ValueError(f"layer {i}: unknown activation {lay.act!r}")
            layers.append(lay)
        shape = cls(vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), norm_eps=float((c.get("norm") or {}).get("eps", 1e-6)),
                    layers=layers, embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)), name=name)
        shape.check()
        return shape

    def check(self) -> None:
        first = self.first_v_mix
        for i, l in enumerate(self.layers):
            if l.kind not in self.KINDS:
                raise ValueError(f"layer {i}: unknown mixer type {l.kind!r}")
            if l.kind == "attention" and l.v_mix and (l.kv_heads, l.vdim) != (self.layers[first].kv_heads, self.layers[first].vdim):
                raise ValueError(f"layer {i}: blends its values with layer {first}'s, which have another shape")

    @classmethod
    def from_dir(cls, path: str) -> "FivesunShape":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_config(json.load(f), name=os.path.basename(os.path.normpath(path)))

    def to_config(self) -> dict:
        """The ``config.json`` form (what ``from_config`` reads)."""
        out = []
        for l in self.layers:
            if l.kind == "attention":
                mixer = {"dim": l.dim, "heads": l.heads, "kv_heads": l.kv_heads, "scale": l.scale, "v_mix": l.v_mix, "vdim": l.vdim}
                if l.rot_dims:
                    mixer["rot"] = {"base": l.rot_base, "dims": l.rot_dims, "scaling": {"factor": l.rot_factor}}
            elif l.kind == "latent_attention":
                mixer = {"dim": l.dim, "heads": l.heads, "kv_rank": l.kv_rank, "rot_dim": l.rot_dim, "scale": l.scale, "vdim": l.vdim,
                         "rot": {"base": l.rot_base, "dims": l.rot_dim}}
                if l.yarn_original:
                    mixer["rot"]["scaling"] = {"factor": l.rot_factor, "fast": l.yarn_fast, "original": l.yarn_original,
                                               "slow": l.yarn_slow}
            else:
                mixer = {"dim": l.dim, "gate_cap": l.gate_cap, "heads": l.heads, "vdim": l.vdim}
            if l.mask:
                mixer["mask"] = {"size": l.mask}
            mlp = {"ff": l.ff, "kind": "dense"} if l.ff else None
            if mlp and l.act != "relu":
                mlp["act"] = l.act
            out.append({"type": l.kind, "mixer": mixer, "mlp": mlp})
        return {"architecture": self.ARCHITECTURE, "embedding": {"scale": self.embed_scale}, "layers": out,
                "norm": {"eps": self.norm_eps}, "vocab": self.vocab_size, "width": self.hidden_size}

    @classmethod
    def uniform(cls, vocab: int, width: int, pattern, heads: int, kv_heads: int, dim: int, ff: int, chunk: int = 0, window: int = 0,
                kv_rank: int = 0, rot_dim: int = 64, name: str = "fivesun") -> "FivesunShape":
        """A stack whose layers follow ``pattern`` (a sequence of mixer kinds), all with the same sizes and feed-forward."""
        layers = []
        for kind in pattern:
            if kind == "attention":
                lay = FivesunLayer(kind, heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=dim ** -0.5, mask=chunk,
                                   rot_base=1000000.0, rot_dims=dim, rot_factor=4.0, v_mix=True)
            elif kind == "latent_attention":
                lay = FivesunLayer(kind, heads=heads, kv_heads=1, dim=dim, vdim=dim, kv_rank=kv_rank or 4 * dim, rot_dim=rot_dim,
                                   rot_dims=rot_dim, scale=(dim + rot_dim) ** -0.5, mask=window, rot_base=10000.0, rot_factor=8.0,
                                   yarn_original=4096.0)
            else:
                lay = FivesunLayer("mlstm", heads=heads, kv_heads=heads, dim=dim, vdim=dim, gate_cap=10.0)
            lay.ff = ff
            layers.append(lay)
        return cls(vocab_size=vocab, hidden_size=width, norm_eps=1e-6, layers=layers, embed_scale=width ** 0.5, name=name)

@dataclass
class BepepelAttention:
    """The softmax half of a Bepepel ``parallel`` mixer: ``heads`` query heads over ``kv_heads`` key/value heads (``dim`` query/key
    and ``vdim`` value columns), projections with biases, a causal convolution of ``conv`` taps per channel on q, k and v (0: none),
    interleaved rotary pairs on the first ``rot_dims`` columns (``rot_scaling``: None, or (factor, low, high, original) of the
    wavelength-dependent frequency scaling), unit-RMS queries and keys, score = ``scale`` q.k, a sliding window of ``window``
    positions (0: all earlier keys) that also keeps the sequence's first ``keep_first`` positions visible."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int = 0
    window: int = 0
    keep_first: int = 0
    rot_base: float = 10000.0
    rot_dims: int = 0
    rot_scaling: Optional[tuple] = None


@dataclass
class BepepelSSD:
    """The state-space half of a Bepepel ``parallel`` mixer (Mamba-2): ``heads`` heads of ``vdim`` channels, a ``state`` x ``vdim``
    matrix state per head with one scalar decay per head and token, B and C shared by the heads of each of ``groups`` groups, a
    causal convolution of ``conv`` taps over x | B | C (0: none), the gated output normed in ``norm_groups`` equal parts."""
    heads: int
    vdim: int
    state: int
    groups: int = 1
    norm_groups: int = 1
    conv: int = 0

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state

    @property
    def in_columns(self) -> int:
        return 2 * self.inner + 2 * self.groups * self.state + self.heads


@dataclass
class BepepelLayer:
    """One layer of a Bepepel stack.  ``kind``: which mixer it has --

    * ``"gla"``: gated linear attention, ``heads`` heads with a ``dim`` x ``vdim`` matrix state each and one decay per key channel
      and token, sigmoid(low-rank projection)^(1 / ``tau``); per-head unit-RMS outputs with a shared gain, a SiLU output gate;
    * ``"parallel"``: ``left`` (``BepepelAttention``) and ``right`` (``BepepelSSD``) read the same input and their results are added
      as ``left_scale`` * left + ``right_scale`` * right.

    ``ff_kind``: "" (no feed-forward), "dense" (a gated unit of width ``ff``, tanh-form GELU) or "moe" (``experts`` gated SiLU units
    of width ``expert_ff`` of which each token uses the ``top`` with the largest router logits, weighted by the softmax over those
    logits, plus -- ``shared_ff`` > 0 -- one unit of that width that every token uses)."""
    kind: str
    heads: int = 0
    dim: int = 0
    vdim: int = 0
    tau: float = 1.0
    a_rank: int = 0
    left: Optional[BepepelAttention] = None
    right: Optional[BepepelSSD] = None
    left_scale: float = 1.0
    right_scale: float = 1.0
    ff_kind: str = ""
    ff: int = 0
    experts: int = 0
    top: int = 0
    expert_ff: int = 0
    shared_ff: int = 0


@dataclass
class BepepelShape:
    """Bepepel: decoder-only, pre-norm layers (layer norms with weight and bias) whose results enter the residual stream times
    ``residual_mult``, mixers gated linear attention or a softmax attention and a Mamba-2 side by side, dense or mixture-of-experts
    feed-forwards, logits times ``logit_scale``.  Every size and constant comes from ``config.json`` (``from_config``); the low rank
    of the decay projection is a tensor's shape and is filled in by the weight loader (``a_rank`` 0: not known yet)."""
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: list
    residual_mult: float = 1.0
    logit_scale: float = 1.0
    name: str = "bepepel"

    ARCHITECTURE = "Bepepel"
    KINDS = ("gla", "parallel")

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_config(cls, c: dict, name: str = "bepepel") -> "BepepelShape":
        if c.get("architecture") != cls.ARCHITECTURE:
            raise ValueError(f"config.json describes {c.get('architecture')!r}, not {cls.ARCHITECTURE}")
        layers = []
        for i, lc in enumerate(c["layers"]):
            kind, m = lc.get("type"), lc.get("mixer") or {}
            if kind == "gla":
                dim = int(m["dim"])
                lay = BepepelLayer(kind, heads=int(m["heads"]), dim=dim, vdim=int(m.get("vdim") or dim), tau=float(m.get("tau", 1.0)),
                                   a_rank=int(m.get("a_rank") or 0))
            elif kind == "parallel":
                a, b = m["left"], m["right"]
                rot, mask = a.get("rot") or {}, a.get("mask") or {}
                sc = rot.get("scaling")
                heads, dim = int(a["heads"]), int(a["dim"])
                left = BepepelAttention(heads=heads, kv_heads=int(a.get("kv_heads") or heads), dim=dim, vdim=int(a.get("vdim") or dim),
                                        scale=float(a.get("scale", dim ** -0.5)), conv=int(a.get("conv") or 0),
                                        window=int(mask.get("size") or 0), keep_first=int(mask.get("keep_first") or 0),
                                        rot_base=float(rot.get("base", 10000.0)), rot_dims=int(rot.get("dims", dim if rot else 0)),
                                        rot_scaling=(float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"]))
                                        if sc else None)
                right = BepepelSSD(heads=int(b["heads"]), vdim=int(b["vdim"]), state=int(b["state"]), groups=int(b.get("groups") or 1),
                                   norm_groups=int(b.get("norm_groups") or 1), conv=int(b.get("conv") or 0))
                lay = BepepelLayer(kind, left=left, right=right, left_scale=float(m.get("left_scale", 1.0)),
                                   right_scale=float(m.get("right_scale", 1.0)))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            mlp = lc.get("mlp")
            if mlp:
                fk = mlp.get("kind", "dense")
                if fk == "dense":
                    lay.ff_kind, lay.ff = "dense", int(mlp["ff"])
                elif fk == "moe":
                    lay.ff_kind, lay.experts, lay.top = "moe", int(mlp["router"]["experts"]), int(mlp["router"]["top"])
                    lay.expert_ff = int(mlp["expert"]["ff"])
                    lay.shared_ff = int((mlp.get("shared") or {}).get("ff") or 0)
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {fk!r}")
            layers.append(lay)
        shape = cls(vocab_size=int(c["vocab"]), hidden_size=int(c["width"]), norm_eps=float((c.get("norm") or {}).get("eps", 1e-6)),
                    layers=layers, residual_mult=float(c.get("residual_mult", 1.0)), logit_scale=float(c.get("logit_scale", 1.0)),
                    name=name)
        shape.check()
        return shape

    def check(self) -> None:
        for i, l in enumerate(self.layers):
            if l.kind not in self.KINDS:
                raise ValueError(f"layer {i}: unknown mixer type {l.kind!r}")
            if l.kind == "gla":
                if min(l.heads, l.dim, l.vdim) < 1 or l.tau <= 0:
                    raise ValueError(f"layer {i}: gated linear attention needs heads, sizes and a positive tau")
            else:
                a, b = l.left, l.right
                if a.heads % a.kv_heads:
                    raise ValueError(f"layer {i}: {a.heads} query heads do not divide over {a.kv_heads} key heads")
                if a.rot_dims % 2 or a.rot_dims > a.dim:
                    raise ValueError(f"layer {i}: {a.rot_dims} rotated columns of {a.dim}")
                if b.heads % b.groups or (b.heads * b.vdim) % b.norm_groups:
                    raise ValueError(f"layer {i}: {b.heads} heads over {b.groups} groups, {b.heads * b.vdim} channels in {b.norm_groups} parts")
            if l.ff_kind == "moe" and not 1 <= l.top <= l.experts:
                raise ValueError(f"layer {i}: top {l.top} of {l.experts} experts")

    @classmethod
    def from_dir(cls, path: str) -> "BepepelShape":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_config(json.load(f), name=os.path.basename(os.path.normpath(path)))

    def to_config(self) -> dict:
        """The ``config.json`` form (what ``from_config`` reads)."""
        out = []
        for l in self.layers:
            if l.kind == "gla":
                mixer = {"dim": l.dim, "heads": l.heads, "tau": l.tau, "vdim": l.vdim}
                if l.a_rank:
                    mixer["a_rank"] = l.a_rank
            else:
                a, b = l.left, l.right
                left = {"dim": a.dim, "heads": a.heads, "kv_heads": a.kv_heads, "scale": a.scale, "vdim": a.vdim}
                if a.conv:
                    left["conv"] = a.conv
                if a.window:
                    left["mask"] = {"keep_first": a.keep_first, "size": a.window}
                if a.rot_dims:
                    left["rot"] = {"base": a.rot_base, "dims": a.rot_dims}
                    if a.rot_scaling:
                        left["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), a.rot_scaling))
                right = {"groups": b.groups, "heads": b.heads, "norm_groups": b.norm_groups, "state": b.state, "vdim": b.vdim}
                if b.conv:
                    right["conv"] = b.conv
                mixer = {"left": left, "left_scale": l.left_scale, "right": right, "right_scale": l.right_scale}
            if l.ff_kind == "dense":
                mlp = {"ff": l.ff, "kind": "dense"}
            elif l.ff_kind == "moe":
                mlp = {"expert": {"ff": l.expert_ff}, "kind": "moe", "router": {"experts": l.experts, "top": l.top}}
                if l.shared_ff:
                    mlp["shared"] = {"ff": l.shared_ff}
            else:
                mlp = None
            out.append({"type": l.kind, "mixer": mixer, "mlp": mlp})
        return {"architecture": self.ARCHITECTURE, "layers": out, "logit_scale": self.logit_scale, "norm": {"eps": self.norm_eps},
                "residual_mult": self.residual_mult, "vocab": self.vocab_size, "width": self.hidden_size}

    @classmethod
    def uniform(cls, vocab: int, width: int, pattern, heads: int, kv_heads: int, dim: int, experts: int = 0, top: int = 0,
                expert_ff: int = 0, dense_ff: int = 0, window: int = 0, keep_first: int = 0, ssd_state: int = 128, ssd_vdim: int = 64,
                name: str = "bepepel") -> "BepepelShape":
        """A stack whose layers follow ``pattern`` (a sequence of mixer kinds), all with the same sizes: ``experts`` > 0 gives every
        layer a mixture-of-experts feed-forward with a shared expert, else ``dense_ff`` > 0 a dense one."""
        layers = []
        for kind in pattern:
            if kind == "gla":
                lay = BepepelLayer(kind, heads=heads, dim=dim, vdim=dim, tau=8.0, a_rank=16)
            else:
                left = BepepelAttention(heads=heads, kv_heads=kv_heads, dim=dim, vdim=dim, scale=1.0 / 8.0, conv=3, window=window,
                                        keep_first=keep_first, rot_base=500000.0, rot_dims=dim // 2,
                                        rot_scaling=(4.0, 1.0, 4.0, 2048.0))
                sh = max(width // ssd_vdim, 1)
                right = BepepelSSD(heads=sh, vdim=ssd_vdim, state=ssd_state, groups=1, norm_groups=1, conv=4)
                lay = BepepelLayer(kind, left=left, right=right, left_scale=1.0, right_scale=1.0)
            if experts:
                lay.ff_kind, lay.experts, lay.top, lay.expert_ff, lay.shared_ff = "moe", experts, top, expert_ff, expert_ff
            elif dense_ff:
                lay.ff_kind, lay.ff = "dense", dense_ff
            layers.append(lay)
        return cls(vocab_size=vocab, hidden_size=width, norm_eps=1e-6, layers=layers, residual_mult=0.5, logit_scale=1.0, name=name)


def architecture_of(path: str) -> str:
    """Which model family a checkpoint directory holds: ``architecture`` (Kazolorn) or HF's ``model_type``."""
    with open(os.path.join(path, "config.json")) as f:
        c = json.load(f)
    if c.get("architecture") == KazolornShape.ARCHITECTURE:
        return "kazolorn"
    if c.get("architecture") == DibizenShape.ARCHITECTURE:
        return "dibizen"
    if c.get("architecture") == FivesunShape.ARCHITECTURE:
        return "fivesun"
    if c.get("architecture") == BepepelShape.ARCHITECTURE:
        return "bepepel"
    return str(c.get("model_type", "llama"))
