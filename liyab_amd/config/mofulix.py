"""Mofulix's typed configuration, read from its own config.json keys.

A decoder of parallel layers: one Dynamic Tanh norm a layer, whose output the mixer and the feed-forward both read, and
their results are added to the stream together. The embedding is scaled; there is no position table: positions enter
inside the mixers. A layer's mixer is one of three kinds. config.json:

    architecture     "Mofulix"
    vocab, width
    embedding.scale  the factor on the embedding's rows
    norm.eps         the epsilon of every root-mean-square norm inside the mixers
    max_positions    optional: the longest context (nothing in the design bounds it; default 32,768)
    layers[i]        type, mixer {...}, mlp (null, or {kind "dense", ff, limit}), weights_of (optional): the layer whose
                     tensors this one runs with, its cache and state being its own
      type "attention": mixer {heads, kv_heads, dim, vdim, scale, softcap (optional), rot {dims, base, scaling {factor, low,
                     high, original} (optional)} (optional)}: values are the keys as projected; queries and keys normed a head
      type "wkv":       mixer {heads, dim}; the decay's rank is the shape of mix.w1
      type "parallel":  mixer {left {heads, kv_heads, dim, vdim, scale, bias_max, q_temp {coef, every} (optional)},
                     right {heads, vdim, state, groups, conv, norm_groups}}: attention with a bias by distance beside a
                     selective state space

Tensors: embed, final.norm(.alpha, .b), head; layer i's start with "l<i>.": norm1(.alpha, .b), mlp.{gate, up, down}, and
  attention: mix.{q, k, q.norm, k.norm, g, o}
  wkv:       mix.mu.{r, k, v, g, w}, mix.{r, k, v, g, w1, w2, w0, u, norm, o}
  parallel:  mix.left.{q, k, v, rel, o, out}, mix.right.{in, conv, conv.b, dt_bias, A_log, D, norm, o, out}
Matrices are stored [out, in].
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, Optional, Tuple

from ..errors import InvalidModel, Unsupported
from .plan import (
    ClampedGLUSpec,
    HeadSpec,
    Init,
    LayerSpec,
    ModelPlan,
    NormSpec,
    OrderEntry,
    RotarySpec,
    ScoredAttentionSpec,
    SideBySideSpec,
    StateSpaceSpec,
    TensorSource,
    TokenEmbeddingSpec,
    WKVSpec,
)
from .registry import register_architecture

_LIMIT = 1 << 24
DEFAULT_MAX_POSITIONS = 1 << 15
DEFAULT_DECAY_RANK = 16


def _int(raw, key: str, what: str, least: int = 1) -> int:
    v = raw.get(key) if isinstance(raw, dict) else None
    if isinstance(v, bool) or not isinstance(v, int) or v < least or v > _LIMIT:
        raise InvalidModel(f"missing or invalid {what}")
    return v


def _number(raw, key: str, what: str, positive: bool = True) -> float:
    v = raw.get(key) if isinstance(raw, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(v) or (positive and v <= 0):
        raise InvalidModel(f"missing or invalid {what}")
    return float(v)


@dataclass(frozen=True)
class MofulixAttention:
    n_head: int
    n_kv_head: int
    head_dim: int
    value_dim: int
    scale: float
    softcap: float  # 0: none
    rot_dims: int  # 0: no rotary encoding
    rot_base: float
    rot_scaling: Optional[Tuple[float, float, float, float]]  # factor, low, high, original


@dataclass(frozen=True)
class MofulixWKV:
    n_head: int
    head_dim: int
    decay_rank: int


@dataclass(frozen=True)
class MofulixBiased:
    n_head: int
    n_kv_head: int
    head_dim: int
    value_dim: int
    scale: float
    bias_max: int
    bias_rows: int
    temp_coef: float
    temp_every: int  # 0: no factor on the query


@dataclass(frozen=True)
class MofulixStateSpace:
    n_head: int
    head_dim: int
    n_state: int
    n_groups: int
    taps: int
    norm_groups: int


@dataclass(frozen=True)
class MofulixLayer:
    kind: str  # "attention" | "wkv" | "parallel"
    mixer: Any  # MofulixAttention | MofulixWKV | (MofulixBiased, MofulixStateSpace)
    ff: int  # 0: no feed-forward
    limit: float
    weights_of: Optional[int]


def _attention(m, where: str) -> MofulixAttention:
    H, G = _int(m, "heads", where + ".heads"), _int(m, "kv_heads", where + ".kv_heads")
    if H % G:
        raise InvalidModel(f"invalid {where}: {H} heads are no multiple of {G} kv_heads")
    rot = m.get("rot")
    dims, base, scaling = 0, 0.0, None
    if rot is not None:
        dims, base = _int(rot, "dims", where + ".rot.dims"), _number(rot, "base", where + ".rot.base")
        sc = rot.get("scaling") if isinstance(rot, dict) else None
        if sc is not None:
            scaling = tuple(_number(sc, k, f"{where}.rot.scaling.{k}") for k in ("factor", "low", "high", "original"))
            if scaling[1] == scaling[2]:
                raise InvalidModel(f"invalid {where}.rot.scaling: low equals high")
    return MofulixAttention(n_head=H, n_kv_head=G, head_dim=_int(m, "dim", where + ".dim"), value_dim=_int(m, "vdim", where + ".vdim"),
                            scale=_number(m, "scale", where + ".scale"),
                            softcap=_number(m, "softcap", where + ".softcap") if m.get("softcap") is not None else 0.0,
                            rot_dims=dims, rot_base=base, rot_scaling=scaling)


def _biased(m, where: str) -> MofulixBiased:
    H, G = _int(m, "heads", where + ".heads"), _int(m, "kv_heads", where + ".kv_heads")
    if H % G:
        raise InvalidModel(f"invalid {where}: {H} heads are no multiple of {G} kv_heads")
    qt = m.get("q_temp")
    coef, every = (_number(qt, "coef", where + ".q_temp.coef", positive=False), _int(qt, "every", where + ".q_temp.every")) if qt is not None else (0.0, 0)
    return MofulixBiased(n_head=H, n_kv_head=G, head_dim=_int(m, "dim", where + ".dim"), value_dim=_int(m, "vdim", where + ".vdim"),
                         scale=_number(m, "scale", where + ".scale"), bias_max=_int(m, "bias_max", where + ".bias_max", 2),
                         bias_rows=_int(m, "bias_rows", where + ".bias_rows", 2) if m.get("bias_rows") is not None else 0,
                         temp_coef=coef, temp_every=every)


def _state_space(m, where: str) -> MofulixStateSpace:
    return MofulixStateSpace(n_head=_int(m, "heads", where + ".heads"), head_dim=_int(m, "vdim", where + ".vdim"),
                             n_state=_int(m, "state", where + ".state"), n_groups=_int(m, "groups", where + ".groups"),
                             taps=_int(m, "conv", where + ".conv"), norm_groups=_int(m, "norm_groups", where + ".norm_groups"))


@dataclass(frozen=True)
class MofulixConfig:
    vocab: int
    width: int
    embedding_scale: float
    eps: float
    max_positions: int
    layers: Tuple[MofulixLayer, ...]

    architecture = "Mofulix"

    @classmethod
    def from_json(cls, raw: dict, shapes: Optional[dict] = None) -> "MofulixConfig":
        """`shapes`: tensor name -> shape, for the two sizes that only a tensor's shape gives (the rows of a bias-by-distance
        table, the rank of a decay); without it config.json's optional keys `bias_rows` and `decay_rank` are read."""
        vocab, width = _int(raw, "vocab", "vocab"), _int(raw, "width", "width")
        eps = _number(raw.get("norm"), "eps", "norm.eps")
        scale = _number(raw.get("embedding"), "scale", "embedding.scale") if raw.get("embedding") is not None else 1.0
        max_positions = _int(raw, "max_positions", "max_positions") if raw.get("max_positions") is not None else DEFAULT_MAX_POSITIONS
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise InvalidModel("missing or invalid layers")
        layers = []
        for i, entry in enumerate(listed):
            if not isinstance(entry, dict):
                raise InvalidModel(f"invalid layers[{i}]")
            weights_of = entry.get("weights_of")
            if weights_of is not None and (isinstance(weights_of, bool) or not isinstance(weights_of, int) or not 0 <= weights_of < len(listed) or weights_of == i):
                raise InvalidModel(f"invalid layers[{i}].weights_of")
            kind, m, where = entry.get("type"), entry.get("mixer"), f"layers[{i}].mixer"
            owner = f"l{weights_of if weights_of is not None else i}"
            if not isinstance(m, dict):
                raise InvalidModel(f"missing or invalid {where}")
            if kind == "attention":
                mixer = _attention(m, where)
            elif kind == "wkv":
                rank = m.get("decay_rank")
                if shapes is not None and owner + ".mix.w1" in shapes and len(shapes[owner + ".mix.w1"]) == 2:
                    rank = int(shapes[owner + ".mix.w1"][0])
                mixer = MofulixWKV(n_head=_int(m, "heads", where + ".heads"), head_dim=_int(m, "dim", where + ".dim"),
                                   decay_rank=rank if isinstance(rank, int) and rank > 0 else DEFAULT_DECAY_RANK)
            elif kind == "parallel":
                left = _biased(m.get("left"), where + ".left")
                name = owner + ".mix.left.rel"
                if shapes is not None and name in shapes and len(shapes[name]) == 2:
                    left = MofulixBiased(**{**left.__dict__, "bias_rows": int(shapes[name][0])})
                if left.bias_rows < 2:
                    raise InvalidModel(f"missing or invalid {where}.left.bias_rows (the rows of '{name}')")
                if left.bias_max <= left.bias_rows // 2:
                    raise InvalidModel(f"invalid {where}.left.bias_max: {left.bias_max} with a table of {left.bias_rows} rows")
                mixer = (left, _state_space(m.get("right"), where + ".right"))
            else:
                raise Unsupported(f"layers[{i}].type '{kind}' is not supported (supported: attention, parallel, wkv)")
            mlp = entry.get("mlp")
            ff, limit = 0, 0.0
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise Unsupported(f"layers[{i}].mlp.kind '{mlp.get('kind') if isinstance(mlp, dict) else mlp}' is not supported (supported: dense)")
                ff, limit = _int(mlp, "ff", f"layers[{i}].mlp.ff"), _number(mlp, "limit", f"layers[{i}].mlp.limit")
            layers.append(MofulixLayer(kind=kind, mixer=mixer, ff=ff, limit=limit, weights_of=weights_of))
        for i, layer in enumerate(layers):
            j = layer.weights_of
            if j is not None:
                seen = {i}
                while layers[j].weights_of is not None:  # a layer that borrows from a borrower: from whom that one borrows
                    if j in seen:
                        raise InvalidModel(f"invalid layers[{i}].weights_of: no layer of the chain has tensors of its own")
                    seen.add(j)
                    j = layers[j].weights_of
                owner = layers[j]
                if (layer.kind, layer.ff) != (owner.kind, owner.ff):
                    raise InvalidModel(f"invalid layers[{i}]: it differs from layer {j}, whose tensors it uses")
                # sizes that only the owner's tensors give are the owner's
                layers[i] = MofulixLayer(kind=layer.kind, mixer=owner.mixer if layer.kind != "attention" else layer.mixer, ff=layer.ff,
                                         limit=layer.limit, weights_of=j)
        return cls(vocab=vocab, width=width, embedding_scale=scale, eps=eps, max_positions=max_positions, layers=tuple(layers))

    def to_json(self) -> dict:
        layers = []
        for layer in self.layers:
            m = layer.mixer
            if layer.kind == "attention":
                mixer = {"heads": m.n_head, "kv_heads": m.n_kv_head, "dim": m.head_dim, "vdim": m.value_dim, "scale": m.scale}
                if m.softcap:
                    mixer["softcap"] = m.softcap
                if m.rot_dims:
                    mixer["rot"] = {"dims": m.rot_dims, "base": m.rot_base}
                    if m.rot_scaling is not None:
                        mixer["rot"]["scaling"] = dict(zip(("factor", "low", "high", "original"), m.rot_scaling))
            elif layer.kind == "wkv":
                mixer = {"heads": m.n_head, "dim": m.head_dim, "decay_rank": m.decay_rank}
            else:
                a, b = m
                left = {"heads": a.n_head, "kv_heads": a.n_kv_head, "dim": a.head_dim, "vdim": a.value_dim, "scale": a.scale,
                        "bias_max": a.bias_max, "bias_rows": a.bias_rows}
                if a.temp_every:
                    left["q_temp"] = {"coef": a.temp_coef, "every": a.temp_every}
                mixer = {"left": left, "right": {"heads": b.n_head, "vdim": b.head_dim, "state": b.n_state, "groups": b.n_groups,
                                                 "conv": b.taps, "norm_groups": b.norm_groups}}
            entry = {"type": layer.kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": layer.ff, "limit": layer.limit} if layer.ff else None}
            if layer.weights_of is not None:
                entry["weights_of"] = layer.weights_of
            layers.append(entry)
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "embedding": {"scale": self.embedding_scale},
                "norm": {"eps": self.eps}, "max_positions": self.max_positions, "layers": layers}

    def plan(self) -> ModelPlan:
        d, V = self.width, self.vocab
        wide = Init(1.0 / math.sqrt(d))

        def dyt(name: str) -> NormSpec:
            return NormSpec(kind="dyt", width=d, eps=self.eps, tensors={
                "weight": TensorSource(name, init=Init(0.1, 1.0)), "bias": TensorSource(name + ".b", init=Init(0.1)),
                "alpha": TensorSource(name + ".alpha", init=Init(0.05, 0.5))})

        layers = []
        for i, layer in enumerate(self.layers):
            p = f"l{layer.weights_of if layer.weights_of is not None else i}"
            m = layer.mixer
            if layer.kind == "attention":
                mixer = self._attention_spec(p + ".mix", m, wide)
            elif layer.kind == "wkv":
                H, D = m.n_head, m.head_dim
                mixer = WKVSpec(kind="wkv", width=d, n_head=H, head_dim=D, decay_rank=m.decay_rank, eps=self.eps, tensors={
                    **{"mu_" + c: TensorSource(f"{p}.mix.mu.{c}", init=Init(0.2, 0.5)) for c in "rkvgw"},
                    **{c: TensorSource(f"{p}.mix.{c}", init=wide) for c in "rkvg"},
                    "w1": TensorSource(p + ".mix.w1", init=wide), "w2": TensorSource(p + ".mix.w2", init=Init(1.0 / math.sqrt(m.decay_rank))),
                    "w0": TensorSource(p + ".mix.w0", init=Init(1.0, -1.0)), "u": TensorSource(p + ".mix.u", init=Init(0.5)),
                    "norm": TensorSource(p + ".mix.norm", init=Init(0.1, 1.0)), "out": TensorSource(p + ".mix.o", init=Init(1.0 / math.sqrt(H * D)))})
            else:
                a, b = m
                left = ScoredAttentionSpec(
                    kind="scored_attention", width=d, n_head=a.n_head, n_kv_head=a.n_kv_head, head_dim=a.head_dim, value_dim=a.value_dim,
                    scale=a.scale, eps=self.eps, q_temp=(a.temp_coef, a.temp_every) if a.temp_every else None, distance_bias=a.bias_max,
                    bias_rows=a.bias_rows, tensors={
                        "q": TensorSource(p + ".mix.left.q", init=wide), "k": TensorSource(p + ".mix.left.k", init=wide),
                        "v": TensorSource(p + ".mix.left.v", init=wide), "rel": TensorSource(p + ".mix.left.rel", init=Init(1.0)),
                        "out": TensorSource(p + ".mix.left.o", init=Init(1.0 / math.sqrt(a.n_head * a.value_dim)))})
                inner = b.n_head * b.head_dim
                right = StateSpaceSpec(
                    kind="state_space", width=d, n_head=b.n_head, head_dim=b.head_dim, n_state=b.n_state, n_groups=b.n_groups, taps=b.taps,
                    norm_groups=b.norm_groups, eps=self.eps, tensors={
                        "in": TensorSource(p + ".mix.right.in", init=wide), "conv": TensorSource(p + ".mix.right.conv", init=Init(0.4)),
                        "conv_bias": TensorSource(p + ".mix.right.conv.b", init=Init(0.1)),
                        "dt_bias": TensorSource(p + ".mix.right.dt_bias", init=Init(0.5, -1.0)), "A_log": TensorSource(p + ".mix.right.A_log", init=Init(0.5)),
                        "D": TensorSource(p + ".mix.right.D", init=Init(0.3, 1.0)), "norm": TensorSource(p + ".mix.right.norm", init=Init(0.1, 1.0)),
                        "out": TensorSource(p + ".mix.right.o", init=Init(1.0 / math.sqrt(inner)))})
                mixer = SideBySideSpec(kind="side_by_side", width=d, left=left, right=right, eps=self.eps, weight=0.5, tensors={
                    "left_out": TensorSource(p + ".mix.left.out", init=Init(0.1, 1.0)), "right_out": TensorSource(p + ".mix.right.out", init=Init(0.1, 1.0))})
            ffn = None
            if layer.ff:
                ffn = ClampedGLUSpec(kind="clamped_glu", width=d, inner=layer.ff, limit=layer.limit, tensors={
                    "gate": TensorSource(p + ".mlp.gate", init=wide), "up": TensorSource(p + ".mlp.up", init=wide),
                    "down": TensorSource(p + ".mlp.down", init=Init(1.0 / math.sqrt(layer.ff)))})
            layers.append(LayerSpec(mixer=mixer, ffn=ffn, norm_mixer=dyt(p + ".norm1"), norm_ffn=None, arrangement="parallel"))
        return ModelPlan(
            architecture=self.architecture, width=d, vocab_size=V, max_positions=self.max_positions,
            embedding=TokenEmbeddingSpec(kind="token_embedding", vocab_size=V, width=d, scale=self.embedding_scale,
                                         tensors={"table": TensorSource("embed", init=Init(1.0 / max(self.embedding_scale, 1e-6)))}),
            residual_position=None,
            layers=layers,
            order=[OrderEntry(layer=i) for i in range(len(layers))],
            final_norm=dyt("final.norm"),
            head=HeadSpec(kind="lm_head", width=d, vocab_size=V, logit_scale=1.0, tensors={"weight": TensorSource("head", init=wide)}),
            ignorable=(), name_prefixes=("",), eos_token_id=None,
        )

    def _attention_spec(self, p: str, m: MofulixAttention, wide: Init) -> ScoredAttentionSpec:
        H, D = m.n_head, m.head_dim
        return ScoredAttentionSpec(
            kind="scored_attention", width=self.width, n_head=H, n_kv_head=m.n_kv_head, head_dim=D, value_dim=m.value_dim, scale=m.scale,
            eps=self.eps, softcap=m.softcap, qk_norm=True,
            rotary=RotarySpec(dims=m.rot_dims, base=m.rot_base, scaling=m.rot_scaling) if m.rot_dims else None,
            values_are_keys=True, gated=True, tensors={
                "q": TensorSource(p + ".q", init=wide), "k": TensorSource(p + ".k", init=wide), "gate": TensorSource(p + ".g", init=wide),
                "q_norm": TensorSource(p + ".q.norm", init=Init(0.1, 1.0)), "k_norm": TensorSource(p + ".k.norm", init=Init(0.1, 1.0)),
                "out": TensorSource(p + ".o", init=Init(1.0 / math.sqrt(H * m.value_dim)))})


register_architecture("Mofulix", MofulixConfig)
