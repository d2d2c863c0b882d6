"""Bokulix's typed configuration, read from its own config.json keys.

A decoder of layers that read the residual stream itself and norm their sublayers' results:
learned positions added to the embedding; per layer an input convolution over time, latent attention
under a sliding window, a routed feed-forward (or none), gates on both results, root-mean-square
norms; a final norm and an untied head. config.json:

    architecture   "Bokulix"
    vocab, width, max_positions
    norm.eps       the epsilon of every norm of a layer, of the final norm and of the cached row's
    canon.taps     the taps of the input convolution (no `canon`: none)
    layers[i]      type ("latent_attention"), mixer {heads, dim, vdim, kv_rank, scale, mask.size (no `mask`: every earlier position)},
                   mlp (null, or {kind "moe", expert.ff, router.experts, router.top}),
                   weights_of (optional): the layer whose tensors this one runs with, its cache and
                   state being its own

Tensors: embed, pos, final.norm, head; layer i's start with "l<i>.": norm1, norm2, canon1, rg1, rg1.b,
rg2, rg2.b, mix.{q, dkv, dkv.norm, uk, uv, g, o}, mlp.router, mlp.router.b, mlp.e<k>.{gate, up, down}.
Matrices are stored [out, in].
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Tuple

from ..errors import InvalidModel, Unsupported
from .plan import (
    CausalConvSpec,
    GateSpec,
    HeadSpec,
    Init,
    LatentAttentionSpec,
    LayerSpec,
    ModelPlan,
    NormSpec,
    OrderEntry,
    PositionSpec,
    RoutedFFNSpec,
    TensorSource,
    TokenEmbeddingSpec,
)
from .registry import register_architecture

_LIMIT = 1 << 24


def _int(raw, key: str, what: str, least: int = 1) -> int:
    v = raw.get(key) if isinstance(raw, dict) else None
    if isinstance(v, bool) or not isinstance(v, int) or v < least or v > _LIMIT:
        raise InvalidModel(f"missing or invalid {what}")
    return v


def _number(raw, key: str, what: str) -> float:
    v = raw.get(key) if isinstance(raw, dict) else None
    if isinstance(v, bool) or not isinstance(v, (int, float)) or not math.isfinite(v) or v < 0:
        raise InvalidModel(f"missing or invalid {what}")
    return float(v)


@dataclass(frozen=True)
class BokulixRouted:
    inner: int
    n_experts: int
    top: int


@dataclass(frozen=True)
class BokulixLayer:
    n_head: int
    head_dim: int
    value_dim: int
    rank: int
    scale: float
    window: int  # 0: every earlier position
    mlp: Optional[BokulixRouted]
    weights_of: Optional[int]


@dataclass(frozen=True)
class BokulixConfig:
    vocab: int
    width: int
    max_positions: int
    eps: float
    taps: int
    layers: Tuple[BokulixLayer, ...]

    architecture = "Bokulix"

    @classmethod
    def from_json(cls, raw: dict) -> "BokulixConfig":
        vocab, width = _int(raw, "vocab", "vocab"), _int(raw, "width", "width")
        max_positions = _int(raw, "max_positions", "max_positions")
        eps = _number(raw.get("norm"), "eps", "norm.eps")
        taps = _int(raw.get("canon"), "taps", "canon.taps") if raw.get("canon") is not None else 0  # (no entry: no input convolution)
        listed = raw.get("layers")
        if not isinstance(listed, list) or not listed:
            raise InvalidModel("missing or invalid layers")
        layers = []
        for i, entry in enumerate(listed):
            if not isinstance(entry, dict):
                raise InvalidModel(f"invalid layers[{i}]")
            kind = entry.get("type")
            if kind != "latent_attention":
                raise Unsupported(f"layers[{i}].type '{kind}' is not supported (supported: latent_attention)")
            m = entry.get("mixer")
            where = f"layers[{i}].mixer"
            mask = m.get("mask") if isinstance(m, dict) else None
            window = _int(mask, "size", where + ".mask.size") if mask is not None and (not isinstance(mask, dict) or mask.get("size") is not None) else 0
            mlp = entry.get("mlp")
            routed = None
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "moe":
                    raise Unsupported(f"layers[{i}].mlp.kind '{mlp.get('kind') if isinstance(mlp, dict) else mlp}' is not supported (supported: moe)")
                routed = BokulixRouted(inner=_int(mlp.get("expert"), "ff", f"layers[{i}].mlp.expert.ff"),
                                       n_experts=_int(mlp.get("router"), "experts", f"layers[{i}].mlp.router.experts"),
                                       top=_int(mlp.get("router"), "top", f"layers[{i}].mlp.router.top"))
                if routed.top > routed.n_experts:
                    raise InvalidModel(f"invalid layers[{i}].mlp.router.top: {routed.top} of {routed.n_experts} experts")
            weights_of = entry.get("weights_of")
            if weights_of is not None:
                if isinstance(weights_of, bool) or not isinstance(weights_of, int) or not 0 <= weights_of < len(listed) or weights_of == i:
                    raise InvalidModel(f"invalid layers[{i}].weights_of")
            layers.append(BokulixLayer(n_head=_int(m, "heads", where + ".heads"), head_dim=_int(m, "dim", where + ".dim"),
                                       value_dim=_int(m, "vdim", where + ".vdim"), rank=_int(m, "kv_rank", where + ".kv_rank"),
                                       scale=_number(m, "scale", where + ".scale"), window=window, mlp=routed, weights_of=weights_of))
        for i, layer in enumerate(layers):
            j = layer.weights_of
            if j is not None:
                seen = {i}
                while layers[j].weights_of is not None:  # a layer that borrows from a borrower: from whom that one borrows
                    if j in seen:
                        raise InvalidModel(f"invalid layers[{i}].weights_of: no layer of the chain has tensors of its own")
                    seen.add(j)
                    j = layers[j].weights_of
                layers[i] = layer = BokulixLayer(**{**layer.__dict__, "weights_of": j})
                a, b = layer, layers[j]
                if (a.n_head, a.head_dim, a.value_dim, a.rank, a.mlp) != (b.n_head, b.head_dim, b.value_dim, b.rank, b.mlp):
                    raise InvalidModel(f"invalid layers[{i}]: its sizes differ from those of layer {j}, whose tensors it uses")
        return cls(vocab=vocab, width=width, max_positions=max_positions, eps=eps, taps=taps, layers=tuple(layers))

    def to_json(self) -> dict:
        layers = []
        for layer in self.layers:
            mixer = {"heads": layer.n_head, "dim": layer.head_dim, "vdim": layer.value_dim, "kv_rank": layer.rank, "scale": layer.scale}
            if layer.window:
                mixer["mask"] = {"size": layer.window}
            entry = {"type": "latent_attention", "mixer": mixer,
                     "mlp": None if layer.mlp is None else {"kind": "moe", "expert": {"ff": layer.mlp.inner},
                                                           "router": {"experts": layer.mlp.n_experts, "top": layer.mlp.top}}}
            if layer.weights_of is not None:
                entry["weights_of"] = layer.weights_of
            layers.append(entry)
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions,
               "norm": {"eps": self.eps}, "layers": layers}
        if self.taps:
            out["canon"] = {"taps": self.taps}
        return out

    def plan(self) -> ModelPlan:
        d, V = self.width, self.vocab
        # What the random-weights mode draws: a norm stands on every sublayer's result, so the products'
        # scales matter little; router and gate biases away from zero and norm weights away from one make
        # a bias or a norm applied in the wrong place visible.
        wide = Init(1.0 / math.sqrt(d))
        layers = []
        for i, layer in enumerate(self.layers):
            p = f"l{layer.weights_of if layer.weights_of is not None else i}"
            H, D, Vd, R = layer.n_head, layer.head_dim, layer.value_dim, layer.rank
            mixer = LatentAttentionSpec(
                kind="latent_attention", width=d, n_head=H, head_dim=D, value_dim=Vd, rank=R, scale=layer.scale,
                window=layer.window, eps=self.eps, gated=True,
                tensors={
                    "q": TensorSource(p + ".mix.q", init=wide),
                    "down": TensorSource(p + ".mix.dkv", init=wide),
                    "down_norm": TensorSource(p + ".mix.dkv.norm", init=Init(0.1, 1.0)),
                    "up_k": TensorSource(p + ".mix.uk", init=Init(1.0 / math.sqrt(R))),
                    "up_v": TensorSource(p + ".mix.uv", init=Init(1.0 / math.sqrt(R))),
                    "gate": TensorSource(p + ".mix.g", init=wide),
                    "out": TensorSource(p + ".mix.o", init=Init(1.0 / math.sqrt(H * Vd))),
                })
            ffn = None
            if layer.mlp is not None:
                F, E = layer.mlp.inner, layer.mlp.n_experts
                tensors = {"router": TensorSource(p + ".mlp.router", init=wide), "router_bias": TensorSource(p + ".mlp.router.b", init=Init(0.2))}
                for e in range(E):
                    tensors[("gate", e)] = TensorSource(f"{p}.mlp.e{e}.gate", init=wide)
                    tensors[("up", e)] = TensorSource(f"{p}.mlp.e{e}.up", init=wide)
                    tensors[("down", e)] = TensorSource(f"{p}.mlp.e{e}.down", init=Init(1.0 / math.sqrt(F)))
                ffn = RoutedFFNSpec(kind="routed_ffn", width=d, inner=F, n_experts=E, top=layer.mlp.top, activation="silu", tensors=tensors)

            def norm(name: str) -> NormSpec:
                return NormSpec(kind="rmsnorm", width=d, eps=self.eps, tensors={"weight": TensorSource(name, init=Init(0.1, 1.0))})

            def gate(name: str) -> GateSpec:
                return GateSpec(kind="sigmoid_gate", width=d, tensors={"weight": TensorSource(name, init=wide),
                                                                       "bias": TensorSource(name + ".b", init=Init(0.5))})

            layers.append(LayerSpec(
                mixer=mixer, ffn=ffn, norm_mixer=norm(p + ".norm1"), norm_ffn=norm(p + ".norm2") if ffn is not None else None,
                arrangement="post_norm_gated",
                input_conv=CausalConvSpec(kind="causal_conv", width=d, taps=self.taps,
                                          tensors={"weight": TensorSource(p + ".canon1", init=Init(0.3))}) if self.taps else None,
                gate_mixer=gate(p + ".rg1"), gate_ffn=gate(p + ".rg2") if ffn is not None else None))
        return ModelPlan(
            architecture=self.architecture, width=d, vocab_size=V, max_positions=self.max_positions,
            embedding=TokenEmbeddingSpec(kind="token_embedding", vocab_size=V, width=d, scale=1.0,
                                         tensors={"table": TensorSource("embed", init=Init(1.0))}),
            residual_position=PositionSpec(kind="learned_positions", where="residual", max_positions=self.max_positions, width=d,
                                           tensors={"table": TensorSource("pos", init=Init(0.5))}),
            layers=layers,
            order=[OrderEntry(layer=i) for i in range(len(layers))],
            final_norm=NormSpec(kind="rmsnorm", width=d, eps=self.eps, tensors={"weight": TensorSource("final.norm", init=Init(0.1, 1.0))}),
            head=HeadSpec(kind="lm_head", width=d, vocab_size=V, logit_scale=1.0,
                          tensors={"weight": TensorSource("head", init=wide), "bias": TensorSource("head.b", required=False)}),
            ignorable=(),
            name_prefixes=("",),
            eos_token_id=None,
        )


register_architecture("Bokulix", BokulixConfig)
