"""Bokulix's configuration, plan and random-weights mode (no GPU needed)."""

import json

import pytest

from liyab_amd.config import config_from_dict
from liyab_amd.errors import InvalidModel, Unsupported


def raw_config():
    m = {"heads": 3, "dim": 8, "vdim": 12, "kv_rank": 16, "scale": 0.25, "mask": {"size": 7}}
    mlp = {"kind": "moe", "expert": {"ff": 20}, "router": {"experts": 4, "top": 2}}
    return {"architecture": "Bokulix", "vocab": 90, "width": 40, "max_positions": 64, "norm": {"eps": 1e-6}, "canon": {"taps": 3},
            "layers": [{"type": "latent_attention", "mixer": m, "mlp": mlp},
                       {"type": "latent_attention", "mixer": dict(m, mask={"size": 11}), "mlp": None},
                       {"type": "latent_attention", "mixer": m, "mlp": mlp, "weights_of": 0},
                       {"type": "latent_attention", "mixer": {k: v for k, v in m.items() if k != "mask"}, "mlp": mlp, "weights_of": 2}]}


def test_config_round_trip_and_plan():
    cfg = config_from_dict(raw_config())
    assert config_from_dict(json.loads(json.dumps(cfg.to_json()))) == cfg
    assert [l.window for l in cfg.layers] == [7, 11, 7, 0]
    assert [l.weights_of for l in cfg.layers] == [None, None, 0, 0]  # a layer that borrows from a borrower: from whom that one borrows
    plan = cfg.plan()
    assert plan.architecture == "Bokulix" and len(plan.layers) == 4 and [e.layer for e in plan.order] == [0, 1, 2, 3]
    assert plan.layers[2].mixer.tensors["q"].name == "l0.mix.q" and plan.layers[3].norm_mixer.tensors["weight"].name == "l0.norm1"
    assert plan.layers[1].ffn is None and plan.layers[1].norm_ffn is None and plan.layers[1].gate_ffn is None
    assert plan.layers[0].ffn.tensors[("down", 3)].name == "l0.mlp.e3.down"
    assert plan.layers[0].input_conv.taps == 3 and plan.layers[0].arrangement == "post_norm_gated"
    assert plan.final_norm.kind == "rmsnorm" and plan.head.tensors["weight"].name == "head"


def test_what_may_be_left_out():
    raw = raw_config()
    del raw["canon"]
    raw["layers"][0]["mixer"]["mask"] = None
    raw["layers"][1]["mixer"]["mask"] = {"size": None}
    cfg = config_from_dict(raw)
    assert cfg.taps == 0 and [l.window for l in cfg.layers[:2]] == [0, 0]
    assert all(l.input_conv is None for l in cfg.plan().layers)
    assert config_from_dict(cfg.to_json()) == cfg


def test_random_weights_name_every_tensor_once():
    from liyab_amd.weights.random_init import random_tensors

    t = random_tensors(config_from_dict(raw_config()), 3)
    own = {"embed": (90, 40), "pos": (64, 40), "final.norm": (40,), "head": (90, 40)}
    for i in (0, 1):
        p = f"l{i}."
        own.update({p + "norm1": (40,), p + "canon1": (40, 3), p + "rg1": (40, 40), p + "rg1.b": (40,), p + "mix.q": (24, 40),
                    p + "mix.dkv": (16, 40), p + "mix.dkv.norm": (16,), p + "mix.uk": (24, 16), p + "mix.uv": (36, 16),
                    p + "mix.g": (36, 40), p + "mix.o": (40, 36)})
    own.update({"l0.norm2": (40,), "l0.rg2": (40, 40), "l0.rg2.b": (40,), "l0.mlp.router": (4, 40), "l0.mlp.router.b": (4,)})
    for e in range(4):
        own.update({f"l0.mlp.e{e}.gate": (20, 40), f"l0.mlp.e{e}.up": (20, 40), f"l0.mlp.e{e}.down": (40, 20)})
    assert {k: tuple(v.shape) for k, v in t.items()} == own


@pytest.mark.parametrize("change,error", [
    (lambda c: c.pop("vocab"), InvalidModel),
    (lambda c: c["norm"].pop("eps"), InvalidModel),
    (lambda c: c["canon"].update(taps=0), InvalidModel),
    (lambda c: c.update(layers=[]), InvalidModel),
    (lambda c: c["layers"][0].update(type="recurrent"), Unsupported),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), Unsupported),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), InvalidModel),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), InvalidModel),
    (lambda c: c["layers"][2].update(weights_of=2), InvalidModel),
    (lambda c: c["layers"][2].update(weights_of=9), InvalidModel),
    (lambda c: c["layers"][2]["mixer"].update(heads=4), InvalidModel),  # other sizes than the layer whose tensors it uses
])
def test_what_the_configuration_refuses(change, error):
    raw = json.loads(json.dumps(raw_config()))
    change(raw)
    with pytest.raises(error):
        config_from_dict(raw)


def test_a_missing_tensor_and_a_wrong_shape_come_as_one_error(tmp_path):
    import torch

    from liyab_amd.models.decoder import DecoderModel
    from liyab_amd.weights.loader import WeightStore
    from liyab_amd.weights.random_init import random_tensors

    cfg = config_from_dict(raw_config())
    t = random_tensors(cfg, 1)
    del t["l1.canon1"]
    t["l0.mlp.e2.up"] = torch.zeros(40, 20)
    t["l5.norm1"] = torch.zeros(40)
    store = WeightStore(t, device="cpu", compute_dtype=torch.float32)
    DecoderModel(cfg.plan(), store, torch.float32)
    with pytest.raises(InvalidModel) as e:
        store.finish()
    text = str(e.value)
    assert "'l1.canon1'" in text and "'l0.mlp.e2.up' has shape [40, 20], expected [20, 40]" in text and "'l5.norm1'" in text
