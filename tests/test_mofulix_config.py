"""Mofulix's configuration and plan without a GPU: config.json's keys, what is refused, the tensors a plan names, the sizes
that only a tensor's shape gives, and the random-weights mode."""

import json

import numpy as np
import pytest

from liyab_amd.config import config_from_dict, load_config
from liyab_amd.config.mofulix import DEFAULT_MAX_POSITIONS, MofulixConfig
from liyab_amd.errors import InvalidModel, Unsupported


def raw_config():
    return {
        "architecture": "Mofulix", "vocab": 90, "width": 48, "embedding": {"scale": 3.0}, "norm": {"eps": 1e-6},
        "layers": [
            {"type": "wkv", "mixer": {"heads": 2, "dim": 8}, "mlp": {"kind": "dense", "ff": 20, "limit": 1.5}},
            {"type": "attention", "mixer": {"heads": 4, "kv_heads": 2, "dim": 12, "vdim": 12, "scale": 0.3, "softcap": 9.0,
                                            "rot": {"dims": 8, "base": 1000.0, "scaling": {"factor": 2.0, "low": 1.0, "high": 4.0, "original": 32}}},
             "mlp": None},
            {"type": "parallel", "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 6, "scale": 0.35, "bias_max": 30, "bias_rows": 10,
                                                    "q_temp": {"coef": 0.5, "every": 16}},
                                           "right": {"heads": 2, "vdim": 10, "state": 6, "groups": 1, "conv": 3, "norm_groups": 2}},
             "mlp": {"kind": "dense", "ff": 16, "limit": 2.0}},
            {"type": "wkv", "mixer": {"heads": 2, "dim": 8}, "mlp": {"kind": "dense", "ff": 20, "limit": 1.5}, "weights_of": 0},
        ],
    }


def test_keys_are_read_and_written_back():
    cfg = config_from_dict(raw_config())
    assert isinstance(cfg, MofulixConfig)
    assert (cfg.vocab, cfg.width, cfg.embedding_scale, cfg.eps, cfg.max_positions) == (90, 48, 3.0, 1e-6, DEFAULT_MAX_POSITIONS)
    assert [l.kind for l in cfg.layers] == ["wkv", "attention", "parallel", "wkv"]
    assert cfg.layers[3].weights_of == 0 and cfg.layers[1].ff == 0
    a = cfg.layers[1].mixer
    assert (a.n_head, a.n_kv_head, a.head_dim, a.softcap, a.rot_dims, a.rot_scaling) == (4, 2, 12, 9.0, 8, (2.0, 1.0, 4.0, 32.0))
    left, right = cfg.layers[2].mixer
    assert (left.bias_rows, left.bias_max, left.temp_every, right.taps, right.norm_groups) == (10, 30, 16, 3, 2)
    again = config_from_dict(json.loads(json.dumps(cfg.to_json())))
    assert again == cfg


def test_sizes_that_only_a_tensors_shape_gives():
    raw = raw_config()
    del raw["layers"][2]["mixer"]["left"]["bias_rows"]
    with pytest.raises(InvalidModel, match="bias_rows"):
        config_from_dict(raw)
    cfg = config_from_dict(raw, {"l2.mix.left.rel": (14, 2), "l0.mix.w1": (5, 48)})
    assert cfg.layers[2].mixer[0].bias_rows == 14
    assert cfg.layers[0].mixer.decay_rank == 5 and cfg.layers[3].mixer.decay_rank == 5  # the borrower's are its owner's


def test_optional_keys():
    raw = raw_config()
    m = raw["layers"][1]["mixer"]
    del m["softcap"], m["rot"]["scaling"]
    del raw["layers"][2]["mixer"]["left"]["q_temp"]
    cfg = config_from_dict(raw)
    assert cfg.layers[1].mixer.softcap == 0.0 and cfg.layers[1].mixer.rot_scaling is None and cfg.layers[2].mixer[0].temp_every == 0
    spec = cfg.plan().layers[1].mixer
    assert spec.softcap == 0.0 and spec.rotary.scaling is None and spec.values_are_keys and spec.gated and spec.qk_norm
    del m["rot"]
    assert config_from_dict(raw).plan().layers[1].mixer.rotary is None


@pytest.mark.parametrize("change,error", [
    (lambda r: r["layers"][0].update(type="conv"), Unsupported),
    (lambda r: r["layers"][0]["mlp"].update(kind="moe"), Unsupported),
    (lambda r: r["layers"][1]["mixer"].update(kv_heads=3), InvalidModel),
    (lambda r: r["layers"][3].update(weights_of=3), InvalidModel),
    (lambda r: r["layers"][3].update(weights_of=1), InvalidModel),
    (lambda r: r["layers"][2]["mixer"]["left"].update(bias_max=5), InvalidModel),
    (lambda r: r.pop("norm"), InvalidModel),
    (lambda r: r.update(vocab=0), InvalidModel),
    (lambda r: r["layers"][2]["mixer"].pop("right"), InvalidModel),
])
def test_what_is_refused(change, error):
    raw = raw_config()
    change(raw)
    with pytest.raises(error):
        config_from_dict(raw)


def test_the_plan_names_the_files_tensors(tmp_path):
    from liyab_amd.weights import write_random_model
    from liyab_amd.weights.safetensors_io import SafetensorsFile

    d = write_random_model(str(tmp_path / "m"), raw_config(), 3)
    f = SafetensorsFile(str(tmp_path / "m" / "model.safetensors"))
    names = set(f.entries)
    assert not any(n.startswith("l3.") for n in names)  # the last layer has no tensors of its own
    for n in ("embed", "head", "final.norm", "final.norm.b", "final.norm.alpha", "l0.norm1.alpha", "l0.mix.mu.w", "l0.mix.w1", "l0.mix.u",
              "l1.mix.q.norm", "l1.mix.k.norm", "l1.mix.g", "l2.mix.left.rel", "l2.mix.left.out", "l2.mix.right.conv.b", "l2.mix.right.A_log",
              "l2.mix.right.out", "l2.mlp.down"):
        assert n in names, n
    assert "l1.mix.v" not in names and "l1.mlp.gate" not in names
    assert f.entries["final.norm.alpha"].shape == () and f.entries["l2.mix.left.rel"].shape == (10, 2)
    assert f.entries["l2.mix.right.in"].shape == (2 * 20 + 2 * 6 + 2, 48) and f.entries["l2.mix.right.conv"].shape == (20 + 12, 3)
    assert f.entries["l0.mix.w1"].shape == (16, 48) and f.entries["l0.mix.u"].shape == (2, 8)
    cfg = load_config(d)  # read back by the architecture's name, the table's rows from the tensor's shape
    assert cfg.layers[2].mixer[0].bias_rows == 10 and cfg.layers[0].mixer.decay_rank == 16
    plan = cfg.plan()
    assert [l.arrangement for l in plan.layers] == ["parallel"] * 4 and plan.residual_position is None
    assert plan.layers[3].mixer.tensors["r"].name == "l0.mix.r" and plan.layers[2].ffn.limit == 2.0


def test_the_distance_table_and_the_frequencies():
    import plain_mofulix as plain
    from liyab_amd.config.plan import RotarySpec
    from liyab_amd.parts.scored_attention import distance_rows, rotary_frequencies

    for rows, far in ((10, 30), (32, 100), (5, 3), (16, 256)):
        assert distance_rows(rows, far).tolist() == [plain.distance_bucket(n, rows, far) for n in range(far + 1)]
    got = rotary_frequencies(RotarySpec(dims=8, base=1000.0, scaling=(2.0, 1.0, 4.0, 32.0)))
    want = plain.rotary_frequencies({"dims": 8, "base": 1000.0, "scaling": {"factor": 2.0, "low": 1.0, "high": 4.0, "original": 32}})
    assert np.allclose(got, want, rtol=1e-14) and got[0] == 1.0 and got[-1] < 1000.0 ** (-6 / 8)
