"""The Tigutar configuration on the CPU: keys, errors, the spec it turns into, tensor names against the plain
implementation's, sizes read off a weight file's shapes."""
import copy

import pytest

import plain_tigutar as P
from rbitnet_amd.config import load_config
from rbitnet_amd.engine.model import expected_tensors
from rbitnet_amd.errors import ConfigError


def _soft(**more):
    return dict(dict(heads=4, kv_heads=2, dim=16, vdim=24, rot={"base": 100.0, "dims": 8}, scale=0.3), **more)


CFG = {"architecture": "Tigutar", "vocab": 50, "width": 32, "residual_mult": 0.5, "norm": {"eps": 1e-5}, "layers": [
    {"type": "attention", "mixer": _soft(), "mlp": {"kind": "dense", "ff": 40}},
    {"type": "delta", "mixer": dict(heads=2, kv_heads=1, dim=8, vdim=4, conv=3),
     "mlp": {"kind": "moe", "expert": {"ff": 12, "limit": 1.5}, "router": {"experts": 5, "top": 2}}},
    {"type": "parallel", "mixer": {"left": _soft(mask={"size": 5}), "right": dict(heads=2, dim=4, vdim=8, tau=4.0)}, "mlp": None},
    {"type": "attention", "mixer": _soft(heads=6, kv_from=0), "mlp": None}]}


def test_tensor_names_and_shapes_are_the_plain_implementations():
    tensors = P.random_tigutar_tensors(CFG, 1, decay_rank=12)
    shapes = {k: tuple(v.shape) for k, v in tensors.items()}
    cfg, spec = load_config(copy.deepcopy(CFG), tensor_shapes=shapes)
    assert cfg.layers[2]["mixer"]["right"]["decay_rank"] == 12            # read off l2.mix.right.a1
    want = expected_tensors(spec)
    assert set(want) == set(tensors)
    assert all(tuple(want[n].shape) == shapes[n] for n in want)
    assert "l3.mix.k" not in want and "l3.mix.sink" in want and "l2.mix.left.sink" not in want
    assert spec.layers[0].block == "parallel" and spec.layers[0].params["residual_scale"] == 0.5
    assert spec.layers[2].mixer.kind == "pair" and spec.layers[2].mixer["left"]["window"] == 5
    assert spec.layers[3].mixer["cache_from"] == 0 and spec.layers[1].feed_forward.kind == "routed_experts"
    again, _ = load_config(cfg.to_dict())
    assert again.to_dict() == cfg.to_dict()


def test_a_model_without_a_weight_file_must_name_the_decay_rank():
    with pytest.raises(ConfigError, match="decay_rank"):
        load_config(copy.deepcopy(CFG))
    cfg = copy.deepcopy(CFG)
    cfg["layers"][2]["mixer"]["right"]["decay_rank"] = 8
    assert expected_tensors(load_config(cfg)[1])["l2.mix.right.a1"].shape == (8, 32)


@pytest.mark.parametrize("change,message", [
    (lambda c: c.pop("residual_mult"), "residual_mult"),
    (lambda c: c["layers"][0].update(type="conv"), "type must be one of"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "cannot share"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=2), "keeps no keys"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), "earlier layer"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=8), "differs from layer 0"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=6), "top 6 of 5"),
    (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "mlp must be"),
    (lambda c: c["layers"][2]["mixer"]["right"].update(tau=0), "tau"),
    (lambda c: c["layers"][2]["mixer"]["left"].update(mask={"size": 0}), "size"),
    (lambda c: c.update(layers=[]), "at least one layer"),
])
def test_errors_name_the_key(change, message):
    cfg = copy.deepcopy(CFG)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        load_config(cfg)
