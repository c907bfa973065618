"""The Bagonex configuration without a GPU: keys, checks, the spec's parts and tensor names, what the cache is asked for."""
import copy

import pytest
import torch

from rbitnet_amd.cache import Cache
from rbitnet_amd.config import load_config
from rbitnet_amd.engine.model import expected_tensors
from rbitnet_amd.errors import ConfigError
from rbitnet_amd.parts import CacheRequest

from plain_bagonex import random_bagonex_tensors

DELTA = {"type": "channel_delta", "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 12, "conv": 3, "decay_rank": 6,
                                            "gate_rank": 10}, "mlp": {"kind": "dense", "ff": 40}}
LATENT = {"type": "latent_attention", "mixer": {"heads": 3, "dim": 8, "vdim": 6, "q_rank": 20, "kv_rank": 16, "scale": 0.3},
          "mlp": None}
SHARED = {"type": "latent_attention", "mixer": {"heads": 2, "dim": 4, "vdim": 10, "q_rank": 12, "kv_rank": 16, "scale": 0.5,
                                                "kv_from": 0}, "mlp": {"kind": "dense", "ff": 24}}
CFG = {"architecture": "Bagonex", "vocab": 50, "width": 32, "streams": 3, "norm": {"eps": 1e-5}, "canon": {"taps": 2},
       "logit_softcap": 9.0, "layers": [LATENT, DELTA, SHARED]}


def test_spec_names_every_tensor_the_oracle_makes():
    cfg, spec = load_config(copy.deepcopy(CFG))
    assert spec.architecture == "Bagonex" and [l.block for l in spec.layers] == ["hyper"] * 3
    want = random_bagonex_tensors(CFG, 0)
    got = expected_tensors(spec)
    assert set(got) == set(want)
    for name, ts in got.items():
        assert tuple(ts.shape) == tuple(want[name].shape), name
    assert "l0.norm2" not in got and "l0.mlp.up" not in got and "l2.mix.dkv" not in got      # no feed-forward; reads layer 0's latents


def test_ranks_come_from_the_weight_file_when_the_file_has_them():
    raw = copy.deepcopy(CFG)
    for key in ("decay_rank", "gate_rank"):
        del raw["layers"][1]["mixer"][key]
    with pytest.raises(ConfigError, match="decay_rank"):
        load_config(copy.deepcopy(raw))
    _, spec = load_config(copy.deepcopy(raw), tensor_shapes={"l1.mix.a1": (5, 32), "l1.mix.g1": (7, 32)})
    got = expected_tensors(spec)
    assert got["l1.mix.a2"].shape == (4 * 8, 5) and got["l1.mix.g2"].shape == (4 * 12, 7)


@pytest.mark.parametrize("edit,match", [
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "stores no latents"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "earlier layer"),
    (lambda c: c["layers"][2]["mixer"].update(kv_rank=8), "differs"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "cannot share"),
    (lambda c: c["layers"][0].update(type="window"), "type must be"),
    (lambda c: c["layers"][1].update(mlp={"kind": "routed", "ff": 8}), "kind 'dense'"),
    (lambda c: c.update(width=0), "width"),
    (lambda c: c.pop("canon"), "canon"),
])
def test_configuration_errors_name_the_key(edit, match):
    raw = copy.deepcopy(CFG)
    edit(raw)
    with pytest.raises(ConfigError, match=match):
        load_config(raw)


def test_a_layer_may_ask_the_cache_for_several_things():
    """Latents as keys and values at once (no second set of pages), two named states beside them, and a reader."""
    reqs = [[CacheRequest("kv", heads=1, head_dim=16, values=False, name="latent"),
             CacheRequest("state", state_shape=(1, 32), name="input_conv")],
            [CacheRequest("state", state_shape=(4, 12, 8), name="delta"), CacheRequest("state", state_shape=(2, 40), name="conv"),
             CacheRequest("state", state_shape=(1, 32), name="input_conv")],
            [CacheRequest("state", state_shape=(1, 32), name="input_conv")]]
    c = Cache(reqs, n_slots=2, max_tokens=128, dtype=torch.float32, device="cpu", readers={2: 0})
    s = c.alloc_slot()
    c.reserve([s], [70])
    tables = {k: torch.tensor(v, dtype=torch.int32) for k, v in c.block_tables([s]).items()}
    v0, v1, v2 = (c.view(l, tables) for l in range(3))
    assert v0.k_pages.shape == (3, 1, 64, 16) and v0.v_pages.data_ptr() == v0.k_pages.data_ptr()
    assert v2.k_pages.data_ptr() == v0.k_pages.data_ptr() and set(v2.states) == {"input_conv"}
    assert v1.states["delta"].shape == (3, 4, 12, 8) and v1.states["conv"].shape == (3, 2, 40) and v1.k_pages is None
    assert v0.states["input_conv"].data_ptr() != v2.states["input_conv"].data_ptr()       # a layer's own
    v1.states["delta"][s] = 3.0
    c.commit([s], [70])
    c.free_slot(s)
    assert c.alloc_slot() == s and float(c.view(1, tables).states["delta"][s].abs().max()) == 0.0     # handed out clean
    with pytest.raises(Exception, match="twice"):
        Cache([[CacheRequest("state", state_shape=(2,)), CacheRequest("state", state_shape=(2,))]], 1, 64, torch.float32, "cpu")


def test_command_line_writes_and_inspects_a_random_model(tmp_path, capsys):
    import json
    from rbitnet_amd import cli
    cfg_path = tmp_path / "config.json"
    cfg_path.write_text(json.dumps(CFG))
    assert cli.main(["random", "--config", str(cfg_path), "--out", str(tmp_path / "m"), "--seed", "3"]) == 0
    capsys.readouterr()
    assert cli.main(["inspect", str(tmp_path / "m")]) == 0
    out = capsys.readouterr().out
    assert "arch=Bagonex" in out and "BagonexConfig" in out and "missing=0 unexpected=0" in out
    # the mixing matrices of a random model start near the identity, so that the copies of the stream survive the layers
    from rbitnet_amd.weights.safetensors_io import WeightFolder
    mix = WeightFolder(str(tmp_path / "m")).tensor("l1.hc2.mix").float()
    assert mix.shape == (3, 3) and float((mix - torch.eye(3)).abs().max()) < 0.2
