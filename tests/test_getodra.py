"""Getodra on the host: its configuration, the model put together from it, the names and
shapes of its tensors, the rotation's scaled table, and what it asks of the cache."""
import copy
import math

import pytest
import torch

import getodra_cases
import plain_getodra


def test_config_and_plan():
    from ninfer_amd import build_spec
    raw = getodra_cases.config_odd()
    cfg, spec = build_spec(raw)
    assert cfg.vocab == 200 and cfg.taps == 3 and len(cfg.layers) == 4
    assert [c.layer for c in spec.plan] == [0, 1, 0, 1] and len(spec.blocks) == 2
    names = spec.tensor_specs()
    assert {"embed", "pos", "head", "final.norm", "l0.norm1", "l0.canon2", "l0.mix.dkv.norm",
            "l1.mix.norm", "l1.mlp.down"} <= set(names)
    assert not any(n.startswith(("l2.", "l3.")) for n in names)
    assert names["l0.norm1"].shape == () and names["final.norm"].shape == ()
    assert names["l0.mix.q"].shape == (3 * 32, 72) and names["l0.mix.dkv"].shape == (48, 72)
    assert names["l0.mix.g"].shape == (3, 72) and names["l1.mix.g"].shape == (100, 72)
    assert names["l0.canon1"].shape == (72, 3)
    assert spec.max_positions() == 160


def test_layer_without_feed_forward_and_state():
    from ninfer_amd import build_spec
    cfg, spec = build_spec(getodra_cases.config_ones())
    names = spec.tensor_specs()
    assert "l0.canon2" not in names and "l0.norm2" not in names and "l1.canon2" in names
    assert spec.blocks[0].state_floats() == 0          # one tap keeps nothing, attention pages
    assert spec.blocks[1].state_floats() == 16 * 16    # the lightning state alone
    cfg, spec = build_spec(getodra_cases.config_odd())
    assert spec.blocks[0].state_floats() == 2 * 2 * 72
    assert spec.blocks[1].state_floats() == 2 * 2 * 72 + 5 * 12 * 20
    need = spec.blocks[0].mixer.cache_need()
    assert need.window is None and need.pools[0].inner == (48,) and need.pools[0].outer == ()
    assert spec.blocks[1].mixer.cache_need() is None


@pytest.mark.parametrize("bad", [
    lambda c: c.pop("vocab"), lambda c: c["norm"].pop("eps"), lambda c: c.__setitem__("canon", 4),
    lambda c: c["layers"][0].__setitem__("type", "conv"),
    lambda c: c["layers"][1]["mixer"].__setitem__("decay", [0.5]),
    lambda c: c["layers"][2].__setitem__("weights_of", 9),
    lambda c: c["layers"][2].__setitem__("weights_of", 1),
    lambda c: c["layers"][0]["mixer"]["rot"].__setitem__("dims", 7),
    lambda c: c["layers"][0]["mlp"].__setitem__("kind", "experts"),
])
def test_config_errors(bad):
    from ninfer_amd import ConfigError, build_spec
    raw = copy.deepcopy(getodra_cases.config_odd())
    bad(raw)
    with pytest.raises(ConfigError):
        build_spec(raw)


@pytest.mark.parametrize("rot", [
    {"base": 30000.0, "dims": 32, "scaling": {"factor": 6.0, "original": 1024, "fast": 24.0, "slow": 1.5}},
    {"base": 10000.0, "dims": 8, "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}},
    {"base": 500.0, "dims": 6},
])
def test_scaled_rotary_table(rot):
    from ninfer_amd.parts import Rotary
    part = Rotary(rot["dims"], rot["base"], scaling=rot.get("scaling"))
    want, mag = plain_getodra.rotary_table(rot)
    torch.testing.assert_close(part.inv_freq().double(), want, rtol=1e-6, atol=0)
    assert part.magnitude == pytest.approx(mag)
    if "scaling" in rot:   # the fastest pair is left alone, the slowest is stretched in full
        plain = [rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)]
        assert want[0].item() == pytest.approx(plain[0])
        assert want[-1].item() == pytest.approx(plain[-1] / rot["scaling"]["factor"])
        assert mag == pytest.approx(0.1 * math.log(rot["scaling"]["factor"]) + 1)


def test_random_model_folder_roundtrip(tmp_path):
    """A folder written for a configuration and a seed holds every tensor the model names,
    single gains included, and the plain implementation runs on it."""
    import ninfer_amd
    import util
    raw = getodra_cases.config_ones()
    ninfer_amd.write_random_model(str(tmp_path), raw, 5, dtype="bfloat16", std=0.2)
    cfg, w = util.read_folder(str(tmp_path))
    assert w["l0.norm1"].shape == () and w["l1.mix.norm"].shape == (16,)
    logits = plain_getodra.forward(w, cfg, [1, 2, 3, 4, 5])
    assert logits.shape == (5, 96) and torch.isfinite(logits).all()


def test_plain_conv_matches_definition():
    torch.manual_seed(0)
    h, w = torch.randn(6, 3, dtype=torch.float64), torch.randn(3, 4, dtype=torch.float64)
    got = plain_getodra.input_conv(h, w)
    # row 5 sees rows 2..5 with taps 0..3; row 1 sees rows 0, 1 with taps 2, 3
    want5 = h[5] + w[:, 0] * h[2] + w[:, 1] * h[3] + w[:, 2] * h[4] + w[:, 3] * h[5]
    want1 = h[1] + w[:, 2] * h[0] + w[:, 3] * h[1]
    torch.testing.assert_close(got[5], want5)
    torch.testing.assert_close(got[1], want1)
