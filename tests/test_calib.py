"""Calibration-file loader: the constrained-parameter transforms of the reference's
ADKVTrainModel getters (train_model.py:127-134), checked against closed forms."""
import math

import pytest
import torch

from adkv_amd import calib


def _raw(n, seed):
    g = torch.Generator().manual_seed(seed)
    return {k: torch.randn(n, generator=g) for k in calib.RAW_FIELDS}


def test_transforms_closed_form():
    sd = {"init_zp": torch.tensor([0.25, -1.0]), "init_log_sc": torch.tensor([0.0, math.log(2.0)]),
          "alpha": torch.tensor([0.0, 100.0]), "beta": torch.tensor([0.0, -100.0]),
          "target": torch.tensor([3.5, 0.5])}
    c = calib.config_from_state_dict(sd)
    assert torch.equal(c.zp_init, sd["init_zp"]) and torch.equal(c.quant_target, sd["target"])
    assert torch.allclose(c.scale_init, torch.tensor([1.0, 2.0]))
    assert torch.allclose(c.alpha, torch.tensor([0.5, 1.0]))
    assert torch.allclose(c.beta, torch.tensor([0.05, 0.0]), atol=1e-30)


def test_round_trip_and_errors(tmp_path):
    raws = [(_raw(64, 2 * l), _raw(64, 2 * l + 1)) for l in range(3)]
    calib.save_calibration(tmp_path, raws)
    got = calib.load_calibration(tmp_path, 3, 64)
    assert len(got) == 3
    for (rk, rv), (ck, cv) in zip(raws, got):
        assert torch.equal(ck.alpha, torch.sigmoid(rk["alpha"]))
        assert torch.equal(cv.beta, 0.1 * torch.sigmoid(rv["beta"]))
        assert torch.equal(cv.scale_init, torch.exp(rv["init_log_sc"]))
    with pytest.raises(FileNotFoundError):
        calib.load_calibration(tmp_path, 4, 64)
    with pytest.raises(ValueError):
        calib.load_calibration(tmp_path, 3, 128)
    with pytest.raises(KeyError):
        calib.config_from_state_dict({"alpha": torch.zeros(2)})


def test_train_model_state_dict_is_loadable(tmp_path):
    """A state_dict saved from the module that mirrors the reference's ADKVTrainModel has the
    reference's key names and goes through the loader; its getters agree with the loader."""
    from adkv_amd.train import ADKVTrainModel
    m = ADKVTrainModel(32)
    with torch.no_grad():
        m.alpha.normal_()
        m.init_log_sc.normal_()
    assert set(m.state_dict()) == set(calib.RAW_FIELDS)
    calib.save_calibration(tmp_path, [(m.state_dict(), m.state_dict())])
    (ck, _), = calib.load_calibration(tmp_path, 1, 32)
    assert torch.equal(ck.alpha, m.get_alpha().detach())
    assert torch.equal(ck.scale_init, m.get_sc().detach())
    assert torch.equal(ck.beta, m.get_beta().detach())


def test_synthetic_config_shapes():
    cfg = calib.synthetic_adkv_config(2, 4, 128)
    assert len(cfg) == 2 and cfg[0][0].alpha.shape == (512,)
    assert not torch.equal(cfg[0][0].alpha, cfg[1][0].alpha)
