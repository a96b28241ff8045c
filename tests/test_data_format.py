"""Input layout and channel schedules: oracle pinned to hand-written cases, host code against the oracle."""
import numpy as np
import pytest
import torch

from oracle import data_format as OD


def test_oracle_layout_hand_written():
    # two degrees: l=0 -> entry 0, l=1 -> entries 1..3
    x = np.array([1 + 2j, 3 + 4j, 5 - 6j, -7 + 8j])
    got = OD.coefficients_to_straight_ref(x, 2)
    want = np.array([[1, 2], [3, 4], [5, -6], [-7, 8]], dtype=np.float32)
    assert got.dtype == np.float32 and np.array_equal(got, want)
    assert np.array_equal(OD.coefficients_to_straight_ref(np.stack([x, 2 * x]), 2)[1], 2 * want)


def test_oracle_tau_schedules_closed_forms():
    assert OD.tau_schedule_ref(1, 12, 3) == [12, 12, 12, 12]
    assert OD.tau_schedule_ref(2, 12, 3) == [12, 4, 3, 2]            # ceil(12 / (1, 3, 5, 7))
    assert OD.tau_schedule_ref(3, 12, 3) == [12, 7, 6, 5]            # ceil(12 / sqrt(1, 3, 5, 7))
    with pytest.raises(ValueError):
        OD.tau_schedule_ref(4, 12, 3)


def test_host_conversion_matches_oracle(tmp_path):
    from cgnet_amd import data, model
    rng = np.random.default_rng(0)
    coefs = (rng.standard_normal((7, 36)) + 1j * rng.standard_normal((7, 36)))
    for n in (6, 4, 1):
        got = data.coefficients_to_straight(coefs, n)
        assert got.dtype == torch.float32 and tuple(got.shape) == (7, n * n, 2)
        assert np.array_equal(got.numpy(), OD.coefficients_to_straight_ref(coefs[:, :n * n], n))
    with pytest.raises(ValueError):
        data.coefficients_to_straight(coefs, 7)
    with pytest.raises(TypeError):
        data.coefficients_to_straight(coefs.real, 6)
    # file form: L_<n>.npy + labels
    np.save(tmp_path / "L_6.npy", coefs)
    np.save(tmp_path / "label.npy", np.arange(7) % 10)
    ds = data.CoefficientFile(str(tmp_path / "L_6.npy"), 4, str(tmp_path / "label.npy"), indices=[5, 0, 3])
    assert len(ds) == 3
    x, y, idx = ds[1]
    assert y == 0 and idx == 1 and np.array_equal(x.numpy(), OD.coefficients_to_straight_ref(coefs[0, :16], 4))
    b = ds.batch([2, 0])
    assert np.array_equal(b.numpy(), OD.coefficients_to_straight_ref(coefs[[3, 5], :16], 4))
    with pytest.raises(IndexError):
        ds[3]
    for mode in (1, 2, 3):
        assert model.define_taus(mode, 12, 11) == OD.tau_schedule_ref(mode, 12, 11)


def test_classifier_parameter_names_on_cpu():
    from cgnet_amd import model
    net = model.MNIST_Net(3, tau_type=2, tau_man=4, nlayers=2, device='cpu')
    keys = set(net.state_dict().keys())
    for k in ("SphericalCNN.cgs.0.bnWMM.W", "SphericalCNN.cgs.1.bnWMM.bn_stds", "SphericalCNN.cgs.0.bnWMM.bn_eps",
              "bm1.weight", "bm1.running_mean", "fcs.0.weight", "fcs.0.bias", "final.weight", "final.bias"):
        assert k in keys, k
    assert net.SphericalCNN.output_length == 2 * (1 + 4 + 4)
    assert net.fcs[0].in_features == net.SphericalCNN.output_length
