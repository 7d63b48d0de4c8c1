"""The pytagi.nn-shaped Python layer (cutagi_amd.nn): construction and field
access without a GPU; on the GPU the README training loop of the reference
(README.md:28-57, the MLP of config 1) gives exactly what the same calls on the
C++ module give -- the wrappers add no arithmetic."""
import numpy as np
import pytest


def test_wrappers_build_and_forward_fields():
    from cutagi_amd import cutagi
    from cutagi_amd.nn import (AvgPool2d, BatchNorm2d, Conv2d, LayerBlock, Linear, MixtureReLU,
                               OutputUpdater, ReLU, ResNetBlock, Sequential, Utils)
    cutagi.manual_seed(0)
    lin = Linear(784, 128)
    assert lin.get_layer_info() == "Linear(784,128)" and lin.input_size == 784
    assert len(lin.mu_w) == 784 * 128
    lin.mu_b = [0.0] * 128                       # writes through to the C++ layer
    assert lin._cpp_backend.mu_b == [0.0] * 128
    net = Sequential(lin, ReLU(), Linear(128, 128), ReLU(), Linear(128, 11))
    assert net.get_layer_stack_info().split() == ["Linear(784,128)", "ReLU()", "Linear(128,128)",
                                                  "ReLU()", "Linear(128,11)"]
    assert net.device == "cpu" and net.z_buffer_size == 784
    net.input_state_update = True
    assert net._cpp_backend.input_state_update is True
    assert sorted(net.state_dict()) == ["Linear.0", "Linear.2", "Linear.4"]
    block = ResNetBlock(LayerBlock(Conv2d(4, 8, 3, bias=False, stride=2, padding=1, padding_type=2),
                                   MixtureReLU(), BatchNorm2d(8)),
                        LayerBlock(Conv2d(4, 8, 2, bias=False, stride=2)))
    cnn = Sequential(Conv2d(3, 4, 3, bias=False, padding=1, in_width=8, in_height=8),
                     BatchNorm2d(4), MixtureReLU(), block, AvgPool2d(4), Linear(8, 5))
    assert "ResNetBlock" in cnn.get_layer_stack_info()
    obs, idx, n_obs = Utils().label_to_obs(np.array([3, 0]), 10)
    assert n_obs == 4 and obs.tolist() == [1, 1, -1, -1, 1, 1, 1, 1]
    assert idx.tolist() == [1, 2, 4, 8, 1, 2, 4, 7] and idx.dtype == np.int32
    with pytest.raises(RuntimeError, match="GPU only"):
        net(np.zeros((2, 784), np.float32))
    assert callable(OutputUpdater("cpu").update_heteros)


def test_label_helpers_match_the_reference_cost_functions(ref_lib):
    """Class probabilities and errors of the hierarchical softmax against the
    compiled reference (get_error over obs_to_class, src/cost.cpp:150-246)."""
    if ref_lib is None or not hasattr(ref_lib.lib, "ref_get_error"):
        pytest.skip("compiled reference not available")
    from cutagi_amd.nn import HRCSoftmaxMetric, Utils
    rng = np.random.default_rng(0)
    for n_classes, n_out in ((10, 11), (4, 3), (7, 7)):
        B = 50
        hs = Utils().get_hierarchical_softmax(n_classes)
        assert hs.len == n_out
        mz = rng.normal(0, 1, (B, hs.len)).astype(np.float32)
        Sz = rng.uniform(0.01, 2, (B, hs.len)).astype(np.float32)
        labels = rng.integers(0, n_classes, B)
        er, prob = ref_lib.get_error(mz, Sz, labels, n_classes)
        e2, p2 = Utils().get_errors(mz.ravel(), Sz.ravel(), labels, hs, n_classes, B)
        assert np.allclose(p2, prob, rtol=1e-5, atol=1e-7) and np.array_equal(e2, er)
        rate = HRCSoftmaxMetric(n_classes).error_rate(mz.ravel(), Sz.ravel(), labels)
        assert rate == pytest.approx(er.mean())


@pytest.mark.gpu
def test_readme_training_loop_matches_the_cpp_module():
    from cutagi_amd import cutagi
    from cutagi_amd.nn import HRCSoftmaxMetric, Linear, OutputUpdater, ReLU, Sequential, Utils
    batch_size, steps = 32, 3
    metric = HRCSoftmaxMetric(num_classes=10)
    rng = np.random.default_rng(0)
    xs = rng.normal(0, 1, (steps, batch_size, 784)).astype(np.float32)
    labels = rng.integers(0, 10, (steps, batch_size))
    var_y = np.full((batch_size * 4,), 1.0, dtype=np.float32)

    cutagi.manual_seed(0)
    net = Sequential(Linear(784, 128), ReLU(), Linear(128, 128), ReLU(), Linear(128, 11))
    net.to_device("cuda")
    udt = OutputUpdater(net.device)
    preds = []
    for i in range(steps):
        y, idx, _ = Utils().label_to_obs(labels[i], 10)
        m_pred, v_pred = net(xs[i])
        udt.update_using_indices(net.output_z_buffer, y, var_y, idx, net.input_delta_z_buffer)
        net.backward()
        net.step()
        preds.append((m_pred, v_pred))
        assert 0.0 <= metric.error_rate(m_pred, v_pred, labels[i]) <= 1.0
    assert preds[0][0].shape == (batch_size * 11,) and np.all(preds[-1][1] > 0)
    assert not np.array_equal(preds[0][0], preds[-1][0])

    cutagi.manual_seed(0)
    raw = cutagi.Sequential([cutagi.Linear(784, 128), cutagi.ReLU(), cutagi.Linear(128, 128),
                             cutagi.ReLU(), cutagi.Linear(128, 11)])
    raw.to_device("cuda")
    upd = cutagi.OutputUpdater(raw.device)
    for i in range(steps):
        y, idx, _ = Utils().label_to_obs(labels[i], 10)
        raw.forward(xs[i])
        m, v = raw.get_outputs()
        assert np.array_equal(m, preds[i][0]) and np.array_equal(v, preds[i][1])
        upd.update_using_indices(raw.output_z_buffer, y.tolist(), var_y.tolist(), idx.tolist(),
                                 raw.input_delta_z_buffer)
        raw.backward()
        raw.step()
    a, b = net.state_dict(), raw.state_dict()
    assert a.keys() == b.keys() and all(a[k] == b[k] for k in a)


@pytest.mark.gpu
def test_mlp_learns_a_synthetic_classification_task():
    """End to end in the manner of the reference's accuracy gate (test/cpp_unit/
    test_mnist.cpp:400-407: error rate below 0.5 after 100 batches of 16), on
    synthetic ten-class data since no dataset travels: noisy copies of ten random
    prototypes. Chance is 0.9."""
    from cutagi_amd import cutagi
    from cutagi_amd.nn import HRCSoftmaxMetric, Linear, OutputUpdater, ReLU, Sequential, Utils
    cutagi.manual_seed(1)
    rng = np.random.default_rng(1)
    protos = rng.normal(0, 1, (10, 784)).astype(np.float32)
    net = Sequential(Linear(784, 128), ReLU(), Linear(128, 128), ReLU(), Linear(128, 11))
    net.to_device("cuda")
    udt = OutputUpdater(net.device)
    metric = HRCSoftmaxMetric(10)
    batch = 16
    var_y = np.full(batch * 4, 1.0, np.float32)
    errors = []
    for _ in range(100):
        label = rng.integers(0, 10, batch)
        x = protos[label] + rng.normal(0, 1.0, (batch, 784)).astype(np.float32)
        y, idx, _ = Utils().label_to_obs(label, 10)
        m_pred, v_pred = net(x)
        errors.append(metric.error_rate(m_pred, v_pred, label))
        udt.update_using_indices(net.output_z_buffer, y, var_y, idx, net.input_delta_z_buffer)
        net.backward()
        net.step()
    assert np.mean(errors[:5]) > 0.6           # starts near chance
    assert np.mean(errors[-20:]) < 0.5, errors[-20:]
