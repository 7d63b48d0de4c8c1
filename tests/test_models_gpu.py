"""The C++ host classes (Sequential, LayerBlock, ResNetBlock, OutputUpdater behind
the pybind11 module `cutagi`) on the GPU against the vectors the compiled reference
wrote with its own drivers on the CPU (tests/golden/models.npz, from
oracle/ref_model.cpp): network outputs of every forward, input innovations, every
parameter (and BatchNorm2d running average) after every step, clamped-variance
counters. Tolerance: the 1e-4 gate of tests/util.py against the reference's fp32
results."""
import os

import numpy as np
import pytest

from model_cases import (CASES, build_host, case_inputs, flat_params_of_host, parse, sample_index,
                         state_dict_of)
from util import assert_close

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "models.npz"),
               allow_pickle=False)


@pytest.mark.parametrize("name", sorted(CASES))
def test_host_classes_match_reference_drivers(name):
    from cutagi_amd import cutagi
    c = CASES[name]
    inp = case_inputs(name)
    _, layers = parse(c["spec"])
    net = build_host(cutagi, c["spec"])
    net.to_device("cuda")
    net.input_state_update = c.get("input_state_update", False)
    net.load_state_dict(state_dict_of(layers, inp["params"]))
    updater = cutagi.OutputUpdater(net.device)
    B, steps = c["B"], c["steps"]
    for s in range(steps):
        if inp["var_x"] is None:
            net.forward(inp["mu_x"][s])
        else:
            net.forward(inp["mu_x"][s], inp["var_x"][s])
        mu, var = net.get_outputs()
        assert_close(mu, GOLD[name + "_out_mu"][s], "%s out_mu step %d" % (name, s))
        assert_close(var, GOLD[name + "_out_var"][s], "%s out_var step %d" % (name, s))
        assert var.min() >= 0
        if c["update"] == 0:
            updater.update(net.output_z_buffer, inp["y"][s], inp["var_y"][s],
                           net.input_delta_z_buffer)
        elif c["update"] == 1:
            updater.update_using_indices(net.output_z_buffer, inp["y"][s], inp["var_y"][s],
                                         inp["sel"][s], net.input_delta_z_buffer)
        else:
            updater.update_heteros(net.output_z_buffer, inp["y"][s], net.input_delta_z_buffer)
        net.backward()
        if c.get("input_state_update"):
            dm, dv = net.get_input_states()
            assert_close(dm, GOLD[name + "_in_dmu"][s], "%s input delta mu step %d" % (name, s))
            assert_close(dv, GOLD[name + "_in_dvar"][s], "%s input delta var step %d" % (name, s))
        net.step()
        got = flat_params_of_host(net, c["spec"])
        ref = GOLD[name + "_params"][s]
        idx = sample_index(got.size)
        assert_close(got[idx], ref, "%s parameters after step %d" % (name, s))
        assert abs(float(got.astype(np.float64).sum()) - float(GOLD[name + "_params_sum"][s])) \
            <= 1e-4 * max(1.0, abs(float(GOLD[name + "_params_sum"][s])))
        counters = {int(k.split(".")[1]): v for k, v in net.get_neg_var_w_counter().items()}
        for i, L in enumerate(layers):
            if L[0] in ("Linear", "Conv2d", "BatchNorm2d"):
                assert counters[i] == int(GOLD[name + "_neg"][s][i]), (name, s, i, counters)
    if c.get("eval_forward"):
        net.eval()
        net.forward(inp["mu_x"][steps - 1])
        mu, var = net.get_outputs()
        assert_close(mu, GOLD[name + "_out_mu"][steps], name + " eval-mode out_mu")
        assert_close(var, GOLD[name + "_out_var"][steps], name + " eval-mode out_var")


def test_eval_then_train_with_another_batch_size():
    """A model first run in eval mode (no delta buffers yet) and then trained at a
    different batch size."""
    from cutagi_amd import cutagi
    rng = np.random.default_rng(0)
    net = cutagi.Sequential([cutagi.Linear(12, 8), cutagi.ReLU(), cutagi.Linear(8, 3)])
    net.to_device("cuda")
    net.eval()
    net.forward(rng.normal(0, 1, (10, 12)).astype(np.float32))
    assert net.get_outputs()[0].shape == (30,)
    net.train()
    x = rng.normal(0, 1, (4, 12)).astype(np.float32)
    net.forward(x)
    updater = cutagi.OutputUpdater(net.device)
    y = rng.normal(0, 1, 12).astype(np.float32)
    updater.update(net.output_z_buffer, y, np.ones(12, np.float32), net.input_delta_z_buffer)
    net.backward()
    net.step()
    net.forward(x)
    assert np.all(np.isfinite(net.get_outputs()[0]))


def test_parameters_loaded_into_a_conv_net_before_its_first_forward():
    """load_state_dict / params_from onto device layers that have not allocated their
    parameters yet (Conv2d creates them lazily): the copy allocates and uploads."""
    from cutagi_amd import cutagi
    rng = np.random.default_rng(1)

    def make():
        return cutagi.Sequential([cutagi.Conv2d(2, 4, 3, True, 1, 1, 1, 6, 6), cutagi.ReLU(),
                                  cutagi.Linear(4 * 36, 3)])
    src = make()
    src.to_device("cuda")
    src.preinit_layer()
    sd = src.state_dict()
    a = make()
    a.to_device("cuda")
    a.load_state_dict(sd)            # nothing allocated on `a` yet
    b = make()
    b.to_device("cuda")
    b.params_from(src)
    x = rng.normal(0, 1, (3, 72)).astype(np.float32)
    outs = []
    for net in (src, a, b):
        net.forward(x)
        outs.append(net.get_outputs())
    for mu, var in outs[1:]:
        assert np.array_equal(mu, outs[0][0]) and np.array_equal(var, outs[0][1])
    assert a.state_dict() == sd and b.state_dict() == sd


def test_raw_update_and_delta_params_to_device():
    """BaseLayer::raw_update_weights / raw_update_biases add the innovations without
    cap or floor; delta_params_to_device uploads host-side innovations."""
    from cutagi_amd import cutagi
    rng = np.random.default_rng(2)
    net = cutagi.Sequential([cutagi.Linear(5, 4)])
    net.to_device("cuda")
    layer = net.layers[0]
    layer.params_to_host()
    mu_w, var_w = np.array(layer.mu_w, np.float32), np.array(layer.var_w, np.float32)
    mu_b, var_b = np.array(layer.mu_b, np.float32), np.array(layer.var_b, np.float32)
    d = [rng.normal(0, 1, n).astype(np.float32) for n in (20, 20, 4, 4)]
    layer.delta_mu_w, layer.delta_var_w = d[0].tolist(), d[1].tolist()
    layer.delta_mu_b, layer.delta_var_b = d[2].tolist(), d[3].tolist()
    layer.delta_params_to_device()
    layer.set_cuda_threads(128)
    layer.raw_update_weights()
    layer.raw_update_biases()
    layer.params_to_host()
    assert np.array_equal(np.array(layer.mu_w, np.float32), mu_w + d[0])
    assert np.array_equal(np.array(layer.var_w, np.float32), var_w + d[1])
    assert np.array_equal(np.array(layer.mu_b, np.float32), mu_b + d[2])
    assert np.array_equal(np.array(layer.var_b, np.float32), var_b + d[3])
