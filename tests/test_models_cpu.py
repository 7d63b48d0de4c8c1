"""The oracle-call emulation of a training step (tests/model_emulation.py) against
the vectors the compiled reference wrote with its own Sequential / LayerBlock /
ResNetBlock / OutputUpdater drivers (tests/golden/models.npz, from
oracle/ref_model.cpp). The emulator chains the bit-exact oracle kernels in the
reference's order, so everything is required to match bit for bit; where the
reference library is present the vectors are also regenerated and compared."""
import os

import numpy as np
import pytest

from model_cases import (CASES, REF_THREADS, build_emulation, case_inputs,
                         flat_params_of_emulation, leaf_sizes, leaves, parse, sample_index)
from model_emulation import Emulator

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "models.npz"),
               allow_pickle=False)


def run_emulation(oracle_lib, name):
    """Steps of a case on the emulator; the same dict ref.model_run returns."""
    c = CASES[name]
    inp = case_inputs(name)
    layers = build_emulation(c["spec"], inp["params"])
    emu = Emulator(oracle_lib, layers, threads=REF_THREADS)
    B, steps = c["B"], c["steps"]
    out_mu, out_var, in_dmu, in_dvar, params, neg = [], [], [], [], [], []
    state = c.get("input_state_update", False)
    for s in range(steps):
        var_x = np.zeros_like(inp["mu_x"][s]) if inp["var_x"] is None else inp["var_x"][s]
        mu, var = emu.forward(inp["mu_x"][s], var_x, B)
        out_mu.append(mu.copy())
        out_var.append(var.copy())
        if c["update"] == 0:
            emu.update_dense(inp["y"][s], inp["var_y"][s])
        elif c["update"] == 1:
            emu.update_indexed(inp["y"][s], inp["var_y"][s], inp["sel"][s], inp["n_out"], c["n_enc"])
        else:
            emu.update_heteros(inp["y"][s])
        emu.backward(input_state_update=state)
        if state:
            in_dmu.append(emu.input_delta[0].copy())
            in_dvar.append(emu.input_delta[1].copy())
        emu.step()
        params.append(flat_params_of_emulation(layers))
        neg.append(dict(emu.neg))
    return dict(out_mu=out_mu, out_var=out_var, in_dmu=in_dmu, in_dvar=in_dvar, params=params,
                neg=neg, emu=emu, layers=layers)


def test_description_parser_and_sizes(ref_lib):
    for name, c in CASES.items():
        _, layers = parse(c["spec"])
        sizes = [s for _, L in leaves(layers) for s in leaf_sizes(L)]
        assert GOLD[name + "_params"].shape == (c["steps"], sample_index(sum(sizes)).size)
        if ref_lib is not None:
            assert ref_lib.model_param_sizes(c["spec"]) == sizes, name


@pytest.mark.parametrize("name", [n for n in CASES if not CASES[n].get("eval_forward")
                                  and not CASES[n].get("big")])
def test_emulation_matches_reference_drivers(oracle_lib, name):
    c = CASES[name]
    r = run_emulation(oracle_lib, name)
    for s in range(c["steps"]):
        assert np.array_equal(r["out_mu"][s], GOLD[name + "_out_mu"][s]), "out_mu step %d" % s
        assert np.array_equal(r["out_var"][s], GOLD[name + "_out_var"][s]), "out_var step %d" % s
        idx = sample_index(r["params"][s].size)
        assert np.array_equal(r["params"][s][idx], GOLD[name + "_params"][s]), "params step %d" % s
        assert float(r["params"][s].astype(np.float64).sum()) == float(GOLD[name + "_params_sum"][s])
        if c.get("input_state_update"):
            assert np.array_equal(r["in_dmu"][s], GOLD[name + "_in_dmu"][s])
            assert np.array_equal(r["in_dvar"][s], GOLD[name + "_in_dvar"][s])
        # the reference counts clamped variances per top-level layer and reports 0 for
        # blocks (BaseLayer::get_neg_var_w_counter is not virtual)
        _, layers = parse(c["spec"])
        for i, L in enumerate(layers):
            if L[0] in ("Linear", "Conv2d", "BatchNorm2d"):
                assert r["neg"][s].get(i, 0) == int(GOLD[name + "_neg"][s][i]), (name, s, i)
    if name == "mlp_negative_variances":
        assert GOLD[name + "_neg"].sum() > 0     # the case does exercise the clamp


def test_small_resnet_with_eval_forward(oracle_lib):
    """Two training steps, then a forward in eval mode (running averages)."""
    name = "small_resnet"
    c = CASES[name]
    r = run_emulation(oracle_lib, name)
    for s in range(c["steps"]):
        assert np.array_equal(r["out_mu"][s], GOLD[name + "_out_mu"][s])
        assert np.array_equal(r["out_var"][s], GOLD[name + "_out_var"][s])
        assert np.array_equal(r["params"][s], GOLD[name + "_params"][s])
    assert GOLD[name + "_out_mu"].shape[0] == c["steps"] + 1


def test_first_layer_of_a_block_without_state_update_is_not_trained(oracle_lib):
    """src/layer_block.cpp:208-213: with state_update false the block never runs its
    first layer's backward, so that layer's parameters stay as they were."""
    name = "resnetblock_first"
    inp = case_inputs(name)
    first = inp["params"][0]      # mu_w of the main block's first convolution
    n = first.size
    assert np.array_equal(GOLD[name + "_params"][1][:n], first)
    # with the state update on, the same layer does move
    assert not np.array_equal(GOLD[name + "_input_update_params"][1][:n],
                              case_inputs(name + "_input_update")["params"][0])


@pytest.mark.parametrize("name", sorted(CASES))
def test_vectors_regenerate_from_the_reference(ref_lib, name):
    if ref_lib is None:
        pytest.skip("the reference library is not built here")
    c = CASES[name]
    if c.get("big") and not os.environ.get("TAGI_SLOW_TESTS"):
        pytest.skip("ten seconds of CPU: runs with TAGI_SLOW_TESTS=1")
    inp = case_inputs(name)
    r = ref_lib.model_run(c["spec"], inp["params"], inp["mu_x"], inp["var_x"], inp["y"],
                          inp["var_y"], inp["sel"], c["B"], c["update"], c.get("n_enc", 0),
                          c.get("input_state_update", False), c.get("eval_forward", False),
                          8 if c.get("big") else REF_THREADS)
    assert np.array_equal(r["out_mu"], GOLD[name + "_out_mu"])
    assert np.array_equal(r["out_var"], GOLD[name + "_out_var"])
    idx = sample_index(r["params"].shape[1])
    assert np.array_equal(r["params"][:, idx], GOLD[name + "_params"])
    assert np.array_equal(r["neg"], GOLD[name + "_neg"])
