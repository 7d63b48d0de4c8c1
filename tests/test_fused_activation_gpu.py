"""Linear / Conv2d forward with the following activation applied in the kernel's
epilogue (tagi_linear_fwd_act, tagi_conv2d_fwd_act); and the host classes with the
fusion switched off against the same reference vectors as with it on.

The fused call is checked in two separate steps, so that neither hides the other:
the layer's sums (the unfused call on the same inputs, which runs the same kernel
without the epilogue) against the oracle's layer at the 1e-4 parity tolerance, and
the epilogue alone - the fused outputs against the oracle's activation applied to
the GPU's OWN sums - at 1e-5 (ReLU: exactly). A non-linearity amplifies the 1e-4
reordering error of its input, which is why the fused outputs are not compared with
oracle-layer-then-oracle-activation at one tolerance."""
import os

import numpy as np
import pytest

from util import assert_close, conv_inputs, linear_inputs

pytestmark = pytest.mark.gpu

# fused epilogue against the oracle's activation of the same fp32 sums: what is left
# is the difference between the device's and the host's erfc / exp
EPILOGUE_TOL = 1e-5

# tiled unsliced / sliced reductions, ragged shapes, the streaming kernels (B <= 8, 9..16)
LINEAR = [(256, 256, 128), (1024, 512, 64), (100, 36, 40), (785, 600, 16), (784, 128, 32),
          (2048, 48, 7), (1536, 260, 12), (5, 3, 2)]


def _dev(d):
    import torch
    return {k: (None if v is None else torch.from_numpy(v).cuda()) for k, v in d.items()}


def _activate(oracle_lib, name, mu, var):
    if name == "relu":
        return oracle_lib.relu_fwd(mu.ravel(), var.ravel())          # mu_a, var_a, jcb
    return oracle_lib.mixture_relu_fwd(mu.ravel(), var.ravel(), 2)


@pytest.mark.parametrize("K,N,B", LINEAR)
@pytest.mark.parametrize("act", ["relu", "mixture_relu"])
@pytest.mark.parametrize("bias", [True, False])
def test_linear_forward_with_activation(oracle_lib, linear_kernel_choice, K, N, B, act, bias):
    import cutagi_amd.functional as F
    d = linear_inputs(K, N, B, seed=3 * K + N + B, bias=bias)
    t = _dev(d)
    got = F.linear_fwd_act(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"], act)
    plain = F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"])
    z = oracle_lib.linear_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"],
                              threads=4)
    if act == "relu":
        # ReLU is a selection: exactly the unfused kernel's sums, gated by their sign
        m = plain[0].cpu().numpy().ravel()
        keep = np.maximum(m, 0) != 0
        assert np.array_equal(got[0].cpu().numpy().ravel(), np.maximum(m, 0))
        assert np.array_equal(got[1].cpu().numpy().ravel(), np.where(keep, plain[1].cpu().numpy().ravel(), 0))
        assert np.array_equal(got[2].cpu().numpy().ravel(), keep.astype(np.float32))
        return
    # the sums, against the oracle's layer
    assert_close(plain[0].cpu().numpy().ravel(), z[0].ravel(), "mu_z")
    assert_close(plain[1].cpu().numpy().ravel(), z[1].ravel(), "var_z", same_sign=True)
    # the epilogue, against the oracle's activation of those very sums
    own = _activate(oracle_lib, act, plain[0].cpu().numpy(), plain[1].cpu().numpy())
    for name, g, r in zip(("mu_a", "var_a", "jcb"), got, own):
        assert_close(g.cpu().numpy().ravel(), r, name, tol=EPILOGUE_TOL)
    assert float(got[1].min()) > 0 and 0 <= float(got[2].min()) and float(got[2].max()) <= 1


# (kernel, stride, pad, pad_type, wi, fi, fo, B): stencil, strided table-driven, sliced
CONV = [(3, 1, 1, 1, 8, 8, 64, 4), (3, 2, 1, 2, 8, 4, 6, 3), (2, 2, 0, 1, 8, 4, 8, 2),
        (3, 1, 1, 1, 4, 64, 64, 8), (5, 1, 2, 1, 9, 2, 3, 1)]


@pytest.mark.parametrize("geom", CONV)
@pytest.mark.parametrize("act", ["relu", "mixture_relu"])
def test_conv2d_forward_with_activation(oracle_lib, geom, act):
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, s, p, pt, wi, fi, fo, B = geom
    idx = capi.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=sum(geom), bias=True)
    t = _dev(d)
    aidx = torch.from_numpy(idx["Fmwa_2"]).cuda()
    got = F.conv2d_fwd_act(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"],
                           aidx, woho, fo, wihi, fi, k, B, act)
    z = oracle_lib.conv2d_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"],
                              idx["Fmwa_2"], woho, fo, wihi, fi, k, B, 2)
    plain = F.conv2d_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"],
                         aidx, woho, fo, wihi, fi, k, B)
    if act == "relu":
        m = plain[0].cpu().numpy()
        assert np.array_equal(got[0].cpu().numpy(), np.maximum(m, 0))
        assert np.array_equal(got[2].cpu().numpy(), (np.maximum(m, 0) != 0).astype(np.float32))
        return
    assert_close(plain[0].cpu().numpy().ravel(), z[0].ravel(), "mu_z")
    assert_close(plain[1].cpu().numpy().ravel(), z[1].ravel(), "var_z", same_sign=True)
    own = _activate(oracle_lib, act, plain[0].cpu().numpy(), plain[1].cpu().numpy())
    for name, g, r in zip(("mu_a", "var_a", "jcb"), got, own):
        assert_close(g.cpu().numpy().ravel(), r, name, tol=EPILOGUE_TOL)


@pytest.mark.parametrize("name", ["mlp_config1", "conv_relu_linear", "small_resnet",
                                  "layerblock_first_input_update"])
def test_host_classes_without_fusion_match_reference_drivers(name):
    """The same reference vectors with every activation as a launch of its own."""
    from cutagi_amd import cutagi
    import test_models_gpu
    cutagi.set_fused_activations(False)
    try:
        test_models_gpu.test_host_classes_match_reference_drivers(name)
    finally:
        cutagi.set_fused_activations(True)


def test_fusion_changes_the_launch_pattern_not_the_layer_list():
    """With the fusion on, the activation layers still exist, keep their place in the
    state dict numbering and report their sizes."""
    from cutagi_amd import cutagi
    net = cutagi.Sequential([cutagi.Linear(12, 8), cutagi.ReLU(), cutagi.Linear(8, 3)])
    net.to_device("cuda")
    x = np.random.default_rng(0).normal(0, 1, (4, 12)).astype(np.float32)
    net.forward(x)
    fused = net.get_outputs()
    assert sorted(net.state_dict()) == ["LinearCuda.0", "LinearCuda.2"]
    assert net.layers[1].input_size == 8 and net.layers[1].output_size == 8
    cutagi.set_fused_activations(False)
    try:
        net.forward(x)
        plain = net.get_outputs()
    finally:
        cutagi.set_fused_activations(True)
    assert np.array_equal(fused[0], plain[0]) and np.array_equal(fused[1], plain[1])
