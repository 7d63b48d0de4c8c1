"""tagi_linear_fwd_static (the Linear forward that allocates nothing) against
tagi_linear_fwd, through the C ABI.

Both entry points run the same kernels on the same slices, so their results are
required to be bit-identical, which is stricter than the 1e-4 gate of the parity
tests; the oracle comparison of tagi_linear_fwd itself is in test_linear_gpu.py.
Every sequence below is two calls in a row on the same GPU, the second with a
smaller input, so the second call meets the array as the first one left it.
"""
import numpy as np
import pytest

from util import assert_close, linear_inputs

pytestmark = pytest.mark.gpu


def _both(d):
    """(static, regular) forward results for one set of host inputs."""
    import torch
    from cutagi_amd import capi
    t = {k: (None if v is None else torch.from_numpy(v).cuda()) for k, v in d.items()}
    N, K = d["mu_w"].shape
    B = d["mu_a"].shape[0]
    bias = int(d["mu_b"] is not None)
    stream = torch.cuda.current_stream().cuda_stream
    out = []
    for fn in (capi.lib.tagi_linear_fwd_static, capi.lib.tagi_linear_fwd):
        # poisoned outputs: anything a call leaves unwritten shows
        mu_z = torch.full((B, N), float("nan"), device="cuda")
        var_z = torch.full((B, N), float("nan"), device="cuda")
        capi.check(fn(capi.ptr(t["mu_w"]), capi.ptr(t["var_w"]), capi.ptr(t["mu_b"]),
                      capi.ptr(t["var_b"]), capi.ptr(t["mu_a"]), capi.ptr(t["var_a"]), K, N, B,
                      bias, capi.ptr(mu_z), capi.ptr(var_z), stream))
        torch.cuda.synchronize()
        out.append((mu_z.cpu().numpy(), var_z.cpu().numpy()))
    return out


# (first call, second and smaller call) as (K, N, B): sliced tile kernel, the
# streaming kernels for up to 8 and for 9..16 samples, a ragged shape, and a
# second call that needs no slices at all
SEQUENCES = [
    ((1024, 512, 64), (512, 256, 32)),
    ((2048, 512, 8), (1024, 96, 3)),
    ((1536, 260, 12), (512, 256, 9)),
    ((785, 600, 40), (100, 36, 40)),
    ((4096, 128, 32), (64, 2048, 256)),
]


@pytest.mark.parametrize("first,second", SEQUENCES)
def test_static_forward_matches_regular_forward(oracle_lib, linear_kernel_choice, first, second):
    for i, (K, N, B) in enumerate((first, second)):
        d = linear_inputs(K, N, B, seed=11 * K + N + B, bias=(i == 0))
        (mu_s, var_s), (mu_r, var_r) = _both(d)
        assert np.array_equal(mu_s, mu_r), "mu_z differs at %r" % ((K, N, B),)
        assert np.array_equal(var_s, var_r), "var_z differs at %r" % ((K, N, B),)
        ref_mu, ref_var = oracle_lib.linear_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"],
                                                d["mu_a"], d["var_a"], threads=4)
        assert_close(mu_s, ref_mu, "mu_z")
        assert_close(var_s, ref_var, "var_z")
        assert float(var_s.min()) >= 0.0


def test_static_forward_rejects_what_does_not_fit():
    """Partial sums beyond the fixed array: an error code, outputs untouched."""
    import torch
    from cutagi_amd import capi
    K, N, B = 2048, 4096, 2048
    w = torch.zeros((N, K), device="cuda")
    a = torch.zeros((B, K), device="cuda")
    mu_z = torch.full((B, N), 7.0, device="cuda")
    var_z = torch.full((B, N), 7.0, device="cuda")
    # 8 slices of a 2048 x 4096 output pair = 512 MiB of partial sums
    capi.tune("linear.fwd.splits", 8)
    try:
        rc = capi.lib.tagi_linear_fwd_static(capi.ptr(w), capi.ptr(w), None, None, capi.ptr(a),
                                             capi.ptr(a), K, N, B, 0, capi.ptr(mu_z),
                                             capi.ptr(var_z), None)
    finally:
        capi.tune("linear.fwd.splits", -1)
    torch.cuda.synchronize()
    assert rc == capi.ERR_UNSUPPORTED
    assert float(mu_z.min()) == 7.0 and float(var_z.max()) == 7.0


def test_static_forward_allocates_no_device_memory():
    """The property the entry point exists for. On a stream that has never been used
    with the library (so it owns no workspace), a sliced shape runs through the static
    entry point without the free device memory moving; the regular entry point, called
    on such a stream, does grow a workspace - which shows that the probe would see an
    allocation."""
    import torch
    from cutagi_amd import capi
    K, N, B = 4096, 2048, 256        # eight reduction slices: 32 MiB of partial sums
    d = linear_inputs(K, N, B, seed=5, bias=True)
    t = {k: torch.from_numpy(v).cuda() for k, v in d.items()}
    mu_z, var_z = torch.empty((B, N), device="cuda"), torch.empty((B, N), device="cuda")
    want_mu, want_var = torch.empty_like(mu_z), torch.empty_like(var_z)
    args = [capi.ptr(t[k]) for k in ("mu_w", "var_w", "mu_b", "var_b", "mu_a", "var_a")] + [K, N, B, 1]
    # first use of the static array on this device (address look-up) happens here
    capi.check(capi.lib.tagi_linear_fwd_static(*args, capi.ptr(want_mu), capi.ptr(want_var), None))
    torch.cuda.synchronize()

    # a stream's first launch makes the runtime set up its queue (device memory of its
    # own): let both streams run something that is not this library first
    fresh, other = torch.cuda.Stream(), torch.cuda.Stream()
    dummy = torch.zeros(1024, device="cuda")
    for s in (fresh, other):
        with torch.cuda.stream(s):
            dummy.add_(1.0)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    capi.check(capi.lib.tagi_linear_fwd_static(*args, capi.ptr(mu_z), capi.ptr(var_z),
                                               fresh.cuda_stream))
    fresh.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the static entry point allocated"
    assert torch.equal(mu_z, want_mu) and torch.equal(var_z, want_var)

    free_before = torch.cuda.mem_get_info()[0]
    capi.check(capi.lib.tagi_linear_fwd(*args, capi.ptr(mu_z), capi.ptr(var_z), other.cuda_stream))
    other.synchronize()
    assert torch.cuda.mem_get_info()[0] < free_before, "probe insensitive: no workspace grew"
    assert torch.equal(mu_z, want_mu)
