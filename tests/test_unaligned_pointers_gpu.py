"""Every Linear / Conv2d entry point of the C ABI with ALL of its float pointers
(inputs and outputs) offset by one float from a 16-byte boundary, on shapes whose
sizes are multiples of four, against the CPU oracle.

The dispatch picks its 16-byte-load kernels by pointer alignment as well as by shape;
with sizes that are multiples of four only the pointer test can send a call down the
scalar / table-driven branches, which is what this file makes it do. The tensors sit
inside larger allocations with a guard value on either side, so a kernel that wrote
or rounded an address down to the boundary would show.
"""
import numpy as np
import pytest

from util import SAME_SIGN, assert_close, conv_inputs, linear_inputs

pytestmark = pytest.mark.gpu

GUARD = 12345.0


def _off(a):
    """Device copy of `a` that starts 4 bytes past a 16-byte boundary."""
    import torch
    if a is None:
        return None
    buf = torch.full((a.size + 8,), GUARD, device="cuda")
    assert buf.data_ptr() % 16 == 0
    view = buf[1:1 + a.size]
    view.copy_(torch.from_numpy(np.ascontiguousarray(a).ravel()))
    assert view.data_ptr() % 16 == 4
    view._guard = buf
    return view


def _out(n):
    import torch
    buf = torch.full((n + 8,), GUARD, device="cuda")
    view = buf[1:1 + n]
    view._guard = buf
    return view


def _host(view):
    """The tensor's values, after checking that its surroundings are untouched."""
    buf = view._guard.cpu().numpy()
    assert buf[0] == GUARD and np.all(buf[1 + view.numel():] == GUARD), "write outside the tensor"
    return buf[1:1 + view.numel()].copy()


# tiled (sliced forward / state backward, side jobs of the weight backward), the
# streaming kernels' shapes (B <= 8 and 9..16), a small layer
LINEAR = [(512, 384, 256), (1024, 256, 8), (1024, 512, 12), (128, 128, 32), (2048, 64, 64)]


@pytest.mark.parametrize("K,N,B", LINEAR)
def test_linear_entry_points_with_offset_pointers(oracle_lib, linear_kernel_choice, K, N, B):
    import torch
    from cutagi_amd import capi
    assert K % 4 == 0 and N % 4 == 0
    d = linear_inputs(K, N, B, seed=5 * K + N + B, bias=True, jcb_random=True)
    t = {k: _off(v) for k, v in d.items()}
    p = capi.ptr
    L = capi.lib

    mu_z, var_z = _out(B * N), _out(B * N)
    capi.check(L.tagi_linear_fwd(p(t["mu_w"]), p(t["var_w"]), p(t["mu_b"]), p(t["var_b"]),
                                 p(t["mu_a"]), p(t["var_a"]), K, N, B, 1, p(mu_z), p(var_z), None))
    ref = oracle_lib.linear_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                d["var_a"], threads=4)
    assert_close(_host(mu_z), ref[0], "mu_z")
    assert_close(_host(var_z), ref[1], "var_z", same_sign=True)

    ref_dz = oracle_lib.linear_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], threads=4)
    ref_dw = oracle_lib.linear_bwd_dw(d["var_w"], d["mu_a"], d["delta_mu"], d["delta_var"], threads=4)
    ref_db = oracle_lib.linear_bwd_db(d["var_b"], d["delta_mu"], d["delta_var"])
    names = ["delta_mu_z", "delta_var_z", "delta_mu_w", "delta_var_w", "delta_mu_b", "delta_var_b"]

    # the one backward call
    outs = [_out(B * K), _out(B * K), _out(N * K), _out(N * K), _out(N), _out(N)]
    capi.check(L.tagi_linear_bwd(p(t["mu_w"]), p(t["var_w"]), p(t["var_b"]), p(t["mu_a"]),
                                 p(t["jcb"]), p(t["delta_mu"]), p(t["delta_var"]), K, N, B, 1, 1, 1,
                                 *[p(o) for o in outs], None))
    for name, got, want in zip(names, outs, ref_dz + ref_dw + ref_db):
        assert_close(_host(got), want, name, same_sign=name in SAME_SIGN)

    # and its three parts as calls of their own
    dz = [_out(B * K), _out(B * K)]
    capi.check(L.tagi_linear_bwd_dz(p(t["mu_w"]), p(t["jcb"]), p(t["delta_mu"]), p(t["delta_var"]),
                                    K, N, B, p(dz[0]), p(dz[1]), None))
    dw = [_out(N * K), _out(N * K)]
    capi.check(L.tagi_linear_bwd_dw(p(t["var_w"]), p(t["mu_a"]), p(t["delta_mu"]), p(t["delta_var"]),
                                    K, N, B, p(dw[0]), p(dw[1]), None))
    db = [_out(N), _out(N)]
    capi.check(L.tagi_linear_bwd_db(p(t["var_b"]), p(t["delta_mu"]), p(t["delta_var"]), N, B,
                                    p(db[0]), p(db[1]), None))
    for name, got, want in zip(names, dz + dw + db, ref_dz + ref_dw + ref_db):
        assert_close(_host(got), want, name + " (own call)", same_sign=name in SAME_SIGN)
    torch.cuda.synchronize()


# (kernel, stride, pad, pad_type, wi, fi, fo, B): the regular-stencil geometry (whole
# channel groups, so only the pointers keep it off the stencil kernels), a strided 3x3,
# a 2x2 projection, a sliced late-stage shape
CONV = [(3, 1, 1, 1, 16, 64, 64, 2), (3, 2, 1, 2, 8, 8, 16, 4), (2, 2, 0, 1, 8, 64, 32, 2),
        (3, 1, 1, 1, 4, 128, 64, 4)]


@pytest.mark.parametrize("geom", CONV)
def test_conv2d_entry_points_with_offset_pointers(oracle_lib, geom):
    import torch
    from cutagi_amd import capi
    k, s, pad, pt, wi, fi, fo, B = geom
    idx = capi.conv2d_build_idx(k, s, wi, wi, pad, pt, k * k * fi * fo + 1)
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=11 + sum(geom), bias=True, jcb_random=True)
    t = {n: _off(v) for n, v in d.items()}
    ti = {n: torch.from_numpy(idx[n]).cuda() for n in ("Fmwa_2", "FCzwa_1", "Szz_ud")}
    p = capi.ptr
    L = capi.lib

    mu_z, var_z = _out(B * fo * woho), _out(B * fo * woho)
    capi.check(L.tagi_conv2d_fwd(p(t["mu_w"]), p(t["var_w"]), p(t["mu_b"]), p(t["var_b"]),
                                 p(t["mu_a"]), p(t["var_a"]), p(ti["Fmwa_2"]), woho, fo, wihi, fi,
                                 k, B, 1, p(mu_z), p(var_z), None))
    ref = oracle_lib.conv2d_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"],
                                idx["Fmwa_2"], woho, fo, wihi, fi, k, B, threads=4)
    assert_close(_host(mu_z), ref[0], "mu_z")
    assert_close(_host(var_z), ref[1], "var_z", same_sign=True)

    dz = [_out(B * fi * wihi), _out(B * fi * wihi)]
    capi.check(L.tagi_conv2d_bwd_dz(p(t["mu_w"]), p(t["jcb"]), p(t["delta_mu"]), p(t["delta_var"]),
                                    p(ti["FCzwa_1"]), p(ti["Szz_ud"]), woho, fo, wihi, fi, k,
                                    idx["h"], B, p(dz[0]), p(dz[1]), None))
    ref_dz = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                      idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k,
                                      idx["h"], B, threads=4)
    assert_close(_host(dz[0]), ref_dz[0], "delta_mu_z")
    assert_close(_host(dz[1]), ref_dz[1], "delta_var_z", same_sign=True)

    dw = [_out(fo * fi * k * k), _out(fo * fi * k * k), _out(fo), _out(fo)]
    capi.check(L.tagi_conv2d_bwd_dw(p(t["var_w"]), p(t["var_b"]), p(t["mu_a"]), p(t["delta_mu"]),
                                    p(t["delta_var"]), p(ti["Fmwa_2"]), B, fo, woho, wihi, fi, k, 1,
                                    *[p(o) for o in dw], None))
    ref_dw = oracle_lib.conv2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], d["delta_mu"],
                                      d["delta_var"], idx["Fmwa_2"], B, fo, woho, wihi, fi, k,
                                      threads=4)
    for name, got, want in zip(["delta_mu_w", "delta_var_w", "delta_mu_b", "delta_var_b"], dw,
                               ref_dw):
        assert_close(_host(got), want, name, same_sign=name in SAME_SIGN)
    torch.cuda.synchronize()
