"""Parity of the HIP Conv2d path (through the C ABI) against the CPU oracle."""
import numpy as np
import pytest

from util import SAME_SIGN, assert_close, conv_inputs

pytestmark = pytest.mark.gpu

# (kernel, stride, pad, pad_type, wi, fi, fo, B): the geometries of the ResNet-18
# configuration (3x3 s1 p1, 3x3 s2 p1 type 2, 2x2 s2 shortcut), odd channel
# counts (27 = 3*9 reduction, the first ResNet conv), 1x1, 5x5 and 7x7 kernels.
GEOMS = [
    (3, 1, 1, 1, 8, 4, 8, 3),
    (3, 1, 1, 1, 16, 3, 16, 2),
    (3, 2, 1, 2, 8, 8, 16, 4),
    (2, 2, 0, 1, 8, 8, 16, 2),
    (1, 1, 0, 1, 6, 5, 7, 3),
    (5, 1, 2, 1, 9, 2, 3, 2),
    (3, 1, 0, 1, 10, 6, 5, 2),
    (3, 1, 1, 1, 32, 16, 32, 2),
    (3, 1, 1, 1, 12, 70, 66, 1),
    (4, 2, 1, 1, 10, 3, 5, 2),
    (7, 2, 3, 1, 17, 3, 40, 2),  # per-tap table + staged tiles exceed 64 KB of LDS
    (10, 1, 0, 1, 12, 2, 3, 2),  # the largest kernel whose per-tap table fits
    (3, 1, 1, 1, 4, 128, 96, 3),  # late-stage shape: few pixels, long reduction (sliced)
    (2, 2, 0, 1, 8, 64, 130, 2),  # projection shortcut, more than 128 output channels
    # 3x3 s1 p1 on square maps with whole groups of channels: the regular-stencil kernels
    (3, 1, 1, 1, 32, 16, 64, 2),  # forward only (state backward wants 64 input channels)
    (3, 1, 1, 1, 32, 64, 64, 1),
    (3, 1, 1, 1, 16, 64, 128, 3),
    (3, 1, 1, 1, 8, 128, 64, 3),  # two images per tile, last tile half empty
    (3, 1, 1, 1, 4, 320, 64, 5),  # eight images per tile, one partial tile, sliced reduction
    # 3x3 s2 with right/bottom padding and whole groups of channels: the strided stencil kernels
    (3, 2, 1, 2, 32, 64, 64, 1),   # 16x16 output maps, half an image per tile
    (3, 2, 1, 2, 16, 128, 96, 2),  # 8x8 output maps, two images per tile
    (3, 2, 1, 2, 8, 64, 160, 8),   # 4x4 output maps, eight images per tile
    (3, 2, 1, 2, 16, 64, 640, 2),  # long reduction: sliced
    (3, 2, 1, 2, 32, 8, 64, 3),    # strided forward stencil only: 8 input channels, last tile partial... (3 x 256 pixels)
    (3, 2, 1, 2, 8, 24, 64, 5),    # 4x4 output maps, 80 pixels: one partial tile
    (2, 2, 0, 1, 16, 40, 128, 3),  # 2x2 forward stencil: 192 pixels, partial second tile
    # 2x2 s2 projections with whole groups of channels: the all-phase state backward
    (2, 2, 0, 1, 32, 64, 64, 1),
    (2, 2, 0, 1, 16, 128, 96, 2),
    (2, 2, 0, 1, 8, 64, 160, 8),
    (2, 2, 0, 1, 16, 64, 640, 2),
]


def _setup(oracle_lib, geom, bias, seed):
    import torch
    from cutagi_amd import capi
    k, s, p, pt, wi, fi, fo, B = geom
    idx = capi.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
    ref_idx = oracle_lib.conv2d_build_idx(k, s, wi, wi, p, pt, k * k * fi * fo + 1)
    for key in ("Fmwa_2", "FCzwa_1", "Szz_ud"):
        assert np.array_equal(idx[key], ref_idx[key]), key
    assert idx["w"] == wi * wi, "every input pixel must be covered"
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=seed, bias=bias, jcb_random=True)
    t = {n: (None if v is None else torch.from_numpy(v).cuda()) for n, v in d.items()}
    ti = {n: torch.from_numpy(idx[n]).cuda() for n in ("Fmwa_2", "FCzwa_1", "Szz_ud")}
    return idx, d, t, ti, wihi, woho


@pytest.mark.parametrize("geom", GEOMS)
@pytest.mark.parametrize("bias", [False, True])
def test_conv2d_forward(oracle_lib, geom, bias):
    import cutagi_amd.functional as F
    k, s, p, pt, wi, fi, fo, B = geom
    idx, d, t, ti, wihi, woho = _setup(oracle_lib, geom, bias, seed=sum(geom))
    mu_z, var_z = F.conv2d_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"],
                               ti["Fmwa_2"], woho, fo, wihi, fi, k, B)
    ref = oracle_lib.conv2d_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                d["var_a"], idx["Fmwa_2"], woho, fo, wihi, fi, k, B, threads=4)
    assert_close(mu_z.cpu().numpy(), ref[0], "mu_z")
    assert_close(var_z.cpu().numpy(), ref[1], "var_z", same_sign=True)
    assert float(var_z.min()) >= 0.0


@pytest.mark.parametrize("geom", GEOMS)
def test_conv2d_backward(oracle_lib, geom):
    import cutagi_amd.functional as F
    k, s, p, pt, wi, fi, fo, B = geom
    idx, d, t, ti, wihi, woho = _setup(oracle_lib, geom, True, seed=3 + sum(geom))
    dz = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"], ti["FCzwa_1"],
                         ti["Szz_ud"], woho, fo, wihi, fi, k, idx["h"], B)
    ref_dz = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                      idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k,
                                      idx["h"], B, threads=4)
    assert_close(dz[0].cpu().numpy(), ref_dz[0], "delta_mu_z")
    assert_close(dz[1].cpu().numpy(), ref_dz[1], "delta_var_z", same_sign=True)
    dw = F.conv2d_bwd_dw(t["var_w"], t["var_b"], t["mu_a"], t["delta_mu"], t["delta_var"],
                         ti["Fmwa_2"], B, fo, woho, wihi, fi, k)
    ref_dw = oracle_lib.conv2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], d["delta_mu"],
                                      d["delta_var"], idx["Fmwa_2"], B, fo, woho, wihi, fi, k,
                                      threads=4)
    for name, got, ref in zip(["delta_mu_w", "delta_var_w", "delta_mu_b", "delta_var_b"], dw,
                              ref_dw):
        assert_close(got.cpu().numpy(), ref, name, same_sign=name in SAME_SIGN)
    assert float(dz[1].max()) <= 0.0 and float(dw[1].max()) <= 0.0


def _same_padding_tables(k, wi, hi, pad_idx):
    """Index tables of a k x k, stride 1, (k-1)/2 padded convolution on a wi x hi map,
    in the reference's layout (the library's own builder makes square maps only)."""
    off, k2, n = (k - 1) // 2, k * k, wi * hi
    fm = np.full((n, k2), -1, np.int32)
    occ = [[] for _ in range(n)]
    for oy in range(hi):
        for ox in range(wi):
            for ky in range(k):
                for kx in range(k):
                    iy, ix = oy + ky - off, ox + kx - off
                    if 0 <= iy < hi and 0 <= ix < wi:
                        fm[oy * wi + ox, ky * k + kx] = iy * wi + ix + 1
                        occ[iy * wi + ix].append((ky * k + kx + 1, oy * wi + ox + 1))
    h = max(len(o) for o in occ)
    zw = np.full((n, h), pad_idx, np.int32)
    zud = np.full((h, n), -1, np.int32)
    for p, lst in enumerate(occ):
        for j, (tap, o) in enumerate(lst):
            zw[p, j], zud[j, p] = tap, o
    return dict(Fmwa_2=fm.ravel(), FCzwa_1=zw.ravel(), Szz_ud=zud.ravel(), h=h)


def test_same_padding_tables_helper_matches_the_builder():
    from cutagi_amd import capi
    a = _same_padding_tables(3, 8, 8, 999)
    b = capi.conv2d_build_idx(3, 1, 8, 8, 1, 1, 999)
    assert all(np.array_equal(a[k], b[k]) for k in ("Fmwa_2", "FCzwa_1", "Szz_ud")) and a["h"] == b["h"]


@pytest.mark.parametrize("wi,hi", [(16, 64), (64, 16)])
def test_conv2d_tables_of_another_geometry_take_the_table_path(oracle_lib, wi, hi):
    """1024 pixels per map are taken for a 32 x 32 map by the launcher; the kernels
    check the tables they are given and fall back to the table-driven loop when
    these describe something else (here a 16 x 64 / 64 x 16 map)."""
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, fi, fo, B = 3, 64, 64, 2
    idx = _same_padding_tables(k, wi, hi, k * k * fi * fo + 1)
    assert wi * hi == 1024 and idx["h"] == 9
    d = conv_inputs(fi, fo, k, 1024, 1024, B, seed=wi, bias=False, jcb_random=True)
    t = {n: (None if v is None else torch.from_numpy(v).cuda()) for n, v in d.items()}
    ti = {n: torch.from_numpy(idx[n]).cuda() for n in ("Fmwa_2", "FCzwa_1", "Szz_ud")}
    mu_z, var_z = F.conv2d_fwd(t["mu_w"], t["var_w"], None, None, t["mu_a"], t["var_a"],
                               ti["Fmwa_2"], 1024, fo, 1024, fi, k, B)
    ref = oracle_lib.conv2d_fwd(d["mu_w"], d["var_w"], None, None, d["mu_a"], d["var_a"],
                                idx["Fmwa_2"], 1024, fo, 1024, fi, k, B, threads=4)
    assert_close(mu_z.cpu().numpy(), ref[0], "mu_z")
    assert_close(var_z.cpu().numpy(), ref[1], "var_z", same_sign=True)
    dz = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"], ti["FCzwa_1"],
                         ti["Szz_ud"], 1024, fo, 1024, fi, k, idx["h"], B)
    ref_dz = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                      idx["FCzwa_1"], idx["Szz_ud"], 1024, fo, 1024, fi, k,
                                      idx["h"], B, threads=4)
    assert_close(dz[0].cpu().numpy(), ref_dz[0], "delta_mu_z")
    assert_close(dz[1].cpu().numpy(), ref_dz[1], "delta_var_z", same_sign=True)
    dw = F.conv2d_bwd_dw(t["var_w"], None, t["mu_a"], t["delta_mu"], t["delta_var"],
                         ti["Fmwa_2"], B, fo, 1024, 1024, fi, k)
    ref_dw = oracle_lib.conv2d_bwd_dw(d["var_w"], None, d["mu_a"], d["delta_mu"], d["delta_var"],
                                      idx["Fmwa_2"], B, fo, 1024, 1024, fi, k, threads=4)
    assert_close(dw[0].cpu().numpy(), ref_dw[0], "delta_mu_w")
    assert_close(dw[1].cpu().numpy(), ref_dw[1], "delta_var_w", same_sign=True)


def test_conv2d_stencil_kernels_agree_with_the_table_path():
    """Same inputs through the regular-stencil kernels and, with them switched off,
    through the table-driven kernels."""
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, wi, fi, fo, B = 3, 16, 64, 64, 8
    idx = capi.conv2d_build_idx(k, 1, wi, wi, 1, 1, k * k * fi * fo + 1)
    d = conv_inputs(fi, fo, k, wi * wi, wi * wi, B, seed=1, bias=True, jcb_random=True)
    t = {n: torch.from_numpy(v).cuda() for n, v in d.items()}
    ti = {n: torch.from_numpy(idx[n]).cuda() for n in ("Fmwa_2", "FCzwa_1", "Szz_ud")}
    out = {}
    try:
        for mode in (1, 0):
            capi.tune("conv2d.stencil", mode)
            z = F.conv2d_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"],
                             ti["Fmwa_2"], wi * wi, fo, wi * wi, fi, k, B)
            dz = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"], ti["FCzwa_1"],
                                 ti["Szz_ud"], wi * wi, fo, wi * wi, fi, k, idx["h"], B)
            dw = F.conv2d_bwd_dw(t["var_w"], t["var_b"], t["mu_a"], t["delta_mu"], t["delta_var"],
                                 ti["Fmwa_2"], B, fo, wi * wi, wi * wi, fi, k)
            out[mode] = [x.cpu().numpy() for x in (*z, *dz, *dw[:2])]
    finally:
        capi.tune("conv2d.stencil", 1)
    for name, a, b in zip(("mu_z", "var_z", "delta_mu_z", "delta_var_z", "delta_mu_w",
                           "delta_var_w"), out[1], out[0]):
        assert_close(a, b, name, same_sign=name in SAME_SIGN)
        # the two paths sum in different orders: identical bits would mean that the
        # switch did not switch
        assert not np.array_equal(a, b), name


def test_conv2d_strided_stencil_kernels_agree_with_the_table_path():
    """3x3 stride 2: the same inputs with the stencil kernels on (the state backward has
    one) and, with them switched off, through the table-driven kernels."""
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, wi, fi, fo, B = 3, 16, 64, 64, 4
    idx = capi.conv2d_build_idx(k, 2, wi, wi, 1, 2, k * k * fi * fo + 1)
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=2, bias=True, jcb_random=True)
    t = {n: torch.from_numpy(v).cuda() for n, v in d.items()}
    ti = {n: torch.from_numpy(idx[n]).cuda() for n in ("Fmwa_2", "FCzwa_1", "Szz_ud")}
    out = {}
    try:
        for mode in (1, 0):
            capi.tune("conv2d.stencil", mode)
            z = F.conv2d_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"],
                             ti["Fmwa_2"], woho, fo, wihi, fi, k, B)
            dz = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"], ti["FCzwa_1"],
                                 ti["Szz_ud"], woho, fo, wihi, fi, k, idx["h"], B)
            dw = F.conv2d_bwd_dw(t["var_w"], t["var_b"], t["mu_a"], t["delta_mu"], t["delta_var"],
                                 ti["Fmwa_2"], B, fo, woho, wihi, fi, k)
            out[mode] = [x.cpu().numpy() for x in (*z, *dz, *dw[:2])]
    finally:
        capi.tune("conv2d.stencil", 1)
    switched = []
    for name, a, b in zip(("mu_z", "var_z", "delta_mu_z", "delta_var_z", "delta_mu_w",
                           "delta_var_w"), out[1], out[0]):
        assert_close(a, b, name, same_sign=name in SAME_SIGN)
        if not np.array_equal(a, b):
            switched.append(name)
    # a different summation order shows that the switch switched all three passes
    assert "delta_mu_z" in switched and "mu_z" in switched and "delta_mu_w" in switched


@pytest.mark.parametrize("k,pad,pt", [(3, 1, 2), (2, 0, 1)])
def test_conv2d_strided_weight_backward_with_an_altered_table_takes_the_table_path(oracle_lib, k,
                                                                                   pad, pt):
    """The same for the weight backward (64 input and output channels, whole 64-pixel
    k-tiles): with one entry of Fmwa_2 altered, the slices that see it run the
    table-driven loop; with the table intact the stencil kernel gives the oracle's result
    in another summation order than the table-driven kernel."""
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    wi, fi, fo, B = 16, 64, 64, 3
    idx = capi.conv2d_build_idx(k, 2, wi, wi, pad, pt, k * k * fi * fo + 1)
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    table = idx["Fmwa_2"].copy()
    table[21 * k * k + 1] = 7
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=13, bias=True, jcb_random=True)
    t = {n: (None if v is None else torch.from_numpy(v).cuda()) for n, v in d.items()}
    for tab in (table, idx["Fmwa_2"]):
        dw = F.conv2d_bwd_dw(t["var_w"], t["var_b"], t["mu_a"], t["delta_mu"], t["delta_var"],
                             torch.from_numpy(tab).cuda(), B, fo, woho, wihi, fi, k)
        ref = oracle_lib.conv2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], d["delta_mu"],
                                       d["delta_var"], tab, B, fo, woho, wihi, fi, k, threads=4)
        assert_close(dw[0].cpu().numpy(), ref[0], "delta_mu_w")
        assert_close(dw[1].cpu().numpy(), ref[1], "delta_var_w", same_sign=True)
    capi.tune("conv2d.stencil", 0)
    try:
        off = F.conv2d_bwd_dw(t["var_w"], t["var_b"], t["mu_a"], t["delta_mu"], t["delta_var"],
                              torch.from_numpy(idx["Fmwa_2"]).cuda(), B, fo, woho, wihi, fi, k)
    finally:
        capi.tune("conv2d.stencil", 1)
    assert not np.array_equal(off[0].cpu().numpy(), dw[0].cpu().numpy())


@pytest.mark.parametrize("k,pad,pt", [(3, 1, 2), (2, 0, 1)])
def test_conv2d_strided_forward_with_an_altered_table_takes_the_table_path(oracle_lib, k, pad, pt):
    """The strided forward stencil is chosen by sizes and checks the table it is given.
    One entry of Fmwa_2 is pointed at another input pixel: the tile that owns it runs the
    table-driven loop, and the result is what the table says."""
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    wi, fi, fo, B = 16, 32, 64, 3
    idx = capi.conv2d_build_idx(k, 2, wi, wi, pad, pt, k * k * fi * fo + 1)
    wihi, woho = wi * wi, idx["wo"] * idx["ho"]
    table = idx["Fmwa_2"].copy()
    table[21 * k * k + 1] = 7          # output pixel 21, tap 1: reads input pixel 7 instead
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=12, bias=True, jcb_random=True)
    t = {n: (None if v is None else torch.from_numpy(v).cuda()) for n, v in d.items()}
    z = F.conv2d_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"],
                     torch.from_numpy(table).cuda(), woho, fo, wihi, fi, k, B)
    ref = oracle_lib.conv2d_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"], d["var_a"],
                                table, woho, fo, wihi, fi, k, B, threads=4)
    assert_close(z[0].cpu().numpy(), ref[0], "mu_z")
    assert_close(z[1].cpu().numpy(), ref[1], "var_z", same_sign=True)
    clean = oracle_lib.conv2d_fwd(d["mu_w"], d["var_w"], d["mu_b"], d["var_b"], d["mu_a"],
                                  d["var_a"], idx["Fmwa_2"], woho, fo, wihi, fi, k, B, threads=4)
    assert not np.array_equal(clean[0], ref[0])


@pytest.mark.parametrize("geom", [(3, 2, 1, 2, 32, 64, 64, 1), (3, 2, 1, 2, 16, 128, 96, 2),
                                  (3, 2, 1, 2, 8, 64, 160, 8), (3, 2, 1, 2, 16, 64, 640, 2),
                                  (2, 2, 0, 1, 16, 64, 96, 2)])
def test_conv2d_strided_state_backward_kernels_agree(oracle_lib, geom):
    """The stride-2 state backward on its stencil kernel (one workgroup for all four
    phases of a pixel block; default) and on the table-driven kernel, switched off either
    by its own switch or with all stencil kernels. All give the oracle's result, and the
    stencil kernel differs from the table-driven one in its summation order."""
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, s, p, pt, wi, fi, fo, B = geom
    idx, d, t, ti, wihi, woho = _setup(oracle_lib, geom, False, seed=21)
    ref = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                   idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k, idx["h"],
                                   B, threads=4)
    got = {}
    try:
        for name, all_phase, stencil in (("all", 1, 1), ("own_switch", 0, 1), ("tables", 1, 0)):
            capi.tune("conv2d.s2_all", all_phase)
            capi.tune("conv2d.stencil", stencil)
            dz = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"], ti["FCzwa_1"],
                                 ti["Szz_ud"], woho, fo, wihi, fi, k, idx["h"], B)
            got[name] = (dz[0].cpu().numpy(), dz[1].cpu().numpy())
            assert_close(got[name][0], ref[0], "delta_mu_z (%s)" % name)
            assert_close(got[name][1], ref[1], "delta_var_z (%s)" % name, same_sign=True)
    finally:
        capi.tune("conv2d.s2_all", 1)
        capi.tune("conv2d.stencil", 1)
    assert not np.array_equal(got["all"][0], got["tables"][0])
    assert np.array_equal(got["own_switch"][0], got["tables"][0])


def test_conv2d_projection_tables_of_another_geometry_take_the_table_path(oracle_lib):
    """2x2 stride 2: every input pixel has one occurrence. One pixel's entry is pointed
    at another output pixel: the workgroup that owns it runs the table-driven loop for
    its four phase tiles, and the result is what the tables say."""
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, wi, fi, fo, B = 2, 16, 64, 32, 2
    idx = capi.conv2d_build_idx(k, 2, wi, wi, 0, 1, k * k * fi * fo + 1)
    wihi, woho, h = wi * wi, idx["wo"] * idx["ho"], idx["h"]
    assert h == 1
    zud = idx["Szz_ud"].copy()
    zud[41] = (zud[41] % woho) + 1
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=10, bias=False, jcb_random=True)
    t = {n: (None if v is None else torch.from_numpy(v).cuda()) for n, v in d.items()}
    dz = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"],
                         torch.from_numpy(idx["FCzwa_1"]).cuda(), torch.from_numpy(zud).cuda(),
                         woho, fo, wihi, fi, k, h, B)
    ref = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                   idx["FCzwa_1"], zud, woho, fo, wihi, fi, k, h, B, threads=4)
    assert_close(dz[0].cpu().numpy(), ref[0], "delta_mu_z")
    assert_close(dz[1].cpu().numpy(), ref[1], "delta_var_z", same_sign=True)
    clean = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                     idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k, h, B,
                                     threads=4)
    assert not np.array_equal(clean[0], ref[0])


def test_conv2d_strided_tables_of_another_geometry_take_the_table_path(oracle_lib):
    """The strided stencil kernel is chosen by sizes (3x3, four input pixels per output
    pixel, lists of four occurrences) and checks the tables it is given. Here the
    tables of the right geometry are altered: the first two occurrences of every
    pixel's list trade places (still the same contraction, which the check accepts in
    any order) and one pixel's list names a wrong output pixel (a different
    contraction, which sends that tile to the table-driven loop). The result must be
    what the tables say."""
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, wi, fi, fo, B = 3, 16, 64, 32, 2
    idx = capi.conv2d_build_idx(k, 2, wi, wi, 1, 2, k * k * fi * fo + 1)
    wihi, woho, h = wi * wi, idx["wo"] * idx["ho"], idx["h"]
    assert h == 4
    zw = idx["FCzwa_1"].reshape(wihi, h).copy()
    zud = idx["Szz_ud"].reshape(h, wihi).copy()
    # (a) reorder: swap the first two occurrences of every pixel that has two
    two = zud[1] > -1
    zw[two, 0], zw[two, 1] = zw[two, 1].copy(), zw[two, 0].copy()
    zud[0, two], zud[1, two] = zud[1, two].copy(), zud[0, two].copy()
    # (b) one wrong entry: pixel 37 takes its first tap from another output pixel
    zud[0, 37] = (zud[0, 37] % woho) + 1
    d = conv_inputs(fi, fo, k, wihi, woho, B, seed=9, bias=False, jcb_random=True)
    t = {n: (None if v is None else torch.from_numpy(v).cuda()) for n, v in d.items()}
    zw_f, zud_f = np.ascontiguousarray(zw.ravel()), np.ascontiguousarray(zud.ravel())
    dz = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"],
                         torch.from_numpy(zw_f).cuda(), torch.from_numpy(zud_f).cuda(), woho, fo,
                         wihi, fi, k, h, B)
    ref = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"], zw_f, zud_f,
                                   woho, fo, wihi, fi, k, h, B, threads=4)
    assert_close(dz[0].cpu().numpy(), ref[0], "delta_mu_z")
    assert_close(dz[1].cpu().numpy(), ref[1], "delta_var_z", same_sign=True)
    # and the corruption did change the contraction
    clean = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                     idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k, h, B,
                                     threads=4)
    assert not np.array_equal(clean[0], ref[0])


@pytest.mark.parametrize("geom", [(3, 2, 1, 2, 16, 16, 64, 4), (2, 2, 0, 1, 8, 64, 32, 3),
                                  (3, 2, 1, 2, 4, 8, 8, 2), (3, 2, 1, 2, 16, 64, 64, 2)])
def test_conv2d_state_backward_column_orders_agree(oracle_lib, geom):
    """Strided layers: columns numbered phase by phase (default) and in natural
    order give the oracle's result both; the order only decides which taps a tile
    can skip."""
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, s, p, pt, wi, fi, fo, B = geom
    idx, d, t, ti, wihi, woho = _setup(oracle_lib, geom, False, seed=7)
    ref = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                   idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k, idx["h"],
                                   B, threads=4)
    try:
        for mode in (1, 0):
            capi.tune("conv2d.phase_order", mode)
            dz = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"], ti["FCzwa_1"],
                                 ti["Szz_ud"], woho, fo, wihi, fi, k, idx["h"], B)
            assert_close(dz[0].cpu().numpy(), ref[0], "delta_mu_z order %d" % mode)
            assert_close(dz[1].cpu().numpy(), ref[1], "delta_var_z order %d" % mode, same_sign=True)
    finally:
        capi.tune("conv2d.phase_order", 1)


def test_conv2d_kernel_too_large_for_the_tap_table_is_refused():
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, wi, fi, fo, B = 11, 12, 1, 2, 1
    idx = capi.conv2d_build_idx(k, 1, wi, wi, 0, 1, k * k * fi * fo + 1)
    woho = idx["wo"] * idx["ho"]
    z = lambda n: torch.zeros(n, device="cuda")
    with pytest.raises(capi.TagiHipError):
        F.conv2d_fwd(z(fo * fi * k * k), z(fo * fi * k * k), None, None, z(B * fi * wi * wi),
                     z(B * fi * wi * wi), torch.from_numpy(idx["Fmwa_2"]).cuda(), woho, fo,
                     wi * wi, fi, k, B)


# stencil kernel, table-driven strided kernel (phase order), sliced reduction
RES_GEOMS = [(3, 1, 1, 1, 8, 64, 64, 3), (3, 2, 1, 2, 8, 8, 16, 4), (3, 1, 1, 1, 4, 128, 96, 3),
             (3, 1, 1, 1, 6, 5, 7, 2), (3, 2, 1, 2, 16, 64, 64, 2)]


@pytest.mark.parametrize("geom", RES_GEOMS)
@pytest.mark.parametrize("mode", [1, 2])
def test_conv2d_state_backward_with_residual(oracle_lib, geom, mode):
    """tagi_conv2d_bwd_dz_res: mode 1 = (sum + res) .* jcb (identity shortcut), mode 2 =
    sum .* jcb + res (a shortcut branch's finished innovations)."""
    import torch
    from cutagi_amd import capi
    k, s, p, pt, wi, fi, fo, B = geom
    idx, d, t, ti, wihi, woho = _setup(oracle_lib, geom, False, seed=sum(geom) + mode)
    rng = np.random.default_rng(sum(geom))
    n_in = B * fi * wihi
    res_mu = rng.normal(0, 0.1, n_in).astype(np.float32)
    res_var = (-rng.uniform(0, 1e-3, n_in)).astype(np.float32)
    ref = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                   idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k, idx["h"],
                                   B, 4)
    if mode == 1:
        want = oracle_lib.add_shortcut_delta(res_mu, res_var, d["jcb"], ref[0].ravel(), ref[1].ravel())
    else:
        want = oracle_lib.add_shortcut(res_mu, res_var, ref[0].ravel(), ref[1].ravel())
    r_mu, r_var = torch.from_numpy(res_mu).cuda(), torch.from_numpy(res_var).cuda()
    om, ov = torch.empty(n_in, device="cuda"), torch.empty(n_in, device="cuda")
    capi.check(capi.lib.tagi_conv2d_bwd_dz_res(
        capi.ptr(t["mu_w"]), capi.ptr(t["jcb"]), capi.ptr(t["delta_mu"]), capi.ptr(t["delta_var"]),
        capi.ptr(ti["FCzwa_1"]), capi.ptr(ti["Szz_ud"]), woho, fo, wihi, fi, k, idx["h"], B,
        capi.ptr(r_mu), capi.ptr(r_var), mode, capi.ptr(om), capi.ptr(ov), None))
    torch.cuda.synchronize()
    assert_close(om.cpu().numpy(), want[0], "delta_mu_z + residual")
    assert_close(ov.cpu().numpy(), want[1], "delta_var_z + residual", same_sign=True)


# eligible for the shared launch (3x3 s1 p1, whole groups of 64 channels, whole 64-pixel
# k-tiles), sliced state backward, and shapes that fall back to two launches
PAIR_GEOMS = [(3, 1, 1, 1, 16, 64, 64, 4), (3, 1, 1, 1, 32, 64, 64, 2), (3, 1, 1, 1, 8, 128, 64, 3),
              (3, 1, 1, 1, 4, 320, 128, 8), (3, 1, 1, 1, 4, 320, 64, 5), (3, 2, 1, 2, 16, 64, 64, 4),
              (2, 2, 0, 1, 8, 64, 130, 2), (3, 1, 1, 1, 8, 4, 8, 3)]


@pytest.mark.parametrize("geom", PAIR_GEOMS)
@pytest.mark.parametrize("res_mode", [0, 1, 2])
def test_conv2d_backward_in_one_call(oracle_lib, geom, res_mode):
    """tagi_conv2d_bwd against the oracle and, bit for bit, against the separate entry
    points (same kernels, whether they share a launch or not); with and without a
    residual, with the parts switched off one at a time."""
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    k, s, p, pt, wi, fi, fo, B = geom
    idx, d, t, ti, wihi, woho = _setup(oracle_lib, geom, True, seed=31 + res_mode)
    rng = np.random.default_rng(5)
    res = None
    if res_mode:
        res = [torch.from_numpy((rng.standard_normal(B * fi * wihi) * 0.1).astype(np.float32)).cuda(),
               torch.from_numpy(rng.uniform(0, 1e-3, B * fi * wihi).astype(np.float32)).cuda()]
    args = (t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"], t["delta_mu"], t["delta_var"],
            ti["Fmwa_2"], ti["FCzwa_1"], ti["Szz_ud"], B, fo, woho, wihi, fi, k, idx["h"])
    kw = dict(res_mu=res[0] if res else None, res_var=res[1] if res else None, res_mode=res_mode)
    got = F.conv2d_bwd(*args, **kw)
    # the separate entry points
    dw = F.conv2d_bwd_dw(t["var_w"], t["var_b"], t["mu_a"], t["delta_mu"], t["delta_var"],
                         ti["Fmwa_2"], B, fo, woho, wihi, fi, k)
    zm, zv = torch.empty(B * fi * wihi, device="cuda"), torch.empty(B * fi * wihi, device="cuda")
    if res_mode:
        capi.check(capi.lib.tagi_conv2d_bwd_dz_res(
            capi.ptr(t["mu_w"]), capi.ptr(t["jcb"]), capi.ptr(t["delta_mu"]), capi.ptr(t["delta_var"]),
            capi.ptr(ti["FCzwa_1"]), capi.ptr(ti["Szz_ud"]), woho, fo, wihi, fi, k, idx["h"], B,
            capi.ptr(res[0]), capi.ptr(res[1]), res_mode, capi.ptr(zm), capi.ptr(zv),
            torch.cuda.current_stream().cuda_stream))
    else:
        zm, zv = F.conv2d_bwd_dz(t["mu_w"], t["jcb"], t["delta_mu"], t["delta_var"], ti["FCzwa_1"],
                                 ti["Szz_ud"], woho, fo, wihi, fi, k, idx["h"], B)
    for name, a, b in zip(("delta_mu_z", "delta_var_z", "delta_mu_w", "delta_var_w", "delta_mu_b",
                           "delta_var_b"), got, (zm, zv) + tuple(dw)):
        assert torch.equal(a, b), name
    # the oracle (the residual is applied as ConvDz does: before or after the Jacobian)
    ref = oracle_lib.conv2d_bwd_dz(d["mu_w"], d["jcb"], d["delta_mu"], d["delta_var"],
                                   idx["FCzwa_1"], idx["Szz_ud"], woho, fo, wihi, fi, k, idx["h"],
                                   B, threads=4)
    if res_mode == 0:
        assert_close(got[0].cpu().numpy(), ref[0], "delta_mu_z")
        assert_close(got[1].cpu().numpy(), ref[1], "delta_var_z", same_sign=True)
    rw = oracle_lib.conv2d_bwd_dw(d["var_w"], d["var_b"], d["mu_a"], d["delta_mu"], d["delta_var"],
                                  idx["Fmwa_2"], B, fo, woho, wihi, fi, k, threads=4)
    assert_close(got[2].cpu().numpy(), rw[0], "delta_mu_w")
    assert_close(got[3].cpu().numpy(), rw[1], "delta_var_w", same_sign=True)
    # parts switched off
    only_w = F.conv2d_bwd(*args, state_update=False)
    assert only_w[0] is None and torch.equal(only_w[2], got[2]) and torch.equal(only_w[4], got[4])
    only_z = F.conv2d_bwd(*args, param_update=False, **kw)
    assert only_z[2] is None and torch.equal(only_z[0], got[0]) and torch.equal(only_z[1], got[1])


def test_conv2d_backward_pair_launch_can_be_switched_off(oracle_lib):
    """"conv2d.bwd_pair" = 0 gives two launches; the results are the same bits."""
    import torch
    import cutagi_amd.functional as F
    from cutagi_amd import capi
    geom = (3, 1, 1, 1, 16, 64, 128, 4)
    k, s, p, pt, wi, fi, fo, B = geom
    idx, d, t, ti, wihi, woho = _setup(oracle_lib, geom, False, seed=40)
    args = (t["mu_w"], t["var_w"], None, t["mu_a"], t["jcb"], t["delta_mu"], t["delta_var"],
            ti["Fmwa_2"], ti["FCzwa_1"], ti["Szz_ud"], B, fo, woho, wihi, fi, k, idx["h"])
    a = F.conv2d_bwd(*args)
    capi.tune("conv2d.bwd_pair", 0)
    try:
        b = F.conv2d_bwd(*args)
    finally:
        capi.tune("conv2d.bwd_pair", 1)
    for x, y in zip(a[:4], b[:4]):
        assert torch.equal(x, y)
