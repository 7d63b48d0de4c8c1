"""Calls on two streams of one device at the same time: every stream owns its
scratch memory, so sliced reductions that overlap in time do not mix partial sums."""
import numpy as np
import pytest

from util import linear_inputs

pytestmark = pytest.mark.gpu


def test_sliced_launches_on_two_streams_do_not_share_partial_sums():
    import torch
    import cutagi_amd.functional as F
    shapes = [(2048, 256, 64), (4096, 192, 48)]   # both forward passes are sliced
    data = [{k: (None if v is None else torch.from_numpy(v).cuda())
             for k, v in linear_inputs(K, N, B, seed=K + B).items()} for K, N, B in shapes]
    fwd = lambda t: F.linear_fwd(t["mu_w"], t["var_w"], t["mu_b"], t["var_b"], t["mu_a"], t["var_a"])
    bwd = lambda t: F.linear_bwd(t["mu_w"], t["var_w"], t["var_b"], t["mu_a"], t["jcb"],
                                 t["delta_mu"], t["delta_var"])
    want = [[x.clone() for x in fwd(t) + tuple(bwd(t))] for t in data]   # one at a time
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for _ in range(20):
        got = [None, None]
        for _rep in range(4):       # interleave: both streams have work queued at once
            for i, (s, t) in enumerate(zip(streams, data)):
                with torch.cuda.stream(s):
                    got[i] = fwd(t) + tuple(bwd(t))
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            for a, b in zip(g, w):
                assert torch.equal(a, b)     # deterministic kernels: same bits


def test_device_info_reports_the_part():
    from cutagi_amd import capi
    cus, mhz, name = capi.device_info()
    assert cus > 0 and mhz > 0 and name
