"""Tensor-level calls into the C ABI.

torch is plumbing here: it owns device memory and the current stream; every
computation is one C-ABI call on raw pointers. Shapes follow the reference:
weights [N, K], activations [B, K], conv weights [fo, fi*k*k], conv activations
flattened NCHW.
"""
import torch

from . import capi


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _chk(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not (t.is_cuda and t.is_contiguous() and t.dtype in (torch.float32, torch.int32)):
            raise ValueError("expected contiguous fp32/int32 device tensors")


def linear_fwd(mu_w, var_w, mu_b, var_b, mu_a, var_a, out=None):
    _chk(mu_w, var_w, mu_b, var_b, mu_a, var_a)
    N, K = mu_w.shape
    B = mu_a.shape[0]
    if mu_a.shape[1] != K:
        raise ValueError("Input size mismatch: %d vs %d" % (K, mu_a.shape[1]))
    mu_z, var_z = out if out is not None else (torch.empty((B, N), device=mu_w.device),
                                                torch.empty((B, N), device=mu_w.device))
    bias = mu_b is not None
    capi.check(capi.lib.tagi_linear_fwd(capi.ptr(mu_w), capi.ptr(var_w), capi.ptr(mu_b),
                                        capi.ptr(var_b), capi.ptr(mu_a), capi.ptr(var_a), K, N, B,
                                        int(bias), capi.ptr(mu_z), capi.ptr(var_z), _stream()))
    return mu_z, var_z


ACTIVATIONS = {"relu": 1, "mixture_relu": 2}


def linear_fwd_act(mu_w, var_w, mu_b, var_b, mu_a, var_a, activation):
    """Linear forward with the following activation ("relu" / "mixture_relu") applied
    in the kernel's epilogue: returns the activation's (mu_a, var_a, jcb)."""
    _chk(mu_w, var_w, mu_b, var_b, mu_a, var_a)
    N, K = mu_w.shape
    B = mu_a.shape[0]
    out = [torch.empty((B, N), device=mu_w.device) for _ in range(3)]
    capi.check(capi.lib.tagi_linear_fwd_act(capi.ptr(mu_w), capi.ptr(var_w), capi.ptr(mu_b),
                                            capi.ptr(var_b), capi.ptr(mu_a), capi.ptr(var_a), K, N,
                                            B, int(mu_b is not None), ACTIVATIONS[activation],
                                            capi.ptr(out[0]), capi.ptr(out[1]), capi.ptr(out[2]),
                                            _stream()))
    return tuple(out)


def linear_bwd_dz(mu_w, jcb, delta_mu, delta_var, out=None):
    _chk(mu_w, jcb, delta_mu, delta_var)
    N, K = mu_w.shape
    B = delta_mu.shape[0]
    om, ov = out if out is not None else (torch.empty((B, K), device=mu_w.device),
                                          torch.empty((B, K), device=mu_w.device))
    capi.check(capi.lib.tagi_linear_bwd_dz(capi.ptr(mu_w), capi.ptr(jcb), capi.ptr(delta_mu),
                                           capi.ptr(delta_var), K, N, B, capi.ptr(om),
                                           capi.ptr(ov), _stream()))
    return om, ov


def linear_bwd_dw(var_w, mu_a, delta_mu, delta_var, out=None):
    _chk(var_w, mu_a, delta_mu, delta_var)
    N, K = var_w.shape
    B = delta_mu.shape[0]
    om, ov = out if out is not None else (torch.empty((N, K), device=var_w.device),
                                          torch.empty((N, K), device=var_w.device))
    capi.check(capi.lib.tagi_linear_bwd_dw(capi.ptr(var_w), capi.ptr(mu_a), capi.ptr(delta_mu),
                                           capi.ptr(delta_var), K, N, B, capi.ptr(om),
                                           capi.ptr(ov), _stream()))
    return om, ov


def linear_bwd_db(var_b, delta_mu, delta_var, out=None):
    _chk(var_b, delta_mu, delta_var)
    B, N = delta_mu.shape
    om, ov = out if out is not None else (torch.empty(N, device=var_b.device),
                                          torch.empty(N, device=var_b.device))
    capi.check(capi.lib.tagi_linear_bwd_db(capi.ptr(var_b), capi.ptr(delta_mu),
                                           capi.ptr(delta_var), N, B, capi.ptr(om), capi.ptr(ov),
                                           _stream()))
    return om, ov


def linear_bwd(mu_w, var_w, var_b, mu_a, jcb, delta_mu, delta_var, state_update=True,
               param_update=True, out=None):
    """All of LinearCuda::backward in one call. Returns (dz_mu, dz_var, dw_mu,
    dw_var, db_mu, db_var); entries not asked for are None."""
    _chk(mu_w, var_w, var_b, mu_a, jcb, delta_mu, delta_var)
    N, K = mu_w.shape
    B = delta_mu.shape[0]
    dev = mu_w.device
    bias = var_b is not None
    if out is None:
        out = [None] * 6
        if state_update:
            out[0], out[1] = torch.empty((B, K), device=dev), torch.empty((B, K), device=dev)
        if param_update:
            out[2], out[3] = torch.empty((N, K), device=dev), torch.empty((N, K), device=dev)
            if bias:
                out[4], out[5] = torch.empty(N, device=dev), torch.empty(N, device=dev)
    capi.check(capi.lib.tagi_linear_bwd(
        capi.ptr(mu_w), capi.ptr(var_w), capi.ptr(var_b), capi.ptr(mu_a), capi.ptr(jcb),
        capi.ptr(delta_mu), capi.ptr(delta_var), K, N, B, int(bias), int(state_update),
        int(param_update), *[capi.ptr(t) for t in out], _stream()))
    return tuple(out)


def conv2d_fwd(mu_w, var_w, mu_b, var_b, mu_a, var_a, aidx, woho, fo, wihi, fi, ki, B):
    _chk(mu_w, var_w, mu_b, var_b, mu_a, var_a, aidx)
    mu_z = torch.empty(B * fo * woho, device=mu_w.device)
    var_z = torch.empty(B * fo * woho, device=mu_w.device)
    bias = mu_b is not None
    capi.check(capi.lib.tagi_conv2d_fwd(capi.ptr(mu_w), capi.ptr(var_w), capi.ptr(mu_b),
                                        capi.ptr(var_b), capi.ptr(mu_a), capi.ptr(var_a),
                                        capi.ptr(aidx), woho, fo, wihi, fi, ki, B, int(bias),
                                        capi.ptr(mu_z), capi.ptr(var_z), _stream()))
    return mu_z, var_z


def conv2d_fwd_act(mu_w, var_w, mu_b, var_b, mu_a, var_a, aidx, woho, fo, wihi, fi, ki, B,
                   activation):
    """Conv2d forward with the following activation applied in the kernel's epilogue:
    returns the activation's (mu_a, var_a, jcb), each [B][fo][woho] flattened."""
    _chk(mu_w, var_w, mu_b, var_b, mu_a, var_a, aidx)
    out = [torch.empty(B * fo * woho, device=mu_w.device) for _ in range(3)]
    capi.check(capi.lib.tagi_conv2d_fwd_act(capi.ptr(mu_w), capi.ptr(var_w), capi.ptr(mu_b),
                                            capi.ptr(var_b), capi.ptr(mu_a), capi.ptr(var_a),
                                            capi.ptr(aidx), woho, fo, wihi, fi, ki, B,
                                            int(mu_b is not None), ACTIVATIONS[activation],
                                            capi.ptr(out[0]), capi.ptr(out[1]), capi.ptr(out[2]),
                                            _stream()))
    return tuple(out)


def conv2d_bwd_dz(mu_w, jcb, delta_mu, delta_var, zw_idx, zud_idx, woho, fo, wihi, fi, ki, nr, B):
    _chk(mu_w, jcb, delta_mu, delta_var, zw_idx, zud_idx)
    om = torch.empty(B * fi * wihi, device=mu_w.device)
    ov = torch.empty(B * fi * wihi, device=mu_w.device)
    capi.check(capi.lib.tagi_conv2d_bwd_dz(capi.ptr(mu_w), capi.ptr(jcb), capi.ptr(delta_mu),
                                           capi.ptr(delta_var), capi.ptr(zw_idx),
                                           capi.ptr(zud_idx), woho, fo, wihi, fi, ki, nr, B,
                                           capi.ptr(om), capi.ptr(ov), _stream()))
    return om, ov


def conv2d_bwd_dw(var_w, var_b, mu_a, delta_mu, delta_var, aidx, B, fo, woho, wihi, fi, ki):
    _chk(var_w, var_b, mu_a, delta_mu, delta_var, aidx)
    nw = ki * ki * fi * fo
    dev = var_w.device
    om, ov = torch.empty(nw, device=dev), torch.empty(nw, device=dev)
    bias = var_b is not None
    bm = torch.empty(fo, device=dev) if bias else None
    bv = torch.empty(fo, device=dev) if bias else None
    capi.check(capi.lib.tagi_conv2d_bwd_dw(capi.ptr(var_w), capi.ptr(var_b), capi.ptr(mu_a),
                                           capi.ptr(delta_mu), capi.ptr(delta_var),
                                           capi.ptr(aidx), B, fo, woho, wihi, fi, ki, int(bias),
                                           capi.ptr(om), capi.ptr(ov), capi.ptr(bm), capi.ptr(bv),
                                           _stream()))
    return om, ov, bm, bv


def conv2d_bwd(mu_w, var_w, var_b, mu_a, jcb, delta_mu, delta_var, aidx, zw_idx, zud_idx, B, fo,
               woho, wihi, fi, ki, nr, state_update=True, param_update=True, res_mu=None,
               res_var=None, res_mode=0):
    """Both backward contractions in one call: (delta_mu_z, delta_var_z, delta_mu_w,
    delta_var_w, delta_mu_b, delta_var_b), None where a part is switched off."""
    _chk(mu_w, var_w, var_b, mu_a, jcb, delta_mu, delta_var, aidx, zw_idx, zud_idx, res_mu, res_var)
    dev = mu_w.device
    nw = ki * ki * fi * fo
    bias = var_b is not None
    zm = torch.empty(B * fi * wihi, device=dev) if state_update else None
    zv = torch.empty(B * fi * wihi, device=dev) if state_update else None
    wm = torch.empty(nw, device=dev) if param_update else None
    wv = torch.empty(nw, device=dev) if param_update else None
    bm = torch.empty(fo, device=dev) if bias and param_update else None
    bv = torch.empty(fo, device=dev) if bias and param_update else None
    capi.check(capi.lib.tagi_conv2d_bwd(
        capi.ptr(mu_w), capi.ptr(var_w), capi.ptr(var_b), capi.ptr(mu_a), capi.ptr(jcb),
        capi.ptr(delta_mu), capi.ptr(delta_var), capi.ptr(aidx), capi.ptr(zw_idx), capi.ptr(zud_idx),
        B, fo, woho, wihi, fi, ki, nr, int(bias), int(state_update), int(param_update),
        capi.ptr(res_mu), capi.ptr(res_var), res_mode, capi.ptr(zm), capi.ptr(zv), capi.ptr(wm),
        capi.ptr(wv), capi.ptr(bm), capi.ptr(bv), _stream()))
    return zm, zv, wm, wv, bm, bv


def store_states(mu_a, jcb, n_in, bwd_mu_a, bwd_jcb, out_jcb, n_out):
    capi.check(capi.lib.tagi_store_states(capi.ptr(mu_a), capi.ptr(jcb), n_in, capi.ptr(bwd_mu_a),
                                          capi.ptr(bwd_jcb), capi.ptr(out_jcb), n_out, _stream()))


def param_update(delta_mu, delta_var, cap_factor, mu, var, neg_var_count=None):
    """In place on mu/var. neg_var_count: int32 device tensor of one element."""
    _chk(delta_mu, delta_var, mu, var, neg_var_count)
    capi.check(capi.lib.tagi_param_update(capi.ptr(delta_mu), capi.ptr(delta_var), cap_factor,
                                          mu.numel(), capi.ptr(mu), capi.ptr(var),
                                          capi.ptr(neg_var_count), _stream()))



def layer_update(delta_mu_w, delta_var_w, mu_w, var_w, delta_mu_b, delta_var_b, mu_b, var_b,
                 cap_factor, neg_var_count=None, slot=0):
    """Weights and biases of a layer in one launch, in place. Bias tensors may be
    None. neg_var_count: int32 device tensor of two elements (counts go to [slot],
    [1 - slot] is zeroed)."""
    _chk(delta_mu_w, delta_var_w, mu_w, var_w, delta_mu_b, delta_var_b, mu_b, var_b, neg_var_count)
    nb = 0 if mu_b is None else mu_b.numel()
    capi.check(capi.lib.tagi_layer_update(
        capi.ptr(delta_mu_w), capi.ptr(delta_var_w), mu_w.numel(), capi.ptr(mu_w), capi.ptr(var_w),
        capi.ptr(delta_mu_b), capi.ptr(delta_var_b), nb, capi.ptr(mu_b), capi.ptr(var_b),
        cap_factor, capi.ptr(neg_var_count), int(slot), _stream()))

def out_update_dense(mu_a, var_a, jcb, obs, var_obs, delta_mu, delta_var):
    _chk(mu_a, var_a, jcb, obs, var_obs, delta_mu, delta_var)
    capi.check(capi.lib.tagi_out_update_dense(capi.ptr(mu_a), capi.ptr(var_a), capi.ptr(jcb),
                                              capi.ptr(obs), capi.ptr(var_obs), obs.numel(),
                                              capi.ptr(delta_mu), capi.ptr(delta_var), _stream()))


def out_update_heteros(mu_a, var_a, jcb, obs, delta_mu, delta_var):
    """obs.numel() observations against 2 * obs.numel() output units."""
    _chk(mu_a, var_a, jcb, obs, delta_mu, delta_var)
    capi.check(capi.lib.tagi_out_update_heteros(capi.ptr(mu_a), capi.ptr(var_a), capi.ptr(jcb),
                                                capi.ptr(obs), obs.numel(), capi.ptr(delta_mu),
                                                capi.ptr(delta_var), _stream()))


def out_update_indexed(mu_a, var_a, jcb, obs, var_obs, selected_idx, n_obs, n_enc, delta_mu,
                       delta_var):
    _chk(mu_a, var_a, jcb, obs, var_obs, selected_idx, delta_mu, delta_var)
    capi.check(capi.lib.tagi_out_update_indexed(capi.ptr(mu_a), capi.ptr(var_a), capi.ptr(jcb),
                                                capi.ptr(obs), capi.ptr(var_obs),
                                                capi.ptr(selected_idx), n_obs, n_enc, obs.numel(),
                                                capi.ptr(delta_mu), capi.ptr(delta_var),
                                                _stream()))


def relu_fwd(mu_z, var_z, mu_a=None, jcb=None, var_a=None):
    _chk(mu_z, var_z, mu_a, jcb, var_a)
    mu_a = torch.empty_like(mu_z) if mu_a is None else mu_a
    jcb = torch.empty_like(mu_z) if jcb is None else jcb
    var_a = torch.empty_like(mu_z) if var_a is None else var_a
    capi.check(capi.lib.tagi_relu_fwd(capi.ptr(mu_z), capi.ptr(var_z), mu_z.numel(),
                                      capi.ptr(mu_a), capi.ptr(jcb), capi.ptr(var_a), _stream()))
    return mu_a, var_a, jcb


def mixture_relu_fwd(mu_z, var_z, mu_a=None, jcb=None, var_a=None):
    _chk(mu_z, var_z, mu_a, jcb, var_a)
    mu_a = torch.empty_like(mu_z) if mu_a is None else mu_a
    jcb = torch.empty_like(mu_z) if jcb is None else jcb
    var_a = torch.empty_like(mu_z) if var_a is None else var_a
    capi.check(capi.lib.tagi_mixture_relu_fwd(capi.ptr(mu_z), capi.ptr(var_z), mu_z.numel(),
                                              capi.ptr(mu_a), capi.ptr(jcb), capi.ptr(var_a),
                                              _stream()))
    return mu_a, var_a, jcb


def batchnorm2d_stats(mu_a, var_a, wihi, fi, B, momentum, mu_ra, var_ra):
    """Batch statistics (returned) and the running averages (updated in place)."""
    _chk(mu_a, var_a, mu_ra, var_ra)
    mu_s, var_s = torch.empty(fi, device=mu_a.device), torch.empty(fi, device=mu_a.device)
    capi.check(capi.lib.tagi_batchnorm2d_stats(capi.ptr(mu_a), capi.ptr(var_a), wihi, fi, B,
                                               momentum, capi.ptr(mu_s), capi.ptr(var_s),
                                               capi.ptr(mu_ra), capi.ptr(var_ra), _stream()))
    return mu_s, var_s


def batchnorm2d_fwd(mu_w, var_w, mu_b, var_b, mu_a, var_a, mu_norm, var_norm, eps, wihi, fi, B):
    _chk(mu_w, var_w, mu_b, var_b, mu_a, var_a, mu_norm, var_norm)
    mu_z, var_z = torch.empty_like(mu_a), torch.empty_like(mu_a)
    capi.check(capi.lib.tagi_batchnorm2d_fwd(capi.ptr(mu_w), capi.ptr(var_w), capi.ptr(mu_b),
                                             capi.ptr(var_b), capi.ptr(mu_a), capi.ptr(var_a),
                                             capi.ptr(mu_norm), capi.ptr(var_norm),
                                             int(mu_b is not None), eps, wihi, fi, B,
                                             capi.ptr(mu_z), capi.ptr(var_z), _stream()))
    return mu_z, var_z


def batchnorm2d_bwd(mu_w, var_w, var_b, mu_a, jcb, mu_norm, var_norm, delta_mu, delta_var, eps,
                    wihi, fi, B, state_update=True, param_update=True):
    """Returns (dz_mu, dz_var, dw_mu, dw_var, db_mu, db_var); entries not asked for are None."""
    _chk(mu_w, var_w, var_b, mu_a, jcb, mu_norm, var_norm, delta_mu, delta_var)
    dev = mu_w.device
    bias = var_b is not None
    out = [None] * 6
    if state_update:
        out[0], out[1] = torch.empty_like(delta_mu), torch.empty_like(delta_mu)
    if param_update:
        out[2], out[3] = torch.empty(fi, device=dev), torch.empty(fi, device=dev)
        if bias:
            out[4], out[5] = torch.empty(fi, device=dev), torch.empty(fi, device=dev)
    capi.check(capi.lib.tagi_batchnorm2d_bwd(
        capi.ptr(mu_w), capi.ptr(var_w), capi.ptr(var_b), capi.ptr(mu_a), capi.ptr(jcb),
        capi.ptr(mu_norm), capi.ptr(var_norm), capi.ptr(delta_mu), capi.ptr(delta_var), eps, wihi,
        fi, B, int(bias), int(state_update), int(param_update), *[capi.ptr(t) for t in out],
        _stream()))
    return tuple(out)


def avgpool2d_fwd(mu_a, var_a, pool_idx, woho, wihi, ki, n_out):
    _chk(mu_a, var_a, pool_idx)
    mu_z, var_z = torch.empty(n_out, device=mu_a.device), torch.empty(n_out, device=mu_a.device)
    capi.check(capi.lib.tagi_avgpool2d_fwd(capi.ptr(mu_a), capi.ptr(var_a), capi.ptr(pool_idx),
                                           woho, wihi, ki, n_out, capi.ptr(mu_z), capi.ptr(var_z),
                                           _stream()))
    return mu_z, var_z


def avgpool2d_bwd_dz(jcb, delta_mu, delta_var, z_ud_idx, woho, wihi, ki, nr, wo, overlap):
    _chk(jcb, delta_mu, delta_var, z_ud_idx)
    om, ov = torch.empty_like(jcb), torch.empty_like(jcb)
    capi.check(capi.lib.tagi_avgpool2d_bwd_dz(capi.ptr(jcb), capi.ptr(delta_mu),
                                              capi.ptr(delta_var), capi.ptr(z_ud_idx), woho, wihi,
                                              ki, nr, wo, jcb.numel(), int(overlap), capi.ptr(om),
                                              capi.ptr(ov), _stream()))
    return om, ov


def add_shortcut(mu_s, var_s, mu_a, var_a):
    """In place on mu_a/var_a."""
    _chk(mu_s, var_s, mu_a, var_a)
    capi.check(capi.lib.tagi_add_shortcut(capi.ptr(mu_s), capi.ptr(var_s), mu_a.numel(),
                                          capi.ptr(mu_a), capi.ptr(var_a), _stream()))


def add_shortcut_delta(mu_s, var_s, jcb_s, mu_a, var_a):
    """In place on mu_a/var_a."""
    _chk(mu_s, var_s, jcb_s, mu_a, var_a)
    capi.check(capi.lib.tagi_add_shortcut_delta(capi.ptr(mu_s), capi.ptr(var_s), capi.ptr(jcb_s),
                                                mu_a.numel(), capi.ptr(mu_a), capi.ptr(var_a),
                                                _stream()))
