"""ctypes front end of the CPU oracle (TEST INFRASTRUCTURE ONLY).

`load()` returns a thin numpy wrapper over ``oracle/liboracle.so`` (this repo's
restatement of the reference CPU algorithms, built by ``oracle/Makefile``);
`load_ref()` returns the same wrapper over ``oracle/_ref/libtagi_ref.so`` (the
reference's own sources compiled in place) or ``None`` when that library was not
built. Only tests, the smoke test and the benchmark's CPU-baseline leg may
import this package; the shipped library never does.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_F = ctypes.POINTER(ctypes.c_float)
_I = ctypes.POINTER(ctypes.c_int)


def _fp(a):
    if a is None:
        return ctypes.cast(None, _F)
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_F)


def _ip(a):
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(_I)


def f32(x):
    return np.ascontiguousarray(x, dtype=np.float32)


def build(ref=False):
    """Compile liboracle.so (and, with ref=True, _ref/libtagi_ref.so)."""
    targets = ["all"] + (["ref"] if ref else [])
    subprocess.run(["make", "-C", _HERE, "-j8"] + targets, check=True,
                   stdout=subprocess.DEVNULL)


class Oracle:
    """Numpy-in / numpy-out calls; `prefix` selects oracle_* or ref_* symbols."""

    def __init__(self, path, prefix):
        self.lib = ctypes.CDLL(path)
        self.prefix = prefix
        self.is_ref = prefix == "ref_"
        for name in ("cap_factor",):
            getattr(self.lib, prefix + name).restype = ctypes.c_float

    def _fn(self, name):
        return getattr(self.lib, self.prefix + name)

    # ---- linear ---------------------------------------------------------
    def linear_fwd(self, mu_w, var_w, mu_b, var_b, mu_a, var_a, threads=1):
        N, K = mu_w.shape
        B = mu_a.shape[0]
        bias = mu_b is not None
        mu_z = np.empty((B, N), np.float32)
        var_z = np.empty((B, N), np.float32)
        self._fn("linear_fwd")(_fp(mu_w), _fp(var_w), _fp(mu_b), _fp(var_b),
                               _fp(mu_a), _fp(var_a), K, N, B, int(bias),
                               threads, _fp(mu_z), _fp(var_z))
        return mu_z, var_z

    def linear_bwd_dz(self, mu_w, jcb, dmu, dvar, threads=1):
        N, K = mu_w.shape
        B = dmu.shape[0]
        om = np.empty((B, K), np.float32)
        ov = np.empty((B, K), np.float32)
        self._fn("linear_bwd_dz")(_fp(mu_w), _fp(jcb), _fp(dmu), _fp(dvar), K,
                                  N, B, threads, _fp(om), _fp(ov))
        return om, ov

    def linear_bwd_dw(self, var_w, mu_a, dmu, dvar, threads=1):
        N, K = var_w.shape
        B = dmu.shape[0]
        om = np.empty((N, K), np.float32)
        ov = np.empty((N, K), np.float32)
        self._fn("linear_bwd_dw")(_fp(var_w), _fp(mu_a), _fp(dmu), _fp(dvar),
                                  K, N, B, threads, _fp(om), _fp(ov))
        return om, ov

    def linear_bwd_db(self, var_b, dmu, dvar, threads=1):
        B, N = dmu.shape
        om = np.empty(N, np.float32)
        ov = np.empty(N, np.float32)
        self._fn("linear_bwd_db")(_fp(var_b), _fp(dmu), _fp(dvar), N, B,
                                  threads, _fp(om), _fp(ov))
        return om, ov

    # ---- conv index tables -------------------------------------------------
    def conv2d_out_size(self, kernel, stride, wi, hi, pad, pad_type):
        wo, ho = ctypes.c_int(0), ctypes.c_int(0)
        rc = self._fn("conv2d_out_size")(kernel, stride, wi, hi, pad, pad_type,
                                         ctypes.byref(wo), ctypes.byref(ho))
        if rc != 0:
            raise ValueError("invalid conv2d geometry")
        return wo.value, ho.value

    def conv2d_build_idx(self, kernel, stride, wi, hi, pad, pad_type,
                         param_pad_idx):
        wo, ho = self.conv2d_out_size(kernel, stride, wi, hi, pad, pad_type)
        k2 = kernel * kernel
        fm = np.zeros(wo * ho * k2, np.int32)
        zw = np.zeros(wi * hi * k2 + 16, np.int32)
        zud = np.zeros(wi * hi * k2 + 16, np.int32)
        w, h = ctypes.c_int(0), ctypes.c_int(0)
        rc = self._fn("conv2d_build_idx")(kernel, stride, wi, hi, wo, ho, pad,
                                          pad_type, param_pad_idx, _ip(fm),
                                          _ip(zw), _ip(zud), ctypes.byref(w),
                                          ctypes.byref(h))
        if rc != 0:
            raise ValueError("conv2d index construction failed (%d)" % rc)
        n = w.value * h.value
        return dict(Fmwa_2=fm, FCzwa_1=zw[:n].copy(), Szz_ud=zud[:n].copy(),
                    w=w.value, h=h.value, wo=wo, ho=ho)

    # ---- conv ---------------------------------------------------------------
    def conv2d_fwd(self, mu_w, var_w, mu_b, var_b, mu_a, var_a, aidx, woho,
                   fo, wihi, fi, ki, B, threads=1):
        bias = mu_b is not None
        mu_z = np.empty(B * fo * woho, np.float32)
        var_z = np.empty(B * fo * woho, np.float32)
        self._fn("conv2d_fwd")(_fp(mu_w), _fp(var_w), _fp(mu_b), _fp(var_b),
                               _fp(mu_a), _fp(var_a), _ip(aidx), woho, fo,
                               wihi, fi, ki, B, int(bias), threads, _fp(mu_z),
                               _fp(var_z))
        return mu_z, var_z

    def conv2d_bwd_dz(self, mu_w, jcb, dmu, dvar, zw_idx, zud_idx, woho, fo,
                      wihi, fi, ki, nr, B, threads=1):
        tmp = np.empty(B * fi * wihi, np.float32)
        om = np.empty(B * fi * wihi, np.float32)
        ov = np.empty(B * fi * wihi, np.float32)
        self._fn("conv2d_bwd_dz")(_fp(mu_w), _fp(jcb), _fp(dmu), _fp(dvar),
                                  _ip(zw_idx), _ip(zud_idx), woho, fo, wihi,
                                  fi, ki, nr, B, threads, _fp(tmp), _fp(om),
                                  _fp(ov))
        return om, ov

    def conv2d_bwd_dw(self, var_w, var_b, mu_a, dmu, dvar, aidx, B, fo, woho,
                      wihi, fi, ki, threads=1):
        bias = var_b is not None
        nw = ki * ki * fi * fo
        t1 = np.empty(B * fo * woho, np.float32)
        t2 = np.empty(B * fo * woho, np.float32)
        om = np.empty(nw, np.float32)
        ov = np.empty(nw, np.float32)
        bm = np.zeros(fo, np.float32)
        bv = np.zeros(fo, np.float32)
        self._fn("conv2d_bwd_dw")(_fp(var_w), _fp(var_b), _fp(mu_a), _fp(dmu),
                                  _fp(dvar), _ip(aidx), B, fo, woho, wihi, fi,
                                  ki, int(bias), threads, _fp(t1), _fp(t2),
                                  _fp(om), _fp(ov), _fp(bm), _fp(bv))
        return (om, ov, bm, bv) if bias else (om, ov, None, None)

    # ---- update / output / relu ----------------------------------------------
    def cap_factor(self, batch_size, prev=1.0):
        return float(self._fn("cap_factor")(int(batch_size),
                                            ctypes.c_float(prev)))

    def param_update(self, mu, var, dmu, dvar, cap, weights=True):
        """In place on copies; returns (mu, var, clamped_count)."""
        mu, var = mu.copy(), var.copy()
        args = [_fp(mu), _fp(var), _fp(dmu), _fp(dvar),
                ctypes.c_size_t(mu.size), ctypes.c_float(cap)]
        if self.is_ref:
            args.append(int(weights))
        cnt = self._fn("param_update")(*args)
        return mu, var, (cnt if weights else 0)

    def out_update_dense(self, mu_a, var_a, jcb, obs, var_obs, dmu, dvar):
        dmu, dvar = dmu.copy(), dvar.copy()
        self._fn("out_update_dense")(_fp(mu_a), _fp(var_a), _fp(jcb), _fp(obs),
                                     _fp(var_obs), obs.size, _fp(dmu),
                                     _fp(dvar))
        return dmu, dvar

    def out_update_heteros(self, mu_a, var_a, jcb, obs, dmu, dvar):
        """obs.size observations against 2*obs.size output units (mean, error variance)."""
        dmu, dvar = dmu.copy(), dvar.copy()
        self._fn("out_update_heteros")(_fp(mu_a), _fp(var_a), _fp(jcb), _fp(obs), obs.size,
                                       _fp(dmu), _fp(dvar))
        return dmu, dvar

    def out_update_indexed(self, mu_a, var_a, jcb, obs, var_obs, sel, n_obs,
                           n_enc, dmu, dvar):
        dmu, dvar = dmu.copy(), dvar.copy()
        args = [_fp(mu_a), _fp(var_a), _fp(jcb), _fp(obs), _fp(var_obs),
                _ip(sel), n_obs, n_enc, obs.size]
        if self.is_ref:
            args.append(int(mu_a.size))
        args += [_fp(dmu), _fp(dvar)]
        self._fn("out_update_indexed")(*args)
        return dmu, dvar

    def relu_fwd(self, mu_z, var_z):
        mu_a = np.empty_like(mu_z)
        jcb = np.empty_like(mu_z)
        var_a = np.empty_like(mu_z)
        self._fn("relu_fwd")(_fp(mu_z), _fp(var_z), mu_z.size, _fp(mu_a),
                             _fp(jcb), _fp(var_a))
        return mu_a, var_a, jcb

    # ---- mixture relu -----------------------------------------------------
    def mixture_relu_fwd(self, mu_z, var_z, threads=1):
        n = mu_z.size
        mu_a, jcb, var_a = (np.empty(n, np.float32) for _ in range(3))
        self._fn("mixture_relu_fwd")(_fp(mu_z), _fp(var_z), n, threads, _fp(mu_a), _fp(jcb),
                                     _fp(var_a))
        return mu_a, var_a, jcb

    # ---- batch norm ---------------------------------------------------------
    def batchnorm2d_stats(self, mu_a, var_a, wihi, fi, B, momentum, mu_ra, var_ra, threads=1):
        """Returns (mu_s, var_s, mu_ra, var_ra): batch statistics and the updated
        running averages (the inputs mu_ra/var_ra are not modified)."""
        mu_s, var_s, tmp = (np.empty(fi, np.float32) for _ in range(3))
        mu_ra, var_ra = f32(mu_ra).copy(), f32(var_ra).copy()
        self._fn("batchnorm2d_stats")(_fp(mu_a), _fp(var_a), wihi, fi, B,
                                      ctypes.c_float(momentum), threads, _fp(tmp), _fp(mu_s),
                                      _fp(var_s), _fp(mu_ra), _fp(var_ra))
        return mu_s, var_s, mu_ra, var_ra

    def batchnorm2d_fwd(self, mu_w, var_w, mu_b, var_b, mu_a, var_a, mu_norm, var_norm, eps,
                        wihi, fi, B, threads=1):
        mu_z, var_z = np.empty(B * fi * wihi, np.float32), np.empty(B * fi * wihi, np.float32)
        self._fn("batchnorm2d_fwd")(_fp(mu_w), _fp(var_w), _fp(mu_b), _fp(var_b), _fp(mu_a),
                                    _fp(var_a), _fp(mu_norm), _fp(var_norm),
                                    int(mu_b is not None), ctypes.c_float(eps), wihi, fi, B,
                                    threads, _fp(mu_z), _fp(var_z))
        return mu_z, var_z

    def batchnorm2d_bwd_dz(self, mu_w, jcb, var_norm, dmu, dvar, eps, wihi, fi, B, threads=1):
        om, ov = np.empty(B * fi * wihi, np.float32), np.empty(B * fi * wihi, np.float32)
        self._fn("batchnorm2d_bwd_dz")(_fp(mu_w), _fp(jcb), _fp(var_norm), _fp(dmu), _fp(dvar),
                                       ctypes.c_float(eps), wihi, fi, B, threads, _fp(om),
                                       _fp(ov))
        return om, ov

    def batchnorm2d_bwd_dw(self, var_w, var_b, mu_a, mu_norm, var_norm, dmu, dvar, eps, wihi,
                           fi, B, threads=1):
        n = B * fi * wihi
        t1, t2 = np.empty(n, np.float32), np.empty(n, np.float32)
        ow, ovw, ob, ovb = (np.zeros(fi, np.float32) for _ in range(4))
        bias = var_b is not None
        self._fn("batchnorm2d_bwd_dw")(_fp(var_w), _fp(var_b), _fp(mu_a), _fp(mu_norm),
                                       _fp(var_norm), _fp(dmu), _fp(dvar), ctypes.c_float(eps),
                                       wihi, fi, B, int(bias), threads, _fp(t1), _fp(t2),
                                       _fp(ow), _fp(ovw), _fp(ob), _fp(ovb))
        return (ow, ovw, ob, ovb) if bias else (ow, ovw, None, None)

    # ---- average pooling -------------------------------------------------------
    def avgpool2d_build_idx(self, kernel, stride, wi, hi, pad, pad_type):
        wo, ho = self.conv2d_out_size(kernel, stride, wi, hi, pad, pad_type)
        k2 = kernel * kernel
        pool = np.zeros(wo * ho * k2, np.int32)
        zud = np.zeros(wi * hi * k2 + 16, np.int32)
        w, h, ov = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
        rc = self._fn("avgpool2d_build_idx")(kernel, stride, wi, hi, wo, ho, pad, pad_type,
                                             _ip(pool), _ip(zud), ctypes.byref(w),
                                             ctypes.byref(h), ctypes.byref(ov))
        if rc != 0:
            raise RuntimeError("avgpool2d_build_idx failed (%d)" % rc)
        return dict(pool_idx=pool, z_ud_idx=zud[:w.value * h.value].copy(), w=w.value,
                    h=h.value, overlap=bool(ov.value), wo=wo, ho=ho)

    def avgpool2d_fwd(self, mu_a, var_a, pool_idx, woho, wihi, ki, n_out, overlap, threads=1):
        mu_z, var_z = np.empty(n_out, np.float32), np.empty(n_out, np.float32)
        self._fn("avgpool2d_fwd")(_fp(mu_a), _fp(var_a), _ip(pool_idx), woho, wihi, ki, n_out,
                                  mu_a.size, int(overlap), threads, _fp(mu_z), _fp(var_z))
        return mu_z, var_z

    def avgpool2d_bwd_dz(self, jcb, dmu, dvar, z_ud_idx, woho, wihi, ki, nr, wo, overlap,
                         threads=1):
        n_in = jcb.size
        om, ov = np.zeros(n_in, np.float32), np.zeros(n_in, np.float32)
        zud = z_ud_idx if z_ud_idx.size else np.zeros(1, np.int32)
        self._fn("avgpool2d_bwd_dz")(_fp(jcb), _fp(dmu), _fp(dvar), _ip(zud), woho, wihi, ki, nr,
                                     wo, n_in, dmu.size, int(overlap), threads, _fp(om),
                                     _fp(ov))
        return om, ov

    # ---- residual connection ----------------------------------------------------
    def add_shortcut(self, mu_s, var_s, mu_a, var_a):
        mu_a, var_a = f32(mu_a).copy(), f32(var_a).copy()
        self._fn("add_shortcut")(_fp(mu_s), _fp(var_s), mu_a.size, _fp(mu_a), _fp(var_a))
        return mu_a, var_a

    def add_shortcut_delta(self, mu_s, var_s, jcb_s, mu_a, var_a):
        mu_a, var_a = f32(mu_a).copy(), f32(var_a).copy()
        self._fn("add_shortcut_delta")(_fp(mu_s), _fp(var_s), _fp(jcb_s), mu_a.size, _fp(mu_a),
                                       _fp(var_a))
        return mu_a, var_a


    # ---- hierarchical softmax (reference build only) -----------------------------
    def class_to_obs(self, n_classes):
        n_obs = int(np.ceil(np.log2(n_classes)))
        obs = np.zeros(n_classes * n_obs, np.float32)
        idx = np.zeros(n_classes * n_obs, np.int32)
        a, b = ctypes.c_int(0), ctypes.c_int(0)
        self._fn("class_to_obs")(n_classes, _fp(obs), _ip(idx), ctypes.byref(a), ctypes.byref(b))
        return obs.reshape(n_classes, n_obs), idx.reshape(n_classes, n_obs), a.value, b.value

    def get_error(self, mz, Sz, labels, n_classes):
        """(errors [B], class probabilities [B][n_classes]) as the reference computes
        them from the output moments [B][len] (reference build only)."""
        mz, Sz = f32(mz), f32(Sz)
        labels = np.ascontiguousarray(labels, np.int32)
        B, length = labels.size, mz.size // labels.size
        er = np.zeros(B, np.int32)
        prob = np.zeros(B * n_classes, np.float32)
        self._fn("get_error")(_fp(mz), _fp(Sz), _ip(labels), n_classes, B, length, _ip(er),
                              _fp(prob))
        return er, prob.reshape(B, n_classes)

    # ---- checkpoint files (reference build only) -----------------------------------
    def checkpoint_save(self, model, path):
        """Writes the reference's binary checkpoint of zoo model `model` with the
        parameter pattern value(leaf, array, i) = leaf+1 + 0.1*(array+1) + 1e-4*i."""
        fn = self._fn("checkpoint_save")
        fn.restype = ctypes.c_int
        return fn(int(model), os.fsencode(path))

    def checkpoint_load(self, model, path, capacity=1 << 16):
        """Loads a binary checkpoint with the reference's loader; returns all
        parameters leaf by leaf in saving order, or None if the loader threw."""
        fn = self._fn("checkpoint_load")
        fn.restype = ctypes.c_int
        out = np.zeros(capacity, np.float32)
        n = fn(int(model), os.fsencode(path), _fp(out), capacity)
        return None if n < 0 else out[:n].copy()

    # ---- whole models through the reference's own drivers (reference build only) ---
    def model_param_sizes(self, spec):
        """Sizes of the parameter arrays of a network description in leaf order
        (oracle/ref_model.cpp), or None if the description does not parse."""
        fn = self._fn("model_param_sizes")
        fn.restype = ctypes.c_int
        sizes = np.zeros(4096, np.int32)
        n = fn(spec.encode(), _ip(sizes), sizes.size)
        return None if n < 0 else sizes[:n].tolist()

    def model_run(self, spec, params, mu_x, var_x, y, var_y, sel, B, update, n_enc=0,
                  input_state_update=False, eval_forward=False, threads=2):
        """Training steps of the reference's Sequential on the CPU: forward, output
        update (0 dense, 1 selected indices, 2 heteroscedastic), backward, step.
        mu_x [steps][B*n_in] etc. Returns a dict of per-step outputs."""
        fn = self._fn("model_run")
        fn.restype = ctypes.c_int
        params = f32(np.concatenate([np.ravel(p) for p in params]))
        mu_x = f32(mu_x)
        steps, nx = mu_x.shape
        n_in = nx // B
        var_x = None if var_x is None else f32(var_x)
        y, var_y = f32(y), f32(var_y)
        sel = np.zeros(1, np.int32) if sel is None else np.ascontiguousarray(sel, np.int32)
        cap = 1 << 22
        out_mu = np.zeros(cap, np.float32)
        out_var = np.zeros(cap, np.float32)
        in_dmu = np.zeros((steps, nx), np.float32)
        in_dvar = np.zeros((steps, nx), np.float32)
        params_out = np.zeros((steps, params.size), np.float32)
        neg = np.zeros((steps, 256), np.int32)
        top = len(_top_level(spec))
        neg = np.zeros((steps, top), np.int32)
        n_out = fn(spec.encode(), int(threads), int(input_state_update), _fp(params), steps, B,
                   n_in, _fp(mu_x), _fp(var_x), int(update), int(n_enc), _fp(y), _fp(var_y),
                   _ip(sel), int(eval_forward), _fp(out_mu), _fp(out_var), _fp(in_dmu),
                   _fp(in_dvar), _fp(params_out), _ip(neg))
        if n_out < 0:
            raise RuntimeError("the reference threw while running: " + spec)
        rows = steps + (1 if eval_forward else 0)
        no = B * n_out
        return dict(n_out=n_out, out_mu=out_mu[:rows * no].reshape(rows, no).copy(),
                    out_var=out_var[:rows * no].reshape(rows, no).copy(), in_dmu=in_dmu,
                    in_dvar=in_dvar, params=params_out, neg=neg)

    def write_csv(self, path, data):
        fn = self._fn("write_csv")
        fn.restype = ctypes.c_int
        data = f32(data)
        return fn(os.fsencode(path), _fp(data), data.size)

    def read_csv(self, path, n):
        fn = self._fn("read_csv")
        fn.restype = ctypes.c_int
        out = np.zeros(n, np.float32)
        return out if fn(os.fsencode(path), _fp(out), n) == 0 else None


def _top_level(spec):
    """Top-level layer names of a network description (brackets skipped)."""
    names, depth = [], 0
    tok = spec.split()
    i = 4 if tok and tok[0] == "input" else 0
    for t in tok[i:]:
        if t == "[":
            depth += 1
        elif t == "]":
            depth -= 1
        elif depth == 0 and t[0].isalpha():
            names.append(t)
    return names


def load():
    path = os.path.join(_HERE, "liboracle.so")
    if not os.path.exists(path):
        build()
    return Oracle(path, "oracle_")


def load_ref():
    path = os.path.join(_HERE, "_ref", "libtagi_ref.so")
    if not os.path.exists(path):
        return None
    return Oracle(path, "ref_")
