"""A numpy emulation of Sequential forward / output update / backward / step built
only from CPU-oracle calls, used to check the C++ host classes end to end."""
import numpy as np


class Lin:
    def __init__(self, mu_w, var_w, mu_b, var_b, K, N):
        self.K, self.N = K, N
        self.mu_w, self.var_w = mu_w.reshape(N, K).copy(), var_w.reshape(N, K).copy()
        self.mu_b = None if mu_b is None or mu_b.size == 0 else mu_b.copy()
        self.var_b = None if var_b is None or var_b.size == 0 else var_b.copy()


class Conv:
    def __init__(self, mu_w, var_w, mu_b, var_b, fi, fo, k, s, p, pt, wi):
        self.fi, self.fo, self.k, self.s, self.p, self.pt, self.wi = fi, fo, k, s, p, pt, wi
        self.mu_w, self.var_w = mu_w.copy(), var_w.copy()
        self.mu_b = None if mu_b is None or mu_b.size == 0 else mu_b.copy()
        self.var_b = None if var_b is None or var_b.size == 0 else var_b.copy()


class Relu:
    pass


class MRelu:
    pass


class BNorm:
    def __init__(self, mu_w, var_w, mu_b, var_b, nf, eps=1e-4, momentum=0.9):
        self.nf, self.eps, self.momentum = nf, eps, momentum
        self.mu_w, self.var_w = mu_w.copy(), var_w.copy()
        self.mu_b = None if mu_b is None or mu_b.size == 0 else mu_b.copy()
        self.var_b = None if var_b is None or var_b.size == 0 else var_b.copy()
        self.mu_ra, self.var_ra = np.zeros(nf, np.float32), np.ones(nf, np.float32)


class Pool:
    def __init__(self, k, s, p, pt, wi, ch):
        self.k, self.s, self.p, self.pt, self.wi, self.ch = k, s, p, pt, wi, ch


class Block:
    def __init__(self, layers):
        self.layers = layers


class Res:
    def __init__(self, main, shortcut=None):
        self.main, self.shortcut = main, shortcut


ACTIVATIONS = (Relu, MRelu)


def param_layers(layers, top=True, suffix=""):
    """(state_dict suffix, layer) of every layer with parameters, with the key
    suffixes the host classes produce: "<i>" at the top level, "main.<i>.<j>" and
    "shortcut.<i>.<j>" inside residual blocks."""
    out = []
    for i, L in enumerate(layers):
        sfx = str(i) if top else suffix + "." + str(i)
        if isinstance(L, (Lin, Conv, BNorm)):
            out.append((sfx, L))
        elif isinstance(L, Block):
            out += param_layers(L.layers, False, sfx)
        elif isinstance(L, Res):
            out += param_layers(L.main.layers, False, "main." + sfx)
            if L.shortcut is not None:
                out += param_layers(L.shortcut.layers, False, "shortcut." + sfx)
    return out


class Emulator:
    def __init__(self, oracle, layers, threads=2):
        self.o, self.layers, self.t = oracle, layers, threads

    # ---- forward -------------------------------------------------------------
    def _fwd(self, L, mu, var, jcb):
        o, B = self.o, self.B
        if isinstance(L, Relu):
            return o.relu_fwd(mu, var)
        if isinstance(L, MRelu):
            return o.mixture_relu_fwd(mu, var, self.t)
        if isinstance(L, Block):
            for sub in L.layers:
                mu, var, jcb = self._fwd(sub, mu, var, jcb)
            return mu, var, jcb
        if isinstance(L, Res):
            L.bwd_jcb = jcb.copy()
            m_mu, m_var, _ = self._fwd(L.main, mu, var, jcb)
            if L.shortcut is not None:
                s_mu, s_var, _ = self._fwd(L.shortcut, mu, var, jcb)
            else:
                s_mu, s_var = mu, var
            mu, var = o.add_shortcut(s_mu, s_var, m_mu, m_var)
            return mu, var, np.ones_like(mu)
        L.bwd_mu_a, L.bwd_jcb = mu.copy(), jcb.copy()
        if isinstance(L, Lin):
            z = o.linear_fwd(L.mu_w, L.var_w, L.mu_b, L.var_b, mu.reshape(B, L.K),
                             var.reshape(B, L.K), self.t)
        elif isinstance(L, Conv):
            L.idx = o.conv2d_build_idx(L.k, L.s, L.wi, L.wi, L.p, L.pt, L.k * L.k * L.fi * L.fo + 1)
            L.wihi, L.woho = L.wi * L.wi, L.idx["wo"] * L.idx["ho"]
            z = o.conv2d_fwd(L.mu_w, L.var_w, L.mu_b, L.var_b, mu, var, L.idx["Fmwa_2"], L.woho,
                             L.fo, L.wihi, L.fi, L.k, B, self.t)
        elif isinstance(L, BNorm):
            L.wihi = mu.size // (B * L.nf)
            L.mu_s, L.var_s, L.mu_ra, L.var_ra = o.batchnorm2d_stats(
                mu, var, L.wihi, L.nf, B, L.momentum, L.mu_ra, L.var_ra, self.t)
            z = o.batchnorm2d_fwd(L.mu_w, L.var_w, L.mu_b, L.var_b, mu, var, L.mu_s, L.var_s, L.eps,
                                  L.wihi, L.nf, B, self.t)
        elif isinstance(L, Pool):
            L.idx = o.avgpool2d_build_idx(L.k, L.s, L.wi, L.wi, L.p, L.pt)
            L.wihi, L.woho = L.wi * L.wi, L.idx["wo"] * L.idx["ho"]
            z = o.avgpool2d_fwd(mu, var, L.idx["pool_idx"], L.woho, L.wihi, L.k,
                                B * L.ch * L.woho, L.idx["overlap"], self.t)
        else:
            raise TypeError(L)
        mu, var = z[0].ravel(), z[1].ravel()
        return mu, var, np.ones_like(mu)

    def forward(self, mu_x, var_x, B):
        mu, var = mu_x.astype(np.float32).ravel(), var_x.astype(np.float32).ravel()
        jcb = np.ones_like(mu)
        self.B = B
        for L in self.layers:
            mu, var, jcb = self._fwd(L, mu, var, jcb)
        self.out = (mu, var, jcb)
        return mu, var

    def update_indexed(self, y, var_y, sel, n_obs, n_enc):
        mu, var, jcb = self.out
        z = np.zeros_like(mu)
        self.delta = self.o.out_update_indexed(mu, var, jcb, y, var_y, sel, n_obs, n_enc, z, z)

    def update_dense(self, y, var_y):
        mu, var, jcb = self.out
        z = np.zeros_like(mu)
        self.delta = self.o.out_update_dense(mu, var, jcb, y, var_y, z, z)

    def update_heteros(self, y):
        mu, var, jcb = self.out
        z = np.zeros_like(mu)
        self.delta = self.o.out_update_heteros(mu, var, jcb, y, z, z)

    # ---- backward --------------------------------------------------------------
    def _bwd_list(self, layers, dmu, dvar, state, block):
        """Layers in reverse. All but the first run with their state update. The
        first one: in a Sequential (src/sequential.cpp:392-410) it runs and only its
        state update depends on `state`; in a LayerBlock (src/layer_block.cpp:208-213)
        it runs only when `state` is set and the block has more than one layer -
        otherwise it gets no backward pass at all, so its parameters see no
        innovation either."""
        for i in range(len(layers) - 1, 0, -1):
            if not isinstance(layers[i], ACTIVATIONS):
                dmu, dvar = self._bwd(layers[i], dmu, dvar, True)
        first = layers[0]
        if isinstance(first, ACTIVATIONS):
            return dmu, dvar
        if block and not (state and len(layers) > 1):
            return dmu, dvar
        return self._bwd(first, dmu, dvar, state)

    def _bwd(self, L, dmu, dvar, state):
        o, B = self.o, self.B
        if isinstance(L, Block):
            return self._bwd_list(L.layers, dmu, dvar, state, True)
        if isinstance(L, Res):
            m = self._bwd(L.main, dmu, dvar, state)
            if L.shortcut is not None:
                s = self._bwd(L.shortcut, dmu, dvar, state)
                return o.add_shortcut(s[0], s[1], m[0], m[1]) if state else (dmu, dvar)
            return o.add_shortcut_delta(dmu, dvar, L.bwd_jcb, m[0], m[1]) if state else (dmu, dvar)
        nz = None
        if isinstance(L, Lin):
            d_m, d_v = dmu.reshape(B, L.N), dvar.reshape(B, L.N)
            L.dw = o.linear_bwd_dw(L.var_w, L.bwd_mu_a.reshape(B, L.K), d_m, d_v, self.t)
            if L.mu_b is not None:
                L.db = o.linear_bwd_db(L.var_b, d_m, d_v, self.t)
            if state:
                nz = o.linear_bwd_dz(L.mu_w, L.bwd_jcb.reshape(B, L.K), d_m, d_v, self.t)
        elif isinstance(L, Conv):
            r = o.conv2d_bwd_dw(L.var_w, L.var_b, L.bwd_mu_a, dmu, dvar, L.idx["Fmwa_2"], B, L.fo,
                                L.woho, L.wihi, L.fi, L.k, self.t)
            L.dw = (r[0], r[1])
            if L.mu_b is not None:
                L.db = (r[2], r[3])
            if state:
                nz = o.conv2d_bwd_dz(L.mu_w, L.bwd_jcb, dmu, dvar, L.idx["FCzwa_1"],
                                     L.idx["Szz_ud"], L.woho, L.fo, L.wihi, L.fi, L.k,
                                     L.idx["h"], B, self.t)
        elif isinstance(L, BNorm):
            r = o.batchnorm2d_bwd_dw(L.var_w, L.var_b, L.bwd_mu_a, L.mu_s, L.var_s, dmu, dvar, L.eps,
                                     L.wihi, L.nf, B, self.t)
            L.dw = (r[0], r[1])
            if L.mu_b is not None:
                L.db = (r[2], r[3])
            if state:
                nz = o.batchnorm2d_bwd_dz(L.mu_w, L.bwd_jcb, L.var_s, dmu, dvar, L.eps, L.wihi, L.nf,
                                          B, self.t)
        elif isinstance(L, Pool):
            if state:
                nz = o.avgpool2d_bwd_dz(L.bwd_jcb, dmu, dvar, L.idx["z_ud_idx"], L.woho, L.wihi, L.k,
                                        L.idx["h"], L.idx["wo"], L.idx["overlap"], self.t)
        else:
            raise TypeError(L)
        if nz is None:
            return dmu, dvar
        return nz[0].ravel(), nz[1].ravel()

    def backward(self, input_state_update=False):
        dmu, dvar = self.delta
        self.input_delta = self._bwd_list(self.layers, dmu, dvar, input_state_update, False)

    # ---- step -------------------------------------------------------------------
    def step(self):
        o = self.o
        cap = o.cap_factor(self.B, 1.0)
        self.neg = {}
        for sfx, L in param_layers(self.layers):
            shape = L.mu_w.shape
            if not hasattr(L, "dw"):  # no backward pass yet: innovations are still zero
                L.dw = (np.zeros(L.mu_w.size, np.float32), np.zeros(L.mu_w.size, np.float32))
                if L.mu_b is not None:
                    L.db = (np.zeros_like(L.mu_b), np.zeros_like(L.mu_b))
            m, v, c = o.param_update(L.mu_w.ravel(), L.var_w.ravel(), L.dw[0].ravel(),
                                     L.dw[1].ravel(), cap, True)
            L.mu_w, L.var_w = m.reshape(shape), v.reshape(shape)
            top = int(sfx.split(".")[0]) if sfx[0].isdigit() else int(sfx.split(".")[1])
            self.neg[top] = self.neg.get(top, 0) + c
            if L.mu_b is not None:
                L.mu_b, L.var_b, _ = o.param_update(L.mu_b, L.var_b, L.db[0], L.db[1], cap, False)
