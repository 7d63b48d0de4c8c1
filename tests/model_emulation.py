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


class Emulator:
    def __init__(self, oracle, layers, threads=2):
        self.o, self.layers, self.t = oracle, layers, threads

    def forward(self, mu_x, var_x, B):
        o = self.o
        mu, var = mu_x.astype(np.float32).ravel(), var_x.astype(np.float32).ravel()
        jcb = np.ones_like(mu)
        self.B = B
        for L in self.layers:
            if isinstance(L, Relu):
                mu, var, jcb = o.relu_fwd(mu, var)
                continue
            L.bwd_mu_a, L.bwd_jcb = mu.copy(), jcb.copy()
            if isinstance(L, Lin):
                z = o.linear_fwd(L.mu_w, L.var_w, L.mu_b, L.var_b, mu.reshape(B, L.K),
                                 var.reshape(B, L.K), self.t)
            else:
                L.idx = o.conv2d_build_idx(L.k, L.s, L.wi, L.wi, L.p, L.pt, L.k * L.k * L.fi * L.fo + 1)
                L.wihi, L.woho = L.wi * L.wi, L.idx["wo"] * L.idx["ho"]
                z = o.conv2d_fwd(L.mu_w, L.var_w, L.mu_b, L.var_b, mu, var, L.idx["Fmwa_2"], L.woho,
                                 L.fo, L.wihi, L.fi, L.k, B, self.t)
            mu, var = z[0].ravel(), z[1].ravel()
            jcb = np.ones_like(mu)
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

    def backward(self, input_state_update=False):
        o, B = self.o, self.B
        dmu, dvar = self.delta
        first = next(i for i, L in enumerate(self.layers) if not isinstance(L, Relu))
        for i in range(len(self.layers) - 1, -1, -1):
            L = self.layers[i]
            if isinstance(L, Relu):
                continue
            state = i != first or input_state_update
            if isinstance(L, Lin):
                d_m, d_v = dmu.reshape(B, L.N), dvar.reshape(B, L.N)
                L.dw = o.linear_bwd_dw(L.var_w, L.bwd_mu_a.reshape(B, L.K), d_m, d_v, self.t)
                if L.mu_b is not None:
                    L.db = o.linear_bwd_db(L.var_b, d_m, d_v, self.t)
                if state:
                    nz = o.linear_bwd_dz(L.mu_w, L.bwd_jcb.reshape(B, L.K), d_m, d_v, self.t)
            else:
                r = o.conv2d_bwd_dw(L.var_w, L.var_b, L.bwd_mu_a, dmu, dvar, L.idx["Fmwa_2"], B, L.fo,
                                    L.woho, L.wihi, L.fi, L.k, self.t)
                L.dw = (r[0], r[1])
                if L.mu_b is not None:
                    L.db = (r[2], r[3])
                if state:
                    nz = o.conv2d_bwd_dz(L.mu_w, L.bwd_jcb, dmu, dvar, L.idx["FCzwa_1"],
                                         L.idx["Szz_ud"], L.woho, L.fo, L.wihi, L.fi, L.k,
                                         L.idx["h"], B, self.t)
            if state:
                dmu, dvar = nz[0].ravel(), nz[1].ravel()
        self.input_delta = (dmu, dvar)

    def step(self):
        o = self.o
        cap = o.cap_factor(self.B, 1.0)
        self.neg = {}
        for i, L in enumerate(self.layers):
            if isinstance(L, Relu):
                continue
            shape = L.mu_w.shape
            m, v, c = o.param_update(L.mu_w.ravel(), L.var_w.ravel(), L.dw[0].ravel(),
                                     L.dw[1].ravel(), cap, True)
            L.mu_w, L.var_w = m.reshape(shape), v.reshape(shape)
            self.neg[i] = c
            if L.mu_b is not None:
                L.mu_b, L.var_b, _ = o.param_update(L.mu_b, L.var_b, L.db[0], L.db[1], cap, False)
