"""The benchmark configurations at their full sizes, with inputs that regenerate
from a seed on any machine (numpy), and the entries of every output that the
reference-CPU fixture (tests/golden/full_size.npz) keeps: a seeded sample of a few
thousand flat indices per tensor, plus float64 sums over the whole tensor."""
import numpy as np

# name -> Linear (K, N, B) of configs 2 and 3, and the 16-sample variant of config 3
LINEAR = {"linear_4096_b256": (4096, 4096, 256), "linear_8192_b8": (8192, 8192, 8),
          "linear_8192_b16": (8192, 8192, 16)}
# config 4: 3x3, stride 1, padding 1, 64 -> 64 channels on 32x32 maps, batch 128, no bias
CONV = {"conv_3x3_64_32_b128": dict(fi=64, fo=64, k=3, wi=32, B=128)}
SAMPLES = 4096


def _normal(rng, shape, scale=1.0):
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(scale)).astype(np.float32)


def _uniform(rng, shape, lo, hi):
    return (np.float32(lo) + np.float32(hi - lo) * rng.random(shape, dtype=np.float32)).astype(np.float32)


def linear_inputs(name):
    """mu_a ~ N(0,1), var_a ~ U(0.01,0.1), jcb ~ U(0,1), mu_w ~ N(0,1/K), var_w ~ U(0.5,1.5)/K,
    bias on, delta_mu ~ N(0, 0.1^2), delta_var ~ -U(0,1e-3)."""
    K, N, B = LINEAR[name]
    rng = np.random.default_rng(K + B)
    return dict(mu_w=_normal(rng, (N, K), K ** -0.5), var_w=_uniform(rng, (N, K), 0.5 / K, 1.5 / K),
                mu_b=_normal(rng, N, 0.5), var_b=_uniform(rng, N, 0.5 / K, 1.5 / K),
                mu_a=_normal(rng, (B, K)), var_a=_uniform(rng, (B, K), 0.01, 0.1),
                jcb=_uniform(rng, (B, K), 0.0, 1.0), delta_mu=_normal(rng, (B, N), 0.1),
                delta_var=-_uniform(rng, (B, N), 0.0, 1e-3))


def conv_inputs(name):
    g = CONV[name]
    fi, fo, k, wi, B = g["fi"], g["fo"], g["k"], g["wi"], g["B"]
    R, pix = k * k * fi, wi * wi
    rng = np.random.default_rng(fi + wi + B)
    return dict(mu_w=_normal(rng, fo * R, R ** -0.5), var_w=_uniform(rng, fo * R, 0.5 / R, 1.5 / R),
                mu_a=_normal(rng, B * fi * pix), var_a=_uniform(rng, B * fi * pix, 0.01, 0.1),
                jcb=_uniform(rng, B * fi * pix, 0.0, 1.0), delta_mu=_normal(rng, B * fo * pix, 0.1),
                delta_var=-_uniform(rng, B * fo * pix, 0.0, 1e-3))


def sample_of(name, tensor, size):
    """Sorted flat indices kept for output `tensor` of case `name`."""
    seed = sum(ord(ch) for ch in name + tensor)
    rng = np.random.default_rng(seed)
    if size <= SAMPLES:
        return np.arange(size)
    return np.sort(rng.choice(size, SAMPLES, replace=False))


def summarize(name, outputs):
    """{tensor: array} -> fixture entries: sampled values, float64 sum and sum of |.|"""
    out = {}
    for tensor, a in outputs.items():
        a = np.asarray(a).ravel()
        idx = sample_of(name, tensor, a.size)
        out["%s_%s" % (name, tensor)] = a[idx].astype(np.float32)
        a64 = a.astype(np.float64)
        out["%s_%s_sums" % (name, tensor)] = np.array([a64.sum(), np.abs(a64).sum()])
    return out


LINEAR_OUTPUTS = ("mu_z", "var_z", "delta_mu_z", "delta_var_z", "delta_mu_w", "delta_var_w",
                  "delta_mu_b", "delta_var_b")
CONV_OUTPUTS = ("mu_z", "var_z", "delta_mu_z", "delta_var_z", "delta_mu_w", "delta_var_w")


# ---- float64 closed forms at sampled entries (numpy, any machine) ---------------------

def _dots(X, rows_x, Y, rows_y, fx=None, fy=None, chunk=256):
    """sum_k fx(X[rows_x[i], k]) * fy(Y[rows_y[i], k]) in float64, for every i."""
    out = np.empty(len(rows_x), np.float64)
    for s in range(0, len(rows_x), chunk):
        x = X[rows_x[s:s + chunk]].astype(np.float64)
        y = Y[rows_y[s:s + chunk]].astype(np.float64)
        if fx is not None:
            x = fx(x)
        if fy is not None:
            y = fy(y)
        out[s:s + chunk] = np.einsum("ik,ik->i", x, y)
    return out


def linear_float64(name, d):
    """{tensor: float64 values at sample_of(name, tensor)} from the layer's closed forms."""
    K, N, B = LINEAR[name]
    f = np.float64
    sq = np.square
    out = {}
    idx = sample_of(name, "mu_z", B * N)
    b, n = idx // N, idx % N
    out["mu_z"] = _dots(d["mu_a"], b, d["mu_w"], n) + d["mu_b"].astype(f)[n]
    idx = sample_of(name, "var_z", B * N)
    b, n = idx // N, idx % N
    m2 = np.square(d["mu_a"].astype(f)) + d["var_a"].astype(f)          # [B][K]
    out["var_z"] = (_dots(m2, b, d["var_w"], n) + _dots(d["var_a"], b, d["mu_w"], n, None, sq)
                    + d["var_b"].astype(f)[n])
    w_t = np.ascontiguousarray(d["mu_w"].T)                               # [K][N]
    idx = sample_of(name, "delta_mu_z", B * K)
    b, k = idx // K, idx % K
    out["delta_mu_z"] = _dots(d["delta_mu"], b, w_t, k) * d["jcb"].astype(f)[b, k]
    idx = sample_of(name, "delta_var_z", B * K)
    b, k = idx // K, idx % K
    out["delta_var_z"] = _dots(d["delta_var"], b, w_t, k, None, sq) * sq(d["jcb"].astype(f)[b, k])
    dmu_t = np.ascontiguousarray(d["delta_mu"].T)                         # [N][B]
    dvar_t = np.ascontiguousarray(d["delta_var"].T)
    a_t = np.ascontiguousarray(d["mu_a"].T)                               # [K][B]
    idx = sample_of(name, "delta_mu_w", N * K)
    n, k = idx // K, idx % K
    out["delta_mu_w"] = _dots(dmu_t, n, a_t, k) * d["var_w"].astype(f)[n, k]
    idx = sample_of(name, "delta_var_w", N * K)
    n, k = idx // K, idx % K
    out["delta_var_w"] = _dots(dvar_t, n, a_t, k, None, sq) * sq(d["var_w"].astype(f)[n, k])
    n = sample_of(name, "delta_mu_b", N)
    out["delta_mu_b"] = d["delta_mu"].astype(f).sum(0)[n] * d["var_b"].astype(f)[n]
    n = sample_of(name, "delta_var_b", N)
    out["delta_var_b"] = d["delta_var"].astype(f).sum(0)[n] * sq(d["var_b"].astype(f)[n])
    return out


def conv_float64(name, d):
    """The same for the 3x3, stride 1, padding 1 convolution (zero padding written
    out: an entry is a sum over channels and the nine taps)."""
    g = CONV[name]
    fi, fo, k, wi, B = g["fi"], g["fo"], g["k"], g["wi"], g["B"]
    pix = wi * wi
    f = np.float64
    W = d["mu_w"].astype(f).reshape(fo, fi, k, k)
    V = d["var_w"].astype(f).reshape(fo, fi, k, k)

    def padded(x, ch):
        p = np.zeros((B, ch, wi + 2, wi + 2), f)
        p[:, :, 1:-1, 1:-1] = x.astype(f).reshape(B, ch, wi, wi)
        return p

    A, VA = padded(d["mu_a"], fi), padded(d["var_a"], fi)
    DM, DV = padded(d["delta_mu"], fo), padded(d["delta_var"], fo)
    out = {}

    def forward(idx, weights, acts):
        b, o, p = idx // (fo * pix), (idx // pix) % fo, idx % pix
        oy, ox = p // wi, p % wi
        acc = np.zeros(len(idx), f)
        for ky in range(k):
            for kx in range(k):
                acc += np.einsum("ic,ic->i", weights[o, :, ky, kx], acts[b, :, oy + ky, ox + kx])
        return acc

    out["mu_z"] = forward(sample_of(name, "mu_z", B * fo * pix), W, A)
    idx = sample_of(name, "var_z", B * fo * pix)
    out["var_z"] = forward(idx, V, A * A + VA) + forward(idx, W * W, VA)

    def backward(idx, weights, deltas):
        b, c, p = idx // (fi * pix), (idx // pix) % fi, idx % pix
        iy, ix = p // wi, p % wi
        acc = np.zeros(len(idx), f)
        for ky in range(k):
            for kx in range(k):
                # output pixel (iy - ky + 1, ix - kx + 1) reaches (iy, ix) through tap (ky, kx)
                acc += np.einsum("io,io->i", weights[:, c, ky, kx].T,
                                 deltas[b, :, iy - ky + 2, ix - kx + 2])
        return acc

    J = d["jcb"].astype(f)
    idx = sample_of(name, "delta_mu_z", B * fi * pix)
    out["delta_mu_z"] = backward(idx, W, DM) * J[idx]
    idx = sample_of(name, "delta_var_z", B * fi * pix)
    out["delta_var_z"] = backward(idx, W * W, DV) * J[idx] ** 2

    def weight(idx, deltas, acts):
        o, c, t = idx // (fi * k * k), (idx // (k * k)) % fi, idx % (k * k)
        ky, kx = t // k, t % k
        acc = np.empty(len(idx), f)
        for i in range(len(idx)):
            acc[i] = np.sum(deltas[:, o[i], 1:-1, 1:-1] *
                            acts[:, c[i], ky[i]:ky[i] + wi, kx[i]:kx[i] + wi])
        return acc

    idx = sample_of(name, "delta_mu_w", fo * fi * k * k)
    out["delta_mu_w"] = weight(idx, DM, A) * V.ravel()[idx]
    idx = sample_of(name, "delta_var_w", fo * fi * k * k)
    out["delta_var_w"] = weight(idx, DV, A * A) * V.ravel()[idx] ** 2
    return out
