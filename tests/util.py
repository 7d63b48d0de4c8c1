"""Shared helpers of the parity tests: the error metric and seeded inputs."""
import numpy as np

# Tolerance of the parity gate: max_i |x_i - ref_i| / max(|ref_i|, rms(ref)).
# Normalising small entries by the tensor's rms keeps reordering noise on
# near-zero means (absolute error ~1e-6) from reading as a large relative error.
TOL = 1e-4


def rel_err(x, ref):
    x = np.asarray(x, dtype=np.float64).ravel()
    ref = np.asarray(ref, dtype=np.float64).ravel()
    assert x.shape == ref.shape
    if ref.size == 0:
        return 0.0
    rms = np.sqrt(np.mean(ref * ref))
    denom = np.maximum(np.abs(ref), max(rms, 1e-30))
    return float(np.max(np.abs(x - ref) / denom))


def max_rel(x, ref):
    """Plain elementwise max |x - ref| / |ref| (entries where both are zero count 0)."""
    x = np.asarray(x, dtype=np.float64).ravel()
    ref = np.asarray(ref, dtype=np.float64).ravel()
    if ref.size == 0:
        return 0.0
    diff = np.abs(x - ref)
    return float(np.max(np.where(diff == 0, 0.0, diff / np.maximum(np.abs(ref), 1e-300))))


def assert_close(x, ref, what, tol=TOL, same_sign=False):
    """The parity gate. same_sign: the tensor is a sum of terms of one sign (var_z,
    the variance innovations), so nothing cancels and the plain elementwise relative
    error is held to the same tolerance as well."""
    e = rel_err(x, ref)
    assert np.all(np.isfinite(np.asarray(x))), what + ": non-finite values"
    assert e <= tol, "%s: rel err %.3e > %.1e" % (what, e, tol)
    if same_sign:
        m = max_rel(x, ref)
        assert m <= tol, "%s: elementwise rel err %.3e > %.1e" % (what, m, tol)
    return e


# outputs of the Linear / Conv2d path that are sums of terms of one sign
SAME_SIGN = ("var_z", "delta_var_z", "delta_var_w", "delta_var_b")


def linear_inputs(K, N, B, seed=0, bias=True, jcb_random=False):
    """Distributions of the benchmark configurations: mu_a ~ N(0,1),
    var_a ~ U(0.01,0.1), mu_w ~ N(0,1/K), var_w ~ 1/K (jittered so that a wrong
    index shows), delta_mu ~ N(0,1e-2), delta_var ~ -U(0,1e-3)."""
    rng = np.random.default_rng(seed)
    f = np.float32
    d = dict(
        mu_w=rng.normal(0, K ** -0.5, (N, K)).astype(f),
        var_w=(rng.uniform(0.5, 1.5, (N, K)) / K).astype(f),
        mu_a=rng.normal(0, 1, (B, K)).astype(f),
        var_a=rng.uniform(0.01, 0.1, (B, K)).astype(f),
        delta_mu=rng.normal(0, 0.1, (B, N)).astype(f),
        delta_var=(-rng.uniform(0, 1e-3, (B, N))).astype(f),
        jcb=(rng.uniform(0, 1, (B, K)) if jcb_random else np.ones((B, K))).astype(f),
    )
    if bias:
        d["mu_b"] = rng.normal(0, 0.5, N).astype(f)
        d["var_b"] = (rng.uniform(0.5, 1.5, N) / K).astype(f)
    else:
        d["mu_b"] = d["var_b"] = None
    return d


def conv_inputs(fi, fo, ki, wihi, woho, B, seed=0, bias=False, jcb_random=False):
    rng = np.random.default_rng(seed)
    f = np.float32
    k2 = ki * ki
    d = dict(
        mu_w=rng.normal(0, (k2 * fi) ** -0.5, fo * fi * k2).astype(f),
        var_w=(rng.uniform(0.5, 1.5, fo * fi * k2) / (k2 * fi)).astype(f),
        mu_a=rng.normal(0, 1, B * fi * wihi).astype(f),
        var_a=rng.uniform(0.01, 0.1, B * fi * wihi).astype(f),
        delta_mu=rng.normal(0, 0.1, B * fo * woho).astype(f),
        delta_var=(-rng.uniform(0, 1e-3, B * fo * woho)).astype(f),
        jcb=(rng.uniform(0, 1, B * fi * wihi) if jcb_random else np.ones(B * fi * wihi)).astype(f),
    )
    if bias:
        d["mu_b"] = rng.normal(0, 0.5, fo).astype(f)
        d["var_b"] = (rng.uniform(0.5, 1.5, fo) / (k2 * fi)).astype(f)
    else:
        d["mu_b"] = d["var_b"] = None
    return d


def batchnorm_inputs(wihi, fi, B, seed=0):
    """A [B][fi][wihi] activation tensor with per-channel parameters, running
    averages and incoming innovations (jittered so that a wrong index shows)."""
    rng = np.random.default_rng(seed)
    n = B * fi * wihi
    f = np.float32
    return dict(
        mu_a=rng.standard_normal(n).astype(f), var_a=rng.uniform(0.01, 0.5, n).astype(f),
        jcb=rng.uniform(0.0, 1.0, n).astype(f),
        mu_w=(1 + 0.1 * rng.standard_normal(fi)).astype(f),
        var_w=rng.uniform(0.01, 0.1, fi).astype(f),
        mu_b=(0.1 * rng.standard_normal(fi)).astype(f), var_b=rng.uniform(0.01, 0.1, fi).astype(f),
        mu_ra=rng.standard_normal(fi).astype(f), var_ra=rng.uniform(0.5, 2.0, fi).astype(f),
        dmu=(0.1 * rng.standard_normal(n)).astype(f), dvar=(-rng.uniform(0, 1e-2, n)).astype(f))


def pool_inputs(wihi, woho, fo, B, seed=0):
    rng = np.random.default_rng(seed)
    f = np.float32
    return dict(
        mu_a=rng.standard_normal(B * fo * wihi).astype(f),
        var_a=rng.uniform(0.01, 0.5, B * fo * wihi).astype(f),
        jcb=rng.uniform(0, 1, B * fo * wihi).astype(f),
        dmu=rng.standard_normal(B * fo * woho).astype(f),
        dvar=(-rng.uniform(0, 1e-2, B * fo * woho)).astype(f))


def heteros_inputs(n, seed=0):
    """Output layer with a learned error variance: 2n units (mean at 2i, expected
    squared error at 2i+1, kept positive as the exponential activation in front of it
    would) and n observations, with the special cases the reference guards: a nan and
    an inf observation, a zero predictive variance, a zero variance of the error unit."""
    rng = np.random.default_rng(seed)
    f = np.float32
    mu_a = rng.normal(0, 1, 2 * n).astype(f)
    mu_a[1::2] = rng.uniform(0.05, 2.0, n)
    var_a = rng.uniform(0.01, 0.5, 2 * n).astype(f)
    jcb = rng.uniform(0.2, 1.0, 2 * n).astype(f)
    obs = rng.normal(0, 1.5, n).astype(f)
    obs[3], obs[8] = np.nan, np.inf
    var_a[2 * 5], mu_a[2 * 5 + 1] = 0.25, -0.25     # var_sum == 0 -> inf -> zeros
    var_a[2 * 11 + 1], jcb[2 * 11 + 1] = 0.0, 0.0   # 0/0 Jacobian ratio -> 0
    return dict(mu_a=mu_a, var_a=var_a, jcb=jcb, obs=obs)
