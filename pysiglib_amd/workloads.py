"""The five benchmark workloads (synthetic, seeded) and their algorithmic flop counts; used by bench.py and the parity tests."""
import numpy as np

CONFIGS = {
    1: dict(name="C1 fwd f64 (32,1000,10) deg 5", batch=32, length=1000, dim=10, degree=5, dtype="float64", kind="points",
            time_aug=False, lead_lag=False, backward=False),
    2: dict(name="C2 fwd f32 Brownian (128,1024,5) deg 7", batch=128, length=1024, dim=5, degree=7, dtype="float32",
            kind="walk", var=1.0 / 1024, time_aug=False, lead_lag=False, backward=False),
    3: dict(name="C3 fwd f64 (64,4096,3) deg 12", batch=64, length=4096, dim=3, degree=12, dtype="float64",
            kind="walk", var=1.0 / 4096, time_aug=False, lead_lag=False, backward=False),
    4: dict(name="C4 fwd f32 augmented (256,500,8) time_aug+lead_lag deg 4", batch=256, length=500, dim=8, degree=4,
            dtype="float32", kind="walk", var=1.0, time_aug=True, lead_lag=True, backward=False),
    5: dict(name="C5 bwd f64 (32,1000,10) deg 5", batch=32, length=1000, dim=10, degree=5, dtype="float64",
            kind="points", time_aug=False, lead_lag=False, backward=True),
}


def make_path(k, batch=None):
    """Path of config k, generated in float64 with numpy's default_rng(1000 + k) and cast to the config dtype."""
    c = CONFIGS[k]
    seed = 1000 + (1 if k == 5 else k)      # config 5 reuses the path of config 1
    rng = np.random.default_rng(seed)
    b = c["batch"]
    if c["kind"] == "points":
        path = rng.standard_normal((b, c["length"], c["dim"]))
    else:
        inc = rng.normal(0.0, np.sqrt(c["var"]), (b, c["length"] - 1, c["dim"]))
        path = np.concatenate([np.zeros((b, 1, c["dim"])), np.cumsum(inc, axis=1)], axis=1)
    if batch is not None:
        path = path[:batch]
    return np.ascontiguousarray(path.astype(c["dtype"]))


def aug_dim(c):
    return (2 * c["dim"] if c["lead_lag"] else c["dim"]) + (1 if c["time_aug"] else 0)


def n_increments(c):
    return (2 * c["length"] - 1 if c["lead_lag"] else c["length"]) - 1


def flops_fwd(d, n):
    """Algorithmic flops per increment per path of the forward Horner step (FMA = 2)."""
    f = 3 * d
    for t in range(2, n + 1):
        f += d + sum(d ** l * (d + 2) for l in range(1, t - 1)) + d ** (t - 1) * (2 * d + 1)
    return f


def flops_bwd(d, n):
    """Algorithmic flops per increment per path of the reverse step (un-multiply + pullback)."""
    f = flops_fwd(d, n) + 3 * d
    for t in range(2, n + 1):
        f += 3 * d + sum(d ** l * (d + 2) for l in range(1, t - 1)) + sum(d ** l * (4 * d + 4) + 2 * d for l in range(1, t))
    return f
