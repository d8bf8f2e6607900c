"""Shared helpers for the parity tests: seeded problems and the error measure."""
import numpy as np

TOL = 1e-4  # max|a-b| / max|b| against the fp64 oracle, per tensor


def relerr(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.max(np.abs(a - b)) / max(np.max(np.abs(b)), 1e-30))


def problem(seed, T, N, C, H, G, zoneout=0.0, forget_bias=None):
    """Seeded float32-representable inputs, returned as float64 arrays."""
    r = np.random.default_rng(seed)
    k = 1.0 / np.sqrt(H)

    def f32(a):
        return a.astype(np.float32).astype(np.float64)
    p = dict(
        W=f32(r.uniform(-k, k, (C, G * H))), R=f32(r.uniform(-k, k, (H, G * H))),
        b=f32(r.uniform(-k, k, G * H)), b2=f32(r.uniform(-k, k, G * H)),
        x=f32(r.standard_normal((T, N, C))), h0=f32(r.standard_normal((N, H)) * 0.5),
        c0=f32(r.standard_normal((N, H)) * 0.5),
        dh_new=f32(r.standard_normal((T + 1, N, H))), dc_new=f32(r.standard_normal((T + 1, N, H))),
        gamma=f32(r.uniform(0.5, 1.5, (2, G * H))), gamma_h=f32(r.uniform(0.5, 1.5, H)),
        beta_h=f32(r.uniform(-0.5, 0.5, H)), u=f32(r.uniform(-1, 1, H)),
        mask=(r.uniform(size=(T, N, H)) >= zoneout).astype(np.float64) if zoneout else None)
    if forget_bias is not None:
        p["b"][:] = 0.0
        p["b"][2 * H:3 * H] = forget_bias
    return p


def dev(a):
    import torch
    if a is None:
        return torch.empty(0, 0, 0, dtype=torch.float32, device="cuda")
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda()


def host(t):
    return t.detach().cpu().numpy().astype(np.float64)
