"""Writes the golden vectors tests/golden/ssd_*.npz and tests/golden/emaseq_*.npz.

The reference repository holds no fixture files for these paths and its comparison provider
(mamba_ssm) is not installed, so the vectors come from the definitions themselves, evaluated
here in float64 with plain numpy loops and no code shared with oracle/ or the HIP library:

  SSD (the recurrence of ssd_step_ref, kernels/mamba_3_kernels/mamba_ssd_fwd.py:795-860 of the
  reference, with the natural exponential of kernels/mamba_kernels/):
      h_t = exp(dt_t * A) * h_{t-1} + dt_t * x_t (outer) B_t,   y_t = C_t . h_t + D * x_t,
      gated y_t * z_t * sigmoid(z_t); h_{-1} = initial state; final state = h_{L-1}.
  EMA, probability form with boundary states (main.py:120-131 of the reference):
      z_t = (1 - p_t) * z_{t-1} + p_t * x_t,  z_{-1} = init, and the gradients of
      sum(z * dz) + sum(final * dfinal) with respect to x, p and init by the reverse recurrence.

Inputs as benchmark configuration 5 describes (x, B, C ~ N(0,1), dt = softplus(N(-2, 0.5)),
A = -exp(U(log 1, log 16))) and stored as float32.  Run `python tests/golden/make_golden_ssd.py`
to rewrite."""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

# name: (batch, seqlen, nheads, hdim, ngroups, dstate, chunk_size, seed)
SSD_CASES = {
    "ssd_small_f32": (1, 200, 2, 64, 1, 64, 64, 2001),
    "ssd_groups_gate_f32": (2, 130, 4, 64, 2, 128, 128, 2002),
}
# name: (batch, nheads, seqlen, dim, seed)
SEQ_CASES = {"emaseq_prob_states_f32": (2, 2, 300, 24, 3001)}


def ssd_case(b, L, nh, P, g, N, seed):
    rng = np.random.default_rng(seed)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    x, B, C, z = f(b, L, nh, P), f(b, L, g, N), f(b, L, g, N), f(b, L, nh, P)
    dt = np.log1p(np.exp(rng.standard_normal((b, L, nh)) * 0.5 - 2.0)).astype(np.float32)
    A = (-np.exp(rng.uniform(0.0, np.log(16.0), nh))).astype(np.float32)
    D = f(nh)
    init = f(b, nh, P, N)
    return x, dt, A, B, C, D, z, init


def ssd_f64(x, dt, A, B, C, D, z, init):
    x, dt, A, B, C, D, z = (a.astype(np.float64) for a in (x, dt, A, B, C, D, z))
    b, L, nh, P = x.shape
    rep = nh // B.shape[2]
    Bh, Ch = np.repeat(B, rep, axis=2), np.repeat(C, rep, axis=2)
    h = init.astype(np.float64).copy()
    y = np.zeros_like(x)
    for t in range(L):
        a = np.exp(dt[:, t] * A)
        h = a[..., None, None] * h + (dt[:, t, :, None] * x[:, t])[..., None] * Bh[:, t, :, None, :]
        out = np.einsum("bhpn,bhn->bhp", h, Ch[:, t]) + D[None, :, None] * x[:, t]
        y[:, t] = out * z[:, t] / (1.0 + np.exp(-z[:, t]))
    return y, h


def seq_case(b, nh, L, d, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((b, L, nh, d)).astype(np.float32)
    p = (1.0 / (1.0 + np.exp(rng.standard_normal((b, L, nh)) + 2.0))).astype(np.float32)
    init = rng.standard_normal((b, nh, d)).astype(np.float32)
    dz = rng.standard_normal((b, L, nh, d)).astype(np.float32)
    dfinal = rng.standard_normal((b, nh, d)).astype(np.float32)
    return x, p, init, dz, dfinal


def seq_f64(x, p, init, dz, dfinal):
    x, p, init, dz, dfinal = (a.astype(np.float64) for a in (x, p, init, dz, dfinal))
    b, L, nh, d = x.shape
    zs = np.zeros_like(x)
    s = init.copy()
    for t in range(L):
        s = (1.0 - p[:, t, :, None]) * s + p[:, t, :, None] * x[:, t]
        zs[:, t] = s
    dx, dp = np.zeros_like(x), np.zeros_like(p)
    r = dfinal.copy()
    for t in range(L - 1, -1, -1):
        r = dz[:, t] + r
        prev = zs[:, t - 1] if t > 0 else init
        dx[:, t] = p[:, t, :, None] * r
        dp[:, t] = np.einsum("bhd,bhd->bh", r, x[:, t] - prev)
        r = (1.0 - p[:, t, :, None]) * r
    return zs, s, dx, dp, r


def main():
    f32 = lambda a: a.astype(np.float32)
    for name, (b, L, nh, P, g, N, Q, seed) in SSD_CASES.items():
        x, dt, A, B, C, D, z, init = ssd_case(b, L, nh, P, g, N, seed)
        y, fin = ssd_f64(x, dt, A, B, C, D, z, init)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), x=x, dt=dt, A=A, B=B, C=C, D=D, z=z, init=init,
                            y=f32(y), final=f32(fin), chunk_size=np.int64(Q))
        print(name, y.shape, float(np.abs(y).max()))
    for name, (b, nh, L, d, seed) in SEQ_CASES.items():
        x, p, init, dz, dfinal = seq_case(b, nh, L, d, seed)
        zs, fin, dx, dp, dinit = seq_f64(x, p, init, dz, dfinal)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), x=x, p=p, init=init, dz=dz, dfinal=dfinal, z=f32(zs),
                            final=f32(fin), dx=f32(dx), dp=f32(dp), dinit=f32(dinit))
        print(name, zs.shape)


if __name__ == "__main__":
    main()
