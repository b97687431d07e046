"""Writes the golden vectors tests/golden/ema_*.npz.

The reference repository holds no fixture files for the EMA path (its tests draw random
inputs and compare two implementations in the same process), so these vectors come from
the definition itself, evaluated here in float64 with plain numpy loops and no code shared
with oracle/ or the HIP library:

    y_t  = exp(A_t) * y_{t-1} + X_t                 (kernels/tests/ema/test_ema_scan_fwd.py:25-37
                                                     of the reference, with P = 1 - exp(A))
    dx_t = dy_t + exp(A_{t+1}) * dx_{t+1}
    dA_t = exp(A_t) * <dx_t, y_{t-1}>

Inputs are drawn as benchmark configuration 1 describes (x ~ N(0,1), alpha = sigmoid(u), u ~ N(2,1),
log-decay log(alpha), input (1 - alpha) * x) and stored as float32; the bf16 cases store
values already rounded to bfloat16.  Run `python tests/golden/make_golden.py` to rewrite."""
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

# name: (batch, nheads, seqlen, head_dim, chunk_size, seed, u_mean, bf16)
CASES = {
    "ema_config1_f32": (1, 2, 512, 64, 128, 1001, 2.0, False),
    "ema_ragged_f32": (2, 1, 300, 40, 64, 1002, 2.0, False),
    "ema_long_memory_f32": (1, 2, 384, 32, 128, 1003, 4.0, False),
    "ema_config1_bf16": (1, 2, 512, 64, 128, 1004, 2.0, True),
    "ema_chunk256_bf16": (1, 2, 768, 32, 256, 1005, 2.0, True),
}


def round_bf16(a):
    """float32 array rounded to the nearest bfloat16 (ties to even), returned as float32."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFF0000
    return u.view(np.float32)


def make_case(b, nh, L, d, seed, u_mean, bf16):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((b, L, nh, d))
    u = rng.standard_normal((b, L, nh)) + u_mean
    alpha = 1.0 / (1.0 + np.exp(-u))
    A = np.log(alpha).astype(np.float32)
    X = ((1.0 - alpha)[..., None] * x).astype(np.float32)
    dy = rng.standard_normal((b, L, nh, d)).astype(np.float32)
    if bf16:
        X, dy = round_bf16(X), round_bf16(dy)
    return A, X, dy


def scan_f64(A, X, dy):
    A64, X64, dy64 = A.astype(np.float64), X.astype(np.float64), dy.astype(np.float64)
    b, L, nh, d = X.shape
    a = np.exp(A64)
    y = np.zeros_like(X64)
    prev = np.zeros((b, nh, d))
    for t in range(L):
        prev = a[:, t, :, None] * prev + X64[:, t]
        y[:, t] = prev
    dx = np.zeros_like(X64)
    carry = np.zeros((b, nh, d))
    for t in range(L - 1, -1, -1):
        carry = dy64[:, t] + (a[:, t + 1, :, None] * carry if t + 1 < L else 0.0)
        dx[:, t] = carry
    dA = np.zeros_like(A64)
    for t in range(1, L):
        dA[:, t] = a[:, t] * np.einsum("bhd,bhd->bh", dx[:, t], y[:, t - 1])
    return y, dx, dA


def main():
    for name, (b, nh, L, d, Q, seed, u_mean, bf16) in CASES.items():
        A, X, dy = make_case(b, nh, L, d, seed, u_mean, bf16)
        y, dx, dA = scan_f64(A, X, dy)
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"),
            A=A, X=X, dy=dy, y=y.astype(np.float32), dx=dx.astype(np.float32), dA=dA.astype(np.float32),
            chunk_size=np.int64(Q), bf16=np.bool_(bf16),
        )
        print(name, X.shape, "chunk", Q, "bf16" if bf16 else "f32")


if __name__ == "__main__":
    main()
