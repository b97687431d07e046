"""Head sizes and state sizes outside what the SSD kernels take natively.

The kernels are built for headdim and dstate in {64, 128} (the Mamba-2 shapes).  The reference's
own tests and benchmarks also call its Mamba launchers on the EMA problem written as an SSD
one, with dstate = 1 and head sizes from 8 to 512 (kernels/tests/ema/test_ema_state_fwd.py:108-141,
kernels/benchmarks/ema/scan_fwd/scan_fwd_bench.py:20-68).  Those shapes are brought to a native
one around the same kernels:

  * a head wider than 128 is cut into sub-heads of 64 features: the recurrence treats the
    features of a head independently and only shares dt, A and D among them, so the sub-heads
    repeat those and per-head gradients are summed over them (views, no copy of x);
  * a narrower head is padded with zero features, a smaller state with zero state components;
    both contribute exact zeros and are cut off again.

The native shapes take none of this."""
import torch
import torch.nn.functional as F

NATIVE = (64, 128)


class Plan:
    def __init__(self, headdim, dstate=None):
        self.hd, self.ds = headdim, dstate
        if headdim in NATIVE:
            self.P, self.split = headdim, 1
        elif headdim < 64:
            self.P, self.split = 64, 1
        elif headdim < 128:
            self.P, self.split = 128, 1
        else:
            self.P, self.split = 64, -(-headdim // 64)
        self.hd_pad = self.P * self.split
        if dstate is None or dstate in NATIVE:
            self.N = dstate
        elif dstate < 64:
            self.N = 64
        elif dstate < 128:
            self.N = 128
        else:
            raise NotImplementedError(f"dstate {dstate} is larger than the SSD kernels take (128)")

    @property
    def native(self):
        return self.split == 1 and self.P == self.hd and self.N == self.ds

    # ---- tensors with a feature axis last: x, z, dout, out, dx (b, L, nh, hd)
    def x(self, t):
        if t is None:
            return None
        if self.hd_pad != self.hd:
            t = F.pad(t, (0, self.hd_pad - self.hd))
        b, L, nh, _ = t.shape
        return t.reshape(b, L, nh * self.split, self.P)

    def x_back(self, t):
        if t is None:
            return None
        b, L, nhs, _ = t.shape
        return t.reshape(b, L, nhs // self.split, self.hd_pad)[..., : self.hd]

    # ---- per-head arrays: dt / dA_cumsum (b, nh, C, Q), dA_chunk (b, nh, C), A / D (nh,)
    def per_head(self, t, axis=1):
        return t if t is None or self.split == 1 else t.repeat_interleave(self.split, dim=axis)

    def per_head_sum(self, t, axis=1):
        if t is None or self.split == 1:
            return t
        shape = list(t.shape)
        shape[axis: axis + 1] = [shape[axis] // self.split, self.split]
        return t.reshape(shape).sum(axis + 1)

    def D(self, D):
        if D is None:
            return None
        if D.dim() == 1:
            return self.per_head(D, 0)
        if self.hd_pad != self.hd:
            D = F.pad(D, (0, self.hd_pad - self.hd))
        return D.reshape(D.shape[0] * self.split, self.P)

    def dD_back(self, dD, D):
        if dD is None:
            return None
        if D.dim() == 1:
            return self.per_head_sum(dD, 0)
        return dD.reshape(D.shape[0], self.hd_pad)[:, : self.hd]

    # ---- B, C, dB, dC (b, L, g, ds)
    def bc(self, t):
        return t if t is None or self.N == self.ds else F.pad(t, (0, self.N - self.ds))

    def bc_back(self, t):
        return t if t is None or self.N == self.ds else t[..., : self.ds]

    # ---- states (b, C, nh, hd, ds)
    def states(self, t):
        if t is None:
            return None
        if self.N != self.ds or self.hd_pad != self.hd:
            t = F.pad(t, (0, self.N - self.ds, 0, self.hd_pad - self.hd))
        b, C, nh = t.shape[:3]
        return t.reshape(b, C, nh * self.split, self.P, self.N)

    def states_back(self, t):
        if t is None:
            return None
        b, C, nhs = t.shape[:3]
        return t.reshape(b, C, nhs // self.split, self.hd_pad, self.N)[..., : self.hd, : self.ds]
