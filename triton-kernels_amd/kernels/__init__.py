"""MI355X-native EMA chunked scan behind the reference's module layout.

`kernels.ema_kernels.*` and `kernels.ema_kernels_bwd.*` carry the same function names and
positional signatures as kartiksrinivas007/triton-kernels; every function launches
hand-written gfx950 kernels through libema_hip.so.  Sequence tensors may be flat
(B, L, T) with a (B, L) log-decay, as in the reference, or headed (b, L, nh, d) with a
(b, L, nh) log-decay; chunked intermediates are indexed by n = b * nh + h.
"""
