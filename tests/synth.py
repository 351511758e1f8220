"""Seeded synthetic expert weights in the GGUF block formats, as "constructed blocks": random bytes with a valid FP16
block scale.  Every bit pattern of the quantized fields of these formats is a legal encoding, so random bytes exercise the
whole decode (the reference's fixtures are built the same way: tools/iq_fixture.py:13-18, 69-83;
tests/hip/expert_kernel_bench.cpp:68-77).  numpy only; no device code here.
"""
import numpy as np

Q8_0, Q4_K, IQ2_XXS, IQ1_S, IQ2_S, IQ1_M = 8, 12, 16, 19, 22, 29
BLOCK_BYTES = {Q8_0: 34, Q4_K: 144, IQ2_XXS: 66, IQ1_S: 50, IQ2_S: 82, IQ1_M: 56}
BLOCK_VALUES = {Q8_0: 32, Q4_K: 256, IQ2_XXS: 256, IQ1_S: 256, IQ2_S: 256, IQ1_M: 256}
# the block scale's range a type (tools/iq_fixture.py:40-60 gives IQ2_S [2e-3, 6e-3]); chosen so that rows of
# thousands of values have O(1) sums
D_RANGE = {Q8_0: (1e-4, 4e-4), Q4_K: (2e-4, 6e-4), IQ2_XXS: (2e-3, 6e-3), IQ1_S: (4e-3, 1.2e-2), IQ2_S: (2e-3, 6e-3),
           IQ1_M: (4e-3, 1.2e-2)}


def row_bytes(t, k):
    assert k % BLOCK_VALUES[t] == 0
    return k // BLOCK_VALUES[t] * BLOCK_BYTES[t]


def _f16_bits(lo, hi, n, rng):
    return rng.uniform(lo, hi, size=n).astype(np.float16).view(np.uint16)


def constructed_rows(t, n_rows, k, rng, d_scale=1.0):
    """n_rows rows of k values of type t -> uint8 [n_rows * row_bytes]."""
    nb = n_rows * (k // BLOCK_VALUES[t])
    bb = BLOCK_BYTES[t]
    blocks = rng.integers(0, 256, size=(nb, bb), dtype=np.uint8)
    lo, hi = D_RANGE[t]
    lo, hi = lo * d_scale, hi * d_scale
    d = _f16_bits(lo, hi, nb, rng)
    if t == IQ1_M:
        # the FP16 super-scale lives in the top nibbles of the four u16 scale words (bytes 48..55)
        sc = blocks[:, 48:56].copy().view(np.uint16).reshape(nb, 4)
        sc[:, 0] = (sc[:, 0] & 0x0FFF) | ((d & 0x000F) << 12)
        sc[:, 1] = (sc[:, 1] & 0x0FFF) | ((d & 0x00F0) << 8)
        sc[:, 2] = (sc[:, 2] & 0x0FFF) | ((d & 0x0F00) << 4)
        sc[:, 3] = (sc[:, 3] & 0x0FFF) | (d & 0xF000)
        blocks[:, 48:56] = sc.view(np.uint8).reshape(nb, 8)
    else:
        blocks[:, 0:2] = d.view(np.uint8).reshape(nb, 2)
        if t == Q4_K:
            dm = _f16_bits(lo, hi, nb, rng)
            blocks[:, 2:4] = dm.view(np.uint8).reshape(nb, 2)
    return blocks.reshape(-1)


def expert_blob(gu_type, d_type, n_embd, n_ff, rng, up_type=None):
    """[gate rows | up rows | down rows] (include/strata/kernels/cpu/native_expert.hpp:26-39) as uint8."""
    up_type = gu_type if up_type is None else up_type
    return np.concatenate([
        constructed_rows(gu_type, n_ff, n_embd, rng),
        constructed_rows(up_type, n_ff, n_embd, rng),
        constructed_rows(d_type, n_embd, n_ff, rng),
    ])


def blob_offsets(gu_type, d_type, n_embd, n_ff, up_type=None):
    """(up_off, down_off, bytes) of an expert blob."""
    up_type = gu_type if up_type is None else up_type
    up_off = n_ff * row_bytes(gu_type, n_embd)
    down_off = up_off + n_ff * row_bytes(up_type, n_embd)
    return up_off, down_off, down_off + n_embd * row_bytes(d_type, n_ff)
