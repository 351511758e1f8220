"""GPU parity, dense mat-vec jobs (maya_mv, the counterpart of glmf::mv): y = alpha * W x + bias against the CPU checker's
row dots on the same seeded rows and activations; every column bit-identical to the single-column call."""
import ctypes as C

import numpy as np
import pytest
import torch

from gpu_util import dev, rel_l2
import synth

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def lib():
    from maya_amd import lib as L
    L.load()
    L.check(L.load().maya_init())
    return L


def want_of(oracle, t, w, n_in, n_out, x, alpha, bias):
    out = np.empty((x.shape[0], n_out), dtype=np.float32)
    for c in range(x.shape[0]):
        dots = oracle.rows(t, w, n_in, n_out, oracle.quant_act(t, x[c]))
        v = np.float32(alpha) * dots
        out[c] = v + bias if bias is not None else v
    return out


CASES = [
    # type, n_in, n_out, columns, alpha, bias
    (8, 512, 64, 1, 1.0, False),
    (8, 2048, 301, 5, 0.5, True),
    (12, 1024, 77, 1, 1.0, True),
    (12, 7168, 512, 3, 1.0, False),
    (19, 1024, 130, 2, 2.0, False),
    (22, 2048, 777, 5, 1.0, True),
    (22, 7168, 256, 16, 0.25, False),
    (29, 1024, 96, 4, 1.0, True),
    (16, 1024, 130, 3, 1.0, True),
    (16, 7168, 64, 1, 0.5, False),
    (22, 16384, 40, 4, 1.0, False),     # long rows: the activations of 4 columns do not fit LDS at once
]


def q80_stream_rows(w, n_out, n_in):
    """Q8_0 rows from the GGUF block order (2-byte scale, 32 codes, ...) to the stream order (a row's codes, then its scales)."""
    g = w.reshape(n_out, n_in // 32, 34)
    return np.ascontiguousarray(np.concatenate([g[:, :, 2:].reshape(n_out, n_in), g[:, :, :2].reshape(n_out, -1)], axis=1)).reshape(-1)


# shapes the position-mapped kernels take (rows of 1024 NW values, n_out a multiple of 32; Q8_0 in the stream packing, Q4_K
# 16-byte aligned): type, n_in, n_out, columns, alpha, bias, packing
POS_CASES = [
    (8, 2048, 64, 1, 1.0, False, 1), (8, 7168, 96, 5, 0.5, True, 1), (8, 4096, 32, 8, 1.0, False, 1), (8, 6144, 64, 16, 1.0, True, 1),
    (8, 8192, 32, 3, 2.0, False, 1), (8, 2048, 16384, 2, 1.0, True, 1),
    (12, 7168, 64, 1, 1.0, True, 0), (12, 2048, 16384, 2, 0.25, False, 0), (12, 4096, 96, 4, 1.0, False, 1), (12, 8192, 32, 1, 1.0, True, 0),
    (12, 6144, 160, 3, 1.0, False, 0), (12, 5120, 64, 2, 1.0, True, 0), (8, 3072, 96, 4, 1.0, False, 1),
]


@pytest.mark.parametrize("t,n_in,n_out,ncol,alpha,with_bias,packing", [c + (0,) for c in CASES] + POS_CASES)
def test_mv_against_the_oracle_rows(lib, oracle, t, n_in, n_out, ncol, alpha, with_bias, packing):
    rng = np.random.default_rng(t * 1000 + n_out)
    w = synth.constructed_rows(t, n_out, n_in, rng)
    x = rng.standard_normal((ncol, n_in)).astype(np.float32)
    bias = rng.standard_normal(n_out).astype(np.float32) if with_bias else None
    want = want_of(oracle, t, w, n_in, n_out, x, alpha, bias)
    w_d, x_d = dev(q80_stream_rows(w, n_out, n_in) if (t == 8 and packing) else w), dev(x)
    job = dict(w=w_d, type=t, x=x_d, n_out=n_out, alpha=alpha, bias=None if bias is None else dev(bias), packing=packing)
    (got,) = lib.mv([job])
    torch.cuda.synchronize()
    assert rel_l2(got.cpu().numpy(), want) <= TOL
    # every column = the single-column call, bit for bit
    for c in range(ncol):
        (one,) = lib.mv([dict(job, x=x_d[c:c + 1].contiguous())])
        assert torch.equal(one[0], got[c]), c


def test_mv_jobs_of_several_types_in_one_call(lib, oracle):
    rng = np.random.default_rng(5)
    specs = [(8, 1024, 200, 2), (12, 2048, 128, 1), (22, 1024, 64, 4), (12, 512, 333, 3), (29, 768, 50, 1), (19, 512, 20, 2), (16, 768, 40, 2)]
    jobs, wants = [], []
    for t, n_in, n_out, ncol in specs:
        w = synth.constructed_rows(t, n_out, n_in, rng)
        x = rng.standard_normal((ncol, n_in)).astype(np.float32)
        wants.append(want_of(oracle, t, w, n_in, n_out, x, 1.0, None))
        jobs.append(dict(w=dev(w), type=t, x=dev(x), n_out=n_out))
    outs = lib.mv(jobs)
    torch.cuda.synchronize()
    for got, want in zip(outs, wants):
        assert rel_l2(got.cpu().numpy(), want) <= TOL


@pytest.mark.parametrize("t", (22, 8))
def test_mv_stream_packed_rows_give_the_same_bits(lib, t):
    """The down matrix of a repacked expert blob as a stream-packed job: the bits of the GGUF-packed job."""
    n_embd, n_ff, ncol = 1024, 512, 3
    rng = np.random.default_rng(9 + t)
    blob = synth.expert_blob(t, t, n_embd, n_ff, rng)
    l, _ = lib.layout(t, t, n_embd, n_ff)
    src = dev(blob)
    packed = torch.zeros_like(src)
    lib.repack(l, src, packed)
    x = dev(rng.standard_normal((ncol, n_ff)).astype(np.float32))
    (a,) = lib.mv([dict(w=src[l.down_off:], type=t, x=x, n_out=n_embd)])
    (b,) = lib.mv([dict(w=packed[l.down_off:], type=t, x=x, n_out=n_embd, packing=lib.PACK_STREAM)])
    torch.cuda.synchronize()
    assert torch.equal(a, b) and float(a.abs().max()) > 0


def test_mv_refusals_launch_nothing(lib):
    L = lib.load()
    x = torch.zeros((1, 512), device="cuda")
    act = lib.quant_act(12, x)
    y = torch.full((1, 8), 7.0, device="cuda")
    w = torch.zeros(lib.row_bytes(12, 512) * 8, dtype=torch.uint8, device="cuda")

    def call(**kw):
        f = dict(w=w.data_ptr(), type=12, packing=0, n_in=512, n_out=8, ncol=1, alpha=1.0, x=act.c(), bias=None,
                 y=y.data_ptr(), y_stride=8)
        f.update(kw)
        arr = (lib.MvJob * 1)(lib.MvJob(*[f[n] for n, _ in lib.MvJob._fields_]))
        return L.maya_mv(arr, 1, lib._stream())

    assert L.maya_mv_supported(12) == 1 and L.maya_mv_supported(10) == 0 and L.maya_mv_supported(16) == 1
    assert call(type=10) == 1            # MAYA_E_UNSUPPORTED
    assert call(n_in=100) == 2           # MAYA_E_SHAPE
    assert call(ncol=17) == 2
    assert call(y=None) == 3             # MAYA_E_ARG
    assert L.maya_mv((lib.MvJob * 1)(), 0, lib._stream()) == 3
    torch.cuda.synchronize()
    assert float(y.min()) == 7.0         # nothing ran
    assert call() == 0
    torch.cuda.synchronize()
    assert float(y.abs().max()) == 0.0   # zero weights
