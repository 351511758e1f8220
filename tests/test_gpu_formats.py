"""GPU parity, format layer: dequantized weights and quantized activations are bit-exact with the CPU checker."""
import numpy as np
import pytest
import torch

import synth

pytestmark = pytest.mark.gpu

TYPES = (8, 12, 16, 19, 22, 29)


@pytest.fixture(scope="module")
def lib():
    from maya_amd import lib as L
    L.load()
    L.check(L.load().maya_init())
    print("device:", L.load().maya_device_info().decode(), flush=True)
    return L


@pytest.mark.parametrize("t", TYPES)
@pytest.mark.parametrize("misalign", (0, 2))
def test_dequant_bit_exact(lib, oracle, t, misalign):
    rng = np.random.default_rng(40 + t)
    n, k = 12, 1024
    w = synth.constructed_rows(t, n, k, rng)
    want = oracle.dequant_rows(t, w, k, n)
    buf = torch.zeros(w.size + 16, dtype=torch.uint8, device="cuda")
    buf[misalign:misalign + w.size] = torch.from_numpy(w).cuda()
    got = lib.dequant_rows(t, buf[misalign:], k, n).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequant_subnormal_scales(lib, oracle):
    """FP16 block scales in the subnormal range and at the extremes decode to the same bits."""
    rng = np.random.default_rng(3)
    for t in (12, 22, 8, 19, 16):
        w = synth.constructed_rows(t, 2, 512, rng).reshape(-1, synth.BLOCK_BYTES[t])
        specials = np.array([0x0001, 0x03FF, 0x0400, 0x7BFF, 0x8001, 0x0000, 0x83FF, 0x3C00], dtype=np.uint16)
        for b in range(w.shape[0]):
            w[b, 0:2] = specials[b % 8: b % 8 + 1].view(np.uint8)
        w = w.reshape(-1)
        want = oracle.dequant_rows(t, w, 512, 2)
        got = lib.dequant_rows(t, torch.from_numpy(w).cuda(), 512, 2).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), t


def _x_cases(k, rng):
    x = rng.standard_normal((6, k)).astype(np.float32)
    x[1] *= 1e-3
    x[2, 256:512] = 0.0
    x[3, :256] = 0.5
    x[3, 300] = -7.0
    x[3, 301] = 7.0                      # equal magnitudes: the first one is the block's maximum
    x[4] = np.round(x[4] * 4) / 4        # many exact .5 products
    x[5, 512:768] = (np.arange(256) - 128).astype(np.float32) / 254.0 * 3.0
    return x


@pytest.mark.parametrize("dt", ("f32", "bf16", "f16"))
def test_q8k_quant_byte_exact(lib, oracle, dt):
    rng = np.random.default_rng(17)
    k = 1024
    x = _x_cases(k, rng)
    xt = torch.from_numpy(x)
    if dt == "bf16":
        xt = xt.to(torch.bfloat16)
    elif dt == "f16":
        xt = xt.to(torch.float16)
    xr = xt.to(torch.float32).numpy()
    act = lib.quant_act(22, xt.cuda().contiguous())
    q, d, bs = act.q.cpu().numpy(), act.d.cpu().numpy(), act.bsums.cpu().numpy()
    for r in range(x.shape[0]):
        wd, wq, wbs = oracle.q8k_fields(oracle.quant_q8k(xr[r]))
        assert np.array_equal(q[r], wq), (dt, r)
        assert np.array_equal(d[r].reshape(-1, 8).view(np.uint32), np.repeat(wd.view(np.uint32)[:, None], 8, 1)), (dt, r)
        assert np.array_equal(bs[r].reshape(-1, 16), wbs), (dt, r)


def test_q80_quant_byte_exact(lib, oracle):
    rng = np.random.default_rng(18)
    k = 512
    x = _x_cases(1024, rng)[:, :k].copy()
    act = lib.quant_act(8, torch.from_numpy(x).cuda())
    q, d = act.q.cpu().numpy(), act.d.cpu().numpy()
    for r in range(x.shape[0]):
        blocks = oracle.quant_act(8, x[r]).reshape(-1, 34)
        wq = blocks[:, 2:].copy().view(np.int8).reshape(-1)
        wd = blocks[:, 0:2].copy().view(np.float16).astype(np.float32).reshape(-1)
        assert np.array_equal(q[r], wq), r
        assert np.array_equal(d[r].view(np.uint32), wd.view(np.uint32)), r


def test_i8x32_quant_byte_exact(lib, oracle):
    rng = np.random.default_rng(19)
    x = _x_cases(1024, rng)
    idx = np.array([5, 0, 3, 3, 1], dtype=np.int32)
    q, d = lib.quant_i8x32(torch.from_numpy(x).cuda(), torch.from_numpy(idx).cuda(), rows=len(idx))
    q, d = q.cpu().numpy(), d.cpu().numpy()
    for r, src in enumerate(idx):
        wq, wd = oracle.quant_i8x32(x[src])
        assert np.array_equal(q[r], wq) and np.array_equal(d[r].view(np.uint32), wd.view(np.uint32))


@pytest.mark.parametrize("gt,dt", ((22, 22), (22, 12), (12, 22), (29, 8), (8, 8), (19, 19), (19, 22), (29, 29), (16, 16), (22, 16)))
def test_stream_packing_round_trip_and_values(lib, oracle, gt, dt):
    """maya_moe_repack regroups bytes only: unpack(repack(blob)) == blob, and the packed rows dequantize to the same bits."""
    n_embd, n_ff = 1024, 512
    rng = np.random.default_rng(gt * 100 + dt)
    blob = synth.expert_blob(gt, dt, n_embd, n_ff, rng)
    l, nbytes = lib.layout(gt, dt, n_embd, n_ff)
    assert nbytes == blob.size
    src = torch.from_numpy(blob).cuda()
    packed = torch.zeros_like(src)
    back = torch.zeros_like(src)
    lib.repack(l, src, packed)
    lib.unpack(l, packed, back)
    torch.cuda.synchronize()
    assert torch.equal(back, src)
    # a permutation of bytes inside each quad of rows: same multiset of bytes per quad
    for t, off, k, rows in ((gt, 0, n_embd, n_ff), (gt, l.up_off, n_embd, n_ff), (dt, l.down_off, n_ff, n_embd)):
        rb = lib.row_bytes(t, k)
        a = src[off:off + rb * rows].view(rows // 4, 4 * rb).cpu().numpy()
        b = packed[off:off + rb * rows].view(rows // 4, 4 * rb).cpu().numpy()
        if t != 29:   # (IQ1_M regroups bits, not bytes: the block scale's four nibbles are put together)
            assert np.array_equal(np.sort(a, axis=1), np.sort(b, axis=1))
        if t == 29:
            # per quad the sub-blocks' index words [u][row], their qh words, then 8 bytes a (block, row): the FP16 block scale
            # gathered from the top nibbles of the four scale words, then their 4 x 12 bits of 3-bit scales in order
            nu = k // 32
            g = src[off:off + rb * rows].view(rows // 4, 4, nu // 8, 56).cpu().numpy()
            p = packed[off:off + rb * rows].view(rows // 4, 4 * rb).cpu().numpy()
            want_i = g[:, :, :, 0:32].reshape(rows // 4, 4, nu, 4).transpose(0, 2, 1, 3).reshape(rows // 4, -1)
            want_h = g[:, :, :, 32:48].reshape(rows // 4, 4, nu, 2).transpose(0, 2, 1, 3).reshape(rows // 4, -1)
            w = g[:, :, :, 48:56].copy().view(np.uint16).astype(np.uint64)        # [quad][row][block][4]
            d = (w[..., 0] >> 12) | ((w[..., 1] >> 8) & 0xf0) | ((w[..., 2] >> 4) & 0xf00) | (w[..., 3] & 0xf000)
            rec = d | ((w[..., 0] & 0xfff) << 16) | ((w[..., 1] & 0xfff) << 28) | ((w[..., 2] & 0xfff) << 40) | ((w[..., 3] & 0xfff) << 52)
            want_s = np.ascontiguousarray(rec.transpose(0, 2, 1)).view(np.uint8).reshape(rows // 4, -1)
            assert np.array_equal(p[:, :16 * nu], want_i) and np.array_equal(p[:, 16 * nu:24 * nu], want_h)
            assert np.array_equal(p[:, 24 * nu:], want_s)
        elif t == 8:
            # Q8_0: a row's codes first, then its scales
            g = src[off:off + rb * rows].view(rows, k // 32, 34).cpu().numpy()
            p = packed[off:off + rb * rows].view(rows, rb).cpu().numpy()
            assert np.array_equal(p[:, :k], g[:, :, 2:].reshape(rows, k)) and np.array_equal(p[:, k:], g[:, :, :2].reshape(rows, -1))
        elif t == 19:
            # IQ1_S: per quad the sub-blocks' index words [u][row], then their qh words, then the block scales [block][row]
            nu = k // 32
            g = src[off:off + rb * rows].view(rows // 4, 4, nu // 8, 50).cpu().numpy()
            p = packed[off:off + rb * rows].view(rows // 4, 4 * rb).cpu().numpy()
            want_i = g[:, :, :, 2:34].reshape(rows // 4, 4, nu, 4).transpose(0, 2, 1, 3).reshape(rows // 4, -1)
            want_h = g[:, :, :, 34:50].reshape(rows // 4, 4, nu, 2).transpose(0, 2, 1, 3).reshape(rows // 4, -1)
            want_d = g[:, :, :, 0:2].transpose(0, 2, 1, 3).reshape(rows // 4, -1)
            assert np.array_equal(p[:, :16 * nu], want_i) and np.array_equal(p[:, 16 * nu:24 * nu], want_h)
            assert np.array_equal(p[:, 24 * nu:], want_d)
        elif t != 22:
            assert np.array_equal(a, b)
        want = oracle.dequant_rows(t, blob[off:off + rb * 16], k, 16)
        got = lib.dequant_rows(t, packed[off:], k, 16, packing=1).cpu().numpy()
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("gt,dt,pad", ((22, 22, 0), (22, 12, 64), (12, 12, 0), (8, 8, 32), (19, 29, 0)))
def test_pack_experts_from_stacked_tensors(lib, gt, dt, pad):
    """A layer's blobs built on the device from ffn_{gate,up,down}_exps as the file stores them ([expert][rows][row bytes]):
    GGUF order = the host concatenation gate | up | down of each expert; stream order = maya_moe_repack of that blob."""
    n_embd, n_ff, ne = 512, 256, 5
    rng = np.random.default_rng(gt * 7 + dt)
    blobs = [synth.expert_blob(gt, dt, n_embd, n_ff, rng) for _ in range(ne)]
    l, nbytes = lib.layout(gt, dt, n_embd, n_ff)
    gate = np.stack([b[:l.up_off] for b in blobs])
    up = np.stack([b[l.up_off:l.down_off] for b in blobs])
    down = np.stack([b[l.down_off:] for b in blobs])
    stride = nbytes + pad
    g_d, u_d, d_d = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (gate, up, down))
    for packing in (0, 1):
        pool = torch.full((ne * stride,), 0xA5, dtype=torch.uint8, device="cuda")
        lib.pack_experts(l, g_d, u_d, d_d, ne, packing, pool, stride)
        torch.cuda.synchronize()
        got = pool.view(ne, stride).cpu().numpy()
        assert (got[:, nbytes:] == 0xA5).all()          # nothing written between the blobs
        for e in range(ne):
            if packing == 0:
                want = blobs[e]
            else:
                w = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
                lib.repack(l, torch.from_numpy(blobs[e]).cuda(), w)
                want = w.cpu().numpy()
            assert np.array_equal(got[e, :nbytes], want), (packing, e)


def test_pack_experts_refusals(lib):
    L = lib.load()
    l, nbytes = lib.layout(22, 22, 512, 256)
    a = torch.zeros(nbytes, dtype=torch.uint8, device="cuda")
    dst = torch.full((nbytes + 16,), 7, dtype=torch.uint8, device="cuda")
    args = lambda **kw: [kw.get("l", l), a.data_ptr(), kw.get("up", a.data_ptr()), a.data_ptr(), kw.get("ne", 1), kw.get("packing", 1),
                         kw.get("dst", dst.data_ptr()), kw.get("stride", nbytes), lib._stream()]
    import ctypes as C
    call = lambda **kw: L.maya_moe_pack_experts(C.byref(args(**kw)[0]), *args(**kw)[1:])
    assert call(up=None) == 3                       # MAYA_E_ARG
    assert call(ne=0) == 2                          # MAYA_E_SHAPE
    assert call(stride=nbytes - 1) == 2
    assert call(packing=2) == 1                     # MAYA_E_UNSUPPORTED
    assert call(dst=dst.data_ptr() + 2) == 3        # a stream blob must be 16-byte aligned
    torch.cuda.synchronize()
    assert int(dst.min()) == 7 and int(dst.max()) == 7
    assert call(dst=dst.data_ptr() + 2, packing=0) == 0   # GGUF order takes any alignment
