"""Pins the oracle's W4 quantiser / layout against independent evidence (CPU only)."""
import numpy as np
import pytest

from oracle import moe_oracle as orc


def _scalar_quantize_group(vals):
    """quantize_tensor of pre_exp/expert_skip_prediction/quant.py:99-106 with bits=4 on ONE
    group, written with scalar numpy.float32/float16 operations only."""
    f32, f16 = np.float32, np.float16
    mn, mx = f32(min(vals)), f32(max(vals))
    scale = f16(f32(mx - mn) / f32(15))
    if not scale > 0:
        scale = f16(1.0)
    s = f32(scale)
    zero = f16(f32(0.0) - f32(mn / s))
    z = f32(zero)
    codes = []
    for v in vals:
        t = f32(f32(f32(v) / s) + z)
        r = float(np.rint(t))           # half-to-even, as torch.round
        codes.append(int(min(max(r, 0.0), 15.0)))
    return codes, scale, zero


def test_quantizer_matches_scalar_closed_form():
    rng = np.random.default_rng(0)
    w = (rng.standard_normal((6, 256)) * 0.02).astype(np.float32)
    w[1, :128] = 0.125                       # constant group
    w[2, 128:] = np.abs(w[2, 128:]) + 0.3    # zero point below 0
    q, s, z = orc.quantize_w4(w)
    codes = orc.unpack_codes(q)
    for n in range(6):
        for g in range(2):
            c, sc, zp = _scalar_quantize_group(list(w[n, 128 * g:128 * g + 128]))
            assert list(codes[n, 128 * g:128 * g + 128]) == c
            assert s[n, g].view(np.uint16) == np.float16(sc).view(np.uint16)
            assert z[n, g].view(np.uint16) == np.float16(zp).view(np.uint16)


def test_quantizer_invariants():
    rng = np.random.default_rng(1)
    w = (rng.standard_normal((32, 512)) * 0.02).astype(np.float32)
    q, s, z = orc.quantize_w4(w)
    codes = orc.unpack_codes(q).reshape(32, 4, 128)
    wg = w.reshape(32, 4, 128)
    assert codes.min() >= 0 and codes.max() <= 15
    # the minimum of each group gets code 0 and the maximum code 15
    assert (np.take_along_axis(codes, wg.argmin(2)[..., None], 2) == 0).all()
    assert (np.take_along_axis(codes, wg.argmax(2)[..., None], 2) == 15).all()
    deq = orc.dequantize_w4(q, s, z).reshape(32, 4, 128)
    sf = s.astype(np.float32)[..., None]
    # half a step, plus the fp16 rounding of the zero point (|zero| <= 16 -> 2^-7 steps)
    assert (np.abs(deq - wg) <= sf * (0.5 + 2.0 ** -6)).all()


def test_dequant_is_q_minus_zero_times_scale():
    q = np.array([[0x10, 0xF2] + [0] * 62], dtype=np.uint8)        # codes 0,1,2,15,0...
    s = np.array([[0.5]], dtype=np.float16)
    z = np.array([[1.25]], dtype=np.float16)
    deq = orc.dequantize_w4(q, s, z)
    assert deq[0, :4].tolist() == [(0 - 1.25) * 0.5, (1 - 1.25) * 0.5, (2 - 1.25) * 0.5, (15 - 1.25) * 0.5]


@pytest.mark.parametrize("stride,offset", [(1, 0), (2, 0), (2, 1)])
def test_pack_layout_bruteforce(stride, offset):
    rng = np.random.default_rng(2)
    n, kd = 32, 256
    q = rng.integers(0, 256, size=(n, kd // 2), dtype=np.uint8)
    s = rng.standard_normal((n, kd // 128)).astype(np.float16)
    z = rng.standard_normal((n, kd // 128)).astype(np.float16)
    qp, sz = orc.pack_w4(q, s, z, stride, offset)
    codes = orc.unpack_codes(q)
    pos = [0, 4, 1, 5, 2, 6, 3, 7]
    for b in range(n // 16):
        bd = b * stride + offset
        for g in range(kd // 128):
            for lane in range(64):
                r, kq = lane % 16, lane // 16
                assert sz[bd, g, r, 0] == s[16 * b + r, g] and sz[bd, g, r, 1] == z[16 * b + r, g]
                for j in range(4):
                    word = 0
                    for i in range(8):
                        word |= int(codes[16 * b + r, 128 * g + 32 * j + 8 * kq + i]) << (4 * pos[i])
                    assert int(qp[bd, g, lane, j]) == word
    # blocks the call did not address stay zero
    other = [b for b in range(qp.shape[0]) if (b - offset) % stride]
    assert not qp[other].any()
    q2, s2, z2 = orc.unpack_w4(qp, sz, stride, offset)
    assert np.array_equal(q2, q) and np.array_equal(s2, s) and np.array_equal(z2, z)


def test_fast_dequant_equals_the_numpy_statement():
    rng = np.random.default_rng(9)
    w = (rng.standard_normal((48, 640)) * 0.05 + rng.standard_normal((48, 1)) * 0.2).astype(np.float32)
    q, s, z = orc.quantize_w4(w)
    a, b = orc.dequantize_w4(q, s, z), orc.dequantize_w4_numpy(q, s, z)
    assert a.dtype == np.float32 and np.array_equal(a.view(np.uint32), b.view(np.uint32))
