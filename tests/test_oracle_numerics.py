"""Pins the CPU oracle's scalar numerics and row quantisers.

Every check compares the oracle with something that is NOT the oracle's own formula: numpy / torch casts,
the reference's byte goldens (tests/ep/unit/test_tilexr_ep_layout.cpp:128-190), the reference's golden
header compiled in place (oracle/_ref), closed forms and hand-picked cases that separate plausible mistakes
(divide vs multiply-by-reciprocal, round-half-even vs half-away, fused vs separate rounding).
"""
import numpy as np
import pytest
import torch

from oracle import ep as O

ALL_U16 = np.arange(65536, dtype=np.uint32).astype(np.uint16)


def test_half_decode_matches_numpy_exhaustive():
    want = ALL_U16.view(np.float16).astype(np.float32)
    got = np.array([O.half_to_float(b) for b in ALL_U16], np.float32)
    finite = np.isfinite(want)
    assert np.array_equal(got[finite].view(np.uint32), want[finite].view(np.uint32))
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_bf16_decode_matches_torch_exhaustive():
    t = torch.from_numpy(ALL_U16.astype(np.int32)).to(torch.int16).view(torch.bfloat16).float().numpy()
    got = np.array([O.bf16_to_float(b) for b in ALL_U16], np.float32)
    ok = ~np.isnan(t)
    assert np.array_equal(got[ok].view(np.uint32), t[ok].view(np.uint32))


def _sample_floats(seed, n):
    rng = np.random.default_rng(seed)
    bits = rng.integers(0, 2**32, size=n, dtype=np.uint64).astype(np.uint32)
    vals = bits.view(np.float32)
    vals = vals[np.isfinite(vals)]
    extra = np.array([0.0, -0.0, 65504.0, 65519.996, 65520.0, 65536.0, 1e9, -1e9, 2.0**-24, 2.0**-25,
                      1.0000001 * 2.0**-25, 2.0**-14, 0.99999 * 2.0**-14, 1.0009766, 1.00048828125,
                      1.00146484375, 3.3895314e38, 1.0 + 2.0**-8, 1.0 + 3 * 2.0**-9], np.float32)
    return np.concatenate([vals, extra, -extra, (rng.standard_normal(n) * 4).astype(np.float32)])


def test_float_to_half_matches_numpy():
    vals = _sample_floats(1, 20000)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([O.float_to_half(v) for v in vals], np.uint16)
    assert np.array_equal(got, want)
    # saturating flavour: identical below 65520, +-65504 (0x7bff) above
    got_sat = np.array([O.float_to_half(v, saturate=True) for v in vals], np.uint16)
    big = np.abs(vals) >= 65520.0
    assert np.array_equal(got_sat[~big], want[~big])
    assert np.all((got_sat[big] & 0x7fff) == 0x7bff)


def test_float_to_bf16_matches_torch():
    vals = _sample_floats(2, 20000)
    want = torch.from_numpy(vals).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([O.float_to_bf16(v) for v in vals], np.uint16)
    assert np.array_equal(got, want)


def test_clamp_int8_known_values():
    # src/ep/kernels/tilexr_ep_dispatch_kernel.cpp:183-193: +-0.5 then truncate: ties go AWAY from zero
    cases = {0.0: 0, 0.49: 0, 0.5: 1, -0.5: -1, 1.5: 2, 2.5: 3, -2.5: -3, 126.5: 127, 127.49: 127, 127.5: 127,
             300.0: 127, -127.5: -128, -128.4: -128, -129.0: -128, -1e20: -128, 1e20: 127}
    for v, want in cases.items():
        assert O.clamp_int8(v) == want, v


def _np_token_int8(row_f32):
    """Independent float32 numpy model of tilexr_ep_dispatch_helpers.h:153-191."""
    amax = np.float32(np.max(np.abs(row_f32))) if row_f32.size else np.float32(0)
    dequant = amax / np.float32(127.0) if amax > 0 else np.float32(1.0)
    quant = np.float32(1.0) / dequant
    v = (row_f32 * quant).astype(np.float32)
    r = np.where(v >= 0, v + np.float32(0.5), v - np.float32(0.5)).astype(np.float32)
    return np.clip(np.trunc(r), -128, 127).astype(np.int8), dequant


@pytest.mark.parametrize("decode", [O.DT_FP16, O.DT_BF16])
def test_token_int8_rows(decode):
    rng = np.random.default_rng(5)
    for h in (1, 7, 64, 1000, 4096):
        f = (rng.standard_normal(h) * 2).astype(np.float32)
        if decode == O.DT_FP16:
            bits = f.astype(np.float16).view(np.uint16)
            dec = bits.view(np.float16).astype(np.float32)
        else:
            bits = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
            dec = (bits.astype(np.uint32) << 16).view(np.float32)
        q, s = O.quant_row_token_int8(bits, decode)
        wq, ws = _np_token_int8(dec)
        assert s == ws
        assert np.array_equal(q, wq)
        # closed-form properties: the absmax element maps to +-127, everything within [-127, 127]
        assert abs(int(q[np.argmax(np.abs(dec))])) == 127
        assert q.min() >= -127 and q.max() <= 127
        # dequantised error is at most half a step (plus float slack)
        assert np.max(np.abs(q.astype(np.float32) * s - dec)) <= 0.5 * s * 1.0001


def test_token_int8_zero_row_and_reciprocal_form():
    q, s = O.quant_row_token_int8(np.zeros(16, np.uint16), O.DT_FP16)
    assert s == np.float32(1.0) and not q.any()
    # The reference multiplies by 1/scale instead of dividing (helpers.h:171-176).  Find an input where the two
    # differ and check the oracle follows the reciprocal form.
    rng = np.random.default_rng(11)
    found = 0
    for _ in range(4000):
        f = (rng.standard_normal(8) * 3).astype(np.float16)
        dec = f.astype(np.float32)
        amax = np.float32(np.max(np.abs(dec)))
        if amax == 0:
            continue
        scale = amax / np.float32(127)
        a = np.trunc(np.where(dec >= 0, dec * (np.float32(1) / scale) + np.float32(0.5),
                              dec * (np.float32(1) / scale) - np.float32(0.5)).astype(np.float32))
        b = np.trunc(np.where(dec >= 0, dec / scale + np.float32(0.5), dec / scale - np.float32(0.5))
                     .astype(np.float32))
        if not np.array_equal(a, b):
            q, _ = O.quant_row_token_int8(f.view(np.uint16), O.DT_FP16)
            assert np.array_equal(q, np.clip(a, -128, 127).astype(np.int8))
            found += 1
    assert found > 0


def test_token_int8_bf16_exhaustive_single_elements():
    """ext (bf16 decode): every finite bf16 value against a few row maxima, numpy float32 model."""
    pats = ALL_U16[(ALL_U16 & 0x7f80) != 0x7f80]
    vals = (pats.astype(np.uint32) << 16).view(np.float32)
    for top in (np.float32(1.0), np.float32(3.140625), np.float32(448.0)):
        keep = np.abs(vals) <= top
        top_bits = np.uint16(np.float32(top).view(np.uint32) >> 16)
        for chunk in np.array_split(np.nonzero(keep)[0], 8):
            row = np.concatenate([[top_bits], pats[chunk]]).astype(np.uint16)
            q, s = O.quant_row_token_int8(row, O.DT_BF16)
            wq, ws = _np_token_int8(np.concatenate([[top], vals[chunk]]).astype(np.float32))
            assert s == ws and np.array_equal(q, wq)


def test_static_int8_row():
    f = np.array([0.0, 1.0, -1.0, 0.5, 2.5, -2.5, 100.0, -100.0, 63.75], np.float16)
    q = O.quant_row_static_int8(f.view(np.uint16), 2.0)
    assert q.tolist() == [0, 2, -2, 1, 5, -5, 127, -128, 127]
    q = O.quant_row_static_int8(f.view(np.uint16), 0.25)
    # 0.5*0.25=0.125 -> 0; 2.5*0.25 = 0.625 -> 1; 63.75*.25 = 15.9375 -> 16
    assert q.tolist() == [0, 0, 0, 0, 1, -1, 25, -25, 16]


# ---------------------------------------------------------------------------------------------
# fp8 / MXFP8
# ---------------------------------------------------------------------------------------------
def test_fp8_reference_byte_goldens(known):
    g = known["mxfp8_bytes"]
    for fmt, dt in (("e4m3", O.DT_FP8E4M3), ("e5m2", O.DT_FP8E5M2)):
        spec = g[fmt]
        row = np.zeros(spec["h"], np.float32)
        for k, v in spec["inputs"].items():
            row[int(k)] = v
        bits = row.astype(np.float16).view(np.uint16)          # all inputs are exact in fp16
        assert np.array_equal(bits.view(np.float16).astype(np.float32), row)
        q, scales = O.quant_row_mxfp8(bits, O.DT_FP16, dt)
        for k, v in spec["elements"].items():
            assert q[int(k)] == v, (fmt, k)
        assert scales[: len(spec["scales"])].tolist() == spec["scales"]
        if "scale_count" in spec:
            assert len(scales) == spec["scale_count"]
    tb = g["two_blocks_e4m3"]
    row = np.full(tb["h"], tb["fill"], np.float32)
    for k, v in tb["inputs"].items():
        row[int(k)] = v
    q, scales = O.quant_row_mxfp8(row.astype(np.float16).view(np.uint16), O.DT_FP16, O.DT_FP8E4M3)
    assert scales.tolist() == tb["scales"] and len(scales) == tb["scale_count"]
    for k, v in tb["round_trip"].items():
        i = int(k)
        assert O.fp8_decode(q[i]) * 2.0 ** (int(scales[i // 32]) - 127) == v
    for d in g["decode"]:
        dt = O.DT_FP8E4M3 if d["fmt"] == "e4m3" else O.DT_FP8E5M2
        assert O.fp8_decode(d["byte"], dt) == d["value"]


@pytest.mark.parametrize("name,dt,tdt", [("e4m3", O.DT_FP8E4M3, torch.float8_e4m3fn),
                                          ("e5m2", O.DT_FP8E5M2, torch.float8_e5m2)])
def test_fp8_codec_matches_torch(name, dt, tdt):
    # decode: all 256 codes
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    want = codes.view(tdt).float().numpy()
    got = np.array([O.fp8_decode(int(c), dt) for c in range(256)], np.float32)
    ok = np.isfinite(want)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    # encode: in-range values round to nearest even exactly like torch's cast
    max_finite = 448.0 if name == "e4m3" else 57344.0
    rng = np.random.default_rng(3)
    vals = np.concatenate([
        (rng.standard_normal(20000) * 50).astype(np.float32),
        (rng.standard_normal(20000) * 2.0 ** rng.integers(-20, 9, 20000)).astype(np.float32),
        want[ok],
        np.array([2.0**-9, 2.0**-10, 3 * 2.0**-10, 2.0**-16, 2.0**-17, 3 * 2.0**-17, 0.0, -0.0], np.float32),
    ])
    vals = vals[np.abs(vals) <= max_finite]
    tw = torch.from_numpy(vals).to(tdt).view(torch.uint8).numpy()
    mine = np.array([O.fp8_encode(v, dt) for v in vals], np.uint8)
    assert np.array_equal(mine, tw)
    # saturation beyond the largest finite value (torch does not saturate, the reference golden does)
    top = 0x7e if name == "e4m3" else 0x7b
    for v in (max_finite * 1.01, max_finite * 1.2, 1e9, 3e38):
        assert O.fp8_encode(v, dt) == top and O.fp8_encode(-v, dt) == (top | 0x80)


def test_fp8_encode_matches_reference_golden_header(ref):
    rng = np.random.default_rng(9)
    vals = np.concatenate([
        (rng.standard_normal(30000) * 2.0 ** rng.integers(-24, 18, 30000)).astype(np.float32),
        (ALL_U16[::7].astype(np.uint32) << 16).view(np.float32),
    ])
    vals = vals[np.isfinite(vals)]
    for e5m2, dt in ((0, O.DT_FP8E4M3), (1, O.DT_FP8E5M2)):
        want = np.array([ref.lib().ref_fp8_encode(float(v), e5m2) for v in vals], np.uint8)
        got = np.array([O.fp8_encode(v, dt) for v in vals], np.uint8)
        assert np.array_equal(got, want)
        for c in range(256):
            a, b = O.fp8_decode(c, dt), ref.lib().ref_fp8_decode(c, e5m2)
            assert (np.isnan(a) and np.isnan(b)) or a == b


@pytest.mark.parametrize("dtype", [O.DT_FP16, O.DT_BF16])
@pytest.mark.parametrize("e5m2", [0, 1])
def test_mxfp8_rows_match_reference_golden_header(ref, dtype, e5m2):
    rng = np.random.default_rng(100 + dtype + e5m2)
    fp8 = O.DT_FP8E5M2 if e5m2 else O.DT_FP8E4M3
    for h in (1, 31, 32, 33, 64, 100, 1024, 7168):
        for scale in (1.0, 1e-3, 300.0, 2.0**-20):
            f = (rng.standard_normal(h) * scale).astype(np.float32)
            f[rng.integers(0, h)] = 0.0
            if h >= 64:
                f[32:64] = 0.0   # an all-zero block
            if dtype == O.DT_FP16:
                with np.errstate(over="ignore"):
                    bits = f.astype(np.float16).view(np.uint16)
                dec = bits.view(np.float16).astype(np.float32)
            else:
                bits = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
                dec = (bits.astype(np.uint32) << 16).view(np.float32)
            if not np.all(np.isfinite(dec)):
                continue
            q, s = O.quant_row_mxfp8(bits, dtype, fp8)
            rq, rs = ref.mxfp8_quant_row(dec, e5m2)
            assert np.array_equal(s, rs), (h, scale)
            assert np.array_equal(q, rq), (h, scale)


def test_mxfp8_scale_count():
    # tests/ep/demo/mxfp8_golden.h:26-30: ceil(h/32) rounded up to even
    assert [O.mxfp8_scale_count(h) for h in (1, 32, 33, 64, 65, 7168, 2048)] == [2, 2, 2, 2, 4, 224, 64]


def test_fp8_block128_matches_torch_cast():
    """ext: the reference has no per-128-column fp32-scale mode, so parity is pinned on torch's e4m3fn cast."""
    rng = np.random.default_rng(21)
    for h in (128, 2048, 200, 7168):
        t = torch.from_numpy(rng.standard_t(3, h).astype(np.float32)).to(torch.bfloat16)
        if h == 2048:
            t[256:384] = 0
        bits = t.view(torch.int16).numpy().view(np.uint16)
        q, s = O.quant_row_fp8_block128(bits, O.DT_BF16)
        x = t.float()
        pad = (-h) % 128
        xp = torch.nn.functional.pad(x, (0, pad)).view(-1, 128)
        amax = xp.abs().amax(dim=1)
        scale = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax))
        want = (xp / scale[:, None]).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).view(-1)[:h]
        assert np.array_equal(s, scale.numpy())
        assert np.array_equal(q, want.numpy())
        # the block maximum always lands on +-448
        for b in range(len(s)):
            blk = q[b * 128:(b + 1) * 128]
            if amax[b] > 0:
                assert (blk & 0x7f).max() == 0x7e
