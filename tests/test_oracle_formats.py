"""Pins the CPU oracle before anything is compared against it.

The reference's own tests hold no vector for this path (its kernels are closed
binaries), so the pins are: the block decoders that ARE in the reference's
text (restated in np_formats.py), closed forms, invariants, brute force over
small inputs and library routines (numpy float16, torch float8_e4m3fn).
"""
import numpy as np
import pytest
import torch

import lowbit_oracle as orc
import np_formats as npf

Q4_0, Q4_1, Q8_0, NF4, FP8 = 2, 3, 8, 10, 15
ALL = [Q4_0, Q4_1, Q8_0, NF4, FP8]


def rng(seed):
    return np.random.default_rng(seed)


# ---------------------------------------------------------------- geometry

def test_block_geometry():
    # gguf.py:167-205 pins the first three; nf4 / fp8_e4m3 are this build's frozen formats
    assert [(orc.qk_size(q), orc.type_size(q)) for q in ALL] == \
        [(32, 18), (32, 20), (32, 34), (64, 34), (128, 132)]
    assert orc.qk_size(12) == 0 and orc.type_size(99) == 0


# -------------------------------------------------------------- fp16 / fp8

def test_f16_to_f32_exhaustive():
    L = orc.lib()
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([L.oracle_f16_to_f32(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f32_to_f16_rne_against_numpy():
    L = orc.lib()
    r = rng(1)
    # every half-way point between consecutive halves, and its two fp32 neighbours
    h = np.arange(0, 0x7c00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    cases = np.concatenate([
        mid, np.nextafter(mid, np.float32(0)), np.nextafter(mid, np.float32(np.inf)),
        -mid, r.standard_normal(20000).astype(np.float32) * 0.02,
        (r.standard_normal(20000) * 1e-6).astype(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 1e9, -1e9, 2.0 ** -25, 2.0 ** -24,
                  np.nextafter(np.float32(2.0 ** -25), np.float32(1))], dtype=np.float32),
        r.integers(0, 2 ** 32, 50000, dtype=np.uint64).astype(np.uint32).view(np.float32)])
    cases = cases[~np.isnan(cases)]
    with np.errstate(over="ignore"):
        want = cases.astype(np.float16).view(np.uint16)
    got = np.array([L.oracle_f32_to_f16(float(c)) for c in cases], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_e4m3fn_decode_all_codes_against_torch():
    L = orc.lib()
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    want = codes.view(torch.float8_e4m3fn).float().numpy()
    got = np.array([L.oracle_e4m3fn_to_f32(int(c)) for c in range(256)], dtype=np.float32)
    nan = np.isnan(want)
    assert nan.sum() == 2 and np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_e4m3fn_encode_rne_against_torch():
    L = orc.lib()
    r = rng(2)
    grid = torch.arange(0, 0x7f, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn)
    g = grid.float().numpy().astype(np.float64)
    mid = ((g[:-1] + g[1:]) / 2).astype(np.float32)
    cases = np.concatenate([
        g.astype(np.float32), mid, np.nextafter(mid, np.float32(0)),
        np.nextafter(mid, np.float32(1e9)), -mid,
        (r.standard_normal(50000) * 100).astype(np.float32),
        (r.standard_normal(20000) * 0.01).astype(np.float32),
        np.array([448.0, 463.9, -448.0, 0.0, -0.0, 2.0 ** -9, 2.0 ** -10, 3 * 2.0 ** -11],
                 dtype=np.float32)])
    cases = cases[np.abs(cases) < 464.0]          # torch maps >= 464 to NaN, the oracle saturates
    want = torch.from_numpy(cases).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    got = np.array([L.oracle_f32_to_e4m3fn(float(c)) for c in cases], dtype=np.uint8)
    assert np.array_equal(got, want)
    # saturation and NaN
    assert L.oracle_f32_to_e4m3fn(1e6) == 0x7e and L.oracle_f32_to_e4m3fn(-500.0) == 0xfe
    assert L.oracle_f32_to_e4m3fn(float("nan")) & 0x7f == 0x7f


# ----------------------------------------- decoders against the reference text

@pytest.mark.parametrize("qtype", ALL)
def test_dequantize_matches_independent_decoder_on_random_blobs(qtype):
    # random *bytes* (not quantizer output): exercises every code and nibble position
    r = rng(10 + qtype)
    nb = 64
    ts, qk = orc.type_size(qtype), orc.qk_size(qtype)
    blob = r.integers(0, 256, nb * ts, dtype=np.uint8).reshape(nb, ts)
    # keep scales finite: overwrite header fields with sane fp16 / fp32 values
    if qtype == FP8:
        blob[:, :4] = (r.random(nb).astype(np.float32) + 0.01).reshape(-1, 1).view(np.uint8)
        body = blob[:, 4:]
        body[(body & 0x7f) == 0x7f] = 0x3c      # no NaN codes
    else:
        blob[:, :2] = (r.standard_normal(nb).astype(np.float16)).reshape(-1, 1).view(np.uint8)
        if qtype == Q4_1:
            blob[:, 2:4] = (r.standard_normal(nb).astype(np.float16)).reshape(-1, 1).view(np.uint8)
    blob = blob.reshape(-1)
    got = orc.dequantize(blob, qtype, (nb, qk))
    want = npf.DECODERS[qtype](blob, (nb, qk))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def test_q4_1_blob_from_reference_writer_layout_decodes():
    # convert.py:417-453 writes [d, m=-(zero*scale), qs]; w = code*scale - zero*scale
    r = rng(3)
    rows, k = 4, 128
    codes = r.integers(0, 16, (rows, k), dtype=np.uint8)
    scales = (r.random((rows, k // 32)) * 0.02 + 0.001).astype(np.float16)
    zeros = r.integers(1, 16, (rows, k // 32)).astype(np.float16)
    blob = npf.write_q4_1_from_codes(codes, scales, zeros)
    got = orc.dequantize(blob, Q4_1, (rows, k))
    s = np.repeat(scales.astype(np.float32), 32, axis=1)
    m = np.repeat((-(zeros * scales)).astype(np.float16).astype(np.float32), 32, axis=1)
    want = codes.astype(np.float32) * s + m
    assert np.array_equal(got, want)


# ------------------------------------------------ quantizer: closed forms

def test_all_zero_blocks():
    z = np.zeros((2, 128), dtype=np.float32)
    b = orc.quantize(z, Q4_0).reshape(-1, 18)
    # d = 0.0f / -8.0f is IEEE negative zero: the scale bytes are 00 80, not 00 00
    assert (b[:, 0] == 0).all() and (b[:, 1] == 0x80).all() and (b[:, 2:] == 0x88).all()
    b = orc.quantize(z, Q4_1).reshape(-1, 20)
    assert (b == 0).all()
    b = orc.quantize(z, Q8_0).reshape(-1, 34)
    assert (b == 0).all()
    b = orc.quantize(z, NF4).reshape(-1, 34)
    assert (b[:, :2] == 0).all() and (b[:, 2:] == 0x77).all()
    b = orc.quantize(z, FP8).reshape(-1, 132)
    assert (b == 0).all()
    for q in ALL:
        assert (orc.dequantize(orc.quantize(z, q), q, z.shape) == 0).all()


def test_q4_0_exact_ramp():
    # block = c * [-8..7, -8..7]: the largest magnitude is -8c (first), d = c, codes 0..15
    for c in (0.5, 0.015625, 3.0):
        x = (np.tile(np.arange(-8, 8), 2) * c).astype(np.float32)
        b = orc.quantize(x.reshape(1, 32), Q4_0)
        assert b[:2].view(np.float16)[0] == np.float16(c)
        codes = np.concatenate([b[2:] & 0xF, b[2:] >> 4])
        assert np.array_equal(codes, np.tile(np.arange(16), 2))
        assert np.array_equal(orc.dequantize(b, Q4_0, (1, 32)).ravel(), x)


def test_q4_0_positive_max_gives_negative_scale_and_clamp():
    # max = +a: d = -a/8, the max itself maps to code 0, and -a would map to 16 -> clamped to 15
    x = np.zeros(32, dtype=np.float32)
    x[5] = 4.0
    x[20] = -4.0            # same magnitude, later: the FIRST largest (+4 at index 5) wins
    b = orc.quantize(x.reshape(1, 32), Q4_0)
    assert b[:2].view(np.float16)[0] == np.float16(-0.5)
    codes = np.concatenate([b[2:] & 0xF, b[2:] >> 4])
    assert codes[5] == 0 and codes[20] == 15
    assert (np.delete(codes, [5, 20]) == 8).all()
    # swapped order: -4 first -> d = +0.5, -4 -> code 0, +4 -> 16 -> 15
    x[5], x[20] = -4.0, 4.0
    b = orc.quantize(x.reshape(1, 32), Q4_0)
    assert b[:2].view(np.float16)[0] == np.float16(0.5)
    codes = np.concatenate([b[2:] & 0xF, b[2:] >> 4])
    assert codes[5] == 0 and codes[20] == 15


def test_q4_0_ties_round_half_up_and_nibble_positions():
    # d = 1 (max = -8 at index 0); x = c - 8 + 0.5 sits exactly between codes c and c+1
    x = np.zeros(32, dtype=np.float32)
    x[0] = -8.0
    x[1:16] = np.arange(0, 15) - 8 + 0.5      # -> codes 1..15
    x[16:32] = np.arange(16) - 8              # -> codes 0..15 in the HIGH nibbles
    b = orc.quantize(x.reshape(1, 32), Q4_0)
    lo, hi = b[2:] & 0xF, b[2:] >> 4
    assert lo[0] == 0 and np.array_equal(lo[1:], np.arange(1, 16))
    assert np.array_equal(hi, np.arange(16))


def test_q4_1_exact_ramp_and_fields():
    for (c, m) in ((0.25, -1.0), (0.125, 3.0)):
        x = (np.tile(np.arange(16), 2) * c + m).astype(np.float32)
        b = orc.quantize(x.reshape(1, 32), Q4_1)
        assert b[:2].view(np.float16)[0] == np.float16(c)
        assert b[2:4].view(np.float16)[0] == np.float16(m)
        codes = np.concatenate([b[4:] & 0xF, b[4:] >> 4])
        assert np.array_equal(codes, np.tile(np.arange(16), 2))
        assert np.array_equal(orc.dequantize(b, Q4_1, (1, 32)).ravel(), x)
    # constant block: d = 0, every code 0, m carries the value
    x = np.full(32, 0.75, dtype=np.float32)
    b = orc.quantize(x.reshape(1, 32), Q4_1)
    assert b[:2].view(np.uint16)[0] == 0 and (b[4:] == 0).all()
    assert np.array_equal(orc.dequantize(b, Q4_1, (1, 32)).ravel(), x)


def test_q8_0_exact_and_half_away_from_zero():
    x = np.zeros(32, dtype=np.float32)
    x[0] = 127.0                  # d = 1
    x[1], x[2], x[3], x[4] = 0.5, -0.5, 1.5, -2.5   # roundf: 1, -1, 2, -3
    x[5], x[6] = 0.49999997, -126.4
    b = orc.quantize(x.reshape(1, 32), Q8_0)
    assert b[:2].view(np.float16)[0] == np.float16(1.0)
    q = b[2:].view(np.int8)
    assert list(q[:7]) == [127, 1, -1, 2, -3, 0, -126]
    x = (np.arange(-16, 16) * 0.5).astype(np.float32)
    x[0] = -63.5                  # amax = 63.5 -> d = 0.5
    b = orc.quantize(x.reshape(1, 32), Q8_0)
    assert np.array_equal(orc.dequantize(b, Q8_0, (1, 32)).ravel(), x)


def test_nf4_codebook_block_is_exact():
    cb = orc.nf4_codebook()
    assert np.array_equal(cb, npf.NF4.astype(np.float32))
    for d in (1.0, 0.25, 0.0234375):
        x = np.concatenate([cb, cb[::-1], cb, cb[::-1]]) * np.float32(d)
        b = orc.quantize(x.reshape(1, 64).astype(np.float32), NF4)
        assert b[:2].view(np.float16)[0] == np.float16(d)
        lo, hi = b[2:] & 0xF, b[2:] >> 4
        want = np.concatenate([np.arange(16), np.arange(15, -1, -1)] * 2)
        assert np.array_equal(np.concatenate([lo, hi]), want)


def test_nf4_index_is_brute_force_nearest():
    # fine grid in [-1, 1] scaled by a power of two so that x * (1/d) is exact
    g = np.linspace(-1, 1, 64 * 257).astype(np.float32)
    g[0], g[-1] = -1.0, 1.0
    x = g.reshape(-1, 64).copy()
    x[:, 0] = 1.0                                   # absmax = 1 in every block
    blob = orc.quantize(x, NF4).reshape(-1, 34)
    idx = np.concatenate([blob[:, 2:] & 0xF, blob[:, 2:] >> 4], axis=1)
    dist = np.abs(x.astype(np.float64)[..., None] - npf.NF4[None, None, :])
    want = dist.argmin(axis=-1)                     # first minimum = lower index on ties
    # fp32 midpoints vs fp64 argmin may differ only within 1 ulp of a midpoint
    mids = (npf.NF4[:-1] + npf.NF4[1:]) / 2
    near = (np.abs(x.astype(np.float64)[..., None] - mids).min(axis=-1) < 1e-7)
    assert np.array_equal(idx[~near], want[~near])
    assert near.sum() < 10


def test_fp8_grid_block_roundtrips_bit_exact():
    codes = torch.arange(0, 0x7f, dtype=torch.int32).to(torch.uint8)
    grid = codes.view(torch.float8_e4m3fn).float().numpy()           # 127 non-negative values
    for s in (1.0, 0.5, 2.0 ** -10):
        x = np.concatenate([grid, [448.0]]).astype(np.float32) * np.float32(s)
        x[1::2] *= -1
        b = orc.quantize(x.reshape(1, 128), FP8)
        assert b[:4].view(np.float32)[0] == np.float32(s)
        assert np.array_equal(orc.dequantize(b, FP8, (1, 128)).ravel(), x)
        want = torch.from_numpy(x / np.float32(s)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(b[4:], want)


# -------------------------------------------------- quantizer: invariants

def _weights(seed, shape, std=0.02, outliers=True):
    r = rng(seed)
    w = (r.standard_normal(shape) * std).astype(np.float32)
    if outliers:
        mask = r.random(shape) < 0.001
        w[mask] = np.where(r.random(mask.sum()) < 0.5, 0.5, -0.5)
    return w


@pytest.mark.parametrize("qtype", [Q4_0, Q4_1, Q8_0])
def test_transcription_agrees_on_seeded_weights(qtype):
    w = _weights(100 + qtype, (64, 512))
    fn = {Q4_0: npf.quant_q4_0, Q4_1: npf.quant_q4_1, Q8_0: npf.quant_q8_0}[qtype]
    assert np.array_equal(orc.quantize(w, qtype), fn(w))


@pytest.mark.parametrize("qtype", ALL)
def test_error_bound_and_scale_sign(qtype):
    w = _weights(200 + qtype, (32, 1024))
    blob = orc.quantize(w, qtype)
    dq = npf.DECODERS[qtype](blob, w.shape)
    qk = orc.qk_size(qtype)
    wb, db = w.reshape(-1, qk), dq.reshape(-1, qk)
    amax = np.abs(wb).max(axis=1, keepdims=True)
    err = np.abs(wb - db)
    if qtype == Q4_0:
        d = amax / 8
        # nearest code: |d|/2; the +8 -> 15 clamp costs up to |d|; fp16 scale slack
        assert (err <= d * (1.0 + 8 * 2.0 ** -10) + 1e-12).all()
        assert (err <= d * (0.5 + 8 * 2.0 ** -10) + 1e-12).mean() > 0.95
        # the largest element decodes to fp16(d) * -8 exactly and has code 0
        t = blob.reshape(-1, 18)
        dh = t[:, :2].copy().view(np.float16).astype(np.float32).ravel()
        i = np.abs(wb).argmax(axis=1)
        mx = wb[np.arange(len(i)), i]
        assert (np.sign(dh) == -np.sign(mx)).all()
        assert np.array_equal(db[np.arange(len(i)), i], dh * -8)
    elif qtype == Q4_1:
        d = (wb.max(axis=1, keepdims=True) - wb.min(axis=1, keepdims=True)) / 15
        assert (err <= d * (0.5 + 16 * 2.0 ** -10) + np.abs(wb).max() * 2.0 ** -10).all()
    elif qtype == Q8_0:
        assert (err <= amax / 127 * (0.5 + 127 * 2.0 ** -10) + 1e-12).all()
    elif qtype == NF4:
        gap = np.diff(npf.NF4).max() / 2
        assert (err <= amax * (gap + 2.0 ** -10) + 1e-12).all()
    else:
        # e4m3: relative 2^-4 for normals, absolute s * 2^-10 near zero
        s = amax / 448
        assert (err <= np.maximum(np.abs(wb) * 2.0 ** -4, s * 2.0 ** -10) * 1.001 + 1e-12).all()


@pytest.mark.parametrize("qtype", ALL)
def test_requantizing_a_dequantized_tensor_is_idempotent(qtype):
    w = _weights(300 + qtype, (16, 512))
    b1 = orc.quantize(w, qtype)
    w1 = orc.dequantize(b1, qtype, w.shape)
    b2 = orc.quantize(w1, qtype)
    w2 = orc.dequantize(b2, qtype, w.shape)
    if qtype in (Q8_0, NF4, FP8, Q4_0):
        assert np.array_equal(w1, w2)
    else:
        # asym_int4: min and scale are re-rounded to fp16, values move by at most a few fp16 ulps
        assert np.abs(w1 - w2).max() <= np.abs(w1).max() * 2.0 ** -9


def test_q4_0_brute_force_nearest_code_on_exact_inputs():
    # d = 2^-4 (max = -0.5 first); inputs are multiples of d/4 so x/d is exact in fp32
    r = rng(7)
    x = (r.integers(-32, 29, (200, 32)) / 64.0).astype(np.float32)
    x[:, 0] = -0.5
    blob = orc.quantize(x, Q4_0).reshape(-1, 18)
    codes = np.concatenate([blob[:, 2:] & 0xF, blob[:, 2:] >> 4], axis=1).astype(np.int64)
    t = x.astype(np.float64) / 0.0625 + 8         # exact
    want = np.minimum(np.floor(t + 0.5), 15).astype(np.int64)   # nearest, ties up, clamp
    assert np.array_equal(codes, want)


def test_shape_errors():
    with pytest.raises(ValueError):
        orc.quantize(np.zeros((2, 48), dtype=np.float32), Q4_0)
    with pytest.raises(ValueError):
        orc.quantize(np.zeros((2, 64), dtype=np.float32), FP8)
    with pytest.raises(ValueError):
        orc.quantize(np.zeros((2, 64), dtype=np.float32), 12)
    assert orc.quantize(np.zeros((0, 64), dtype=np.float32), Q4_0).size == 0
