"""Independent numpy witnesses for the block formats.

Decoders restate the pure-torch block readers that ARE in the reference
(python/llm/src/ipex_llm/transformers/gguf/gguf.py:273-296,332-342) and the
Q4_1 writer (python/llm/src/ipex_llm/transformers/convert.py:417-453).  The
quantizer transcriptions follow the published ggml quantize_row_*_reference
routines those files point to; they share the formula with the oracle but not
its code, so they catch indexing / ordering slips, while closed forms and
brute force in the tests pin the formula itself.
"""
import numpy as np

F32 = np.float32


# ---- decoders (gguf.py) ---------------------------------------------------

def decode_q4_0(blob, shape):
    t = np.asarray(blob, dtype=np.uint8).reshape(-1, 18)
    scales = t[:, :2].copy().view(np.float16).astype(F32)          # [nb,1]
    data = t[:, 2:]
    q = np.concatenate([data & 0xF, data >> 4], axis=-1).astype(np.int8) - 8
    return (q.astype(F32) * scales).reshape(shape)


def decode_q4_1(blob, shape):
    t = np.asarray(blob, dtype=np.uint8).reshape(-1, 20)
    scales = t[:, :2].copy().view(np.float16).astype(F32)
    base = t[:, 2:4].copy().view(np.float16).astype(F32)
    data = t[:, 4:]
    q = np.concatenate([data & 0xF, data >> 4], axis=-1)
    return (q.astype(F32) * scales + base).reshape(shape)


def decode_q8_0(blob, shape):
    t = np.asarray(blob, dtype=np.uint8).reshape(-1, 34)
    scales = t[:, :2].copy().view(np.float16).astype(F32)
    q = t[:, 2:].copy().view(np.int8)
    return (q.astype(F32) * scales).reshape(shape)


# ---- Q4_1 writer (convert.py:417-453, reduced to its layout statement) -----

def write_q4_1_from_codes(codes, scales, zeros):
    """codes uint8 [rows, K] in 0..15, scales/zeros fp16 [rows, K/32].
    Field order d, m, qs; m = -(zero * scale) in fp16; byte j of a block packs
    code j (low nibble) and code j+16 (high nibble)."""
    rows, k = codes.shape
    w = codes.reshape(rows, k // 32, 2, 16)
    w = np.swapaxes(w, 2, 3)                                       # [rows, nb, 16, 2]
    packed = (w[..., 0] | (w[..., 1] << 4)).astype(np.uint8)       # [rows, nb, 16]
    d = scales.astype(np.float16).reshape(rows, k // 32, 1)
    m = (-(zeros.astype(np.float16) * scales.astype(np.float16))).astype(np.float16)
    m = m.reshape(rows, k // 32, 1)
    blob = np.concatenate([d.view(np.uint8), m.view(np.uint8), packed], axis=-1)
    return blob.reshape(-1)


# ---- quantizer transcriptions (vectorised, fp32 arithmetic, no FMA) --------

def _roundf(v):
    r = np.trunc(v)
    frac = v - r
    return r + np.where(np.abs(frac) >= 0.5, np.sign(v), 0).astype(F32)


def quant_q4_0(w):
    x = np.asarray(w, dtype=F32).reshape(-1, 32)
    idx = np.argmax(np.abs(x), axis=1)                             # first largest wins
    mx = x[np.arange(x.shape[0]), idx]
    d = (mx / F32(-8.0)).astype(F32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, F32(1.0) / d, F32(0)).astype(F32)
    v = (x * inv[:, None]).astype(F32) + F32(8.5)
    q = np.minimum(np.trunc(v).astype(np.int32).astype(np.int8), 15).astype(np.uint8)
    out = np.empty((x.shape[0], 18), dtype=np.uint8)
    out[:, :2] = d.astype(np.float16).reshape(-1, 1).view(np.uint8)
    out[:, 2:] = q[:, :16] | (q[:, 16:] << 4)
    return out.reshape(-1)


def quant_q4_1(w):
    x = np.asarray(w, dtype=F32).reshape(-1, 32)
    mn = x.min(axis=1)
    mx = x.max(axis=1)
    d = ((mx - mn) / F32(15.0)).astype(F32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, F32(1.0) / d, F32(0)).astype(F32)
    v = ((x - mn[:, None]).astype(F32) * inv[:, None]).astype(F32) + F32(0.5)
    q = np.minimum(np.trunc(v).astype(np.int32).astype(np.int8), 15).astype(np.uint8)
    out = np.empty((x.shape[0], 20), dtype=np.uint8)
    out[:, :2] = d.astype(np.float16).reshape(-1, 1).view(np.uint8)
    out[:, 2:4] = mn.astype(np.float16).reshape(-1, 1).view(np.uint8)
    out[:, 4:] = q[:, :16] | (q[:, 16:] << 4)
    return out.reshape(-1)


def quant_q8_0(w):
    x = np.asarray(w, dtype=F32).reshape(-1, 32)
    amax = np.abs(x).max(axis=1)
    d = (amax / F32(127.0)).astype(F32)
    with np.errstate(divide="ignore"):
        inv = np.where(d != 0, F32(1.0) / d, F32(0)).astype(F32)
    q = _roundf((x * inv[:, None]).astype(F32)).astype(np.int8)
    out = np.empty((x.shape[0], 34), dtype=np.uint8)
    out[:, :2] = d.astype(np.float16).reshape(-1, 1).view(np.uint8)
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(-1)


NF4 = np.array([-1.0, -0.6961928009986877, -0.5250730514526367, -0.39491748809814453,
                -0.28444138169288635, -0.18477343022823334, -0.09105003625154495, 0.0,
                0.07958029955625534, 0.16093020141124725, 0.24611230194568634,
                0.33791524171829224, 0.44070982933044434, 0.5626170039176941,
                0.7229568362236023, 1.0], dtype=np.float64)


def decode_nf4(blob, shape):
    t = np.asarray(blob, dtype=np.uint8).reshape(-1, 34)
    d = t[:, :2].copy().view(np.float16).astype(F32)
    data = t[:, 2:]
    idx = np.concatenate([data & 0xF, data >> 4], axis=-1)
    return (NF4.astype(F32)[idx] * d).reshape(shape)


def decode_fp8(blob, shape):
    import torch
    t = np.asarray(blob, dtype=np.uint8).reshape(-1, 132)
    s = t[:, :4].copy().view(np.float32)
    codes = torch.from_numpy(t[:, 4:].copy()).view(torch.float8_e4m3fn).float().numpy()
    return (codes * s).reshape(shape)


DECODERS = {2: decode_q4_0, 3: decode_q4_1, 8: decode_q8_0, 10: decode_nf4, 15: decode_fp8}
