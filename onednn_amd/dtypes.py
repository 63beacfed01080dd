"""numpy views of the path's low-precision data types (host-side data prep).

Bit contract: the reference's software types (src/common/bfloat16.cpp:22-49,
float16.hpp:50-135, float8.cpp:29-45/:216-281/:341-374, float4.cpp:28-84,
nibble.hpp:33).  Used to build inputs (quantize f32 data to e4m3 / e2m1 /
bf16, pack nibbles) and to decode outputs; the kernels carry their own device
versions.
"""
import numpy as np

E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0,
                        -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], dtype=np.float32)


def f32_to_bf16(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    expo = (u >> 23) & 0xFF
    man = u & 0x7FFFFF
    rounded = ((u.astype(np.uint64) + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32)
    out = np.where(expo == 0, (u >> 16) & 0x8000, rounded)
    out = np.where((expo == 0xFF) & (man != 0), (u >> 16) | 0x40, out)
    out = np.where((expo == 0xFF) & (man == 0), u >> 16, out)
    return out.astype(np.uint16)


def bf16_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << 16).view(np.float32)


def f32_to_f16_bits(x):
    x = np.ascontiguousarray(x, dtype=np.float32)
    with np.errstate(over="ignore"):
        return x.astype(np.float16).view(np.uint16)


def f16_bits_to_f32(h):
    return np.ascontiguousarray(h, dtype=np.uint16).view(np.float16).astype(np.float32)


def f16_bits_to_e4m3(h):
    h = np.ascontiguousarray(h, dtype=np.uint16).astype(np.uint32)
    s8 = (h & 0x8000) >> 8
    a = h & 0x7FFF
    e16 = a >> 10
    # e4m3-normal range
    x = a - (8 << 10)
    normal = ((x + 0x3F + ((x >> 7) & 1)) >> 7) & 0xFF
    # e4m3 subnormal range (e16 in 5..8)
    sig = 1024 + (a & 0x3FF)
    shift = np.clip(16 - e16.astype(np.int64), 1, 31).astype(np.uint32)
    q = sig >> shift
    rem = sig & ((np.uint32(1) << shift) - 1)
    half = np.uint32(1) << (shift - 1)
    q = q + ((rem > half) | ((rem == half) & ((q & 1) == 1)))
    out = np.where(e16 >= 9, normal, q)
    out = np.where(a <= 0x1400, 0, out)
    out = np.where(a > 0x5F40, 0x7F, out)
    return (s8 | out).astype(np.uint8)


def f32_to_e4m3(x):
    return f16_bits_to_e4m3(f32_to_f16_bits(x))


def _e4m3_table():
    t = np.zeros(256, dtype=np.float32)
    for b in range(256):
        e, m = (b >> 3) & 0xF, b & 7
        if e == 0xF and m == 7:
            v = np.nan
        elif e == 0:
            v = m * 2.0 ** -9
        else:
            v = (8 + m) * 2.0 ** (e - 10)
        t[b] = -v if (b & 0x80) else v
    return t


E4M3_VALUES = _e4m3_table()


def e4m3_to_f32(b):
    return E4M3_VALUES[np.ascontiguousarray(b, dtype=np.uint8)]


def f32_to_e8m0(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u >> 23) & 0xFF).astype(np.uint8)


def e8m0_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint8).astype(np.uint32)
    bits = np.where(b == 0xFF, 0xFFC00000, np.where(b == 0, 0x00400000, b << 23)).astype(np.uint32)
    return bits.view(np.float32)


def f32_to_e2m1_codes(x):
    """One 4-bit code per element (unpacked, uint8 in 0..15)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    sign = ((u >> 28) & 0x8).astype(np.uint8)
    naninf = (u & 0x7F800000) == 0x7F800000
    a = np.minimum(np.abs(np.where(naninf, 0, x)), np.float32(6.0))
    c = np.full(x.shape, 7, dtype=np.uint8)
    c = np.where(a <= 5.0, 6, c)
    c = np.where(a < 3.5, 5, c)
    c = np.where(a <= 2.5, 4, c)
    c = np.where(a < 1.75, 3, c)
    c = np.where(a <= 1.25, 2, c)
    c = np.where(a < 0.75, 1, c)
    c = np.where(a <= 0.25, 0, c)
    c = np.where(naninf, 7, c)
    return (sign | c).astype(np.uint8)


def pack_nibbles(codes):
    """Pack 4-bit codes two per byte along the flattened (logical-offset)
    order: even offset -> low nibble."""
    flat = np.ascontiguousarray(codes, dtype=np.uint8).reshape(-1)
    if flat.size % 2:
        flat = np.concatenate([flat, np.zeros(1, np.uint8)])
    return ((flat[0::2] & 0xF) | ((flat[1::2] & 0xF) << 4)).astype(np.uint8)


def unpack_nibbles(packed, n):
    packed = np.ascontiguousarray(packed, dtype=np.uint8).reshape(-1)
    out = np.empty(packed.size * 2, dtype=np.uint8)
    out[0::2] = packed & 0xF
    out[1::2] = packed >> 4
    return out[:n]


def s4_codes_to_int(codes):
    c = np.ascontiguousarray(codes, dtype=np.uint8).astype(np.int32)
    return np.where(c & 8, c - 16, c)
