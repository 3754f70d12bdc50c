"""Storage-dtype rounding for the oracle.

Float tensors are carried as float32 arrays (float64 for "f64") whose values
are exactly representable in the storage dtype; `rnd` applies the storage
rounding a primitive's output undergoes (round-to-nearest-even, like the
`half` crate used by candle: rai-core/src/dtype.rs, backend/candle.rs:762-774).
"""
import numpy as np

FLOAT_DTYPES = ("f16", "bf16", "f32", "f64")
INT_DTYPES = {"u8": np.uint8, "u32": np.uint32, "i64": np.int64}


def f32_to_bf16_bits(x):
    """float32 -> uint16 bf16 bit patterns, round-to-nearest-even, NaN kept quiet."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    rounded = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    out = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), rounded)
    return out.astype(np.uint16)


def bf16_bits_to_f32(b):
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def carrier(dt):
    if dt == "f64":
        return np.float64
    if dt in FLOAT_DTYPES:
        return np.float32
    return INT_DTYPES[dt]


def rnd(x, dt):
    """Round an array computed in the carrier type to storage dtype `dt`."""
    if dt == "f64":
        return np.asarray(x, dtype=np.float64)
    if dt == "f32":
        return np.asarray(x, dtype=np.float32)
    if dt == "bf16":
        x = np.asarray(x, dtype=np.float32)
        return bf16_bits_to_f32(f32_to_bf16_bits(x)).reshape(x.shape)
    if dt == "f16":
        with np.errstate(over="ignore"):
            return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)
    return np.asarray(x, dtype=INT_DTYPES[dt])


def to_storage(x, dt):
    """Carrier array -> the bytes-on-device representation (bf16 as uint16 bits)."""
    if dt == "bf16":
        x = np.asarray(x, dtype=np.float32)
        return f32_to_bf16_bits(x).reshape(x.shape)
    if dt == "f16":
        return np.asarray(x, dtype=np.float32).astype(np.float16)
    return np.ascontiguousarray(x, dtype=carrier(dt))


def from_storage(a, dt):
    if dt == "bf16":
        a = np.asarray(a, dtype=np.uint16)
        return bf16_bits_to_f32(a).reshape(a.shape)
    if dt == "f16":
        return np.asarray(a, dtype=np.float16).astype(np.float32)
    return np.asarray(a, dtype=carrier(dt))
