"""Shared test helpers: seeded inputs of the benchmark configurations, the int4 packing of the
reference test, numpy<->torch conversions (bf16 travels as uint16 bit patterns on the numpy side)
and the parity metrics."""
import numpy as np

from oracle import ofq_oracle as O


def rng_for(cfg, tensor):
    """One PCG64 stream per (configuration, tensor)."""
    return np.random.Generator(np.random.PCG64(1000 + cfg * 10 + tensor))


def pack_int4(codes):
    """Two 4-bit codes per byte along the last axis, element 2i in the HIGH nibble
    (python/oneflow/test/modules/test_groupwise_quantization.py:26-34)."""
    l = codes[..., 0::2]
    r = codes[..., 1::2]
    l = np.left_shift(l, 4)
    if codes.dtype == np.int8:
        r = np.bitwise_and(r, np.int8(0xF))
    return np.bitwise_or(l, r).astype(codes.dtype)


def unpack_int4(packed):
    """Inverse of pack_int4 (test_groupwise_quantization.py:37-43)."""
    l = np.right_shift(packed, 4)
    r = np.right_shift(np.left_shift(packed, 4).astype(packed.dtype), 4)
    out = np.stack((l, r), axis=-1).reshape(packed.shape[:-1] + (packed.shape[-1] * 2,))
    return out.astype(packed.dtype)


def as_T(a_f32, t):
    """fp32 ndarray -> storage of T ('f32' | 'f16' | 'bf16')."""
    if t == "f32":
        return np.ascontiguousarray(a_f32, dtype=np.float32)
    if t == "f16":
        return np.ascontiguousarray(a_f32, dtype=np.float32).astype(np.float16)
    return O.f32_to_bf16_bits(a_f32)


def quantize_groupwise(x, num_bits, symmetric, group_dim, group_size, quant_dtype, t):
    """The weight quantiser of the reference test (test_groupwise_quantization.py:46-81) in
    numpy: returns (packed codes, scale as T, zero as T or None)."""
    x = np.asarray(x, dtype=np.float32)
    shp = x.shape
    xr = x.reshape(shp[:group_dim] + (shp[group_dim] // group_size, group_size) + shp[group_dim + 1:])
    ax = group_dim + 1
    if symmetric:
        signed_max = float(2 ** (num_bits - 1)) - 1
        offset = signed_max if quant_dtype == np.uint8 else 0.0
        scale = np.abs(xr).max(axis=ax, keepdims=True) / signed_max
        scale = np.where(scale == 0, 1.0, scale).astype(np.float32)
        q = np.rint(xr / scale + offset).reshape(shp).astype(quant_dtype)
        zero = None
    else:
        unsigned_max = float(2 ** num_bits) - 1
        mn = xr.min(axis=ax, keepdims=True)
        mx = xr.max(axis=ax, keepdims=True)
        scale = ((mx - mn) / unsigned_max).astype(np.float32)
        scale = np.where(scale == 0, 1.0, scale).astype(np.float32)
        q = np.rint((xr - mn) / scale).reshape(shp).astype(np.uint8)
        zero = as_T(np.squeeze(mn, axis=ax), t)
    if num_bits == 4:
        q = pack_int4(q)
    return q, as_T(np.squeeze(scale, axis=ax), t), zero


def to_torch(a, device="cuda"):
    import torch
    if a is None:
        return None
    if a.dtype == np.uint16:  # bf16 bits
        return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).to(device)
    return torch.from_numpy(np.ascontiguousarray(a)).to(device)


def to_numpy(t):
    import torch
    t = t.detach().cpu()
    if t.dtype == torch.bfloat16:
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()


def rel_l2(got, ref):
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    den = np.sqrt((ref ** 2).sum())
    return float(np.sqrt(((got - ref) ** 2).sum()) / (den if den > 0 else 1.0))


def ulp_of(ref_f32, t):
    """Spacing of T at |ref| (for 'one output ulp' bounds)."""
    mant = {"f32": 23, "f16": 10, "bf16": 7}[t]
    a = np.abs(np.asarray(ref_f32, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(a, 1e-30)))
    return np.exp2(e - mant)


def assert_linear_parity(got_T, ref_T, t, what=""):
    """The stated contract for fp16/bf16 linear outputs: rel-L2 <= 1e-3 and max-abs <= 2e-2
    against the dequantize -> matmul (fp32 accumulate) composition.  Where outputs are so large
    that one ulp of T exceeds 2e-2 the absolute bound cannot be met by ANY implementation that
    accumulates in a different order, so the absolute bound is max(2e-2, 1 ulp of T at |ref|)."""
    got = O.to_f32(got_T).astype(np.float64)
    ref = O.to_f32(ref_T).astype(np.float64)
    r = rel_l2(got, ref)
    assert r <= 1e-3, f"{what}: rel-L2 {r:.3e} > 1e-3"
    bound = np.maximum(2e-2, ulp_of(ref, t))
    err = np.abs(got - ref)
    worst = float((err / bound).max())
    assert worst <= 1.0, f"{what}: max-abs {err.max():.4e} exceeds max(2e-2, 1 ulp) by x{worst:.2f}"
    return r, float(err.max())
