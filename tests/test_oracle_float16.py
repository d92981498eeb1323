"""Pins the oracle's f32->bf16 / f32->f16 conversions against library
round-to-nearest-even conversions and the reference's documented special cases."""
import numpy as np
import torch

from oracle import pyoracle as O


def _bits_grid():
    hi = np.arange(1 << 16, dtype=np.uint32) << 16
    lows = np.array([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x4000, 0xC000], dtype=np.uint32)
    return (hi[:, None] | lows[None, :]).reshape(-1)


def test_bf16_normals_equal_torch_rne():
    bits = _bits_grid()
    exp = (bits >> 23) & 0xFF
    normal = (exp > 0) & (exp < 255)
    x = bits[normal].view(np.float32)
    got = O.f32_to_bf16(x)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    # random mantissas too
    rng = np.random.default_rng(0)
    rb = rng.integers(0, 1 << 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    e = (rb >> 23) & 0xFF
    rb = rb[(e > 0) & (e < 255)]
    x = rb.view(np.float32)
    want = torch.from_numpy(x.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(O.f32_to_bf16(x), want)


def test_bf16_special_cases():
    def cvt(b):
        return int(O.f32_to_bf16(np.array([b], dtype=np.uint32).view(np.float32))[0])
    # NaN -> 0x7fff regardless of sign/payload (Float16.cpp:524-526,626-627)
    for b in (0x7FC00000, 0xFFC00000, 0x7F800001, 0xFF812345):
        assert cvt(b) == 0x7FFF
    # +-inf kept
    assert cvt(0x7F800000) == 0x7F80 and cvt(0xFF800000) == 0xFF80
    # +-0 kept
    assert cvt(0x00000000) == 0x0000 and cvt(0x80000000) == 0x8000
    # fp32 denormals flush to signed zero ...
    for b in (0x00000001, 0x00400000, 0x007F0000, 0x007F7FFF, 0x80000001, 0x807F7FFF, 0x00123456):
        assert cvt(b) == (0x8000 if b >> 31 else 0)
    # ... except 0x007f8000..0x007fffff, which round up to the smallest normal
    for b in (0x007F8000, 0x007FFFFF, 0x807F8000, 0x807FABCD):
        assert cvt(b) == ((0x8000 if b >> 31 else 0) | 0x0080)
    # largest finite rounds up to infinity, ties go to even
    assert cvt(0x7F7FFFFF) == 0x7F80
    assert cvt(0x3F808000) == 0x3F80 and cvt(0x3F818000) == 0x3F82 and cvt(0x3F808001) == 0x3F81


def test_bf16_cv18xx_variant():
    # add 0x7fff + lsb then truncate; any result with all-ones exponent becomes 0x7f7f
    rng = np.random.default_rng(1)
    rb = rng.integers(0, 1 << 32, size=500_000, dtype=np.uint64).astype(np.uint32)
    got = O.f32_to_bf16(rb.view(np.float32), cv18xx=True)
    u = rb.astype(np.uint64)
    u = (u + 0x7FFF + ((u >> 16) & 1)) & 0xFFFFFFFF
    h = (u >> 16).astype(np.uint16)
    want = np.where((h & 0x7F80) == 0x7F80, np.uint16(0x7F7F), h)
    assert np.array_equal(got, want)
    # hardware behaviour: infinities (either sign) become the max finite positive value
    inf = np.array([0x7F800000, 0xFF800000, 0x7F7FFFFF], dtype=np.uint32).view(np.float32)
    assert O.f32_to_bf16(inf, cv18xx=True).tolist() == [0x7F7F, 0x7F7F, 0x7F7F]


def test_f16_equals_numpy_rne():
    bits = _bits_grid()
    rng = np.random.default_rng(2)
    rb = rng.integers(0, 1 << 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    # dense sampling of the f16 subnormal / normal boundary exponents (97..114) and overflow edge
    e = rng.integers(96, 145, size=1_000_000, dtype=np.uint64).astype(np.uint32)
    m = rng.integers(0, 1 << 23, size=1_000_000, dtype=np.uint64).astype(np.uint32)
    s = rng.integers(0, 2, size=1_000_000, dtype=np.uint64).astype(np.uint32)
    dense = (s << 31) | (e << 23) | m
    allb = np.concatenate([bits, rb, dense])
    x = allb.view(np.float32)
    isnan = np.isnan(x)
    got = O.f32_to_f16(x)
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(got[~isnan], want[~isnan])
    assert np.all(got[isnan] == 0x7FFF)  # NaN -> 0x7fff (Float16.cpp:655-659,691-692)


def test_f16_to_f32_roundtrip():
    h = np.arange(1 << 16, dtype=np.uint16)
    f = O.f16_to_f32(h)
    ref = h.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(f[~nan].view(np.uint32), ref[~nan].view(np.uint32))
    assert np.all(f[nan].view(np.uint32) == 0xFFC00000)  # Float16.cpp:778-783
    # F16(x) is idempotent and the identity on representable values
    assert np.array_equal(O.F16(f[~nan]).view(np.uint32), f[~nan].view(np.uint32))
