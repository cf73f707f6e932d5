"""16-bit narrowing/widening of the oracle: exhaustive and against numpy float16."""
import numpy as np


def test_f16_roundtrip_all_patterns(oracle):
    bits = np.arange(1 << 16, dtype=np.uint16)
    f = oracle.f16_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    np.testing.assert_array_equal(f.view(np.uint32)[~nan], ref.view(np.uint32)[~nan])
    assert np.isnan(f[nan]).all()
    back = oracle.f32_to_f16(f)
    np.testing.assert_array_equal(back[~nan], bits[~nan])


def test_f32_to_f16_matches_numpy(oracle):
    r = np.random.Generator(np.random.PCG64(1))
    # random bit patterns cover normals, subnormals, overflow, tiny values
    u = r.integers(0, 1 << 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        ref = x.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(oracle.f32_to_f16(x), ref)
    # values concentrated where half is interesting: around ties, subnormal edge, max
    y = np.concatenate([
        r.normal(0, 1, 500000), r.normal(0, 1e-5, 500000), r.normal(0, 3e4, 500000),
        np.array([65504.0, 65519.99, 65520.0, 65536.0, 2.0**-24, 2.0**-25, 2.0**-25 * 1.0000001,
                  2.0**-14, 2.0**-14 - 2.0**-25, 0.0, -0.0, np.inf, -np.inf]),
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        ref = y.astype(np.float16).view(np.uint16)
    np.testing.assert_array_equal(oracle.f32_to_f16(y), ref)


def _bf16_rne_reference(x):
    """Independent statement of RNE: pick the nearer of the two neighbouring bf16 values,
    ties to the one with an even last bit; computed in float64."""
    u = x.view(np.uint32)
    lo = (u & np.uint32(0xFFFF0000))
    hi = lo + np.uint32(0x10000)  # next bf16 away from zero (may become inf)
    flo = lo.view(np.float32).astype(np.float64)
    fhi = hi.view(np.float32).astype(np.float64)
    xd = x.astype(np.float64)
    dlo, dhi = np.abs(xd - flo), np.abs(fhi - xd)
    # distance to inf is not meaningful in float: compare on the integer remainder instead
    rem = (u & np.uint32(0xFFFF)).astype(np.int64)
    take_hi = (rem > 0x8000) | ((rem == 0x8000) & (((lo >> 16) & 1) == 1))
    finite_hi = np.isfinite(fhi)
    assert ((dhi < dlo) == (rem > 0x8000))[finite_hi & (rem != 0x8000)].all()
    return np.where(take_hi, hi >> 16, lo >> 16).astype(np.uint16)


def test_f32_to_bf16(oracle):
    r = np.random.Generator(np.random.PCG64(2))
    u = r.integers(0, 1 << 32, size=2_000_000, dtype=np.uint64).astype(np.uint32)
    x = u.view(np.float32)
    x = x[np.isfinite(x)]
    np.testing.assert_array_equal(oracle.f32_to_bf16(x), _bf16_rne_reference(x))
    # ties
    ties = np.array([0x3F808000, 0x3F818000, 0x3F80FFFF, 0x7F7FFFFF, 0x00008000, 0x80018000],
                    np.uint32).view(np.float32)
    assert oracle.f32_to_bf16(ties).tolist() == [0x3F80, 0x3F82, 0x3F81, 0x7F80, 0x0000, 0x8002]
    # all bf16 patterns survive widening and narrowing
    bits = np.arange(1 << 16, dtype=np.uint16)
    f = oracle.bf16_to_f32(bits)
    keep = ~np.isnan(f)
    np.testing.assert_array_equal(oracle.f32_to_bf16(f)[keep], bits[keep])
    assert np.isnan(oracle.bf16_to_f32(oracle.f32_to_bf16(np.array([np.nan], np.float32)))).all()


def test_workload_helpers_agree_with_oracle(oracle):
    from cudaintro_amd import workloads as wl
    r = np.random.Generator(np.random.PCG64(3))
    x = r.normal(0, 10, 100000).astype(np.float32)
    np.testing.assert_array_equal(wl.f32_to_bf16_bits(x), oracle.f32_to_bf16(x))
    np.testing.assert_array_equal(wl.bf16_bits_to_f32(wl.f32_to_bf16_bits(x)),
                                  oracle.bf16_to_f32(oracle.f32_to_bf16(x)))
