"""The bit-level identities the few-row GEMM kernels rest on (rustane_amd/csrc/hipdec_prefill.h), worked
through with integers and exact floats on the CPU: a plausible slip in a mask, a shift, the element order
or the correction constant fails one of them."""
import numpy as np

from oracle_lib import lib as oracle_lib


def bf16_bits_to_f64(bits):
    return (np.asarray(bits, dtype=np.uint32) << 16).view(np.float32).astype(np.float64)


def f32_to_bf16_bits(x):
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint32)


def unpack_dword(q):
    """The kernel's four operations on one dword of eight offset-binary nibbles: four dwords of two bf16 each."""
    q = np.asarray(q, dtype=np.uint64)
    mask, bias = 0x00780078, 0x41804180
    return [(((q << 3) & 0xFFFFFFFF) & mask) | bias, ((q >> 1) & mask) | bias, ((q >> 5) & mask) | bias, ((q >> 9) & mask) | bias]


def test_every_nibble_lands_as_sixteen_plus_itself():
    # all 2^16 patterns of a half dword, in both halves at once (the halves must not leak into each other)
    half = np.arange(1 << 16, dtype=np.uint64)
    q = half | (((half * 40503) & 0xFFFF) << 16)            # another pattern in the upper half
    words = unpack_dword(q)
    for j, w in enumerate(words):
        lo, hi = w & 0xFFFF, w >> 16
        want_lo = 16 + ((q >> (4 * j)) & 15)
        want_hi = 16 + ((q >> (16 + 4 * j)) & 15)
        assert np.array_equal(bf16_bits_to_f64(lo), want_lo.astype(np.float64))
        assert np.array_equal(bf16_bits_to_f64(hi), want_hi.astype(np.float64))


def test_unpacked_order_is_the_staged_order_of_the_activations():
    # storage: element 2i of a row is the low nibble of byte i, so nibble m of a dword is element m of its eight
    rng = np.random.default_rng(1)
    nib = rng.integers(0, 16, size=(1000, 8), dtype=np.uint64)
    q = sum(nib[:, m] << (4 * m) for m in range(8))
    words = unpack_dword(q)
    got = np.stack([bf16_bits_to_f64(h) for w in words for h in (w & 0xFFFF, w >> 16)], axis=1)   # register order
    assert np.array_equal(got, 16.0 + nib[:, [0, 4, 1, 5, 2, 6, 3, 7]])
    # the staged activations: a 16-byte chunk (x, y, z, w) = elements (0 1)(2 3)(4 5)(6 7) becomes
    # (x.lo z.lo)(x.hi z.hi)(y.lo w.lo)(y.hi w.hi)
    e = np.arange(8)
    x, y, z, w = e[0:2], e[2:4], e[4:6], e[6:8]
    staged = [x[0], z[0], x[1], z[1], y[0], w[0], y[1], w[1]]
    assert staged == [0, 4, 1, 5, 2, 6, 3, 7]


def test_group_product_with_the_tile_of_minus_twenty_fours_is_the_signed_product():
    rng = np.random.default_rng(2)
    for _ in range(200):
        nib = rng.integers(0, 16, size=128)
        xs = bf16_bits_to_f64(f32_to_bf16_bits(rng.normal(size=128).astype(np.float32) * 10.0 ** rng.integers(-3, 4)))
        signed = float(np.sum(xs * (nib - 8.0)))
        biased = float(np.sum(xs * (16.0 + nib)) + np.sum(xs * -24.0))      # every term and sum exact in fp64
        assert biased == signed
    assert bf16_bits_to_f64(np.uint32(0xC1C0)) == -24.0
    assert bf16_bits_to_f64(np.uint32(0x4180)) == 16.0


def test_every_e4m3_code_is_a_bf16_number():
    L = oracle_lib()
    vals = np.array([L.orc_e4m3_to_f32(b) for b in range(256)], dtype=np.float32)
    finite = np.isfinite(vals)
    assert finite.sum() >= 252
    assert np.array_equal(bf16_bits_to_f64(f32_to_bf16_bits(vals[finite])), vals[finite].astype(np.float64))


def test_hi_lo_pair_keeps_sixteen_bits():
    rng = np.random.default_rng(3)
    v = (rng.normal(size=200000) * 10.0 ** rng.integers(-6, 6, size=200000)).astype(np.float32)
    hi = bf16_bits_to_f64(f32_to_bf16_bits(v))
    lo = bf16_bits_to_f64(f32_to_bf16_bits((v.astype(np.float64) - hi).astype(np.float32)))
    err = np.abs(v.astype(np.float64) - (hi + lo))
    assert np.all(err <= np.abs(v.astype(np.float64)) * 2.0 ** -16)


def test_row_of_a_staged_chunk_without_a_division():
    # t = int((cc + 0.5) * (1 / cpr)) in fp32 equals cc // cpr for every chunk count per row (a multiple of 16
    # with 4-bit weights; any count up to 1280 is covered here) and every chunk index a workgroup stages (at
    # most 1280 + a round of 512 threads), also with the reciprocal one unit in the last place off either way
    for cpr in range(1, 1281):
        cc = np.arange(0, 1280 + 512, dtype=np.int64)
        rcp = np.float32(1.0) / np.float32(cpr)
        for r in (rcp, np.nextafter(rcp, np.float32(0)), np.nextafter(rcp, np.float32(1))):
            t = ((cc.astype(np.float32) + np.float32(0.5)) * np.float32(r)).astype(np.int64)
            assert np.array_equal(t, cc // cpr), cpr
