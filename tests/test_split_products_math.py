"""The arithmetic behind dsx_fc_forward_split, checked on the CPU with numpy: an fp32 value is the exact sum of three bf16
values obtained by rounding to nearest-even what the pieces before left, and the six products of such pieces that the kernel
keeps carry all but 2^-24 of an fp32 x fp32 product.  (The kernel itself is compared with fp64 on the GPU in
test_gpu_split_products.py; this pins the scheme those tests rely on, including the term list.)"""
import numpy as np


def bf16_rn(x):
    """Round float32 to bfloat16 (nearest, ties to even), returned as float32."""
    u = np.asarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    return (r.astype(np.uint32) << 16).view(np.float32)


def split3(x):
    x = np.asarray(x, dtype=np.float32)
    hi = bf16_rn(x)
    r1 = x - hi
    mid = bf16_rn(r1)
    r2 = r1 - mid
    lo = bf16_rn(r2)
    return hi, mid, lo, r1, r2


def samples():
    rng = np.random.default_rng(42)
    a = (rng.standard_normal(200000) * np.exp(6 * rng.standard_normal(200000))).astype(np.float32)
    edge = np.array([0.0, -0.0, 1.0, -1.0, 1 + 2.0 ** -23, 1 - 2.0 ** -24, 2 - 2.0 ** -23, 255.5, 0.1, 1 / 3, 3.0e38 * 0.99, 1.1754944e-38,
                     16777215.0, 16777217.0, 0.99999994, 1.0000001, 65504.0, 3.1415927, 2.0 ** -100, 1.5 * 2.0 ** 100], dtype=np.float32)
    bits = rng.integers(0, 2 ** 32, 200000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    bits = bits[np.isfinite(bits) & (np.abs(bits) < 3.0e38) & (np.abs(bits) > 1e-30)]      # every exponent and mantissa pattern
    return np.concatenate([a, edge, -edge, bits])


def test_three_bf16_pieces_are_the_value_exactly():
    x = samples()
    hi, mid, lo, r1, r2 = split3(x)
    # the subtractions are exact in fp32 (the pieces cancel leading bits), and so is the last rounding
    assert np.array_equal(r1.astype(np.float64), x.astype(np.float64) - hi.astype(np.float64))
    assert np.array_equal(r2.astype(np.float64), r1.astype(np.float64) - mid.astype(np.float64))
    assert np.array_equal(lo, r2)
    assert np.array_equal(hi.astype(np.float64) + mid.astype(np.float64) + lo.astype(np.float64), x.astype(np.float64))
    nz = hi != 0
    assert np.all(np.abs(mid[nz]) <= np.abs(hi[nz]) * 2.0 ** -8) and np.all(np.abs(lo[nz]) <= np.abs(hi[nz]) * 2.0 ** -16)
    # every piece is a bf16 value: the low 16 bits of its fp32 pattern are zero
    for piece in (hi, mid, lo):
        assert not (piece.view(np.uint32) & 0xFFFF).any()


def test_six_terms_carry_an_fp32_product_to_2_pow_minus_24():
    x = samples()
    rng = np.random.default_rng(7)
    y = rng.permutation(x)
    big = (np.abs(x.astype(np.float64) * y.astype(np.float64)) < 1e37) & (np.abs(x.astype(np.float64) * y.astype(np.float64)) > 1e-25)
    x, y = x[big], y[big]
    xs = [p.astype(np.float64) for p in split3(x)[:3]]
    ys = [p.astype(np.float64) for p in split3(y)[:3]]
    exact = x.astype(np.float64) * y.astype(np.float64)
    terms = [(2, 0), (0, 2), (1, 1), (1, 0), (0, 1), (0, 0)]       # (piece of x, piece of y) as the kernel lists them
    kept = sum(xs[a] * ys[b] for a, b in terms)                     # each bf16 x bf16 product is exact in fp32, and in fp64
    rel = np.abs(kept - exact) / np.abs(exact)
    assert rel.max() < 2.0 ** -24, rel.max()
    # every kept term matters at fp32 accuracy: without the smallest three the error is 2^-17, hundreds of fp32 roundings
    coarse = sum(xs[a] * ys[b] for a, b in terms[3:])
    assert (np.abs(coarse - exact) / np.abs(exact)).max() > 2.0 ** -18
    # and a bf16 x bf16 product needs no more than fp32's 24 bits: the matrix instruction adds exact terms
    p = (xs[0] * ys[0])
    assert np.array_equal(p.astype(np.float32).astype(np.float64), p)
