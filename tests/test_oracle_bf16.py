"""Pins oracle.bf16_linear_ref (the plain bf16 linear, kernels/k-core/src/gemm.rs:128-167) without the reference: cases
whose answer the mathematics fixes, chosen so that a transposed operand, a single rounding of the residual add or a wrong
bf16 rounding fails one of them."""
import numpy as np


def bits(x):
    b = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((b + 0x7FFF + ((b >> 16) & 1)) >> 16).astype(np.uint16)


def f32(b):
    return (np.asarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def test_one_hot_weights_copy_the_input(oracle):
    rng = np.random.default_rng(1)
    m, k = 5, 64
    x = bits(rng.normal(size=(m, k)))
    perm = rng.permutation(k)[:48]
    w = np.zeros((48, k), np.float32)
    w[np.arange(48), perm] = 1.0
    y, _ = oracle.bf16_linear_ref(x, bits(w))
    assert np.array_equal(y, x[:, perm])  # y[r][n] = x[r][perm[n]]: W is [n][k], not [k][n]


def test_all_ones_sum_to_k(oracle):
    y, acc = oracle.bf16_linear_ref(bits(np.ones((2, 256))), bits(np.ones((8, 256))))
    assert (acc == 256.0).all() and (f32(y) == 256.0).all()


def test_brute_force_tiny(oracle):
    rng = np.random.default_rng(2)
    x, w = bits(rng.normal(size=(3, 64))), bits(rng.normal(size=(8, 64)))
    y, acc = oracle.bf16_linear_ref(x, w)
    for r in range(3):
        for n in range(8):
            s = sum(float(f32(x[r, i])) * float(f32(w[n, i])) for i in range(64))
            assert acc[r, n] == np.float32(s)
            assert y[r, n] == bits(np.float32(s))


def test_rounds_to_nearest_even(oracle):
    # 1 + 2^-8 is halfway between the bf16 neighbours 1 and 1 + 2^-7: ties go to the even mantissa (1.0);
    # 1 + 2^-7 + 2^-8 is halfway between 1 + 2^-7 and 1 + 2^-6: even is 1 + 2^-6
    x = bits(np.float32([[1.0, 2.0 ** -8] + [0.0] * 62, [1.0 + 2.0 ** -7, 2.0 ** -8] + [0.0] * 62]))
    w = bits(np.ones((8, 64), np.float32))
    y, acc = oracle.bf16_linear_ref(x, w)
    assert acc[0, 0] == np.float32(1.00390625) and f32(y)[0, 0] == 1.0
    assert f32(y)[1, 0] == np.float32(1.0 + 2.0 ** -6)


def test_residual_is_added_after_rounding(oracle):
    # sum = 1 + 2^-9 -> bf16 1.0; + res 2^-8 = 1 + 2^-8, a tie -> 1.0. One rounding of 1 + 2^-9 + 2^-8 would give 1 + 2^-7.
    x = bits(np.float32([[1.0, 2.0 ** -9] + [0.0] * 62]))
    w = bits(np.ones((8, 64), np.float32))
    res = bits(np.full((1, 8), 2.0 ** -8, np.float32))
    y, _ = oracle.bf16_linear_ref(x, w, res)
    assert (f32(y) == 1.0).all()
    assert bits(np.float32(1.0 + 2.0 ** -9 + 2.0 ** -8)) == bits(np.float32(1.0 + 2.0 ** -7))
