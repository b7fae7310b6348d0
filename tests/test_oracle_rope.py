"""Pins of the rotary oracle that do not retype its formula: complex multiplication in
float64, identity at position 0, which elements pair up, which table row a token uses,
norm preservation, and the table generator against closed forms."""
import numpy as np

from oracle import rope_cpu as RO
from helpers import rand_f16


def _tables(T, D, seed):
    rng = np.random.default_rng(seed)
    ang = rng.uniform(-np.pi, np.pi, size=(T, D // 2))
    return np.cos(ang).astype(np.float16), np.sin(ang).astype(np.float16)


def test_matches_complex_multiplication_within_one_fp16_ulp():
    rng = np.random.default_rng(0)
    T, H, D = 37, 5, 128
    x = rand_f16(rng, T, H, D)
    cos, sin = _tables(T, D, 1)
    got = RO.rotate_rows(x, cos, sin).astype(np.float64)
    z = (x[:, :, :64].astype(np.float64) + 1j * x[:, :, 64:].astype(np.float64)) * \
        (cos.astype(np.float64) + 1j * sin.astype(np.float64))[:, None, :]
    want = np.concatenate([z.real, z.imag], axis=2)
    ulp = np.spacing(np.abs(want).astype(np.float16)).astype(np.float64)
    # one rounded product + one rounded fma: at most 0.5 ulp of the product plus 0.5 ulp of the result
    prod_ulp = np.spacing(np.maximum(np.abs(x[:, :, :64]), np.abs(x[:, :, 64:])).astype(np.float16)).astype(np.float64)
    bound = 0.5 * ulp + 0.5 * np.concatenate([prod_ulp, prod_ulp], axis=2) + 1e-12
    assert np.all(np.abs(got - want) <= bound)


def test_identity_at_angle_zero_and_quarter_turn():
    rng = np.random.default_rng(2)
    x = rand_f16(rng, 4, 3, 128)
    one, zero = np.ones((4, 64), np.float16), np.zeros((4, 64), np.float16)
    assert np.array_equal(RO.rotate_rows(x, one, zero), x)                  # cos 1, sin 0
    quarter = RO.rotate_rows(x, zero, one)                                  # cos 0, sin 1: (x0, x1) -> (-x1, x0)
    assert np.array_equal(quarter[:, :, :64], -x[:, :, 64:]) and np.array_equal(quarter[:, :, 64:], x[:, :, :64])


def test_pairing_is_d_with_d_plus_half_and_rows_follow_tokens():
    T, H, D = 6, 2, 128
    cos, sin = _tables(T, D, 3)
    for d in (0, 1, 17, 63):
        x = np.zeros((T, H, D), np.float16)
        x[:, :, d] = 1.0
        y = RO.rotate_rows(x, cos, sin)
        touched = np.nonzero(np.any(y != 0, axis=(0, 1)))[0].tolist()
        assert set(touched) <= {d, d + 64}
        assert np.array_equal(y[:, 0, d], cos[:, d]) and np.array_equal(y[:, 1, d + 64], sin[:, d])
    # token t uses row t: permuting tokens and table rows together permutes the output
    rng = np.random.default_rng(4)
    x = rand_f16(rng, T, H, D)
    perm = rng.permutation(T)
    assert np.array_equal(RO.rotate_rows(x[perm], cos[perm], sin[perm]), RO.rotate_rows(x, cos, sin)[perm])


def test_norm_of_each_pair_is_preserved():
    rng = np.random.default_rng(5)
    x = rand_f16(rng, 50, 4, 128)
    pos = rng.integers(0, 4000, size=50)
    ct, st = RO.rotary_tables(128, 4096)
    y = RO.rotate_rows(x, ct[pos], st[pos]).astype(np.float64)
    n_in = x[:, :, :64].astype(np.float64) ** 2 + x[:, :, 64:].astype(np.float64) ** 2
    n_out = y[:, :, :64] ** 2 + y[:, :, 64:] ** 2
    assert np.allclose(n_out, n_in, rtol=4e-3, atol=1e-4)                   # fp16 tables: cos^2 + sin^2 = 1 +- 1e-3


def test_tables_closed_forms():
    ct, st = RO.rotary_tables(128, 2048, rope_theta=10000.0)
    assert ct.shape == (2048 + 128, 64) and ct.dtype == np.float16
    assert np.all(ct[0] == 1) and np.all(st[0] == 0)                        # position 0
    # pair 0 turns by one radian per position; the last pair by theta^(-126/128)
    assert np.array_equal(ct[:, 0], np.cos(np.arange(2176, dtype=np.float32)).astype(np.float16))
    assert abs(float(st[1, 63]) - 10000.0 ** (-126 / 128)) < 1e-6
    c2, s2 = RO.rotary_tables(64, 1024, rope_theta=500000.0, rope_scaling=2.0)
    assert c2.shape == (2048 + 128, 32)
    assert np.array_equal(c2[::2, 0], np.cos(np.arange(1088, dtype=np.float32)).astype(np.float16))   # t / scaling
