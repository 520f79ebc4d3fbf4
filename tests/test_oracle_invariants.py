"""Known answers and invariants the mathematics fixes, restated from the reference's
own unit tests (tests/unit/core/test_lattice.py, test_codec.py, test_quantizer.py,
test_packing.py).  Each is chosen so a plausible slip in the oracle (wrong tie rule,
transposed generator, dropped dither term, wrong nibble order) fails it."""

from itertools import product

import numpy as np
import pytest

from conftest import Q


def _brute_force_e8(x):
    """Finite-neighbourhood search in float64 (test_lattice.py:11-25)."""
    best, best_pt = np.inf, None
    for offset in (0.0, 0.5):
        floors = np.floor(x - offset).astype(int)
        for cand in product(*[range(f - 1, f + 3) for f in floors]):
            if sum(cand) % 2:
                continue
            p = np.array(cand, dtype=np.float64) + offset
            d = float(((x - p) ** 2).sum())
            if d < best:
                best, best_pt = d, p
    return best, best_pt


def test_nearest_e8_agrees_with_brute_force(oracle):
    rng = np.random.default_rng(58)
    x = (rng.standard_normal((6, 8)) * 1.7).astype(np.float32)
    point, dist = oracle.nearest_e8(x)
    for row, p, d in zip(x.astype(np.float64), point, dist):
        best, _ = _brute_force_e8(row)
        assert abs(d - best) < 1e-5
        assert abs(((row - p) ** 2).sum() - best) < 1e-5


def test_tie_goes_to_half_integer_coset(oracle):
    point, dist = oracle.nearest_e8(np.full((1, 8), 0.25, dtype=np.float32))
    assert np.array_equal(point, np.full((1, 8), 0.5, dtype=np.float32))   # test_lattice.py:29-33
    assert dist[0] == 0.5


def test_lattice_points_of_both_cosets_are_fixed(oracle):
    x = np.array([[1, 1, 0, 0, 0, 0, 0, 0], [0.5] * 8, [-1.5, 0.5, 0.5, 0.5, 0.5, 0.5, 0.5, 0.5]], dtype=np.float32)
    point, dist = oracle.nearest_e8(x)
    assert np.array_equal(point, x) and not dist.any()


def test_outputs_are_e8_points(oracle):
    rng = np.random.default_rng(3)
    point, _ = oracle.nearest_e8((rng.standard_normal((5000, 8)) * 4).astype(np.float32))
    doubled = point * 2
    assert np.array_equal(doubled, np.round(doubled))
    all_int = (doubled % 2 == 0).all(axis=1)
    all_half = (doubled % 2 == 1).all(axis=1)
    assert (all_int | all_half).all()
    assert (point.sum(axis=1) % 2 == 0).all()


def test_all_binary_residues_round_trip(oracle):
    codes = np.array(list(product(range(2), repeat=8)), dtype=np.int32)     # test_codec.py:16-28
    reps = oracle.decode_nested(codes, 2)
    assert np.array_equal(oracle.encode_nested(reps, 2), codes)
    assert np.array_equal(oracle.decode_nested(oracle.encode_nested(reps, 2), 2), reps)
    closest, _ = oracle.nearest_e8(reps)
    assert np.array_equal(closest, reps)


def test_q14_decode_encode_decode_is_idempotent(oracle):
    rng = np.random.default_rng(11)
    codes = rng.integers(0, Q, (20000, 8)).astype(np.int32)
    reps = oracle.decode_nested(codes, Q)
    assert np.array_equal(oracle.encode_nested(reps, Q), codes)
    # representatives are minimum-energy: inside (or on the boundary of) 14 * Voronoi(E8)
    nearest, _ = oracle.nearest_e8(reps / np.float32(Q))
    shifted = reps - Q * nearest
    assert np.allclose((shifted ** 2).sum(1), (reps ** 2).sum(1))


def test_coset_shift_invariance(oracle):
    x = np.array([[1, 1, 0, 0, 0, 0, 0, 0], [2, 0, 0, 0, 0, 0, 0, 0]], dtype=np.float32)
    q = 3
    shift = np.array([2, -2, 0, 0, 0, 0, 0, 0], dtype=np.float32) * q      # test_codec.py:42-53
    assert np.array_equal(oracle.encode_nested(x, q), oracle.encode_nested(x + shift, q))


def test_generator_matrix_closed_form(oracle):
    """decode of a unit code = the matching generator column (codec.py:30-42), q large."""
    G = np.array([[2, -1, 0, 0, 0, 0, 0, 0.5], [0, 1, -1, 0, 0, 0, 0, 0.5], [0, 0, 1, -1, 0, 0, 0, 0.5],
                  [0, 0, 0, 1, -1, 0, 0, 0.5], [0, 0, 0, 0, 1, -1, 0, 0.5], [0, 0, 0, 0, 0, 1, -1, 0.5],
                  [0, 0, 0, 0, 0, 0, 1, 0.5], [0, 0, 0, 0, 0, 0, 0, 0.5]])
    eye = np.eye(8, dtype=np.int32)
    out = oracle.decode_nested(eye, 64)
    assert np.array_equal(out, (eye @ G.T).astype(np.float32))
    rng = np.random.default_rng(5)
    lattice = (rng.integers(-3, 4, (500, 8)) @ G.T).astype(np.float32)
    codes = oracle.encode_nested(lattice, 64)
    assert np.array_equal(oracle.decode_nested(codes, 64), lattice)


def test_dithered_round_trip(oracle):
    rng = np.random.default_rng(91)                                          # test_codec.py:71-79
    x = rng.standard_normal((64, 8)).astype(np.float32)
    d = oracle.dither_stateless(64, 17)
    codes = oracle.encode_nested(x, Q, d)
    rec = oracle.decode_nested(codes, Q, d)
    assert np.array_equal(oracle.encode_nested(rec, Q, d), codes)
    # subtractive dither: x - rec is bounded by the covering radius (1) of E8
    assert ((x - rec) ** 2).sum(1).max() <= 1.0 + 1e-5


def test_hash_is_the_integer_closed_form(oracle):
    counters = np.array([0, 1, 7, 8, 123456789, 2**31 - 1, 2**31, 2**33 + 5], dtype=np.uint64)
    for seed in (0, 1, 20261025, 2**31 - 1):
        expected = []
        for c in counters.tolist():
            m = 1 << 31
            v = (c + seed) % m
            v ^= v >> 16
            v = (v * 1103515245 + 12345) % m
            v ^= v >> 13
            v = (v * 134775813 + 1) % m
            v ^= v >> 16
            expected.append(v)
        assert oracle.hash_lcg31(counters, seed).tolist() == expected


def test_stateless_dither_chunk_invariance_and_range(oracle):
    full = oracle.dither_stateless(37, 20261025)                            # test_codec.py:91-102
    chunks = np.concatenate([oracle.dither_stateless(11, 20261025, 0),
                             oracle.dither_stateless(19, 20261025, 11),
                             oracle.dither_stateless(7, 20261025, 30)])
    assert np.array_equal(full, chunks)
    big = oracle.dither_stateless(20000, 5)
    nearest, _ = oracle.nearest_e8(big)
    assert (np.abs(big) <= 1.0).all() and (big ** 2).sum(1).max() <= 1.0
    assert not nearest[(big ** 2).sum(1) < 0.49].any()                      # interior points map to 0
    with pytest.raises(ValueError):
        oracle.dither_stateless(1, 2**31)
    with pytest.raises(ValueError):
        oracle.dither_stateless(2, 0, block_offset=(1 << 28) - 1)


def test_quantize_rows_selects_min_error_beta(oracle):
    rng = np.random.default_rng(17)                                          # test_quantizer.py:11-25, 50-58
    x = rng.standard_normal((5, 64)).astype(np.float32)
    betas = (0.25, 0.5, 1.0)
    codes, idx, norms = oracle.quantize_rows(x, Q, betas)
    assert codes.max() < Q and idx.max() < 3
    y = x * ((1.0 / norms) * np.float32(8.0))[:, None]
    sel = oracle.dequantize_rows(codes, idx, np.full(5, 8.0, np.float32), betas, Q)   # norm/sqrt(n) = 1
    err_sel = ((sel - y) ** 2).reshape(5, 8, 8).sum(-1)
    singles = []
    for b in betas:
        c1, i1, _ = oracle.quantize_rows(x, Q, (b,))
        r1 = oracle.dequantize_rows(c1, i1, np.full(5, 8.0, np.float32), (b,), Q)
        singles.append(((r1 - y) ** 2).reshape(5, 8, 8).sum(-1))
    assert np.allclose(err_sel, np.min(singles, axis=0), rtol=1e-5, atol=1e-7)
    # first index wins a tie: with duplicate betas index 1 is never chosen over 0
    _, dup, _ = oracle.quantize_rows(x, Q, (0.5, 0.5))
    assert not dup.any()


def test_zero_rows_stay_zero(oracle):
    x = np.stack([np.zeros(16, np.float32), np.ones(16, np.float32)])     # test_quantizer.py:43-48
    codes, idx, norms = oracle.quantize_rows(x, Q, (0.5, 1.0, 2.0))
    out = oracle.dequantize_rows(codes, idx, norms, (0.5, 1.0, 2.0), Q)
    assert not out[0].any() and np.isfinite(out).all() and norms[0] == 0


def test_row_norm_is_the_l2_norm(oracle):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((7, 2048)).astype(np.float32)
    exact = np.sqrt((x.astype(np.float64) ** 2).sum(1))
    assert np.allclose(oracle.row_norms(x), exact, rtol=1e-6)


def test_packing_bit_order(oracle):
    def reference(values, width):                                           # test_packing.py:19-23
        result = bytearray((len(values) * width + 7) // 8)
        for index, value in enumerate(values):
            result[index * width // 8] |= int(value) << (index * width % 8)
        return bytes(result)

    for cardinality, width in ((2, 1), (4, 2), (14, 4), (256, 8)):
        values = (np.arange(27) % cardinality).astype(np.uint8)
        packed = oracle.pack_unsigned(values, width)
        assert packed.tobytes() == reference(values.tolist(), width)
        assert np.array_equal(oracle.unpack_unsigned(packed, 27, width), values)
    assert oracle.pack_unsigned(np.array([0, 3], np.uint8), 2).tobytes() == bytes([0b00001100])  # :36-51


def test_hadamard_is_orthogonal_involution(oracle):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((3, 64)).astype(np.float32)
    h = oracle.hadamard(x)
    assert np.allclose(oracle.hadamard(h), x, atol=1e-5)
    assert np.allclose((h ** 2).sum(1), (x ** 2).sum(1), rtol=1e-5)
    e0 = np.zeros((1, 8), np.float32); e0[0, 0] = 1
    assert np.allclose(oracle.hadamard(e0), 1 / np.sqrt(8))
    e1 = np.zeros((1, 8), np.float32); e1[0, 1] = 1
    assert np.allclose(oracle.hadamard(e1), np.array([1, -1, 1, -1, 1, -1, 1, -1]) / np.sqrt(8))


def test_attention_dense_matches_numpy_softmax(oracle):
    rng = np.random.default_rng(4)
    q = rng.standard_normal((8, 64)).astype(np.float32)
    k = rng.standard_normal((37, 2, 64)).astype(np.float32)
    v = rng.standard_normal((37, 2, 64)).astype(np.float32)
    out = oracle.attention_dense(q, k, v)
    for h in range(8):
        g = h // 4
        s = (k[:, g] @ q[h]) / 8.0
        p = np.exp(s - s.max()); p /= p.sum()
        assert np.allclose(out[h], p @ v[:, g], atol=1e-5)


def test_three_operation_division_by_14_is_ieee_exact(oracle):
    """The HIP kernels divide by 14 with q0 = p*c, r = fma(-14, q0, p), q = fma(r, c, q0);
    checked against IEEE division for every finite float32 in [1e-30, 1e30]."""
    assert oracle.count_div14_mismatches() == 0


def test_division_through_the_reciprocal_is_ieee_exact(oracle):
    """The many-row encoder forms y / beta as two exact-remainder corrections of y * (1 / beta);
    checked against IEEE division over every float32 of the range the kernel uses it on, for
    the activation, key and value betas and a few awkward divisors."""
    import numpy as np
    betas = [v / 14 for v in (3.47, 4.74, 6.90, 18.11, 3.50, 4.58, 6.47, 17.06, 3.53, 5.59, 9.62, 29.03)]
    betas += [1.0 / 3.0, 0.7, 1.9999999, 1.0000001, 3.1415927]
    for beta in betas:
        assert oracle.count_reciprocal_division_mismatches(float(np.float32(beta))) == 0, beta


def test_hinted_decode_needs_the_exact_quotient():
    """The hinted KV decode rounds p / 14 - h (h = 0 or 1/2) per coordinate.  A single fused multiply-add
    p * RN(1/14) - h in place of the correctly rounded quotient would be cheaper, and is wrong: for the
    coset-point coordinate p = 14 in the half-integer coset the exact value is the tie 0.5 (rounds to 0),
    the fused form gives 0.50000006 (rounds to 1).  This test keeps the counter-example, and checks that it
    is the only kind: every disagreement over the coordinates a coset point can have (multiples of 1/2;
    code digits up to 15 give [-15, 37.5]) sits on an exact tie of the reference's form."""
    c = np.float32(1.0) / np.float32(14.0)
    disagreements = []
    for twice in range(-30, 76):
        p = np.float32(twice / 2.0)
        exact = p / np.float32(14.0)                               # IEEE division, correctly rounded
        for half in (np.float32(0.0), np.float32(0.5)):
            reference = np.float32(exact - half)
            fused = np.float32(np.float64(p) * np.float64(c) - np.float64(half))   # one rounding of the exact value
            if np.rint(reference) != np.rint(fused):
                disagreements.append((float(p), float(half)))
                assert abs(float(reference) - np.floor(float(reference))) == 0.5
    assert (14.0, 0.5) in disagreements
