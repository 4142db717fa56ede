"""Pins the CPU oracle before anything is compared against it.

Nothing here retypes the oracle's formula and calls that a check: each test
confronts the C restatement with independent evidence -- the reference's own
closed-form fixtures evaluated separately in numpy, a second formulation of
the same unpacking (llama.cpp's kmask words), exact rational arithmetic
rounded step by step, a cross-format identity (Q3_K rewritten as Q6_K),
special cases that reduce to integer dots, and the literal expectations in
the reference's router tests.
"""
from fractions import Fraction

import numpy as np
import pytest

import ferrum_fixtures as fx
import oracle

Q4_K, Q6_K = 12, 14
F = np.float32


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


# ------------------------------------------------------------ conversions

def test_f16_widening_is_exact_for_every_bit_pattern():
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.f16_to_f32(int(v)) for v in h], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(bits(got)[~nan], bits(want)[~nan])


def test_f16_narrowing_rounds_to_nearest_even():
    rng = np.random.default_rng(7)
    samples = np.concatenate([
        rng.standard_normal(4000).astype(F) * F(3.0),
        (rng.standard_normal(2000) * 1e-6).astype(F),           # subnormal halves
        (rng.standard_normal(500) * 7e4).astype(F),              # overflow edge
        # exact ties between neighbouring halves, even and odd
        np.array([1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 2.0 ** -25, 3 * 2.0 ** -25,
                  65504.0, 65519.99, 65520.0, 0.0, -0.0, np.inf, -np.inf], dtype=F),
    ])
    want = samples.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16(v) for v in samples], dtype=np.uint16)
    assert np.array_equal(got, want)


def test_bf16_rounding_ties_and_nan():
    # tests/correctness.rs:300-318: 1 + 2^-8 is a tie that rounds to even (1.0),
    # 1.0078125 + 2^-8 is a tie that rounds up to 1.015625; NaN stays NaN.
    r = oracle.round_storage(np.array([1.0 + 0.00390625, 1.0078125 + 0.00390625, np.inf], dtype=F), 2)
    assert r[0] == 1.0 and r[1] == 1.015625 and r[2] == np.inf
    nan_bits = oracle.f32_to_bf16(float("nan"))
    assert (nan_bits & 0x7F80) == 0x7F80 and (nan_bits & 0x7F) != 0


# --------------------------------------------------------- 6-bit scale/min

def kmask_unpack(scales12: np.ndarray):
    """llama.cpp's word form (the `utmp` shuffle of ggml's q4_K dot product),
    an independent statement of the same packing."""
    u = scales12.view("<u4").astype(np.uint64)
    kmask1, kmask2, kmask3 = 0x3F3F3F3F, 0x0F0F0F0F, 0x03030303
    u0, u1, u2 = int(u[0]), int(u[1]), int(u[2])
    mins_hi = ((u2 >> 4) & kmask2) | (((u1 >> 6) & kmask3) << 4)
    sc_hi = (u2 & kmask2) | (((u0 >> 6) & kmask3) << 4)
    sc = np.array([(u0 & kmask1), sc_hi], dtype="<u4").view(np.uint8)
    mn = np.array([(u1 & kmask1), mins_hi], dtype="<u4").view(np.uint8)
    return sc, mn


def test_scale_min_matches_the_kmask_word_form():
    rng = np.random.default_rng(11)
    for _ in range(300):
        s = rng.integers(0, 256, 12, dtype=np.uint8)
        sc, mn = kmask_unpack(s)
        for g in range(8):
            assert oracle.q4_k_scale_min(s, g) == (int(sc[g]), int(mn[g]))


def test_scale_min_bruteforce_over_interacting_bytes():
    # group g >= 4 reads bytes g+4, g-4 and g; sweep every value of each pair.
    for g in range(8):
        for a in range(0, 256, 5):
            for b in range(0, 256, 3):
                s = np.zeros(12, dtype=np.uint8)
                if g < 4:
                    s[g], s[g + 4] = a, b
                    want = (a & 63, b & 63)
                else:
                    s[g + 4], s[g - 4], s[g] = a, b, (a * 7 + b) & 255
                    want = ((a & 15) | ((b >> 6) << 4), (a >> 4) | ((int(s[g]) >> 6) << 4))
                assert oracle.q4_k_scale_min(s, g) == want


def test_scale_pack_roundtrip_in_synthetic_generator():
    from ferrum_amd import synth
    rng = np.random.default_rng(3)
    sc = rng.integers(0, 64, (50, 8), dtype=np.uint8)
    mn = rng.integers(0, 64, (50, 8), dtype=np.uint8)
    packed = synth.pack_q4_k_scales(sc, mn)
    for i in range(50):
        for g in range(8):
            assert oracle.q4_k_scale_min(packed[i], g) == (int(sc[i, g]), int(mn[i, g]))


# ------------------------------------------------------------ dequantize

@pytest.mark.parametrize("rows,cols", [(5, 512), (7, 256), (3, 1024)])
def test_q4_k_block_decoder_equals_reference_closed_form(rows, cols):
    packed = fx.q4k_packed(rows, cols)
    assert packed.size == rows * (cols // 256) * 144
    dense = oracle.dequantize(Q4_K, packed, rows, cols)
    assert np.array_equal(bits(dense), bits(fx.q4k_dense(rows, cols)))


@pytest.mark.parametrize("rows,cols", [(5, 512), (7, 256)])
def test_q6_k_block_decoder_equals_reference_closed_form(rows, cols):
    packed = fx.q6k_packed(rows, cols)
    assert packed.size == rows * (cols // 256) * 210
    dense = oracle.dequantize(Q6_K, packed, rows, cols)
    assert np.array_equal(bits(dense), bits(fx.q6k_dense(rows, cols)))
    # the second Q6_K generator (inside qk_tests)
    packed = fx.qk_q6_packed(rows, cols)
    dense = oracle.dequantize(Q6_K, packed, rows, cols)
    want = np.array([[fx.qk_q6_value(r, c) for c in range(cols)] for r in range(rows)], dtype=F)
    assert np.array_equal(bits(dense), bits(want))


@pytest.mark.parametrize("ggml_type", [Q4_K, Q6_K])
def test_block_form_equals_per_element_form_on_random_blocks(ggml_type):
    rows, cols = 6, 768
    packed = fx.xorshift_blocks(ggml_type, rows * cols // 256)
    dense = oracle.dequantize(ggml_type, packed, rows, cols)
    rng = np.random.default_rng(5)
    for _ in range(3000):
        r, c = int(rng.integers(rows)), int(rng.integers(cols))
        got = np.float32(oracle.weight(ggml_type, packed, r, c, cols))
        assert bits(got) == bits(dense[r, c])


def round_f32(value: Fraction) -> np.float32:
    """Correctly rounded (nearest-even) float32 of an exact rational."""
    if value == 0:
        return F(0.0)
    sign = -1 if value < 0 else 1
    v = abs(value)
    e = 0
    while v >= (1 << 24):
        v /= 2
        e += 1
    while v < (1 << 23) and e > -149:
        v *= 2
        e -= 1
    q, r = divmod(v.numerator, v.denominator)
    twice = 2 * r
    if twice > v.denominator or (twice == v.denominator and q & 1):
        q += 1
    return F(sign * float(q) * 2.0 ** e)


def test_q4_k_expression_order_against_exact_rationals():
    # ((d*sc)*q) - (dmin*m), one rounding per step.  Because d and dmin are
    # f16 (11 significant bits), d*sc (<= 17 bits), (d*sc)*q (<= 21 bits) and
    # dmin*m (<= 17 bits) are all exact in f32: only the subtraction rounds,
    # so the value must also equal the correctly rounded exact rational
    # d*sc*q - dmin*m.  A wrong scale, nibble or sign fails both comparisons.
    rng = np.random.default_rng(23)
    for _ in range(400):
        block = rng.integers(0, 256, 144, dtype=np.uint8)
        block[0:2] = np.frombuffer(np.float16(abs(rng.standard_normal()) * 0.01).tobytes(), np.uint8)
        block[2:4] = np.frombuffer(np.float16(abs(rng.standard_normal()) * 0.005).tobytes(), np.uint8)
        dense = oracle.dequantize(Q4_K, block, 1, 256)[0]
        d = Fraction(float(block[0:2].view(np.float16)[0]))
        dmin = Fraction(float(block[2:4].view(np.float16)[0]))
        for w in rng.integers(0, 256, 12):
            group = int(w) // 32
            sc, mn = fx._unpack_scale_min(block[4:16], group)
            byte = int(block[16 + (int(w) // 64) * 32 + int(w) % 32])
            q = byte & 15 if group % 2 == 0 else byte >> 4
            a = round_f32(d * sc)
            b = round_f32(Fraction(float(a)) * q)
            c = round_f32(dmin * mn)
            want = round_f32(Fraction(float(b)) - Fraction(float(c)))
            assert bits(dense[int(w)]) == bits(want)
            assert Fraction(float(a)) == d * sc and Fraction(float(b)) == d * sc * q
            assert bits(round_f32(d * sc * q - dmin * mn)) == bits(want)


def test_q6_k_expression_order_against_exact_rationals():
    # (d*scale)*q: 11 + 7 + 6 significant bits fit f32's 24, so for normal
    # results both products are exact and the value equals the exact rational.
    rng = np.random.default_rng(29)
    for _ in range(300):
        block = rng.integers(0, 256, 210, dtype=np.uint8)
        block[208:210] = np.frombuffer(np.float16(abs(rng.standard_normal()) * 0.002 + 1e-4).tobytes(), np.uint8)
        dense = oracle.dequantize(Q6_K, block, 1, 256)[0]
        d = Fraction(float(block[208:210].view(np.float16)[0]))
        for w in rng.integers(0, 256, 12):
            w = int(w)
            group, lane = w // 32, w % 32
            half, slc = group // 4, group % 4
            byte = int(block[half * 64 + (slc & 1) * 32 + lane])
            low = byte & 15 if slc < 2 else byte >> 4
            high = (int(block[128 + half * 32 + lane]) >> (2 * slc)) & 3
            q = (low | (high << 4)) - 32
            scale = int(block[192 + half * 8 + slc * 2 + lane // 16].view(np.int8))
            a = round_f32(d * scale)
            want = round_f32(Fraction(float(a)) * q)
            if want == 0 and (scale < 0) != (q < 0):
                want = F(-0.0)          # IEEE sign of a zero product
            assert bits(dense[w]) == bits(want)
            assert round_f32(d * scale * q) == want


# --- Q3_K rewritten as Q6_K keeps every value (src/hybrid/iq_tests.rs:1503-1527)

def dequant_q3_k_numpy(q3: np.ndarray) -> np.ndarray:
    """ggml's dequantize_row_q3_K (110-byte blocks: hmask[32], qs[64],
    scales[12], f16 d), written from the published algorithm."""
    out = []
    for b in q3.reshape(-1, 110):
        hm, qs = b[:32], b[32:96]
        d_all = F(b[108:110].view(np.float16)[0])
        aux = [int(v) for v in b[96:108].view("<u4")] + [0]
        k1, k2 = 0x03030303, 0x0F0F0F0F
        tmp = aux[2]
        aux[2] = ((aux[0] >> 4) & k2) | (((tmp >> 4) & k1) << 4)
        aux[3] = ((aux[1] >> 4) & k2) | (((tmp >> 6) & k1) << 4)
        aux[0] = (aux[0] & k2) | ((tmp & k1) << 4)
        aux[1] = (aux[1] & k2) | (((tmp >> 2) & k1) << 4)
        scales = np.array(aux, dtype="<u4").view(np.int8)
        y = np.zeros(256, dtype=F)
        is_, m, at = 0, 1, 0
        for n in range(2):
            q = qs[32 * n:]
            for shift in (0, 2, 4, 6):
                for half in range(2):
                    dl = F(d_all * F(int(scales[is_]) - 32))
                    is_ += 1
                    for l in range(16 * half, 16 * half + 16):
                        v = ((int(q[l]) >> shift) & 3) - (0 if int(hm[l]) & m else 4)
                        y[at] = F(dl * F(v))
                        at += 1
                m <<= 1
        out.append(y)
    return np.concatenate(out)


def q3k_to_q6k_numpy(q3: np.ndarray) -> np.ndarray:
    """The value-preserving rewrite (src/hybrid/weights.rs:761-805)."""
    blocks = q3.reshape(-1, 110)
    out = np.zeros((blocks.shape[0], 210), dtype=np.uint8)
    for x, y in zip(blocks, out):
        hmask, qs, packed = x[:32], x[32:96], x[96:108]
        scales = np.zeros(16, dtype=np.int8)
        for j in range(16):
            low = int(packed[j]) & 0xF if j < 8 else int(packed[j - 8]) >> 4
            high = (int(packed[8 + j % 4]) >> (2 * (j // 4))) & 3
            scales[j] = (low | (high << 4)) - 32
        q = np.zeros(256, dtype=np.int32)
        for i in range(256):
            half, rest = divmod(i, 128)
            shift, l = divmod(rest, 32)
            low = (int(qs[32 * half + l]) >> (2 * shift)) & 3
            high = (int(hmask[l]) >> (4 * half + shift)) & 1
            q[i] = low + 4 * high + 28
        for half in range(2):
            for l in range(32):
                at = [q[128 * half + l + 32 * k] for k in range(4)]
                y[64 * half + l] = (at[0] & 0xF) | ((at[2] & 0xF) << 4)
                y[64 * half + l + 32] = (at[1] & 0xF) | ((at[3] & 0xF) << 4)
                y[128 + 32 * half + l] = (at[0] >> 4) | ((at[1] >> 4) << 2) | ((at[2] >> 4) << 4) | ((at[3] >> 4) << 6)
        y[192:208] = scales.view(np.uint8)
        y[208:210] = x[108:110]
    return out.reshape(-1)


def test_q6_k_decoder_agrees_with_q3_k_through_the_rewrite():
    blocks = 24
    q3 = fx.iq_random_blocks(blocks, 110, 5).reshape(blocks, 110)
    for b in q3:
        b[108:110] = np.frombuffer(
            np.array([F(0.002) + F(0.001) * F(b[0]) / F(255.0)], dtype=F).astype(np.float16).tobytes(), np.uint8)
    q3 = q3.reshape(-1)
    want = dequant_q3_k_numpy(q3)
    got = oracle.dequantize(Q6_K, q3k_to_q6k_numpy(q3), blocks, 256).reshape(-1)
    assert np.any(want != 0)
    assert np.array_equal(bits(got), bits(want))


# ---------------------------------------------------------------- validate

def test_payload_validation_rejects_partial_blocks_and_nonfinite_scales():
    good = fx.q4k_packed(2, 256)
    assert oracle.validate_payload(Q4_K, good) == 0
    assert oracle.validate_payload(Q4_K, good[:-1]) == 1
    bad = good.copy()
    bad[144:146] = np.frombuffer(np.float16(np.inf).tobytes(), np.uint8)
    assert oracle.validate_payload(Q4_K, bad) == 2
    bad = good.copy()
    bad[2:4] = np.frombuffer(np.float16(np.nan).tobytes(), np.uint8)
    assert oracle.validate_payload(Q4_K, bad) == 2
    good6 = fx.q6k_packed(2, 256)
    assert oracle.validate_payload(Q6_K, good6) == 0
    bad6 = good6.copy()
    bad6[208:210] = np.frombuffer(np.float16(-np.inf).tobytes(), np.uint8)
    assert oracle.validate_payload(Q6_K, bad6) == 2


# ----------------------------------------------------------------- project

def integer_q4_k_blocks(rows, cols, rng):
    """d = 1, dmin = 0, every scale 1: the matrix is its own nibbles."""
    nb = rows * cols // 256
    blocks = np.zeros((nb, 144), dtype=np.uint8)
    blocks[:, 0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    sc = np.ones((nb, 8), dtype=np.uint8)
    mn = np.zeros((nb, 8), dtype=np.uint8)
    from ferrum_amd import synth
    blocks[:, 4:16] = synth.pack_q4_k_scales(sc, mn)
    blocks[:, 16:] = rng.integers(0, 256, (nb, 128), dtype=np.uint8)
    return blocks.reshape(-1)


def test_project_integer_special_case_is_an_exact_integer_dot():
    rng = np.random.default_rng(41)
    n, k, m = 9, 1024, 3
    packed = integer_q4_k_blocks(n, k, rng)
    qs = packed.reshape(n, k // 256, 144)[:, :, 16:]
    w = np.zeros((n, k // 256, 256), dtype=np.int64)
    for chunk in range(4):
        w[:, :, 64 * chunk:64 * chunk + 32] = qs[:, :, 32 * chunk:32 * chunk + 32] & 15
        w[:, :, 64 * chunk + 32:64 * chunk + 64] = qs[:, :, 32 * chunk:32 * chunk + 32] >> 4
    w = w.reshape(n, k)
    x = rng.integers(-8, 9, (m, k)).astype(F)
    want = (x.astype(np.int64) @ w.T).astype(F)      # |sum| < 2^24: exact in f32
    for acc in ("f32", "f64"):
        got = oracle.project(Q4_K, packed, n, k, x, accumulate=acc)
        assert np.array_equal(got, want)
    # a transposed operand or swapped nibble order would fail the line above
    assert not np.array_equal(want, (x.astype(np.int64) @ w[:, ::-1].T).astype(F))


def test_project_zero_quants_reduce_to_minus_dmin_m_sum_x():
    rng = np.random.default_rng(43)
    n, k = 4, 512
    packed = fx.xorshift_blocks(Q4_K, n * k // 256).reshape(-1, 144)
    packed[:, 16:] = 0
    x = rng.integers(-4, 5, (1, k)).astype(F)
    got = oracle.project(Q4_K, packed.reshape(-1), n, k, x, accumulate="f64")[0]
    for row in range(n):
        total = 0.0
        for b in range(k // 256):
            blk = packed[row * (k // 256) + b]
            dmin = float(blk[2:4].view(np.float16)[0])
            for g in range(8):
                _, mn = fx._unpack_scale_min(blk[4:16], g)
                total -= float(F(F(dmin) * F(mn))) * float(x[0, b * 256 + g * 32:b * 256 + g * 32 + 32].sum())
        assert got[row] == pytest.approx(total, rel=1e-6, abs=1e-7)


@pytest.mark.parametrize("ggml_type", [Q4_K, Q6_K])
def test_project_matches_numpy_float64_matmul_of_the_dequantized_matrix(ggml_type):
    n, k, m = 37, 1280, 5
    packed = fx.xorshift_blocks(ggml_type, n * k // 256)
    dense = oracle.dequantize(ggml_type, packed, n, k)
    x = fx.xorshift_uniform(m * k, 31).reshape(m, k)
    want = x.astype(np.float64) @ dense.astype(np.float64).T
    got64 = oracle.project(ggml_type, packed, n, k, x, accumulate="f64", threads=3)
    assert np.array_equal(got64, want.astype(F)) or np.abs(got64 - want).max() <= 1e-6 * np.abs(want).max()
    got32 = oracle.project(ggml_type, packed, n, k, x, accumulate="f32")
    assert np.abs(got32 - want).max() <= 2e-5 * np.abs(want).max()
    # threads only split rows: bitwise the same
    assert np.array_equal(got32, oracle.project(ggml_type, packed, n, k, x, accumulate="f32", threads=4))


def test_project_reproduces_the_reference_gemv_gemm_expectations():
    # src/ops/transformer.rs:2982-3002 and :4251-4269: (N, K) = (5, 512), M in
    # {1,2,3,4,5,7}; the sequential-f32 answer built from the closed form.
    n, k = 5, 512
    p4, d4 = fx.q4k_packed(n, k), fx.q4k_dense(n, k)
    p6, d6 = fx.q6k_packed(n, k), fx.q6k_dense(n, k)
    for m in (1, 2, 3, 4, 5, 7):
        x = fx.q4k_input(m, k)
        assert np.array_equal(oracle.project(Q4_K, p4, n, k, x), fx.expected_f32seq(x, d4))
        x = fx.q6k_input(m, k)
        assert np.array_equal(oracle.project(Q6_K, p6, n, k, x), fx.expected_f32seq(x, d6))


def test_project_weight_rounding_mirrors_the_tile_tests():
    # src/ops/transformer.rs:3130-3141: weights rounded to the tile dtype first.
    n, k, m = 5, 512, 4
    packed = fx.q4k_packed(n, k)
    x = oracle.round_storage(fx.q4k_input(m, k), oracle.BF16)
    dense = oracle.round_storage(fx.q4k_dense(n, k), oracle.BF16)
    want = fx.expected_f32seq(x, dense)
    got = oracle.project(Q4_K, packed, n, k, x, weight_round=oracle.BF16)
    assert np.array_equal(got, want)


# ------------------------------------------------------------------ router

def test_sigmoid_top_k_routes_normalize_and_apply_scale():
    # src/nn/moe.rs:666-703
    r = oracle.select_routes([0.0, 2.0, -2.0], 3, 2, sigmoid=True, normalize=True, eps=1e-6,
                             scaling=1.5).reshape(-1)
    assert bits(r[0]) == 0 and bits(r[1]) == 0 and bits(r[3]) == 1
    s0, s2 = 0.5, 1.0 / (1.0 + np.exp(-2.0))
    den = s0 + s2 + 1e-6
    assert abs(r[2] - s0 / den * 1.5) < 1e-6 and abs(r[5] - s2 / den * 1.5) < 1e-6
    assert abs(r[2] + r[5] - 1.5) < 2e-6


def test_sigmoid_expert_bias_changes_selection_not_scores():
    # src/nn/moe.rs:705-739
    r = oracle.select_routes([2.0, 1.0, 0.0], 3, 2, sigmoid=True, normalize=True, eps=1e-6,
                             scaling=1.0, bias=[-10.0, 0.0, 2.0]).reshape(-1)
    s1, s0 = 1.0 / (1.0 + np.exp(-1.0)), 0.5
    den = s1 + s0 + 1e-6
    assert bits(r[0]) == 1 and abs(r[2] - s1 / den) < 1e-6
    assert bits(r[3]) == 2 and abs(r[5] - s0 / den) < 1e-6


def test_router_tie_break_order_and_softmax_weights():
    # src/nn/moe.rs:741-819 logits; all-equal scores break ties by lower id
    # after the bias reorders them; softmax weights vs float64.
    logits = np.array([[0, 0, 0, 0, 0], [2, 0.5, -1, 1.5, 0]], dtype=F)
    bias = np.array([0.1, 0.05, 0.1, -0.3, 0.1], dtype=F)
    r = oracle.select_routes(logits, 5, 3, normalize=True, eps=1e-6, scaling=1.25, bias=bias)
    ids = bits(r[:, 0]).reshape(2, 3)
    assert ids[0].tolist() == [0, 2, 4]          # 0.3, 0.3, 0.3 beat 0.25 and -0.1
    p = np.exp(logits[1].astype(np.float64) - 2.0)
    p /= p.sum()
    order = sorted(range(5), key=lambda e: (-(np.float32(p[e]) + bias[e]), e))[:3]
    assert ids[1].tolist() == sorted(order)
    sel = sorted(order)
    want = p[sel] / (p[order].sum() + 1e-6) * 1.25
    assert np.allclose(r[3:, 2], want, atol=2e-6)
    assert bits(r[:, 1]).tolist() == [0, 0, 0, 1, 1, 1]


def test_top_k_equal_to_experts_with_equal_logits_is_a_uniform_mean():
    r = oracle.select_routes(np.zeros((1, 8), dtype=F), 8, 8, normalize=True)
    assert bits(r[:, 0]).tolist() == list(range(8))
    assert np.allclose(r[:, 2], 0.125, atol=1e-7)


def test_invalid_logits_are_rejected():
    with pytest.raises(ValueError):
        oracle.select_routes([0.0, np.nan, 1.0], 3, 2)


# -------------------------------------------------------------- MoE stages

def test_expert_pipeline_matches_a_float64_restatement():
    rng = np.random.default_rng(61)
    experts, hidden, inter, tokens, top_k = 4, 256, 256, 6, 2
    w_in = fx.xorshift_blocks(Q4_K, experts * 2 * inter * hidden // 256)
    w_out = fx.xorshift_blocks(Q6_K, experts * hidden * inter // 256)
    d_in = oracle.dequantize(Q4_K, w_in, experts * 2 * inter, hidden).astype(np.float64)
    d_out = oracle.dequantize(Q6_K, w_out, experts * hidden, inter).astype(np.float64)
    x = rng.standard_normal((tokens, hidden)).astype(F)
    logits = rng.standard_normal((tokens, experts)).astype(F)
    meta = oracle.select_routes(logits, experts, top_k, normalize=True)
    assigned = oracle.expert_assign(x, meta)
    up = oracle.expert_project(Q4_K, w_in, experts, 2 * inter, hidden, assigned, meta)
    act = oracle.expert_silu_mul(up, inter)
    down = oracle.expert_project(Q6_K, w_out, experts, hidden, inter, act, meta)
    got = oracle.expert_combine(down, meta, tokens, hidden, top_k)

    want = np.zeros((tokens, hidden))
    ids = bits(meta[:, 0]).reshape(tokens, top_k)
    for t in range(tokens):
        for rank in range(top_k):
            e = int(ids[t, rank])
            h = d_in[e * 2 * inter:(e + 1) * 2 * inter] @ x[t].astype(np.float64)
            g, u = h[:inter], h[inter:]
            a = g / (1.0 + np.exp(-g)) * u
            want[t] += float(meta[t * top_k + rank, 2]) * (d_out[e * hidden:(e + 1) * hidden] @ a)
    assert np.abs(want).max() > 1e-3
    assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max())


def test_storage_rounding_points_of_silu_mul_and_combine():
    # ops.metal:2223-2246: silu is rounded before the product; each gated term
    # is rounded before it joins the f32 running total.
    gate, up = F(0.7312), F(1.3377)
    out = oracle.expert_silu_mul(np.array([[gate, up]], dtype=F), 1, oracle.BF16)[0, 0]
    s = oracle.round_storage([gate * (1.0 / (1.0 + np.exp(-np.float64(gate))))], oracle.BF16)[0]
    assert out == oracle.round_storage([F(s * up)], oracle.BF16)[0]
    meta = np.array([[0, 0, 0.30078125 + 2 ** -10], [0, 0, 0.7]], dtype=F)
    meta[:, 0] = np.array([1, 3], dtype=np.uint32).view(F)
    vals = np.array([[1.2345], [2.5]], dtype=F)
    got = oracle.expert_combine(vals, meta, 1, 1, 2, oracle.BF16)[0, 0]
    r = lambda v: oracle.round_storage([v], oracle.BF16)[0]
    want = r(F(r(F(r(meta[0, 2]) * vals[0, 0])) + r(F(r(meta[1, 2]) * vals[1, 0]))))
    assert got == want


def test_argmax_rows_is_the_first_maximal_index_and_flags_non_finite_rows():
    # numpy's argmax (first occurrence of the maximum) pins the finite case; the
    # flagged cases follow the reference kernel's own scan and merge order
    rng = np.random.default_rng(17)
    for width in (1, 31, 1024, 1025, 5000):
        x = rng.standard_normal((6, width)).astype(np.float32)
        if width > 40:
            x[1, 5] = x[1, width - 3] = 9.0       # a tie: the lower index wins
            x[2, 7] = -np.inf                     # non-finite but not maximal
            x[3, 11] = np.inf
        got = oracle.argmax_rows(x)
        assert np.array_equal(got[:, 0], x.argmax(axis=1).astype(np.uint32)), width
        assert np.array_equal(got[:, 1], (~np.isfinite(x)).any(axis=1).astype(np.uint32))
    x = rng.standard_normal((3, 3000)).astype(np.float32)
    x[0, 0] = np.nan        # thread 0 starts on NaN and never leaves it
    x[1, 2047] = np.nan     # a NaN later in a thread's scan is skipped
    x[2, :] = np.nan
    got = oracle.argmax_rows(x)
    assert got[:, 1].tolist() == [1, 1, 1]
    assert got[0, 0] == 0 and got[2, 0] == 0
    y = x[1].copy(); y[2047] = -np.inf
    assert got[1, 0] == y.argmax()


def test_add_rmsnorm_closed_forms():
    eps = 1e-6
    # constant rows: every element is c / sqrt(c^2 + eps) times its weight
    width = 96
    w = (1.0 + fx.deterministic(width)).astype(np.float32)
    a = np.full((2, width), 0.75, np.float32)
    b = np.full((2, width), -0.25, np.float32)
    residual, normed = oracle.add_rmsnorm(a, b, w, eps)
    assert np.array_equal(residual, np.full((2, width), 0.5, np.float32))
    assert np.allclose(normed, (0.5 / np.sqrt(0.25 + eps)) * w.astype(np.float64), rtol=1e-7, atol=0)
    # a one-hot row: mean of squares is v^2 / width
    a = np.zeros((1, width), np.float32); b = np.zeros((1, width), np.float32)
    a[0, 17] = 3.0; b[0, 17] = 1.0
    residual, normed = oracle.add_rmsnorm(a, b, w, eps)
    want = np.zeros(width); want[17] = 4.0 / np.sqrt(16.0 / width + eps) * float(w[17])
    assert np.allclose(normed[0], want, rtol=1e-7, atol=0)
    # scale invariance up to eps, and unit mean square of normed / weight
    x = fx.deterministic(4 * 1000).reshape(4, 1000)
    y = fx.deterministic(4 * 1000 + 11)[11:].reshape(4, 1000)
    w = (2.0 + fx.deterministic(1003)[3:]).astype(np.float32)      # 0.25 .. 3.8, never zero
    r1, n1 = oracle.add_rmsnorm(x, y, w, eps)
    r4, n4 = oracle.add_rmsnorm(4 * x, 4 * y, w, eps)
    assert np.array_equal(r4, 4 * r1)
    assert np.allclose(n4, n1, rtol=2e-6, atol=0)
    ms = ((n1.astype(np.float64) / w) ** 2).mean(axis=1)
    assert np.allclose(ms, 1.0, atol=1e-5)
    # the residual of 16-bit rows is the rounded sum, and the norm is taken of the rounded values
    for code in (oracle.F16, oracle.BF16):
        xs = oracle.round_storage(x, code).reshape(x.shape); ys = oracle.round_storage(y, code).reshape(y.shape)
        ws = oracle.round_storage(w, code)
        residual, normed = oracle.add_rmsnorm(xs, ys, ws, eps, code)
        assert np.array_equal(residual, oracle.round_storage(xs + ys, code).reshape(x.shape))
        r64 = residual.astype(np.float64)
        want = r64 / np.sqrt((r64 ** 2).mean(axis=1, keepdims=True) + eps) * ws.astype(np.float64)
        assert np.allclose(normed, want, rtol=1e-6, atol=0)


def _ranked_by_numpy(logits, top_k, sigmoid, norm):
    """The CPU procedure of the reference's own routing test
    (src/hybrid/engine.rs:5004-5024) in float64 numpy."""
    ids, weights = [], []
    for row in logits.astype(np.float64):
        scores = 1 / (1 + np.exp(-row)) if sigmoid else np.exp(row - row.max()) / np.exp(row - row.max()).sum()
        order = np.lexsort((np.arange(row.size), -scores))[:top_k]
        w = scores[order]
        ids.append(order)
        weights.append(w / w.sum() if norm else w)
    return np.array(ids), np.array(weights)


def test_ranked_routing_follows_the_hybrid_engines_cpu_procedure():
    rng = np.random.default_rng(21)
    experts, top_k, tokens = 256, 6, 3
    logits = (rng.standard_normal((tokens, experts)) * 3).astype(np.float32)
    for sigmoid, norm in ((True, True), (False, True), (True, False)):
        meta = oracle.select_routes_ranked(logits, experts, top_k, sigmoid=sigmoid, normalize=norm)
        want_ids, want_w = _ranked_by_numpy(logits, top_k, sigmoid, norm)
        assert np.array_equal(meta[:, 0].view(np.uint32).reshape(tokens, top_k), want_ids)
        assert np.array_equal(meta[:, 1].view(np.uint32).reshape(tokens, top_k),
                              np.repeat(np.arange(tokens), top_k).reshape(tokens, top_k))
        assert np.abs(meta[:, 2].reshape(tokens, top_k) - want_w).max() < 1e-6
    # equal logits: ties go to the lower index, in rank order
    meta = oracle.select_routes_ranked(np.zeros((1, 8), np.float32), 8, 3)
    assert meta[:, 0].view(np.uint32).tolist() == [0, 1, 2]
    # the same selection as the id-ordered form, in a different row order
    plain = oracle.select_routes(logits, experts, top_k)
    ranked = oracle.select_routes_ranked(logits, experts, top_k)
    for t in range(tokens):
        a = plain[t * top_k:(t + 1) * top_k]
        b = ranked[t * top_k:(t + 1) * top_k]
        assert sorted(a[:, 0].view(np.uint32)) == sorted(b[:, 0].view(np.uint32))
        assert np.all(np.diff(b[:, 2]) <= 0)


def test_shared_gate_and_combine_with_a_shared_expert():
    rng = np.random.default_rng(22)
    tokens, hidden, top_k = 3, 64, 2
    x = rng.standard_normal((tokens, hidden)).astype(np.float32)
    w = rng.standard_normal(hidden).astype(np.float32)
    gate = oracle.shared_gate(x, w)
    assert np.allclose(gate, 1 / (1 + np.exp(-(x.astype(np.float64) @ w.astype(np.float64)))), rtol=1e-6)
    down = rng.standard_normal((tokens * top_k, hidden)).astype(np.float32)
    shared = rng.standard_normal((tokens, hidden)).astype(np.float32)
    meta = np.zeros((tokens * top_k, 3), np.float32)
    meta[:, 2] = rng.random(tokens * top_k).astype(np.float32)
    got = oracle.expert_combine_shared(down, meta, tokens, hidden, top_k, shared, gate)
    want = (meta[:, 2:3].astype(np.float64) * down).reshape(tokens, top_k, hidden).sum(1) + gate[:, None] * shared
    assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    plain = oracle.expert_combine(down, meta, tokens, hidden, top_k)
    assert np.array_equal(oracle.expert_combine_shared(down, meta, tokens, hidden, top_k, np.zeros_like(shared)), plain)


# ------------------------------------------------------------------ Q5_K

Q5_K = 13


@pytest.mark.parametrize("rows,cols", [(5, 512), (7, 256), (3, 1024)])
def test_q5_k_block_decoder_equals_reference_closed_form(rows, cols):
    # the Q5_K branch of the reference's qk_tests (src/ops/transformer.rs:2843-2952)
    packed = fx.q5k_packed(rows, cols)
    assert packed.size == rows * (cols // 256) * 176 == rows * (cols // 256) * oracle.block_bytes(Q5_K)
    dense = oracle.dequantize(Q5_K, packed, rows, cols)
    assert np.array_equal(bits(dense), bits(fx.q5k_dense(rows, cols)))


def test_q5_k_block_form_per_element_form_and_the_q4_k_special_case_agree():
    from ferrum_amd import synth
    rows, cols = 6, 768
    packed = synth.matrix(Q5_K, rows, cols, seed=71)
    dense = oracle.dequantize(Q5_K, packed, rows, cols)
    rng = np.random.default_rng(6)
    for _ in range(3000):
        r, c = int(rng.integers(rows)), int(rng.integers(cols))
        assert bits(np.float32(oracle.weight(Q5_K, packed, r, c, cols))) == bits(dense[r, c])
    # with every fifth bit clear a Q5_K block is the Q4_K block with the same header and nibbles
    blocks = packed.reshape(-1, 176).copy()
    blocks[:, 16:48] = 0
    as_q4 = np.concatenate([blocks[:, :16], blocks[:, 48:]], axis=1)
    assert np.array_equal(bits(oracle.dequantize(Q5_K, blocks.reshape(-1), rows, cols)),
                          bits(oracle.dequantize(Q4_K, as_q4.reshape(-1), rows, cols)))
    # and setting them all adds 16 * d * sc to every weight
    blocks[:, 16:48] = 255
    up = oracle.dequantize(Q5_K, blocks.reshape(-1), rows, cols).astype(np.float64)
    base = oracle.dequantize(Q4_K, as_q4.reshape(-1), rows, cols).astype(np.float64)
    d = blocks[:, 0:2].copy().view(np.float16).astype(np.float64).reshape(rows, cols // 256, 1)
    sc = np.array([[oracle.q4_k_scale_min(b[4:16], g)[0] for g in range(8)] for b in blocks], dtype=np.float64)
    step = (16 * d * sc.reshape(rows, cols // 256, 8)).repeat(32, axis=2).reshape(rows, cols)
    assert np.abs(up - base - step).max() <= 1e-6 * np.abs(step).max()
    x = fx.xorshift_uniform(3 * cols, 9).reshape(3, cols)
    want = x.astype(np.float64) @ dense.astype(np.float64).T
    assert np.abs(oracle.project(Q5_K, packed, rows, cols, x, accumulate="f64") - want).max() <= 1e-6 * np.abs(want).max()


# ---------------------------------------------------------------- IQ4_XS

IQ4_XS = 23


def test_iq4_xs_two_reference_statements_agree_and_values_are_exact():
    # block form = dequantize_iq4_xs, per-element form = the indexing of mv_iq4_xs
    rows, cols = 13, 1024          # the geometry of the hybrid engine's own format tests
    packed = fx.hybrid_random_blocks(rows * cols // 256, 136, 136)
    assert oracle.block_bytes(IQ4_XS) == 136 and oracle.validate_payload(IQ4_XS, packed) == 0
    dense = oracle.dequantize(IQ4_XS, packed, rows, cols)
    rng = np.random.default_rng(23)
    for _ in range(4000):
        r, c = int(rng.integers(rows)), int(rng.integers(cols))
        assert bits(np.float32(oracle.weight(IQ4_XS, packed, r, c, cols))) == bits(dense[r, c])
    # every value is d * (ls - 32) * codebook exactly: no rounding happens in f32
    blocks = packed.reshape(-1, 136)
    for bi in (0, 7, 51):
        b = blocks[bi]
        d = Fraction(float(b[0:2].copy().view(np.float16)[0]))
        scales_h = int(b[2]) | (int(b[3]) << 8)
        for sub in range(8):
            ls = ((int(b[4 + sub // 2]) >> (4 * (sub % 2))) & 15) | (((scales_h >> (2 * sub)) & 3) << 4)
            for j in range(32):
                byte = int(b[8 + 16 * sub + (j & 15)])
                value = int(fx.IQ4_VALUES[byte & 15 if j < 16 else byte >> 4])
                want = d * (ls - 32) * value
                got = Fraction(float(dense.reshape(-1, 256)[bi, 32 * sub + j]))
                assert got == want


def test_iq4_xs_reduces_to_the_reference_iq4_nl_decoder():
    # with ls = 33 every sub-block is an IQ4_NL block of the same d and the same 16 bytes
    count = 40
    rng = np.random.default_rng(5)
    d = (0.01 + 0.02 * rng.random(count)).astype(np.float16)
    index = rng.integers(0, 16, (count, 256), dtype=np.uint8)
    packed = fx.iq4_xs_pack(d, np.full((count, 8), 33), index)
    dense = oracle.dequantize(IQ4_XS, packed.reshape(-1), count, 256)
    nl = np.empty((count, 8, 18), dtype=np.uint8)
    nl[:, :, 0:2] = d.view(np.uint8).reshape(count, 1, 2)
    nl[:, :, 2:] = packed[:, 8:].reshape(count, 8, 16)
    assert np.array_equal(bits(dense), bits(fx.iq4_nl_dense(nl).reshape(count, 256)))


def test_iq4_xs_scale_bits_at_every_position():
    # all 64 scale values at each of the 8 sub-block positions, the others held at 32 (zero)
    d = np.float16(0.03125)
    index = np.full((1, 256), 15, dtype=np.uint8)        # codebook value 113
    for position in range(8):
        for ls in range(64):
            scales = np.full((1, 8), 32)
            scales[0, position] = ls
            dense = oracle.dequantize(IQ4_XS, fx.iq4_xs_pack([d], scales, index).reshape(-1), 1, 256)[0]
            want = np.zeros(256, dtype=np.float32)
            want[32 * position: 32 * position + 32] = np.float32(d) * np.float32(ls - 32) * np.float32(113)
            assert np.array_equal(bits(dense), bits(want)), (position, ls)


def test_iq4_xs_projection_is_the_float64_product_of_the_dequantised_matrix():
    from ferrum_amd import synth
    rows, cols = 9, 1280
    packed = synth.matrix(IQ4_XS, rows, cols, seed=81)
    dense = oracle.dequantize(IQ4_XS, packed, rows, cols)
    assert np.isfinite(dense).all() and np.abs(dense).max() > 0
    # the synthetic packer and the fixture packer are separate code: same fields, same bytes
    blocks = packed.reshape(-1, 136)
    scales_h = blocks[:, 2].astype(np.uint32) | (blocks[:, 3].astype(np.uint32) << 8)
    ls = np.stack([((blocks[:, 4 + i // 2] >> (4 * (i % 2))) & 15) | (((scales_h >> (2 * i)) & 3) << 4)
                   for i in range(8)], axis=1)
    q = blocks[:, 8:].reshape(-1, 8, 16)
    index = np.concatenate([q & 15, q >> 4], axis=2).reshape(-1, 256)
    assert np.array_equal(fx.iq4_xs_pack(blocks[:, 0:2].copy().view(np.float16).reshape(-1), ls, index), blocks)
    x = fx.xorshift_uniform(3 * cols, 9).reshape(3, cols)
    want = x.astype(np.float64) @ dense.astype(np.float64).T
    assert np.abs(oracle.project(IQ4_XS, packed, rows, cols, x, accumulate="f64") - want).max() <= 1e-6 * np.abs(want).max()
    assert oracle.validate_payload(IQ4_XS, packed[:-1]) == 1
    bad = packed.copy(); bad[0:2] = np.frombuffer(np.float16(np.inf).tobytes(), dtype=np.uint8)
    assert oracle.validate_payload(IQ4_XS, bad) == 2


# ------------------------------------------------------------------ Q8_0

Q8_0 = 8


def test_q8_0_decoder_equals_numpy_on_the_reference_generator():
    # value = q * d (src/hybrid/draft/gguf.rs:331-338); 256 weights are eight 34-byte blocks
    rows, cols = 13, 1024
    packed = fx.hybrid_random_blocks(rows * cols // 32, 34, 34)
    assert oracle.block_bytes(Q8_0) == 272 and oracle.validate_payload(Q8_0, packed) == 0
    b = packed.reshape(-1, 34)
    want = (b[:, 2:].view(np.int8).astype(np.float32)
            * b[:, 0:2].copy().view(np.float16).astype(np.float32)).reshape(rows, cols)
    dense = oracle.dequantize(Q8_0, packed, rows, cols)
    assert np.array_equal(bits(dense), bits(want))
    rng = np.random.default_rng(8)
    for _ in range(3000):
        r, c = int(rng.integers(rows)), int(rng.integers(cols))
        assert bits(np.float32(oracle.weight(Q8_0, packed, r, c, cols))) == bits(dense[r, c])
    x = fx.xorshift_uniform(3 * cols, 9).reshape(3, cols)
    ref = x.astype(np.float64) @ dense.astype(np.float64).T
    assert np.abs(oracle.project(Q8_0, packed, rows, cols, x, accumulate="f64") - ref).max() <= 1e-6 * np.abs(ref).max()
    assert oracle.validate_payload(Q8_0, packed[:-1]) == 1
    bad = packed.copy(); bad[34 * 5: 34 * 5 + 2] = np.frombuffer(np.float16(np.nan).tobytes(), dtype=np.uint8)
    assert oracle.validate_payload(Q8_0, bad) == 2


@pytest.mark.parametrize("rows,cols", [(8, 32), (16, 288), (8, 2880), (24, 224)])
def test_q8_0_rows_that_end_inside_a_run_of_eight_blocks(rows, cols):
    # a row is cols / 32 * 34 bytes (src/hybrid/weights.rs:1167): the same byte stream read as rows of
    # 256 weights must give the same values in the same order, and every row the plain numpy product
    blocks = rows * cols // 32
    assert cols % 256 and blocks % 8 == 0
    packed = fx.hybrid_random_blocks(blocks, 34, 34 + cols)
    assert oracle.row_bytes(Q8_0, cols) == cols // 32 * 34 and oracle.validate_payload(Q8_0, packed) == 0
    dense = oracle.dequantize(Q8_0, packed, rows, cols)
    as_runs = oracle.dequantize(Q8_0, packed, blocks // 8, 256)
    assert np.array_equal(bits(dense.reshape(-1)), bits(as_runs.reshape(-1)))
    b = packed.reshape(-1, 34)
    want = (b[:, 2:].view(np.int8).astype(np.float32)
            * b[:, 0:2].copy().view(np.float16).astype(np.float32)).reshape(rows, cols)
    assert np.array_equal(bits(dense), bits(want))
    rng = np.random.default_rng(cols)
    for _ in range(500):
        r, c = int(rng.integers(rows)), int(rng.integers(cols))
        assert bits(np.float32(oracle.weight(Q8_0, packed, r, c, cols))) == bits(dense[r, c])
    x = fx.xorshift_uniform(3 * cols, 9).reshape(3, cols)
    ref = x.astype(np.float64) @ dense.astype(np.float64).T
    assert np.abs(oracle.project(Q8_0, packed, rows, cols, x, accumulate="f64") - ref).max() <= 1e-6 * np.abs(ref).max()
    # sequential f32 accumulation, K ascending: the loop itself
    acc = np.zeros(rows, dtype=np.float32)
    for c in range(cols):
        acc = (acc + x[0, c] * dense[:, c]).astype(np.float32)
    assert np.array_equal(bits(oracle.project(Q8_0, packed, rows, cols, x[:1])[0]), bits(acc))
    # routed rows: each assignment its own expert's slice
    experts = 2
    meta = np.zeros((3, 3), dtype=np.uint32)
    meta[:, 0] = [1, 0, 1]
    got = oracle.expert_project(Q8_0, packed, experts, rows // experts, cols, x, meta.view(np.float32), accumulate="f64")
    per = rows // experts
    for a, e in enumerate(meta[:, 0]):
        assert np.abs(got[a] - ref[a, e * per:(e + 1) * per]).max() <= 1e-6 * np.abs(ref).max()
    with pytest.raises(ValueError):
        oracle.row_bytes(Q8_0, cols + 16)
    assert oracle.validate_payload(Q8_0, packed[:-1]) == 1
    bad = packed.copy(); bad[34 * 3: 34 * 3 + 2] = np.frombuffer(np.float16(np.inf).tobytes(), dtype=np.uint8)
    assert oracle.validate_payload(Q8_0, bad) == 2


# ----------------------------------------------- the hybrid engine's route map and combine

def test_moe_map_is_numpy_stable_argsort():
    rng = np.random.default_rng(31)
    for experts, routes in ((4, 1), (8, 40), (256, 4096), (60, 1000)):
        ids = rng.integers(0, experts, routes).astype(np.uint32)
        if routes > 10:
            ids[ids == 3] = 5                      # an empty expert
        offsets, order, position = oracle.moe_map(ids, experts)
        counts = np.bincount(ids, minlength=experts)
        assert np.array_equal(offsets, np.concatenate([[0], np.cumsum(counts)]).astype(np.uint32))
        want = np.argsort(ids, kind="stable").astype(np.uint32)
        assert np.array_equal(order, want)
        assert np.array_equal(position[want], np.arange(routes, dtype=np.uint32))
    ids = np.array([1, 9, 0, 1], dtype=np.uint32)     # 9 is not an expert: left out
    offsets, order, position = oracle.moe_map(ids, 2)
    assert offsets.tolist() == [0, 1, 3] and order[:3].tolist() == [2, 0, 3] and position.tolist() == [1, 0xFFFFFFFF, 0, 2]


def test_hybrid_combine_is_the_weighted_sum_plus_gated_shared_rows():
    rng = np.random.default_rng(32)
    tokens, used, hidden = 5, 4, 24
    down = rng.standard_normal((tokens * used, hidden)).astype(np.float32)
    weights = rng.random(tokens * used).astype(np.float32)
    shared = rng.standard_normal((tokens, hidden)).astype(np.float32)
    gate = rng.random(tokens).astype(np.float32)
    position = rng.permutation(tokens * used).astype(np.uint32)
    for pos in (None, position):
        rows = down if pos is None else down[pos]
        want = (weights[:, None].astype(np.float64) * rows).reshape(tokens, used, hidden).sum(1) + gate[:, None] * shared.astype(np.float64)
        got = oracle.hybrid_combine(down, weights, pos, shared, gate, used)
        assert np.allclose(got, want, rtol=1e-5, atol=1e-6)
    # one route of weight 1, no shared contribution: the row itself
    one = oracle.hybrid_combine(down[:tokens], np.ones(tokens, np.float32), None, shared, np.zeros(tokens, np.float32), 1)
    assert np.array_equal(one, down[:tokens])
