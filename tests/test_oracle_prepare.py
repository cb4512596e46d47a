"""Pins for the preparation oracle (CPU).  Each check is something the mathematics or
the reference's own tests fix, chosen so that a wrong sign, index or dropped
term fails: none of them re-types the oracle's formula."""

import numpy as np
import pytest
import torch

from oracle import prepare
from oracle.ieee import fma32

rng = np.random.default_rng(7)


def sylvester(n):
    h = np.array([[1.0]])
    while h.shape[0] < n:
        h = np.block([[h, h], [h, -h]])
    return h


def test_fma32_is_single_rounding():
    from fractions import Fraction

    a = rng.standard_normal(400).astype(np.float32)
    b = rng.standard_normal(400).astype(np.float32)
    c = (-(a.astype(np.float64) * b.astype(np.float64))).astype(np.float32) + np.float32(1e-7) * rng.standard_normal(400).astype(np.float32)
    got = fma32(a, b, c)
    for i in range(400):
        exact = Fraction(float(a[i])) * Fraction(float(b[i])) + Fraction(float(c[i]))
        guess = np.float32(float(exact))
        candidates = [guess, np.nextafter(guess, np.float32(np.inf)), np.nextafter(guess, np.float32(-np.inf))]
        best = min(candidates, key=lambda z: (abs(Fraction(float(z)) - exact), int(np.float32(z).view(np.uint32)) & 1))
        assert best == got[i]


@pytest.mark.parametrize("mode,dim", [("h4", 64), ("h4", 128), ("h64", 64), ("h128_plain", 128),
                                      ("h128_plain", 256), ("h128_signed", 128)])
def test_rotation_is_the_documented_hadamard(mode, dim):
    """y = H_n diag(s) x / sqrt(n) in natural (Sylvester) order, n = 4, 64 or 128 per block
    (reference quantize_qk_impl.cuh:69-147; docs of int8_attention, dense.py:95-103)."""
    x = rng.standard_normal((5, dim)).astype(np.float32)
    y = prepare.rotate(x, mode)
    block = {"h4": 4, "h64": 64, "h128_plain": 128, "h128_signed": 128}[mode]
    h = sylvester(block) / np.sqrt(block)
    xs = x.astype(np.float64).reshape(5, dim // block, block)
    if mode == "h128_signed":
        xs = xs * prepare.sign_diagonal().astype(np.float64)
    expected = (xs @ h.T).reshape(5, dim)
    np.testing.assert_allclose(y, expected, rtol=0, atol=2e-6)
    # orthogonal: norms and dot products are preserved
    np.testing.assert_allclose(np.linalg.norm(y, axis=1), np.linalg.norm(x, axis=1), rtol=2e-6)
    np.testing.assert_allclose(y[0] @ y[1], x[0].astype(np.float64) @ x[1].astype(np.float64), atol=2e-5)


def test_sign_diagonal_bits():
    signs = prepare.sign_diagonal()
    # word 0 = 0x1035997b: bits 0,1 set, bit 2 clear, bit 7 clear, bit 8 set
    assert list(signs[:4]) == [1, 1, -1, 1]
    assert signs[7] == -1 and signs[8] == 1
    # word 3 = 0x71132418: bit 31 clear, bits 30,29,28 set
    assert signs[127] == -1 and signs[126] == 1 and signs[125] == 1 and signs[124] == 1
    assert int((signs > 0).sum()) == sum(bin(w).count("1") for w in prepare.SIGN_WORDS)


def test_rotation_mode_policy():
    assert prepare.rotation_mode(128, 256) == "h4"
    assert prepare.rotation_mode(128, 257) == "h128_signed"
    assert prepare.rotation_mode(64, 257) == "h64"
    assert prepare.rotation_mode(256, 257) == "h128_plain"
    assert prepare.select_key_block_size(128, 1025, False) == 128
    assert prepare.select_key_block_size(128, 1024, False) == 64
    assert prepare.select_key_block_size(128, 4096, True) == 64
    assert prepare.select_key_block_size(64, 4096, False) == 64
    assert [prepare.kernel_head_dim(d) for d in (1, 64, 65, 128, 129, 256)] == [64, 64, 128, 128, 256, 256]


@pytest.mark.parametrize("dim,length,key_length", [(128, 70, 300), (64, 45, 300), (256, 40, 300), (128, 33, 100)])
def test_query_groups_by_brute_force(dim, length, key_length):
    """Scale of token n covers the tokens congruent to n mod 8 inside its 32-row
    (16-row for head dim 256) slice; codes are the rotated values over that scale."""
    q = rng.standard_normal((1, 2, length, dim)).astype(np.float32)
    codes, scales = prepare.quantize_queries(q, key_length)
    y = prepare.rotate(q, prepare.rotation_mode(dim, key_length)).astype(np.float64)
    width = 16 if dim == 256 else 32
    assert scales.shape[-1] == (length + 127) // 128 * (128 // width) * 8
    for h in range(2):
        for n in range(length):
            members = [t for t in range(n // width * width, min(length, (n // width + 1) * width)) if t % 8 == n % 8]
            mx = np.abs(y[0, h, members]).max()
            index = (n // width) * 8 + n % 8
            assert scales[0, h, index] == pytest.approx(mx / 127 + 1e-7, rel=1e-6)
            expected = np.rint(y[0, h, n] / float(scales[0, h, index]))
            assert np.abs(codes[0, h, n] - expected).max() <= 1  # ties only
            assert np.abs(codes[0, h, n]).max() <= 127
    # empty groups (tokens past the end) carry the epsilon only
    tail = scales[0, 0, ((length - 1) // width + 1) * 8 :]
    assert np.all(tail == np.float32(1e-7))


@pytest.mark.parametrize("key_block,length", [(64, 150), (128, 300)])
def test_key_groups_by_brute_force(key_block, length):
    k = rng.standard_normal((1, 1, length, 128)).astype(np.float32)
    codes, scales, anchor = prepare.quantize_keys(k, key_block)
    assert anchor[0, 0] == -1
    y = prepare.rotate(k, prepare.rotation_mode(128, length)).astype(np.float64)
    for n in range(length):
        tile = n // key_block
        members = [t for t in range(tile * key_block, min(length, (tile + 1) * key_block)) if (t % 8) // 2 == (n % 8) // 2]
        mx = np.abs(y[0, 0, members]).max()
        index = tile * 4 + (n % 8) // 2
        assert scales[0, 0, index] == pytest.approx(mx / 127 + 1e-7, rel=1e-6)
    dequantised = codes[0, 0].astype(np.float64) * np.repeat(
        scales[0, 0].reshape(-1, 4)[:, (np.arange(key_block) % 8) // 2].reshape(-1), 1)[:length, None]
    assert np.abs(dequantised - y[0, 0]).max() <= 0.5 * scales.max() * (1 + 1e-5)


def test_zero_inputs_give_zero_codes_and_epsilon_scale():
    q = np.zeros((1, 1, 9, 128), np.float32)
    codes, scales = prepare.quantize_queries(q, 500)
    assert not codes.any() and np.all(scales == np.float32(1e-7))


def test_anchor_decision_matches_float64_criterion():
    """Anchor = sampled row minimising sum_c (9 x_c - sum)^2, accepted when it lowers the
    sampled energy and keeps the peak within 12.5% (reference quantize_qk_impl.cuh:430-438)."""
    for seed, offset, expect in [(0, 4.0, True), (1, 0.0, False), (2, -3.0, True)]:
        r = np.random.default_rng(seed)
        k = (r.standard_normal((2, 3, 257, 128)) * (0.1 if offset else 1.0) + offset).astype(np.float32)
        anchor = prepare.detect_key_anchor(k)
        rows = np.array([s * 256 // 8 for s in range(9)])
        for b in range(2):
            for h in range(3):
                x = k[b, h, rows].astype(np.float64)
                cost = ((9 * x - x.sum(0)) ** 2).sum(1)
                best = int(np.argmin(cost))
                res = x - x[best]
                accept = (res**2).sum() < (x**2).sum() and np.abs(res).max() <= 1.125 * np.abs(x).max()
                assert accept == expect
                assert anchor[b, h] == (rows[best] if accept else -1)


def test_anchor_is_the_sampled_row_nearest_the_sample_centroid():
    """sum_c (9 x_a[c] - sum_c)^2 = 81 |x_a - mean|^2, so the candidate the detector settles on
    is the sampled row closest to the mean of the nine sampled rows (reference
    quantize_qk_impl.cuh:442-577): a closed form that shares no expression with the oracle."""
    r = np.random.default_rng(11)
    for length in (9, 64, 257, 1000):
        k = (r.standard_normal((1, 4, length, 128)) * 0.05 + r.standard_normal((1, 4, 1, 128))).astype(np.float32)
        anchor = prepare.detect_key_anchor(k)
        rows = [s * (length - 1) // 8 for s in range(9)]
        for h in range(4):
            sampled = k[0, h, rows].astype(np.float64)
            nearest = int(np.argmin(np.linalg.norm(sampled - sampled.mean(0), axis=1)))
            assert anchor[0, h] == rows[nearest]  # a tight cluster far from the origin always fires


def test_anchor_accept_and_reject_rules_on_hand_built_keys():
    """Accepted iff the shifted samples have less energy and a peak within 12.5 % of the
    original one (reference quantize_qk_impl.cuh:430-438)."""
    length, dim = 65, 128
    rows = [s * (length - 1) // 8 for s in range(9)]
    # constant offset, tiny spread: shifting removes nearly all the energy -> fires, and on
    # the row made equal to the offset itself (distance 0 from ... the centroid is nearest to it)
    k = np.full((1, 1, length, dim), 3.0, np.float32)
    k[0, 0, rows] += (np.arange(9, dtype=np.float32)[:, None] - 4.0) * 1e-3  # centroid = row of sample 4
    assert prepare.detect_key_anchor(k)[0, 0] == rows[4]
    # zero-mean samples: +e and -e alternate, so every candidate's shift raises the energy -> no anchor
    k = np.zeros((1, 1, length, dim), np.float32)
    for index, row in enumerate(rows):
        k[0, 0, row] = 1.0 if index % 2 == 0 else -1.0
    assert prepare.detect_key_anchor(k)[0, 0] == -1
    # energy falls but the peak grows by more than 12.5 %: eight samples at +1 and one at -0.2;
    # the best candidate is a +1 row, which leaves a residual peak of 1.2 > 1.125
    k = np.zeros((1, 1, length, dim), np.float32)
    k[0, 0, rows] = 1.0
    k[0, 0, rows[8]] = -0.2
    assert prepare.detect_key_anchor(k)[0, 0] == -1
    # same construction with the odd sample at +0.2 (residual peak 0.8): accepted, first +1 row wins
    k[0, 0, rows[8]] = 0.2
    assert prepare.detect_key_anchor(k)[0, 0] == rows[0]
    # all samples zero: the energy does not fall strictly -> rejected
    assert prepare.detect_key_anchor(np.zeros((1, 1, length, dim), np.float32))[0, 0] == -1


def test_key_shift_is_softmax_invariant():
    """Subtracting the anchor changes every score of a row by the same amount."""
    r = np.random.default_rng(5)
    k = (r.standard_normal((1, 1, 300, 128)) * 0.1 + 4).astype(np.float32)
    q = r.standard_normal((1, 1, 8, 128)).astype(np.float32)
    codes, scales, anchor = prepare.quantize_keys(k, 64)
    assert anchor[0, 0] >= 0
    qc, qs = prepare.quantize_queries(q, 300)
    ks = scales[0, 0].reshape(-1, 4)[np.arange(300) // 64, (np.arange(300) % 8) // 2]
    deq_k = codes[0, 0].astype(np.float64) * ks[:, None]
    deq_q = qc[0, 0].astype(np.float64) * qs[0, 0][np.arange(8) // 32 * 8 + np.arange(8) % 8][:, None]
    approx = deq_q @ deq_k.T
    exact = q[0, 0].astype(np.float64) @ (k[0, 0] - k[0, 0, anchor[0, 0]]).astype(np.float64).T
    assert np.abs(approx - exact).max() < 0.05 * np.abs(exact).max()


@pytest.mark.parametrize("length", [1025, 2049])
def test_absmax_values_known_answer(length):
    """reference tests/cuda/test_value_quantization.py:18-52: v = code * 2^(c%4-2)."""
    heads, channels = 3, 128
    tokens = np.arange(length)[None, :, None]
    head_offsets = np.arange(heads)[:, None, None]
    codes = ((tokens + head_offsets) % 255 - 127) * np.ones((1, 1, channels), np.int64)
    scales = 2.0 ** ((np.arange(channels) % 4) - 2.0)
    v = (codes * scales).astype(np.float32)[None]
    got, got_scale, got_center = prepare.quantize_values(v, 128, False)
    padded = got.shape[1]
    assert padded == (length + 127) // 128 * 128
    expected = np.zeros((heads, channels, padded), np.int8)
    expected[..., :length] = codes.transpose(0, 2, 1)
    np.testing.assert_array_equal(got.reshape(heads, channels, padded), expected)
    np.testing.assert_array_equal(got_scale.reshape(heads, channels), np.broadcast_to(scales.astype(np.float32), (heads, channels)))
    assert not got_center.any()
    # the reference's physical order is a fixed table
    packed = prepare.reference_value_order(got)
    order = [0, 1, 8, 9, 2, 3, 10, 11, 4, 5, 12, 13, 6, 7, 14, 15]
    np.testing.assert_array_equal(packed.reshape(-1, 16), got.reshape(-1, 16)[:, order])


def test_midpoint_affine_center_reproduces_the_mean():
    """Uniform attention over V must return the mean of V: sum(code)*scale/L + center == mean
    (reference tests/cuda/test_probability_mass.py:148-155)."""
    g = torch.Generator().manual_seed(3)
    v = (torch.randn(1, 1, 512, 128, generator=g) + 3).to(torch.bfloat16)
    v[..., ::53, :] += 12
    vf = v.float().numpy()
    codes, scale, center = prepare.quantize_values(vf, 64, True)
    mean_codes = codes[:, :512].astype(np.float64).mean(1)
    rebuilt = mean_codes * scale + center
    np.testing.assert_allclose(rebuilt, vf[0, 0].astype(np.float64).mean(0), rtol=0, atol=3e-6)
    mn, mx = vf[0, 0].min(0), vf[0, 0].max(0)
    np.testing.assert_allclose(scale, (mx - mn) / 2 / 127, rtol=1e-6)
    assert np.abs(codes).max() <= 127


def test_value_tile_sums_and_padding():
    v = rng.standard_normal((1, 2, 200, 64)).astype(np.float32)
    codes, _, _ = prepare.quantize_values(v, 64, False)
    assert codes.shape == (128, 256) and not codes[:, 200:].any()
    sums = prepare.value_tile_sums(codes, 64)
    assert sums.shape == (128, 4)
    assert sums[5, 3] == codes[5, 192:256].astype(int).sum()


@pytest.mark.parametrize("dim", [64, 128, 256])
def test_lse_shift_closed_form(dim):
    """reference tests/cuda/test_lse_correction.py:9-31."""
    r = np.random.default_rng(35)
    q = r.standard_normal((2, 4, 17, dim)).astype(np.float32)
    k = r.standard_normal((2, 2, 9, dim)).astype(np.float32)
    anchors = np.array([[-1, 0], [3, 2]], np.int32)
    out = prepare.lse_shift(q, k, anchors, dim**-0.5)
    for b in range(2):
        for h in range(4):
            a = anchors[b, h // 2]
            ref = 0.0 if a < 0 else (q[b, h].astype(np.float64) @ k[b, h // 2, a].astype(np.float64)) * dim**-0.5
            np.testing.assert_allclose(out[b, h], ref, rtol=2e-5, atol=5e-6)
    assert not out[0, :2].any()
