"""Pins the CPU checker (oracle/) before anything is compared against it.

What each group rules out:
  * golden / _ref        — bit equality with the reference's own compiled
                           csrc/cpu/layernorm.cpp: wrong operation order, wrong value
                           squared (rounded vs unrounded), wrong value re-read;
  * closed forms         — dropped eps, mean vs sum, missing weight, wrong sign;
  * numpy restatements   — rounding mode, P-sum order, in-place / aliasing contract;
  * float64 witness      — gross arithmetic error on random data at full width.
"""
import os

import numpy as np
import pytest

from helpers import assert_close_bits, bits_to_f32, ulp_distance

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def _cases(npz):
    names = sorted({k.split(".")[0] for k in npz.files})
    return [(n, {k.split(".", 1)[1]: npz[k] for k in npz.files if k.startswith(n + ".")})
            for n in names]


def rand_bits(rng, shape, scale=1.0):
    from oracle import tw_oracle as O
    return O.f32_to_bf16((rng.standard_normal(shape) * scale).astype(np.float32))


# ---------------------------------------------------------------------------
# golden vectors produced by the reference's compiled CPU path
# ---------------------------------------------------------------------------
def test_golden_fused_add_rms_norm_bit_exact(oracle):
    npz = np.load(os.path.join(GOLDEN, "ref_fused_add_rms_norm.npz"))
    cases = _cases(npz)
    assert len(cases) >= 8
    for name, c in cases:
        x, r = c["x"].copy(), c["r"].copy()
        oracle.fused_add_rms_norm(x, r, c["w"], float(c["eps"]), mode=oracle.ROUND_TRUNC)
        assert np.array_equal(r, c["r_ref"]), name
        assert np.array_equal(x, c["y_ref"]), name


def test_golden_rms_norm_bit_exact(oracle):
    npz = np.load(os.path.join(GOLDEN, "ref_rms_norm.npz"))
    for name, c in _cases(npz):
        out = oracle.rms_norm(c["x"], c["w"], float(c["eps"]), mode=oracle.ROUND_TRUNC)
        assert np.array_equal(out, c["y_ref"]), name


def test_golden_rne_within_one_ulp_of_truncating_reference(oracle):
    """RNE and truncation differ by at most one ulp per rounding; y has two roundings
    in its history (residual, then output)."""
    npz = np.load(os.path.join(GOLDEN, "ref_fused_add_rms_norm.npz"))
    for name, c in _cases(npz):
        x, r = c["x"].copy(), c["r"].copy()
        oracle.fused_add_rms_norm(x, r, c["w"], float(c["eps"]))
        finite = np.isfinite(bits_to_f32(c["r_ref"]))
        assert ulp_distance(r, c["r_ref"])[finite].max() <= 1, name
        assert_close_bits(x[finite], c["y_ref"][finite], name)


# ---------------------------------------------------------------------------
# the reference's own build, on the reference's own test grid
# (tests/kernels/test_layernorm.py:11-15 with hidden_size % 8 == 0)
# ---------------------------------------------------------------------------
REF_GRID = [(T, H) for T in (7, 83, 4096) for H in (8, 768, 5120, 8192)]


@pytest.mark.parametrize("T,H", REF_GRID)
def test_matches_compiled_reference_bitwise(oracle, T, H):
    if not oracle.have_ref():
        pytest.skip("oracle/_ref not built (reference tree absent)")
    rng = np.random.default_rng(0)
    scale = 1.0 / (2 * H)
    x, r = rand_bits(rng, (T, H), scale), rand_bits(rng, (T, H), scale)
    w = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    x1, r1, x2, r2 = x.copy(), r.copy(), x.copy(), r.copy()
    oracle.fused_add_rms_norm(x1, r1, w, 1e-6, mode=oracle.ROUND_TRUNC)
    oracle.ref_fused_add_rms_norm(x2, r2, w, 1e-6)
    assert np.array_equal(r1, r2) and np.array_equal(x1, x2)
    assert np.array_equal(oracle.rms_norm(x, w, 1e-6, mode=oracle.ROUND_TRUNC),
                          oracle.ref_rms_norm(x, w, 1e-6))


@pytest.mark.parametrize("T,H", REF_GRID)
def test_within_reference_test_tolerance_of_forward_native(oracle, T, H):
    """The reference's unit test accepts atol = rtol = 1e-2 between its kernels and
    forward_native (tests/kernels/test_layernorm.py:53-57)."""
    rng = np.random.default_rng(0)
    scale = 1.0 / (2 * H)
    x, r = rand_bits(rng, (T, H), scale), rand_bits(rng, (T, H), scale)
    w = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    y_nat, r_nat = oracle.forward_native_np(x, r, w, 1e-6)
    xo, ro = x.copy(), r.copy()
    oracle.fused_add_rms_norm(xo, ro, w, 1e-6)
    assert np.array_equal(ro, r_nat)  # both: bf16_rne(fp32 sum)
    assert_close_bits(xo, y_nat, "vs forward_native", rtol=1e-2, atol=1e-2)
    assert_close_bits(oracle.rms_norm(x, w, 1e-6), oracle.forward_native_np(x, None, w, 1e-6),
                      "rms_norm vs forward_native", rtol=1e-2, atol=1e-2)


# ---------------------------------------------------------------------------
# closed forms
# ---------------------------------------------------------------------------
def test_constant_row(oracle):
    H, eps = 512, 1e-5
    for c in (0.5, -3.0, 96.0):
        x = oracle.f32_to_bf16(np.full((1, H), c, np.float32))
        r = np.zeros((1, H), np.uint16)
        w = oracle.f32_to_bf16(np.full(H, 1.25, np.float32))
        oracle.fused_add_rms_norm(x, r, w, eps)
        want = np.float32(c) * (np.float32(1) / np.sqrt(np.float32(c * c) + np.float32(eps))) * np.float32(1.25)
        assert np.array_equal(x, oracle.f32_to_bf16(np.full((1, H), want, np.float32)))
        assert np.array_equal(r, oracle.f32_to_bf16(np.full((1, H), c, np.float32)))


def test_one_hot_row_uses_mean_not_sum(oracle):
    H, eps, a, k = 1024, 1e-5, 4.0, 77
    x = np.zeros((1, H), np.float32); x[0, k] = a
    xb, r = oracle.f32_to_bf16(x), np.zeros((1, H), np.uint16)
    w = oracle.f32_to_bf16(np.ones(H, np.float32))
    oracle.fused_add_rms_norm(xb, r, w, eps)
    y = bits_to_f32(xb)
    inv = 1.0 / np.sqrt(a * a / H + eps)
    assert abs(y[0, k] - a * inv) <= 2 ** -8 * a * inv
    assert (np.delete(y[0], k) == 0).all()


def test_zero_row_is_finite_and_zero(oracle):
    H = 256
    x, r = np.zeros((2, H), np.uint16), np.zeros((2, H), np.uint16)
    w = oracle.f32_to_bf16(np.full(H, 2.0, np.float32))
    oracle.fused_add_rms_norm(x, r, w, 1e-6)
    assert (x == 0).all() and (r == 0).all()


def test_eps_is_inside_the_square_root(oracle):
    """Tiny inputs: y = s / sqrt(eps) to first order (eps dropped or added outside
    the root gives a different magnitude)."""
    H, eps = 64, 1e-2
    x = oracle.f32_to_bf16(np.full((1, H), 1e-4, np.float32))
    r = np.zeros((1, H), np.uint16)
    oracle.fused_add_rms_norm(x, r, oracle.f32_to_bf16(np.ones(H, np.float32)), eps)
    got = bits_to_f32(x)[0, 0]
    assert abs(got - 1e-4 / np.sqrt(eps)) < 1e-2 * 1e-4 / np.sqrt(eps)


def test_scale_law_and_weight_factor(oracle):
    rng = np.random.default_rng(3)
    H = 2048
    x, r = rand_bits(rng, (4, H)), rand_bits(rng, (4, H))
    ones = oracle.f32_to_bf16(np.ones(H, np.float32))
    w = oracle.f32_to_bf16((0.5 + rng.random(H)).astype(np.float32))
    y1, _ = oracle.reduce_add_rms_norm([x], r.copy(), ones, 1e-12)
    # power-of-two scaling of the inputs is exact in bf16 and must not change y
    x4 = oracle.f32_to_bf16(bits_to_f32(x) * 4); r4 = oracle.f32_to_bf16(bits_to_f32(r) * 4)
    y4, _ = oracle.reduce_add_rms_norm([x4], r4, ones, 1e-12)
    assert ulp_distance(y1, y4).max() <= 1
    yw, _ = oracle.reduce_add_rms_norm([x], r.copy(), w, 1e-12)
    assert_close_bits(yw, oracle.f32_to_bf16(bits_to_f32(y1) * bits_to_f32(w)), "weight", rtol=2 ** -7, atol=1e-6)


# ---------------------------------------------------------------------------
# P-way sum, rounding, aliasing
# ---------------------------------------------------------------------------
def test_residual_is_rne_of_fixed_order_fp32_sum(oracle):
    rng = np.random.default_rng(5)
    P, T, H = 8, 5, 1024
    parts = [rand_bits(rng, (T, H), 0.35) for _ in range(P)]
    r = rand_bits(rng, (T, H))
    s = bits_to_f32(parts[0]).copy()
    for p in parts[1:]:
        s = s + bits_to_f32(p)
    s = s + bits_to_f32(r)
    r2 = r.copy()
    oracle.reduce_add_rms_norm(parts, r2, oracle.f32_to_bf16(np.ones(H, np.float32)), 1e-5)
    assert np.array_equal(r2, oracle.f32_to_bf16(s))
    r3 = r.copy()
    oracle.reduce_add_rms_norm(parts, r3, oracle.f32_to_bf16(np.ones(H, np.float32)), 1e-5,
                               mode=oracle.ROUND_TRUNC)
    assert np.array_equal(r3, oracle.f32_to_bf16(s, oracle.ROUND_TRUNC))


def test_rne_rounding_against_torch(oracle):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(11)
    f = np.concatenate([rng.standard_normal(100000).astype(np.float32) * 10.0 ** rng.integers(-30, 30, 100000),
                        np.array([0.0, -0.0, np.inf, -np.inf, 1.00390625, 1.01171875, 3.3895314e38], np.float32)])
    want = torch.from_numpy(f).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.f32_to_bf16(f), want)
    # the C rounding agrees with the numpy one (ones weight, zero residual, P = 1 copy)
    H = f.size - f.size % 8
    x = oracle.f32_to_bf16(f[:H]).reshape(1, H)
    out, r = oracle.reduce_add_rms_norm([x], np.zeros((1, H), np.uint16), oracle.f32_to_bf16(np.ones(H, np.float32)), 1.0)
    assert np.array_equal(r, x)


def test_zero_partials_reduce_to_p1_and_order_free_inputs(oracle):
    rng = np.random.default_rng(7)
    T, H = 9, 768
    x, r = rand_bits(rng, (T, H)), rand_bits(rng, (T, H))
    w = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    x1, r1 = x.copy(), r.copy()
    oracle.fused_add_rms_norm(x1, r1, w, 1e-5)
    zeros = [np.zeros((T, H), np.uint16) for _ in range(7)]
    y8, r8 = oracle.reduce_add_rms_norm([x] + zeros, r.copy(), w, 1e-5)
    assert np.array_equal(y8, x1) and np.array_equal(r8, r1)
    # multiples of 2^-6 below 4: every fp32 partial sum is exact, so any order agrees
    parts = [oracle.f32_to_bf16((rng.integers(-255, 256, (T, H)) / 64.0).astype(np.float32)) for _ in range(8)]
    rr = oracle.f32_to_bf16((rng.integers(-255, 256, (T, H)) / 64.0).astype(np.float32))
    ya, ra = oracle.reduce_add_rms_norm(parts, rr.copy(), w, 1e-5)
    yb, rb = oracle.reduce_add_rms_norm(parts[::-1], rr.copy(), w, 1e-5)
    assert np.array_equal(ya, yb) and np.array_equal(ra, rb)


def test_output_may_alias_a_partial_and_weight_is_untouched(oracle):
    rng = np.random.default_rng(9)
    P, T, H = 4, 6, 512
    parts = [rand_bits(rng, (T, H), 0.5) for _ in range(P)]
    r = rand_bits(rng, (T, H))
    w = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    w0 = w.copy()
    y, r_new = oracle.reduce_add_rms_norm([p.copy() for p in parts], r.copy(), w, 1e-5)
    alias = [p.copy() for p in parts]
    y2, r2 = oracle.reduce_add_rms_norm(alias, r.copy(), w, 1e-5, y=alias[2])
    assert y2 is alias[2] and np.array_equal(y2, y) and np.array_equal(r2, r_new)
    assert np.array_equal(w, w0)
    for i in (0, 1, 3):
        assert np.array_equal(alias[i], parts[i])


def test_rms_norm_inplace_copies_then_normalises(oracle):
    rng = np.random.default_rng(13)
    T, H = 5, 1024
    x = rand_bits(rng, (T, H))
    w = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    want = oracle.rms_norm(x, w, 1e-5)
    out, xi = np.zeros_like(x), x.copy()
    oracle.rms_norm_inplace(out, xi, w, 1e-5)
    assert np.array_equal(out, x) and np.array_equal(xi, want)


def test_rows_are_independent_and_permutation_equivariant(oracle):
    rng = np.random.default_rng(17)
    P, T, H = 3, 11, 256
    parts = [rand_bits(rng, (T, H)) for _ in range(P)]
    r = rand_bits(rng, (T, H))
    w = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    y, rn = oracle.reduce_add_rms_norm(parts, r.copy(), w, 1e-5)
    perm = rng.permutation(T)
    yp, rp = oracle.reduce_add_rms_norm([np.ascontiguousarray(p[perm]) for p in parts],
                                        np.ascontiguousarray(r[perm]), w, 1e-5)
    assert np.array_equal(yp, y[perm]) and np.array_equal(rp, rn[perm])
    y1, r1 = oracle.reduce_add_rms_norm([np.ascontiguousarray(p[4:5]) for p in parts],
                                        np.ascontiguousarray(r[4:5]), w, 1e-5)
    assert np.array_equal(y1, y[4:5]) and np.array_equal(r1, rn[4:5])


def test_float64_witness_at_full_width(oracle):
    rng = np.random.default_rng(19)
    P, T, H = 8, 16, 8192
    parts = [rand_bits(rng, (T, H), 8 ** -0.5) for _ in range(P)]
    r = rand_bits(rng, (T, H))
    w = oracle.f32_to_bf16((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    y64, s64 = oracle.reduce_add_rms_norm_f64(parts, r, w, 1e-5)
    y, rn = oracle.reduce_add_rms_norm(parts, r.copy(), w, 1e-5)
    # residual: one bf16 rounding of the exact sum (fp32 partial-sum error is far below)
    assert np.max(np.abs(bits_to_f32(rn) - s64) / np.maximum(np.abs(s64), 1e-30)) <= 2 ** -8 * 1.01
    # y: two bf16 roundings (residual, output)
    err = np.abs(bits_to_f32(y) - y64)
    assert np.max(err - (2 ** -7 * np.abs(y64) + 1e-6)) <= 0


def test_gemm_oracle_against_float64(oracle):
    rng = np.random.default_rng(23)
    M, N, K = 33, 40, 96
    a, b = rand_bits(rng, (M, K)), rand_bits(rng, (N, K), 0.02)
    want = bits_to_f32(a).astype(np.float64) @ bits_to_f32(b).astype(np.float64).T
    got = bits_to_f32(oracle.gemm_bf16_nt(a, b))
    assert np.max(np.abs(got - want) - (2 ** -8 * np.abs(want) + 1e-5)) <= 0


def test_rejects_hidden_size_not_multiple_of_8(oracle):
    """TORCH_CHECK(hidden_size % VEC_ELEM_NUM == 0), csrc/cpu/layernorm.cpp:11,52."""
    x = np.zeros((2, 12), np.uint16)
    with pytest.raises(RuntimeError):
        oracle.fused_add_rms_norm(x, x.copy(), np.zeros(12, np.uint16), 1e-5)
    with pytest.raises(RuntimeError):
        oracle.rms_norm(x, np.zeros(12, np.uint16), 1e-5)


def test_empty_input_is_a_no_op(oracle):
    x = np.zeros((0, 64), np.uint16)
    oracle.fused_add_rms_norm(x, x.copy(), np.zeros(64, np.uint16), 1e-5)
    assert oracle.rms_norm(x, np.zeros(64, np.uint16), 1e-5).shape == (0, 64)


def test_fp8_quant_matches_torch_cast_on_every_bf16_pattern(oracle):
    """Pins the e4m3fn conversion of the checker against an independent
    implementation (torch's CPU cast), on all 65536 bf16 inputs and three scales."""
    torch = pytest.importorskip("torch")
    bits = np.arange(65536, dtype=np.uint16)
    vals = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).float()
    finite = torch.isfinite(vals).numpy()
    for scale in (1.0, 0.01, 10.0, 0.37):
        got = oracle.static_fp8_quant(bits, scale)
        inv = torch.tensor(1.0, dtype=torch.float32) / torch.tensor(scale, dtype=torch.float32)
        want = (vals * inv).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        assert np.array_equal(got[finite], want[finite]), scale
    # spot values: 448 saturates, ties go to even, subnormal grid is 2^-9
    f = np.array([448.0, 1000.0, -1000.0, 0.0, 2 ** -9, 2 ** -10, 3 * 2 ** -10, 17.0, 19.0], np.float32)
    got = oracle.static_fp8_quant(oracle.f32_to_bf16(f), 1.0)
    assert list(got) == [0x7E, 0x7E, 0xFE, 0x00, 0x01, 0x00, 0x02, 0x58, 0x5A]


# ---------------------------------------------------------------------------
# dynamic per-token quantisation: pinned by the composition the reference's own
# test compares its fused kernel with (tests/kernels/test_fused_quant_layernorm.py
# :51-72): forward_native, then per-token scales, then the element conversion — here
# in numpy, with torch's CPU cast as the fp8 converter.
# ---------------------------------------------------------------------------
FP8_MAX, FP8_MIN_SCALE = np.float32(448.0), np.float32(1.0 / (448.0 * 512.0))
I8_MAX, I8_MIN_SCALE = np.float32(127.0), np.float32(np.finfo(np.float32).eps)


def _composed_dynamic_quant(oracle, x_f32_exact_bits, r, w, eps, qkind, ub):
    """x_f32_exact_bits: bf16 bits of the (already summed) input; returns codes, scales, r'."""
    import torch
    res = oracle.forward_native_np(x_f32_exact_bits, r, w, eps)
    y, r_new = res if r is not None else (res, None)
    n = bits_to_f32(y)
    amax = np.abs(n).max(axis=-1, keepdims=True).astype(np.float32)
    if qkind == oracle.QUANT_FP8:
        s = amax if ub is None else np.minimum(amax, np.float32(ub))
        scales = np.maximum(s / FP8_MAX, FP8_MIN_SCALE).astype(np.float32)
        q = np.clip(n / scales, -FP8_MAX, FP8_MAX).astype(np.float32)
        codes = torch.from_numpy(q).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    else:
        scales = np.maximum(amax / I8_MAX, I8_MIN_SCALE).astype(np.float32)
        q = np.rint(n * (np.float32(1.0) / scales)).astype(np.float32)
        codes = np.clip(q, -128, 127).astype(np.int8).view(np.uint8)
    return codes, scales, r_new


def _order_free_bits(rng, shape, kmax=64):
    """bf16 values k/64, |k| <= kmax: squares and their sums over <= 4096 elements are
    exact in fp32 in any order, so every implementation agrees on the mean bit for bit."""
    from oracle import tw_oracle as O
    k = rng.integers(-kmax, kmax + 1, size=shape)
    return O.f32_to_bf16((k / 64.0).astype(np.float32))


@pytest.mark.parametrize("qkind", [0, 1])
@pytest.mark.parametrize("add_residual", [False, True])
@pytest.mark.parametrize("use_ub", [False, True])
@pytest.mark.parametrize("T,H", [(1, 64), (7, 1024), (83, 2048), (5, 4096), (3, 1032)])
def test_dynamic_quant_equals_reference_test_composition_bitwise(oracle, qkind, add_residual, use_ub, T, H):
    if use_ub and qkind == oracle.QUANT_INT8:
        pytest.skip("scale_ub is fp8-only (fused_layernorm_dynamic_per_token_quant.cu:144-146)")
    rng = np.random.default_rng(100 * T + H + 7 * qkind)
    x = _order_free_bits(rng, (T, H), kmax=32)
    r = _order_free_bits(rng, (T, H), kmax=32) if add_residual else None
    w = oracle.f32_to_bf16(rng.normal(1.0, 0.1, H).astype(np.float32))
    eps = 1e-6
    ub = None
    if use_ub:
        # as in the reference test (:139-141): the mean of the normalised output
        yy = oracle.forward_native_np(x, r, w, eps)
        yy = yy[0] if add_residual else yy
        ub = float(np.abs(bits_to_f32(yy)).mean())
    want_codes, want_scales, want_r = _composed_dynamic_quant(oracle, x, r, w, eps, qkind, ub)
    r_io = r.copy() if add_residual else None
    codes, scales = oracle.rms_norm_dynamic_per_token_quant([x], w, eps, qkind, scale_ub=ub, r=r_io)
    assert np.array_equal(scales, want_scales)
    assert np.array_equal(codes, want_codes), int((codes != want_codes).sum())
    if add_residual:
        assert np.array_equal(r_io, want_r)
    if use_ub:
        assert (np.abs(bits_to_f32(yy)).max(axis=-1) > ub).any(), "the bound never bites: test is vacuous"


@pytest.mark.parametrize("qkind", [0, 1])
def test_dynamic_quant_partials_sum_in_fp32_before_anything_is_rounded(oracle, qkind):
    """P order-free partials == one input holding their exact sum."""
    rng = np.random.default_rng(5)
    T, H, P = 6, 2048, 8
    parts = [_order_free_bits(rng, (T, H), kmax=4) for _ in range(P)]
    total = oracle.f32_to_bf16(sum(bits_to_f32(p) for p in parts))   # |k| <= 32: exact in bf16
    r = _order_free_bits(rng, (T, H), kmax=32)
    w = oracle.f32_to_bf16(rng.normal(1.0, 0.1, H).astype(np.float32))
    r1, r2 = r.copy(), r.copy()
    c1, s1 = oracle.rms_norm_dynamic_per_token_quant(parts, w, 1e-6, qkind, r=r1)
    c2, s2 = oracle.rms_norm_dynamic_per_token_quant([total], w, 1e-6, qkind, r=r2)
    assert np.array_equal(c1, c2) and np.array_equal(s1, s2) and np.array_equal(r1, r2)


@pytest.mark.parametrize("T,H", [(7, 768), (83, 5120), (16, 8192)])
@pytest.mark.parametrize("qkind", [0, 1])
def test_dynamic_quant_random_rows_within_reference_test_tolerance(oracle, qkind, T, H):
    """Random data (the reference test's distribution): the mean of squares may differ
    from numpy's pairwise mean in the last bit, which can move a rounding; the reference's
    test allows rtol 1e-5 on scales and one step on int8 codes
    (test_fused_quant_layernorm.py:151-159).  Here: almost every row exact, none off by
    more than one bf16 step of the row maximum."""
    rng = np.random.default_rng(11 * T + H)
    x = rand_bits(rng, (T, H), 1.0 / H)
    r = rand_bits(rng, (T, H), 1.0 / H)
    w = oracle.f32_to_bf16(rng.normal(1.0, 0.1, H).astype(np.float32))
    want_codes, want_scales, want_r = _composed_dynamic_quant(oracle, x, r, w, 1e-6, qkind, None)
    r_io = r.copy()
    codes, scales = oracle.rms_norm_dynamic_per_token_quant([x], w, 1e-6, qkind, r=r_io)
    assert np.array_equal(r_io, want_r)
    rel = np.abs(scales - want_scales) / want_scales
    assert rel.max() <= 2.0 ** -7 and (rel > 1e-5).mean() <= 0.05
    same_scale = (rel[:, 0] == 0)
    a = codes[same_scale].view(np.int8).astype(np.int32)
    b = want_codes[same_scale].view(np.int8).astype(np.int32)
    if qkind == oracle.QUANT_FP8:   # sign-magnitude codes -> monotone line
        a = np.where(a < 0, -(a & 0x7F), a)
        b = np.where(b < 0, -(b & 0x7F), b)
    d = np.abs(a - b)
    assert d.max() <= 1 and (d != 0).mean() <= 2e-3


def test_dynamic_quant_closed_forms(oracle):
    H = 512
    w1 = oracle.f32_to_bf16(np.ones(H, np.float32))
    # constant row: every element is the row maximum -> every code is the largest one
    x = oracle.f32_to_bf16(np.full((1, H), -0.75, np.float32))
    c, s = oracle.rms_norm_dynamic_per_token_quant([x], w1, 1e-6, oracle.QUANT_FP8)
    assert (c == 0xFE).all()                      # -448
    assert abs(s[0, 0] * 448.0 - 1.0) < 2.0 ** -8  # |n| = bf16(0.75 / sqrt(0.5625 + eps)) ~ 1
    c, s = oracle.rms_norm_dynamic_per_token_quant([x], w1, 1e-6, oracle.QUANT_INT8)
    assert (c.view(np.int8) == -127).all() and abs(s[0, 0] * 127.0 - 1.0) < 2.0 ** -8
    # one-hot row: n_k = a / sqrt(a^2 / H) = sqrt(H) up to the eps term, scale = n_k / qmax
    x = np.zeros((1, H), np.float32); x[0, 5] = 3.0
    c, s = oracle.rms_norm_dynamic_per_token_quant([oracle.f32_to_bf16(x)], w1, 1e-6, oracle.QUANT_FP8)
    assert c[0, 5] == 0x7E and (np.delete(c[0], 5) == 0).all()
    assert abs(s[0, 0] * 448.0 / np.sqrt(H) - 1.0) < 2.0 ** -7
    # zero row: the scale floor, zero codes
    z = np.zeros((2, H), np.uint16)
    c, s = oracle.rms_norm_dynamic_per_token_quant([z], w1, 1e-6, oracle.QUANT_FP8)
    assert (c == 0).all() and (s == FP8_MIN_SCALE).all()
    c, s = oracle.rms_norm_dynamic_per_token_quant([z], w1, 1e-6, oracle.QUANT_INT8)
    assert (c == 0).all() and (s == I8_MIN_SCALE).all()
    # upper bound below the maximum: scale = ub / 448 and everything above ub saturates
    rng = np.random.default_rng(3)
    x = rand_bits(rng, (4, H))
    c, s = oracle.rms_norm_dynamic_per_token_quant([x], w1, 1e-6, oracle.QUANT_FP8, scale_ub=0.5)
    assert np.array_equal(s, np.full((4, 1), np.float32(0.5) / FP8_MAX, np.float32))
    n = bits_to_f32(oracle.forward_native_np(x, None, w1, 1e-6))
    assert ((c & 0x7F) == 0x7E)[np.abs(n) >= 0.5].all() and (np.abs(n) >= 0.5).any()


def test_dynamic_quant_dequantises_to_the_normalised_output(oracle):
    """codes * scale reproduces forward_native's output to the format's precision:
    fp8 e4m3 relative 2^-4 (plus its subnormal step), int8 half a step."""
    import torch
    rng = np.random.default_rng(17)
    T, H = 9, 4096
    x, r = rand_bits(rng, (T, H)), rand_bits(rng, (T, H))
    w = oracle.f32_to_bf16(rng.uniform(0.5, 1.5, H).astype(np.float32))
    n = bits_to_f32(oracle.forward_native_np(x, r, w, 1e-5)[0]).astype(np.float64)
    c, s = oracle.rms_norm_dynamic_per_token_quant([x], w, 1e-5, oracle.QUANT_FP8, r=r.copy())
    deq = torch.from_numpy(c.copy()).view(torch.float8_e4m3fn).float().numpy().astype(np.float64) * s
    assert (np.abs(deq - n) <= np.abs(n) * 2.0 ** -4 + s * 2.0 ** -10 + 1e-2 * np.abs(n)).all()
    c, s = oracle.rms_norm_dynamic_per_token_quant([x], w, 1e-5, oracle.QUANT_INT8, r=r.copy())
    deq = c.view(np.int8).astype(np.float64) * s
    assert (np.abs(deq - n) <= 0.5 * s * (1 + 1e-6) + 1e-2 * np.abs(n)).all()
