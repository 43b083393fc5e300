"""Pins the floating-point half of the oracle against independent routines
(numpy / scipy / math) and the reference's own known answers."""
import math

import numpy as np
import pytest

import oracle as orc


def test_h2f_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    got = orc.h2f(bits)
    want = bits.view(np.float16).astype(np.float32)
    assert np.array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])
    assert np.all(np.isnan(got[np.isnan(want)]))


def test_f2h_round_to_nearest_even():
    rng = np.random.default_rng(0)
    vals = np.concatenate([
        rng.standard_normal(200000).astype(np.float32) * 10.0 ** rng.integers(-9, 6, 200000),
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25,
                  np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 6.1e-5, 5.96e-8,
                  1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, np.inf, -np.inf], dtype=np.float32),
        # every half value and every midpoint between neighbouring halves
        np.arange(0, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float32),
        ((np.arange(0, 0x7bff, dtype=np.uint16).view(np.float16).astype(np.float64)
          + np.arange(1, 0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)) / 2).astype(np.float32),
    ])
    vals = np.concatenate([vals, -vals]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    assert np.array_equal(orc.f2h(vals), want)
    assert math.isnan(float(orc.f2h(np.array([np.nan], np.float32)).view(np.float16)[0]))


def test_gemm_matrixmul_known_answer():
    # EX/twoMatMuls/matrixMul.cu:149-152,243,259: A = 1, B = D = 0.01, 256^3.
    n = 256
    a = np.ones((n, n), np.float16)
    b = np.full((n, n), 0.01, np.float16)
    c = orc.gemm(a, b)
    b16 = float(np.float16(0.01))
    # fp32 accumulation of 256 equal terms is exact here up to fp32 rounding; compare to fp16(256*b16)
    assert np.all(c == np.float16(np.float32(n) * np.float32(b16)))
    assert abs(float(c[0, 0]) - 2.56) < 2e-3
    e = orc.gemm(c, b)
    assert np.all(np.abs(e.astype(np.float32) - 2.56 * 2.56) < 1e-2)


@pytest.mark.parametrize("shape", [(7, 33, 129), (1, 64, 256), (64, 48, 1000)])
def test_gemm_vs_numpy(shape):
    M, N, K = shape
    rng = np.random.default_rng(1)
    a = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    b = (rng.standard_normal((K, N)) * 0.02).astype(np.float16)
    got = orc.gemm(a, b).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    # fp32 accumulation error bound + one fp16 rounding
    assert np.allclose(got, want, rtol=2e-3, atol=1e-4)
    # a transposed operand or dropped row fails this
    assert not np.allclose(got, (a.astype(np.float64)[::-1] @ b.astype(np.float64)), rtol=2e-3, atol=1e-4) or M == 1


def test_gemm_exact_small_integers():
    # integer-valued inputs: fp32 accumulation is exact, any indexing slip shows up bit-exactly
    rng = np.random.default_rng(2)
    a = rng.integers(-4, 5, (5, 24)).astype(np.float16)
    b = rng.integers(-4, 5, (24, 9)).astype(np.float16)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float16)
    assert np.array_equal(orc.gemm(a, b), want)
    relu = np.maximum(want, 0)
    assert np.array_equal(orc.gemm(a, b, orc.EPI_RELU), relu)


def test_gelu_silu_closed_forms():
    L = orc.lib()
    for x in [-6.0, -1.0, -0.25, 0.0, 0.3, 1.0, 2.5, 6.0]:
        assert abs(L.orc_gelu(x) - 0.5 * x * (1 + math.erf(x / math.sqrt(2)))) < 2e-7 * max(1, abs(x))
        assert abs(L.orc_silu(x) - x / (1 + math.exp(-x))) < 2e-7 * max(1, abs(x))
    # cross-check with torch's erf GeLU and SiLU
    import torch
    xs = torch.linspace(-8, 8, 4001)
    got = np.array([L.orc_gelu(float(v)) for v in xs])
    assert np.allclose(got, torch.nn.functional.gelu(xs).numpy(), atol=1e-6)
    got = np.array([L.orc_silu(float(v)) for v in xs])
    assert np.allclose(got, torch.nn.functional.silu(xs).numpy(), atol=1e-6)


def test_gemm_gelu_epilogue_applied_on_fp32_accumulator():
    rng = np.random.default_rng(3)
    a = rng.uniform(-1, 1, (4, 64)).astype(np.float16)
    b = rng.uniform(-1, 1, (64, 8)).astype(np.float16)
    acc = a.astype(np.float32) @ b.astype(np.float32)
    from scipy.special import erf
    want = (0.5 * acc * (1 + erf(acc / np.sqrt(2)))).astype(np.float16)
    got = orc.gemm(a, b, orc.EPI_GELU)
    assert np.max(np.abs(got.astype(np.float32) - want.astype(np.float32))) <= 2e-3


def test_swiglu():
    rng = np.random.default_rng(4)
    gu = rng.uniform(-3, 3, (5, 16)).astype(np.float16)
    g, u = gu[:, :8].astype(np.float32), gu[:, 8:].astype(np.float32)
    want = (g / (1 + np.exp(-g)) * u).astype(np.float16)
    got = orc.swiglu(gu, 8)
    assert np.max(np.abs(got.astype(np.float32) - want.astype(np.float32))) <= 4e-3
    # swapping gate and up must not pass
    wrong = (u / (1 + np.exp(-u)) * g).astype(np.float16)
    assert np.max(np.abs(got.astype(np.float32) - wrong.astype(np.float32))) > 0.05


def test_gemm_swiglu_fused_on_the_accumulators():
    # silu(X Wg) * (X Wu) with one rounding at the end: against numpy in float64, against the two-step form
    # (round gate|up to fp16, then orc.swiglu) within fp16 rounding, and not symmetric in gate and up
    rng = np.random.default_rng(14)
    M, K, d = 7, 96, 24
    x = rng.uniform(-1, 1, (M, K)).astype(np.float16)
    w = (rng.standard_normal((K, 2 * d)) * 0.3).astype(np.float16)
    got = orc.gemm_swiglu(x, w, d).astype(np.float64)
    acc = x.astype(np.float64) @ w.astype(np.float64)
    g, u = acc[:, :d], acc[:, d:]
    want = g / (1 + np.exp(-g)) * u
    assert np.max(np.abs(got - want)) <= 2e-3 + 1e-3 * np.max(np.abs(want))
    two_step = orc.swiglu(orc.gemm(x, w), d).astype(np.float64)
    assert np.max(np.abs(got - two_step)) <= 1e-2 * np.max(np.abs(want)) + 1e-3
    wrong = u / (1 + np.exp(-u)) * g
    assert np.max(np.abs(got - wrong)) > 0.05
    # integer data with gate = 0 columns: silu(0) * u == 0 exactly; with up = 1: silu(gate) alone
    xi = rng.integers(-2, 3, (M, K)).astype(np.float16)
    wi = rng.integers(-1, 2, (K, 2 * d)).astype(np.float16)
    wi[:, :d // 2] = 0
    hi = orc.gemm_swiglu(xi, wi, d)
    assert np.all(hi[:, :d // 2] == 0)


def test_attention_invariants_and_numpy():
    rng = np.random.default_rng(5)
    S, heads, hd = 37, 3, 16
    qkv = rng.uniform(-1, 1, (S, 3 * heads * hd)).astype(np.float16)
    out = orc.attention(qkv, heads, hd, causal=True).astype(np.float32)
    D = heads * hd
    q, k, v = (qkv[:, i * D:(i + 1) * D].astype(np.float64) for i in range(3))
    # row 0 attends only to itself: O[0] == V[0]
    assert np.allclose(out[0], v[0], atol=1e-3)
    want = np.zeros((S, D))
    for h in range(heads):
        sl = slice(h * hd, (h + 1) * hd)
        s = q[:, sl] @ k[:, sl].T / math.sqrt(hd)
        s[np.triu_indices(S, 1)] = -np.inf
        p = np.exp(s - s.max(1, keepdims=True))
        p /= p.sum(1, keepdims=True)
        assert np.allclose(p.sum(1), 1)
        want[:, sl] = p @ v[:, sl]
    assert np.allclose(out, want, atol=2e-3)
    # constant V => output equals that constant whatever the scores are
    qkv2 = qkv.copy()
    qkv2[:, 2 * D:] = np.float16(0.5)
    assert np.allclose(orc.attention(qkv2, heads, hd).astype(np.float32), 0.5, atol=1e-3)
    # non-causal differs (mask is really applied)
    assert not np.allclose(orc.attention(qkv, heads, hd, causal=False).astype(np.float32), out, atol=2e-3)


def test_conv_all_ones_closed_form():
    # all-ones input and filter, 3x3 pad 1: interior 9C, edges 6C, corners 4C
    C_, K_ = 8, 4
    x = np.ones((2, 6, 7, C_), np.float16)
    w = np.ones((K_, 3, 3, C_), np.float16)
    y = orc.conv2d_nhwc(x, w).astype(np.float32)
    assert y.shape == (2, 6, 7, K_)
    assert np.all(y[:, 1:-1, 1:-1] == 9 * C_)
    assert np.all(y[:, 0, 1:-1] == 6 * C_) and np.all(y[:, 1:-1, 0] == 6 * C_)
    assert np.all(y[:, 0, 0] == 4 * C_) and np.all(y[:, -1, -1] == 4 * C_)


def test_conv_1x1_is_gemm_and_matches_scipy():
    rng = np.random.default_rng(6)
    x = rng.integers(-3, 4, (2, 5, 6, 8)).astype(np.float16)
    w1 = rng.integers(-3, 4, (4, 1, 1, 8)).astype(np.float16)
    y = orc.conv2d_nhwc(x, w1, pad=0)
    want = orc.gemm(x.reshape(-1, 8), np.ascontiguousarray(w1.reshape(4, 8).T)).reshape(2, 5, 6, 4)
    assert np.array_equal(y, want)
    # 3x3 against scipy's correlate (cross-correlation, zero padding), integer data => exact
    from scipy.signal import correlate
    w = rng.integers(-2, 3, (3, 3, 3, 8)).astype(np.float16)
    y = orc.conv2d_nhwc(x, w).astype(np.float64)
    xf, wf = x.astype(np.float64), w.astype(np.float64)
    for n in range(2):
        for k in range(3):
            acc = sum(correlate(xf[n, :, :, c], wf[k, :, :, c], mode="same") for c in range(8))
            assert np.array_equal(y[n, :, :, k], acc)
    yr = orc.conv2d_nhwc(x, w, epilogue=orc.EPI_RELU).astype(np.float64)
    assert np.array_equal(yr, np.maximum(y, 0))


def test_equals_branches():
    # TB/common.h:104-137
    h = lambda *v: np.array(v, np.float16)
    assert orc.equals(h(0.01, 0.05), h(0.09, 0.0), 0.1)        # both below tol -> equal
    assert not orc.equals(h(0.01), h(0.5), 0.1)                 # one below tol -> differ
    assert orc.equals(h(1.0), h(1.05), 0.1)                     # relative within tol
    assert not orc.equals(h(1.0), h(1.5), 0.1)
    assert orc.equals(h(-1.0), h(1.0), 0.1)                     # the reference compares magnitudes


def test_count_mismatch():
    a = np.array([1.0, 2.0, 0.0], np.float16)
    b = np.array([1.005, 2.1, 0.0009], np.float16)
    bad, mx = orc.count_mismatch(a, b, 1e-2, 1e-3)
    assert bad == 1 and abs(mx - 0.1) < 2e-3


def test_attention_with_cache_is_the_tail_of_full_causal_attention():
    # queries behind a key/value cache see exactly what the same rows see in causal attention over
    # the whole sequence; without cache rows the two functions are one
    rng = np.random.default_rng(6)
    heads, hd = 2, 16
    for total, cached in ((50, 0), (50, 13), (70, 64), (33, 32)):
        qkv = rng.uniform(-1, 1, (total, 3 * heads * hd)).astype(np.float16)
        full = orc.attention(qkv, heads, hd, causal=True)
        tail = orc.attention_kv(qkv, cached, heads, hd, causal=True)
        assert np.array_equal(tail.view(np.uint16), full[cached:].view(np.uint16))
    # not causal: every query sees all rows; permuting the cache rows changes nothing but rounding order
    qkv = rng.uniform(-1, 1, (40, 3 * heads * hd)).astype(np.float16)
    a = orc.attention_kv(qkv, 10, heads, hd, causal=False).astype(np.float32)
    b = orc.attention(qkv, heads, hd, causal=False).astype(np.float32)[10:]
    assert np.allclose(a, b, atol=1e-3)
