"""Pins for the CPU oracle: each check is chosen so that a plausible mistake (a transposed
factor, a wrong nibble, truncation instead of round-half-even, a dropped rounding) fails it.
None of these retype the oracle's own formula: they use exact rational arithmetic, closed forms
(scipy's Sylvester matrix, Kronecker products in float64), brute force and invariants."""
import hashlib
from fractions import Fraction

import numpy as np
import pytest
import scipy.linalg
import torch

from oracle import quarot_oracle as o

F16, F32 = np.float16, np.float32


def all_finite_f16():
    v = np.arange(65536, dtype=np.uint16).view(F16)
    return v[np.isfinite(v)]


def round_fraction_to_f16(fr):
    """Correctly rounded (nearest, ties to even) binary16 of an exact Fraction, by search over
    the two neighbouring representable values.  Independent of numpy's float casts except for
    the (exact) float16 -> Fraction conversion."""
    if fr == 0:
        return F16(0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    # exponent of the binade
    e = 0
    while Fraction(2) ** (e + 1) <= a:
        e += 1
    while Fraction(2) ** e > a:
        e -= 1
    e = max(e, -14)                       # subnormal grid below 2^-14
    ulp = Fraction(2) ** (e - 10)
    k = a / ulp
    lo = int(k)                           # floor
    rem = k - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    val = lo * ulp
    if val >= Fraction(65520):
        return F16(sign * np.inf)
    return F16(sign * float(val))


# ------------------------------------------------------------------ tables and get_hadK

SHA = {12: "5ed24dfa527572b5", 20: "f1f0309c0a997831", 28: "388c0b2f668d130f", 36: "d56db1cfa5877c3f",
       40: "e697ab89f5bb9140", 52: "f80473403896af66", 60: "73c41ef814c170ec", 108: "a213b05e570867de",
       140: "3c0c825cdc56ba9e", 156: "a53703a157ee01fb", 172: "891685e890ac3afd"}


def test_tables_hash_and_orthogonality():
    t = o.hadamard_tables()
    assert sorted(t) == sorted(SHA)
    for k, h in t.items():
        assert h.shape == (k, k) and set(np.unique(h)) == {-1, 1}
        assert hashlib.sha256(np.packbits(h.reshape(-1) > 0).tobytes()).hexdigest()[:16] == SHA[k]
        hh = h.astype(np.int64)
        assert np.array_equal(hh @ hh.T, k * np.eye(k, dtype=np.int64))
    # orientation matters: several tables are not symmetric
    assert np.array_equal(t[28], t[28].T) and np.array_equal(t[36], t[36].T)
    assert not np.array_equal(t[172], t[172].T) and not np.array_equal(t[12], t[12].T)


@pytest.mark.parametrize("n,k", [(4096, 1), (8192, 1), (128, 1), (32, 1), (64, 1), (11008, 172), (28672, 28),
                                 (13824, 108), (5120, 40), (6656, 52), (17920, 140), (14336, 28), (12288, 12),
                                 (72, 36), (19968, 156), (15360, 60), (160, 40), (80, 40), (20, 20)])
def test_get_hadK_known_answers(n, k):
    h, kk = o.get_hadK(n)
    assert kk == k
    assert (h is None) == (k == 1)
    if h is not None:
        assert np.array_equal(o.get_hadK(n, transpose=True)[0], h.T)


@pytest.mark.parametrize("n", [324, 3 * 172, 100, 7, 0])
def test_get_hadK_rejects(n):
    with pytest.raises(AssertionError):
        o.get_hadK(n)


def test_sylvester_matches_scipy():
    for m in (1, 2, 8, 64, 256):
        assert np.array_equal(o.sylvester(m), scipy.linalg.hadamard(m))


# ------------------------------------------------------------------ Hadamard transforms

@pytest.mark.parametrize("n", [8, 16, 64, 24, 40, 56, 72, 344, 104])
def test_matmul_hadU_equals_kron_closed_form(n):
    rng = np.random.default_rng(n)
    x = rng.standard_normal((5, n))
    hadk, k = o.get_hadK(n)
    hm = scipy.linalg.hadamard(n // k).astype(np.float64)
    full = hm if k == 1 else np.kron(hadk, hm)
    want = x @ full.T / np.sqrt(n)
    got = o.matmul_hadU(x)
    # float32 sqrt(n) inside matmul_hadU limits agreement to ~1e-7 relative
    np.testing.assert_allclose(got, want, rtol=2e-7, atol=1e-12)
    np.testing.assert_allclose(o.hadamard_closed_form(x), want, rtol=1e-13, atol=1e-13)
    # transposed factor inverts it (orthonormal), and differs when hadK is not symmetric
    back = o.matmul_hadU(got, transpose=True) if k > 1 else o.matmul_hadU(got)
    np.testing.assert_allclose(back, x, rtol=1e-6, atol=1e-6)


def test_matmul_hadU_unit_vectors_give_columns():
    n = 344  # 172 * 2
    hadk, k = o.get_hadK(n)
    full = np.kron(hadk, scipy.linalg.hadamard(2))
    eye = np.eye(n)
    got = o.matmul_hadU(eye) * np.sqrt(F32(n)).astype(np.float64)
    np.testing.assert_allclose(got, full.T, atol=1e-9)   # row i of output = column i of kron(...)


@pytest.mark.parametrize("n,dtype", [(64, F16), (4096, F16), (688, F16), (688, F32), (224, F32), (11008, F16)])
def test_hadamard_staged_close_to_closed_form(n, dtype):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((3, n)).astype(dtype)
    hadk, k = o.get_hadK(n)
    got = o.hadamard_staged(x, hadk, k, dtype).astype(np.float64)
    want = o.hadamard_closed_form(x.astype(np.float64))
    tol = 2e-3 if dtype == F16 else 2e-6
    np.testing.assert_allclose(got, want, rtol=tol, atol=tol)
    # norm preservation
    np.testing.assert_allclose(np.linalg.norm(got, axis=-1), np.linalg.norm(x.astype(np.float64), axis=-1), rtol=1e-3)


def test_fwht_butterfly_had_scale_and_online_hadamard_directly():
    """The three thin helpers on their own (their callers pin them only indirectly):
    fwht_butterfly on integer-valued input is the exact product with scipy's natural-order Hadamard matrix, in the
    layout the reference's loop leaves ([rows, stop_len, n / stop_len], transformed index trailing); stopping at length K
    leaves K untouched blocks; a swapped (a - b, a + b) pair or a transform over the wrong axis fails these.
    had_scale is the float32 quotient 1 / sqrt(float32(n)).  online_hadamard casts to fp32 and back exactly when told
    to, and otherwise rounds to fp16 between the two factors (it differs from the fp32 form in that case only)."""
    rng = np.random.default_rng(21)
    for n in (2, 8, 64):
        x = rng.integers(-50, 50, (3, n)).astype(np.float64)
        got = o.fwht_butterfly(x)
        assert got.shape == (3, 1, n)
        assert np.array_equal(got[:, 0, :], x @ scipy.linalg.hadamard(n).T)
    # 24 = 12 blocks of 2 (the order in which matmul_hadU leaves them: block index k = i // 2 leading)
    x = rng.integers(-50, 50, (2, 24)).astype(np.float64)
    got = o.fwht_butterfly(x, stop_len=12)
    assert got.shape == (2, 12, 2)
    blocks = x.reshape(2, 12, 2)
    assert np.array_equal(got[..., 0], blocks[..., 0] + blocks[..., 1]) and np.array_equal(got[..., 1], blocks[..., 0] - blocks[..., 1])
    # fp16 input: every stage rounds (65504 + 65504 overflows in the first stage, whatever comes later)
    big = np.array([[65504, 65504, -65504, -65504]], F16)
    with np.errstate(over="ignore", invalid="ignore"):
        got = o.fwht_butterfly(big)[0, 0]
    # exact result [0, 0, 4a, 0]; with a + b = inf and c + d = -inf: inf + -inf = NaN, inf - -inf = inf
    assert got.dtype == F16 and np.isnan(got[0]) and got[1] == 0 and got[2] == np.inf and got[3] == 0
    for n in (1, 2, 128, 11008, 28672):
        s = o.had_scale(n)
        assert s.dtype == F32 and s == F32(1.0) / np.sqrt(F32(n))
        assert abs(float(s) * float(s) * n - 1.0) < 1e-6
    assert o.had_scale(4096) == F32(1 / 64) and o.had_scale(64) == F32(0.125)
    # online_hadamard: output dtype is the input's; force_fp32 = one rounding of the fp32 transform
    x = (rng.standard_normal((4, 24)) * 3).astype(F16)
    y16, y32 = o.online_hadamard(x), o.online_hadamard(x, force_fp32=True)
    assert y16.dtype == F16 and y32.dtype == F16
    exact = o.hadamard_closed_form(x.astype(np.float64))
    assert np.all(np.abs(y32.astype(np.float64) - exact) <= np.abs(exact) * 2.0 ** -10 + 1e-6)     # half an fp16 step + fp32 noise
    assert np.all(np.abs(y16.astype(np.float64) - exact) <= 4e-3 * np.abs(exact).max())
    hadk, k = o.get_hadK(24)
    assert np.array_equal(y16, o.hadamard_staged(x, hadk, k, F16)) and np.array_equal(y32, o.hadamard_staged(x.astype(F32), hadk, k, F32).astype(F16))
    # a power of two: no second factor, so the two modes differ by nothing but the fp32 scale's rounding
    x = (rng.standard_normal((4, 64))).astype(F16)
    assert np.array_equal(o.online_hadamard(x), o.online_hadamard(x, force_fp32=True))


def test_fwht_natural_brute_force():
    rng = np.random.default_rng(2)
    for m in (1, 2, 4, 32, 128):
        x = rng.standard_normal((4, m))
        np.testing.assert_allclose(o.fwht_natural(x), x @ scipy.linalg.hadamard(m).astype(float).T, atol=1e-10)


def test_kv_hadamard_involution_and_value():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((6, 128)).astype(F16)
    y = o.kv_hadamard(x)
    want = x.astype(np.float64) @ scipy.linalg.hadamard(128) / np.sqrt(128)
    np.testing.assert_allclose(y.astype(np.float64), want, rtol=1e-3, atol=1e-3)
    np.testing.assert_allclose(o.kv_hadamard(y).astype(np.float64), x.astype(np.float64), rtol=3e-3, atol=3e-3)


# ------------------------------------------------------------------ quantizer

def test_scale_is_correctly_rounded_for_every_amax():
    amax = np.abs(all_finite_f16())
    amax = np.unique(amax)
    got = o.quantizer_scales(amax.reshape(-1, 1))
    step = 97  # every 97th value by exact rational rounding (the full sweep is 31k Fractions; keep it quick)
    for a, g in zip(amax[::step], got[::step]):
        assert round_fraction_to_f16(Fraction(float(a)) / 7) == g, a
    # clip ratio: torch evaluates half_tensor * python_float in float32 and rounds the float32
    # product to fp16 (two roundings), so the pin here is torch's own CPU kernel on every amax.
    import torch
    t = torch.from_numpy(amax.copy()).reshape(-1, 1)
    for clip in (0.9, 0.85, 1.0):
        want = ((torch.max(torch.abs(t), dim=-1)[0].unsqueeze(1) / 7).to(torch.float16) * clip).numpy().reshape(-1)
        assert np.array_equal(o.quantizer_scales(amax.reshape(-1, 1), clip=clip), want)


def test_codes_match_torch_cpu_half_ops():
    """The reference's CPU-capable statement of the same quantiser is torch.round(x / scale) on
    fp16 tensors (quarot/functional/quantization.py:31); torch's CPU half kernels are an
    independent implementation of the IEEE operations the oracle spells out in numpy."""
    import torch
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((64, 512)) * 4).astype(F16)
    s = o.quantizer_scales(x)
    tx, ts = torch.from_numpy(x), torch.from_numpy(s).reshape(-1, 1)
    want = torch.clamp(torch.round(tx / ts), -8, 7).to(torch.int8).numpy()
    assert np.array_equal(o.sym_quant_codes(x, s), want)
    q = torch.from_numpy(rng.integers(-30000, 30000, (64, 48)).astype(np.int32))
    sc = torch.from_numpy((np.abs(rng.standard_normal(48)) * 0.01).astype(F16))
    wantd = (ts * sc.reshape(1, -1)) * q.to(torch.float16)
    assert np.array_equal(o.sym_dequant(q.numpy(), s, sc.numpy()).view(np.uint16), wantd.numpy().view(np.uint16))


def test_codes_exact_rational_random_and_ties():
    rng = np.random.default_rng(4)
    xs = rng.standard_normal(400).astype(F16) * F16(3)
    ss = np.abs(rng.standard_normal(400).astype(F16)) + F16(0.01)
    got = o.sym_quant_codes(xs.reshape(-1, 1), ss)
    for x, s, g in zip(xs, ss, got[:, 0]):
        d = round_fraction_to_f16(Fraction(float(x)) / Fraction(float(s)))
        fr = Fraction(float(d))
        fl = fr.numerator // fr.denominator
        rem = fr - fl
        r = fl + (1 if (rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1)) else 0)
        assert g == max(-8, min(7, r)), (x, s)
    # constructed ties: x = s * (j + 0.5) exactly -> round half to even
    s = F16(0.25)
    halves = np.array([-8.5, -7.5, -2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 3.5, 6.5, 7.5, 8.5, 100.0, -100.0])
    x = (halves * float(s)).astype(F16)
    want = np.array([-8, -8, -2, -2, 0, 0, 2, 2, 4, 6, 7, 7, 7, -8])
    assert np.array_equal(o.sym_quant_codes(x.reshape(1, -1), np.array([s]))[0], want)
    # truncation toward zero (the HIP __half2int_rn trap) would give 0 for 0.75 and 1 for 1.75
    x = np.array([0.75, 1.75, -0.75, -1.75], F16)
    assert np.array_equal(o.sym_quant_codes(x.reshape(1, -1), np.array([F16(1)]))[0], [1, 2, -1, -2])


def test_codes_double_rounding_case():
    # x/s slightly below 2.5 but within half an fp16 ulp of it: fp16 division gives exactly 2.5,
    # which then rounds to even (2); 3.5-eps likewise becomes 3.5 -> 4 (exact rounding would say 3).
    s = F16(1 / 3)            # 0.33325195
    found = 0
    for target, want in ((3.5, 4), (2.5, 2), (5.5, 6)):
        for xb in all_finite_f16():
            if xb <= 0:
                continue
            exact = Fraction(float(xb)) / Fraction(float(s))
            if exact < Fraction(target) and round_fraction_to_f16(exact) == F16(target):
                assert o.sym_quant_codes(np.array([[xb]], F16), np.array([s]))[0, 0] == want
                found += 1
                break
    assert found >= 1


def test_zero_row_gives_zero_codes_and_zero_scale():
    x = np.zeros((2, 8), F16)
    p, s = o.quantizer(x)
    assert np.all(s == 0) and np.all(p == 0)
    # explicit zero scale with non-zero x: +-inf -> clamp
    c = o.sym_quant_codes(np.array([[1, -1, 0]], F16), np.array([0], F16))
    assert np.array_equal(c[0], [7, -8, 0])


def test_pack_unpack_all_bytes_and_nibble_order():
    b = np.arange(256, dtype=np.uint8).reshape(16, 16)
    assert np.array_equal(o.pack_i4(o.unpack_i4(b)), b)
    assert np.array_equal(o.unpack_i4(np.array([[0x2F]], np.uint8)), [[-1, 2]])      # low nibble first
    assert np.array_equal(o.pack_i4(np.array([[-8, 7, 3]])), [[0x78, 0x03]])         # odd tail -> high nibble 0
    assert o.unpack_i4(b).min() == -8 and o.unpack_i4(b).max() == 7
    with pytest.raises(AssertionError):
        o.pack_i4(np.array([[8, 0]]))


# ------------------------------------------------------------------ GEMM and dequant

def test_int4_matmul_known_answers():
    k = 128
    a = o.pack_i4(np.full((3, k), 7))
    b = o.pack_i4(np.full((5, k), -8))
    assert np.all(o.int4_matmul(a, b) == -56 * k)
    assert np.all(o.int4_matmul(a, b, exact_int=True) == -56 * k)
    # one-hot rows pick out columns of B^T
    rng = np.random.default_rng(5)
    bq = rng.integers(-8, 8, (7, 64))
    onehot = np.zeros((64, 64), np.int64)
    onehot[np.arange(64), np.arange(64)] = 1
    assert np.array_equal(o.int4_matmul(o.pack_i4(onehot), o.pack_i4(bq)), bq.T)


def test_int4_matmul_float_path_equals_int64():
    rng = np.random.default_rng(6)
    aq = rng.integers(-8, 8, (33, 448))
    bq = rng.integers(-8, 8, (17, 448))
    want = aq.astype(np.int64) @ bq.astype(np.int64).T
    assert np.array_equal(o.int4_matmul(o.pack_i4(aq), o.pack_i4(bq)), want)
    assert np.array_equal(o.int4_matmul(o.pack_i4(aq), o.pack_i4(bq), exact_int=True), want)


def test_dequant_three_roundings_exact():
    rng = np.random.default_rng(7)
    q = rng.integers(-40000, 40000, (6, 9)).astype(np.int32)
    q[0, 0], q[0, 1], q[0, 2] = 2049, 65519, 65520          # 2049 -> 2048 (tie to even), 65519 -> 65504, 65520 -> inf
    sr = (np.abs(rng.standard_normal(6)) * 0.1).astype(F16)
    sc = (np.abs(rng.standard_normal(9)) * 0.01).astype(F16)
    bias = rng.standard_normal(9).astype(F16)
    got = o.sym_dequant(q, sr, sc)
    gotb = o.sym_dequant(q, sr, sc, bias)
    for i in range(6):
        for j in range(9):
            qh = round_fraction_to_f16(Fraction(int(q[i, j])))
            ss = round_fraction_to_f16(Fraction(float(sr[i])) * Fraction(float(sc[j])))
            if not np.isfinite(qh):
                assert not np.isfinite(got[i, j])
                continue
            y = round_fraction_to_f16(Fraction(float(ss)) * Fraction(float(qh)))
            assert y == got[i, j]
            assert round_fraction_to_f16(Fraction(float(y)) + Fraction(float(bias[j]))) == gotb[i, j]
    assert o.sym_dequant(np.array([[2049]]), [F16(1)], [F16(1)])[0, 0] == F16(2048)


def test_linear4bit_close_to_float_product():
    rng = np.random.default_rng(8)
    x = rng.standard_normal((16, 256)).astype(F16)
    w = (rng.standard_normal((24, 256)) * 0.02).astype(F16)
    ws = (np.max(np.abs(w), axis=1, keepdims=True).astype(F32) / 7).astype(F16)
    wq = o.weight_codes_from_float(w, ws)
    xq, xs = o.quantizer(x)
    y = o.linear4bit(xq, xs, wq, ws).astype(np.float64)
    ref = x.astype(np.float64) @ w.astype(np.float64).T
    # 4-bit noise: correlation, not equality
    assert np.corrcoef(y.ravel(), ref.ravel())[0, 1] > 0.95


# ------------------------------------------------------------------ KV asymmetric int4

def test_kv_asym_invariants():
    rng = np.random.default_rng(9)
    x = rng.standard_normal((64, 128)).astype(F16)
    p, s, z = o.kv_asym_quant(x)
    assert p.shape == (64, 64) and s.shape == (64, 1) and z.shape == (64, 1)
    nib = np.stack([p & 0xF, p >> 4], -1).reshape(64, 128)
    assert nib[np.arange(64), x.argmin(1)].max() == 0          # min -> code 0
    assert nib[np.arange(64), x.argmax(1)].min() == 15         # max -> code 15
    xh = o.kv_asym_dequant(p, s, z).astype(np.float64)
    err = np.abs(xh - x.astype(np.float64))
    assert np.all(err <= s.astype(np.float64) / 2 + 4e-3)
    # constant vector: range clamps to fp16(1e-5), all codes 0
    c = np.full((1, 128), 0.5, F16)
    p, s, z = o.kv_asym_quant(c)
    assert np.all(p == 0) and s[0, 0] == (F16(1e-5).astype(F32) / F32(15)).astype(F16) and z[0, 0] == F16(-0.5)


def test_kv_asym_exact_rational_spot():
    rng = np.random.default_rng(10)
    x = (rng.standard_normal((3, 128)) * 2).astype(F16)
    p, s, z = o.kv_asym_quant(x)
    nib = np.stack([p & 0xF, p >> 4], -1).reshape(3, 128)
    for r in range(3):
        mx, mn = Fraction(float(x[r].max())), Fraction(float(x[r].min()))
        rg = round_fraction_to_f16(mx - mn)
        sc = round_fraction_to_f16(Fraction(float(rg)) / 15)
        assert sc == s[r, 0] and z[r, 0] == F16(-float(mn))
        for c in range(0, 128, 5):
            sh = round_fraction_to_f16(Fraction(float(x[r, c])) - mn)
            d = Fraction(float(round_fraction_to_f16(Fraction(float(sh)) / Fraction(float(sc)))))
            fl = d.numerator // d.denominator
            rem = d - fl
            q = fl + (1 if (rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1)) else 0)
            assert nib[r, c] == max(0, min(15, q))
            back = round_fraction_to_f16(Fraction(float(round_fraction_to_f16(int(nib[r, c]) * Fraction(float(sc))))) + mn)
            assert back == o.kv_asym_dequant(p, s, z)[r, c]


def test_rmsnorm_closed_form_and_special_cases():
    """x / sqrt(sum(x^2) / mean_dim + eps) in exact rational arithmetic, rounded once to fp16, on a
    handful of rows (the square root bracketed by exact integer comparison); then properties a wrong
    divisor, a missing eps or a mean over the wrong axis would break."""
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((3, 24)) * 3).astype(F16)
    got = o.rmsnorm(x, 24, 1e-5)
    x64 = x.astype(np.float64)
    want64 = x64 / np.sqrt((x64 ** 2).sum(-1, keepdims=True) / 24 + np.float64(F32(1e-5)))
    # float64 carries 53 bits: its rounding to fp16 is the exact answer unless within 2^-40 of a tie
    assert np.array_equal(got, want64.astype(F16))
    # exact rational check of one element: y^2 * (S / d + eps) == x^2 up to the fp16 rounding interval
    S = sum(Fraction(float(v)) ** 2 for v in x[0])
    denom = S / 24 + Fraction(float(F32(1e-5)))
    for j in (0, 7, 23):
        y = Fraction(float(got[0, j]))
        ulp = Fraction(float(np.spacing(np.abs(got[0, j]).astype(F16))))
        lo, hi = abs(y) - ulp / 2, abs(y) + ulp / 2
        assert lo ** 2 * denom <= Fraction(float(x[0, j])) ** 2 <= hi ** 2 * denom
        assert (y < 0) == (x[0, j] < 0)
    # constant row c with mean_dim = length: c / sqrt(c^2 + eps) ~ sign(c)
    c = np.full((1, 64), -2.0, F16)
    assert np.array_equal(o.rmsnorm(c, 64, 1e-5), np.full((1, 64), F16(-2.0 / np.sqrt(4.0 + 1e-5)), F16))
    # mean_dim is a parameter, not the row length: quadrupling it doubles the output (eps negligible)
    big = (rng.standard_normal((2, 32)) * 8).astype(F16)
    a, b = o.rmsnorm(big, 32, 0.0).astype(np.float64), o.rmsnorm(big, 128, 0.0).astype(np.float64)
    assert np.allclose(b, 2 * a, rtol=2e-3)
    # eps matters for tiny rows: an all-zero row stays zero instead of dividing by zero
    assert np.array_equal(o.rmsnorm(np.zeros((1, 16), F16), 16, 1e-5), np.zeros((1, 16), F16))
    # each row is normalised on its own
    assert np.array_equal(o.rmsnorm(x, 24, 1e-5)[1], o.rmsnorm(x[1:2], 24, 1e-5)[0])
    # torch's CPU kernels on the same statement (the timed CPU baseline uses them): same values up to
    # the order of the fp32 sum
    import torch
    from oracle import cpu_baseline as cb
    wide = (rng.standard_normal((16, 4096)) * 2).astype(F16)
    t = cb.rmsnorm(torch.from_numpy(wide)).numpy()
    w = o.rmsnorm(wide, 4096, 1e-5)
    assert np.mean(t == w) > 0.999 and np.allclose(t.astype(F32), w.astype(F32), rtol=1e-3, atol=1e-3)


def test_cpu_baseline_port_agrees_with_oracle():
    """The torch chain timed as the CPU baseline computes what the oracle computes (Hadamard to
    tolerance; given the same Hadamard output, identical codes and identical fp16 outputs)."""
    import torch
    from oracle import cpu_baseline as cb
    rng = np.random.default_rng(12)
    x = rng.standard_normal((8, 688)).astype(F16)
    wq = rng.integers(-8, 8, (24, 688))
    ws = (np.abs(rng.standard_normal(24)) * 0.01).astype(F16)
    xh = cb.matmul_hadU(torch.from_numpy(x).float())
    np.testing.assert_allclose(xh.numpy(), o.hadamard_closed_form(x.astype(np.float64)), rtol=1e-4, atol=1e-4)
    xh16 = xh.half()
    q, sx = cb.quantize(xh16)
    assert np.array_equal(q.numpy(), o.sym_quant_codes(xh16.numpy(), o.quantizer_scales(xh16.numpy())))
    y = cb.linear4bit_path(torch.from_numpy(x), torch.from_numpy(wq.astype(np.int32)), torch.from_numpy(ws))
    want = o.linear4bit(o.pack_i4(q.numpy()), sx.numpy().reshape(-1), o.pack_i4(wq), ws)
    assert np.array_equal(y.numpy().view(np.uint16), want.view(np.uint16))


def test_heads_hadamard_is_the_transform_over_the_head_axis():
    """The composition transpose -> OnlineHadamard(num_heads) -> transpose -> reshape against an
    independent float64 einsum with scipy's Sylvester matrix, and cases that a transform over the
    wrong axis, a missing 1/sqrt(H) or a transposed result would fail."""
    import scipy.linalg
    rng = np.random.default_rng(21)
    for heads, dim in ((32, 128), (64, 128), (16, 8), (8, 4)):
        x = rng.standard_normal((3, heads, dim)).astype(F16)
        got = o.heads_hadamard(x, heads)
        assert got.shape == (3, heads * dim) and got.dtype == F16
        H = scipy.linalg.hadamard(heads).astype(np.float64)
        want = np.einsum("gh,rhd->rgd", H, x.astype(np.float64)) / np.sqrt(np.float64(heads))
        # the oracle multiplies by the float32 scale 1/sqrt(H) before its single rounding: one fp16 ulp
        assert np.allclose(got.astype(np.float64), want.reshape(3, -1), rtol=2e-3, atol=2e-3)
        assert np.mean(got == want.reshape(3, -1).astype(F16)) > 0.99
    # constant across heads: everything lands in head 0, scaled by sqrt(H) (exact for H = 16, 64)
    c = np.broadcast_to(rng.standard_normal((1, 1, 128)).astype(F16), (1, 64, 128)).copy()
    y = o.heads_hadamard(c, 64).reshape(64, 128)
    assert np.array_equal(y[0], (c[0, 0].astype(F32) * F32(8)).astype(F16)) and not y[1:].any()
    # a single non-zero head h: output head g is Had[g, h] / sqrt(H) times that head's vector
    e = np.zeros((1, 16, 128), F16)
    e[0, 5] = rng.standard_normal(128).astype(F16)
    y = o.heads_hadamard(e, 16).reshape(16, 128)
    H16 = scipy.linalg.hadamard(16)
    for g in range(16):
        assert np.array_equal(y[g], (e[0, 5].astype(F32) * F32(0.25 * H16[g, 5])).astype(F16))


# ------------------------------------------------------------------------------ paged KV cache

def bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def _paged_case(rng, batch, heads, page_size, lens, layers=2, spare_pages=3, shuffle=True):
    """A cache with every sequence's pages scattered over the page pool."""
    per = [max(1, -(-n // page_size)) for n in lens]
    total = sum(per) + spare_pages
    order = rng.permutation(total) if shuffle else np.arange(total)
    indptr = np.concatenate([[0], np.cumsum(per)]).astype(np.int32)
    indices = order[: sum(per)].astype(np.int32)
    last = np.array([n - (p - 1) * page_size for n, p in zip(lens, per)], np.int32)
    data = rng.integers(0, 256, (total, layers, 2, heads, page_size, 64), dtype=np.uint8)
    param = rng.standard_normal((total, layers, 2, heads, page_size, 2)).astype(F16)
    return data, param, indptr, indices, last


def test_paged_append_follows_the_reference_offset_formulas():
    """The numpy-indexed oracle against an element-by-element walk over FLAT buffers with the offset
    formulas of page.cuh:75-103 spelled out, prefill (ragged lengths, pages partly filled before) and
    one-token append; bytes of other layers, pages and entries must stay untouched."""
    rng = np.random.default_rng(5)
    heads, P, L, layer = 3, 4, 2, 1
    lens = [6, 1, 9, 4]                                   # lengths AFTER the append
    add = [3, 1, 9, 2]
    data, param, indptr, indices, last = _paged_case(rng, 4, heads, P, lens, layers=L)
    app = np.concatenate([[0], np.cumsum(add)]).astype(np.int32)
    T = int(app[-1])
    k, v = rng.integers(0, 256, (T, heads, 64), dtype=np.uint8), rng.integers(0, 256, (T, heads, 64), dtype=np.uint8)
    kp, vp = rng.standard_normal((T, heads, 2)).astype(F16), rng.standard_normal((T, heads, 2)).astype(F16)
    want_d, want_p = data.copy().reshape(-1), param.copy().reshape(-1, 2)
    for b in range(4):
        seq = (indptr[b + 1] - indptr[b] - 1) * P + last[b]
        for j in range(add[b]):
            pos = seq - add[b] + j
            page, entry = indices[indptr[b] + pos // P], pos % P
            for h in range(heads):
                for kv, src, sp in ((0, k, kp), (1, v, vp)):
                    # get_k_elem_offset / get_v_elem_offset in elements of 4 bits -> bytes / 2; parameters in half2
                    slot = (((page * L + layer) * 2 + kv) * heads + h) * P + entry
                    for f in range(64):
                        want_d[slot * 64 + f] = src[app[b] + j, h, f]
                    want_p[slot] = sp[app[b] + j, h]
    before = data.copy()
    o.paged_append(data, param, indptr, indices, last, k, v, kp, vp, layer, app)
    assert np.array_equal(data.reshape(-1), want_d) and np.array_equal(bits(param.reshape(-1, 2)), bits(want_p))
    assert np.array_equal(data[:, 0], before[:, 0])                           # the other layer
    # one token per sequence
    d2, p2 = data.copy(), param.copy()
    k1, v1 = k[:4], v[:4]
    o.paged_append(d2, p2, indptr, indices, last, k1, v1, kp[:4], vp[:4], layer, None)
    for b in range(4):
        kc, kpar, vc, vpar = o.paged_gather(d2, p2, indptr, indices, last, layer, b)
        assert kc.shape == (lens[b], heads, 64)
        assert np.array_equal(kc[-1], k1[b]) and np.array_equal(vc[-1], v1[b]) and np.array_equal(bits(vpar[-1]), bits(vp[b]))
        if lens[b] > 1:                                                       # earlier positions: what the prefill wrote
            kc0, _, _, _ = o.paged_gather(data, param, indptr, indices, last, layer, b)
            assert np.array_equal(kc[:-1], kc0[:-1])


def test_paged_append_then_gather_round_trip():
    rng = np.random.default_rng(6)
    heads, P = 2, 16
    lens = [16, 33, 5]
    data, param, indptr, indices, last = _paged_case(rng, 3, heads, P, lens, layers=1)
    app = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(app[-1])
    k, v = rng.integers(0, 256, (T, heads, 64), dtype=np.uint8), rng.integers(0, 256, (T, heads, 64), dtype=np.uint8)
    kp, vp = rng.standard_normal((T, heads, 2)).astype(F16), rng.standard_normal((T, heads, 2)).astype(F16)
    o.paged_append(data, param, indptr, indices, last, k, v, kp, vp, 0, app)
    for b in range(3):
        kc, kpar, vc, vpar = o.paged_gather(data, param, indptr, indices, last, 0, b)
        sl = slice(app[b], app[b + 1])
        assert np.array_equal(kc, k[sl]) and np.array_equal(vc, v[sl])
        assert np.array_equal(bits(kpar), bits(kp[sl])) and np.array_equal(bits(vpar), bits(vp[sl]))
    assert np.array_equal(o.paged_seq_lens(indptr, last, P), lens)


def test_paged_dequant_is_one_float32_rounding_of_the_exact_value():
    """float(nibble) * scale is exact in float32 (4 + 11 significant bits); subtracting zero rounds once."""
    rng = np.random.default_rng(7)
    codes = rng.integers(0, 256, (40, 64), dtype=np.uint8)
    param = (rng.standard_normal((40, 2)) * np.array([0.3, 2.0])).astype(F16)
    got = o.paged_dequant(codes, param)
    assert got.dtype == F32 and got.shape == (40, 128)
    for r in range(0, 40, 7):
        s, z = Fraction(float(param[r, 0])), Fraction(float(param[r, 1]))
        for i in (0, 1, 2, 63, 126, 127):
            nib = int(codes[r, i // 2]) >> (4 * (i % 2)) & 0xF                # even element in the low nibble
            exact = nib * s - z
            assert got[r, i] == F32(float(exact)) or abs(Fraction(float(got[r, i])) - exact) <= abs(exact) * Fraction(1, 1 << 24)
            assert Fraction(float(F32(nib) * F32(float(param[r, 0])))) == nib * s


def test_paged_batch_decode_against_textbook_attention():
    """torch's scaled_dot_product_attention in float64 on the gathered, dequantised vectors; and special
    cases a wrong softmax axis, a missing 1/sqrt(D) or K/V swapped would fail."""
    rng = np.random.default_rng(8)
    heads, P = 4, 8
    lens = [1, 8, 19, 40]
    data, param, indptr, indices, last = _paged_case(rng, 4, heads, P, lens, layers=2)
    param[..., 0] = (np.abs(param[..., 0].astype(F32)) * 0.05 + 0.01).astype(F16)      # positive scales
    q = rng.standard_normal((4, heads, 128)).astype(F16)
    got = o.paged_batch_decode(q, data, param, indptr, indices, last, 1)
    for b in range(4):
        kc, kp, vc, vp = o.paged_gather(data, param, indptr, indices, last, 1, b)
        kf = torch.from_numpy(o.paged_dequant(kc, kp)).double().permute(1, 0, 2)      # [H, seq, D]
        vf = torch.from_numpy(o.paged_dequant(vc, vp)).double().permute(1, 0, 2)
        want = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q[b]).double().unsqueeze(1), kf, vf)
        np.testing.assert_allclose(got[b], want.squeeze(1).numpy(), rtol=1e-10, atol=1e-10)
    # a sequence of one token returns v_0 whatever q is
    _, _, vc, vp = o.paged_gather(data, param, indptr, indices, last, 1, 0)
    np.testing.assert_allclose(got[0], o.paged_dequant(vc, vp)[0].astype(np.float64), rtol=1e-12)
    # q = 0: uniform weights, the mean of V
    g0 = o.paged_batch_decode(np.zeros_like(q), data, param, indptr, indices, last, 1)
    _, _, vc, vp = o.paged_gather(data, param, indptr, indices, last, 1, 3)
    np.testing.assert_allclose(g0[3], o.paged_dequant(vc, vp).astype(np.float64).mean(axis=0), rtol=1e-10, atol=1e-12)
    # the other layer holds different data: a wrong layer offset changes the result
    assert not np.allclose(o.paged_batch_decode(q, data, param, indptr, indices, last, 0), got)


def test_paged_batch_decode_over_fp16_pages_against_textbook_attention():
    """The fp16-page form: torch's scaled_dot_product_attention in float64 on the vectors gathered page by page with
    explicit loops, a cache whose int4 twin holds the same values (both oracles must agree), and the one-token and
    q = 0 cases."""
    rng = np.random.default_rng(9)
    heads, P = 3, 8
    lens = [1, 8, 19, 40]
    _, _, indptr, indices, last = _paged_case(rng, 4, heads, P, lens, layers=2)
    pool = int(indices.max()) + 4
    data = rng.standard_normal((pool, 2, 2, heads, P, 128)).astype(F16)
    q = rng.standard_normal((4, heads, 128)).astype(F16)
    got = o.paged_batch_decode_f16(q, data, indptr, indices, last, 1)
    for b in range(4):
        ks, vs = [], []
        for pos in range(lens[b]):
            page = int(indices[int(indptr[b]) + pos // P])
            ks.append(data[page, 1, 0, :, pos % P, :])
            vs.append(data[page, 1, 1, :, pos % P, :])
        kf = torch.from_numpy(np.stack(ks)).double().permute(1, 0, 2)
        vf = torch.from_numpy(np.stack(vs)).double().permute(1, 0, 2)
        want = torch.nn.functional.scaled_dot_product_attention(torch.from_numpy(q[b]).double().unsqueeze(1), kf, vf)
        np.testing.assert_allclose(got[b], want.squeeze(1).numpy(), rtol=1e-10, atol=1e-10)
        if b == 0:
            np.testing.assert_allclose(got[0], np.stack(vs)[0].astype(np.float64), rtol=1e-12)      # one token: v_0
        if b == 3:
            g0 = o.paged_batch_decode_f16(np.zeros_like(q), data, indptr, indices, last, 1)
            np.testing.assert_allclose(g0[3], np.stack(vs).astype(np.float64).mean(axis=0), rtol=1e-10, atol=1e-12)
    assert not np.allclose(o.paged_batch_decode_f16(q, data, indptr, indices, last, 0), got)
    # values that int4 codes hold exactly (code * 0.25 - 1): the int4 oracle over the coded cache gives the same
    codes = rng.integers(0, 16, (pool, 2, 2, heads, P, 128)).astype(np.uint8)
    packed = (codes[..., 0::2] | (codes[..., 1::2] << 4)).astype(np.uint8)
    param = np.zeros((pool, 2, 2, heads, P, 2), F16)
    param[..., 0], param[..., 1] = 0.25, 1.0
    exact = (codes.astype(F32) * F32(0.25) - F32(1.0)).astype(F16)
    np.testing.assert_allclose(o.paged_batch_decode_f16(q, exact, indptr, indices, last, 0),
                               o.paged_batch_decode(q, packed, param, indptr, indices, last, 0), rtol=1e-12, atol=1e-12)

