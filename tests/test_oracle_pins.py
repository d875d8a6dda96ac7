"""Pins for the CPU oracle: each check is independent of the oracle's own formula
(library FFT, brute-force loops, closed forms, invariants), so that a dropped
term, wrong sign, wrong period or transposed operand fails at least one."""
import math

import numpy as np
import pytest

from oracle import fourier_oracle as fo


def rng(seed=0):
    return np.random.default_rng(seed)


# ---------------------------------------------------------------- periods ---
def test_period_pair_known_values():
    # T_c = int(1/(1/T_x)) drops by one for some integers (CPython float64)
    assert fo.periods(130044 + 4 + 1024, 4, 1024)[0::2] == (130044, 130043)
    assert fo.periods(93 + 10, 4, 6)[0::2] == (93, 92)
    assert fo.periods(31868 + 1028, 4, 1024)[0::2] == (31868, 31868)
    bad = [x for x in range(1, 2000) if fo.periods(x, 0, 0)[2] != x]
    assert bad[:5] == [93, 99, 105, 117, 123]
    for x in range(1, 5000):
        assert fo.periods(x, 0, 0)[2] in (x, x - 1)


# ------------------------------------------------------------ compression ---
@pytest.mark.parametrize("L,T", [(37, 37), (20, 37), (50, 37), (64, 64), (5, 9)])
def test_compress_equals_library_fft(L, T):
    # zero-pad when L < T, truncate when L > T (torch.fft.fft(n=T) semantics == numpy's)
    x = rng(1).standard_normal((2, L, 3))
    nf = 4
    c = fo.compress_prefill(x, nf, T)
    f = np.fft.fft(x, n=T, axis=1)[:, :nf, :]
    assert c.shape == (2, 2 * nf, 3)
    np.testing.assert_allclose(c[:, :nf], f.real, atol=1e-10)
    np.testing.assert_allclose(c[:, nf:], -f.imag, atol=1e-10)


def test_compress_brute_force_loops():
    x = rng(2).standard_normal((1, 7, 2))
    nf, T = 3, 11
    c = fo.compress_prefill(x, nf, T)
    for n in range(nf):
        for j in range(2):
            cc = sum(x[0, t, j] * math.cos(2 * math.pi * n * t / T) for t in range(7))
            ss = sum(x[0, t, j] * math.sin(2 * math.pi * n * t / T) for t in range(7))
            assert abs(c[0, n, j] - cc) < 1e-12
            assert abs(c[0, nf + n, j] - ss) < 1e-12
    # n = 0: cos row is the plain column sum, sin row is zero
    np.testing.assert_allclose(c[0, 0], x[0].sum(0), atol=1e-12)
    np.testing.assert_allclose(c[0, nf], 0.0, atol=1e-12)


def test_update_is_difference_of_batch_transforms():
    # transform of t in [0, L] minus transform of t in [0, L) == rank-1 term at phase L
    x = rng(3).standard_normal((2, 13, 4))
    nf, T = 5, 29
    full = fo.compress_prefill(x, nf, T)
    part = fo.compress_prefill(x[:, :12], nf, T)
    upd = fo.coeff_update(part, x[:, 12, :], 12, T)
    np.testing.assert_allclose(upd, full, atol=1e-10)
    # additivity: two updates commute
    a = fo.coeff_update(fo.coeff_update(part, x[:, 3], 40, T), x[:, 5], 41, T)
    b = fo.coeff_update(fo.coeff_update(part, x[:, 5], 41, T), x[:, 3], 40, T)
    np.testing.assert_allclose(a, b, atol=1e-10)
    # phase is periodic in T
    np.testing.assert_allclose(fo.coeff_update(part, x[:, 3], 7, T), fo.coeff_update(part, x[:, 3], 7 + T, T), atol=1e-9)


# ------------------------------------------------------------------ stats ---
def test_stats_definitions():
    x = rng(4).standard_normal((2, 50, 3))
    avg, dev = fo.mean_max_dev(x)
    for b in range(2):
        for j in range(3):
            col = x[b, :, j]
            m = col.mean()
            assert abs(avg[b, j] - m) < 1e-12
            assert abs(dev[b, j] - max(col.max() - m, m - col.min())) < 1e-12
    a16, d16 = fo.stats_reconstructed(fo.compress_prefill(x, 4, 50), 50, 50)
    assert a16.dtype == np.float32 and np.array_equal(a16, a16.astype(np.float16).astype(np.float32))
    ab, _ = fo.stats_original(x, "bf16")
    assert np.all((ab.view(np.uint32) & 0xFFFF) == 0)


def test_round_bf16_known_values():
    v = np.array([1.0, 1.00390625, 1.005859375, 3.14159265, -2.71828], dtype=np.float32)
    r = fo.round_bf16(v)
    # 1 + 2^-8 is a tie between 1.0 and 1.0078125 -> even (1.0); 1.005859375 -> 1.0078125
    np.testing.assert_array_equal(r[:3], np.array([1.0, 1.0, 1.0078125], dtype=np.float32))
    assert abs(r[3] - 3.140625) < 1e-7 and abs(r[4] + 2.71875) < 1e-7


# --------------------------------------------------------- reconstruction ---
def test_reconstruct_brute_force():
    c = rng(5).standard_normal((1, 6, 2))
    T, K = 17, 9
    r = fo.reconstruct(c, K, T)
    for l in range(K):
        for j in range(2):
            s = sum(math.cos(2 * math.pi * n * l / T) * c[0, n, j] + math.sin(2 * math.pi * n * l / T) * c[0, 3 + n, j]
                    for n in range(3)) / 3
            assert abs(r[0, l, j] - s) < 1e-12


def test_reconstruct_dirichlet_identity():
    # with one period T for both directions: r[t] = (1/N_f) sum_s x[s] Dir(t - s)
    x = rng(6).standard_normal((1, 40, 2))
    nf, T = 6, 40
    r = fo.reconstruct(fo.compress_prefill(x, nf, T), 40, T)
    u = np.arange(40)[:, None] - np.arange(40)[None, :]
    dirk = sum(np.cos(2 * np.pi * n * u / T) for n in range(nf))
    np.testing.assert_allclose(r[0], dirk @ x[0] / nf, atol=1e-10)


def test_reconstruct_amplitude_of_single_tone():
    # a pure in-band tone cos(2 pi f t / T): reconstruction = (T / (2 N_f)) * tone  (f != 0),
    # i.e. the 1/N_f scaling is NOT an inverse DFT; the affine statistics repair the amplitude.
    T, nf, f = 64, 8, 3
    t = np.arange(T)
    x = np.cos(2 * np.pi * f * t / T)[None, :, None]
    r = fo.reconstruct(fo.compress_prefill(x, nf, T), T, T)
    np.testing.assert_allclose(r[0, :, 0], (T / (2 * nf)) * x[0, :, 0], atol=1e-9)
    scale, u_avg, i_avg = fo.prefill_stats(x, fo.compress_prefill(x, nf, T), T, "fp32")
    k = fo.denormalize(r, i_avg, scale, u_avg)
    np.testing.assert_allclose(k[0, :, 0], x[0, :, 0], atol=2e-3)  # fp16 statistics


# -------------------------------------------------------------- attention ---
def _attn_case(seed=7, B=2, Hq=6, Hkv=2, D=8, nil=5, L=11, nf=3, T=23):
    r = rng(seed)
    hid = Hkv * D
    kc = np.sort(r.choice(hid, 7, replace=False)); kn = np.setdiff1d(np.arange(hid), kc)
    vc = np.sort(r.choice(hid, 9, replace=False)); vn = np.setdiff1d(np.arange(hid), vc)
    a = dict(
        q=r.standard_normal((B, 1, Hq * D)), k_il=r.standard_normal((B, nil, hid)), v_il=r.standard_normal((B, nil, hid)),
        k_mc=r.standard_normal((B, 2 * nf, kc.size)), v_mc=r.standard_normal((B, 2 * nf, vc.size)),
        k_mn=r.standard_normal((B, L, kn.size)), v_mn=r.standard_normal((B, L, vn.size)),
        avg_k_u=r.standard_normal((B, kc.size)), avg_k_d=r.standard_normal((B, kc.size)), scale_k=r.uniform(0.5, 2, (B, kc.size)),
        avg_v_u=r.standard_normal((B, vc.size)), avg_v_d=r.standard_normal((B, vc.size)), scale_v=r.uniform(0.5, 2, (B, vc.size)),
        kc_list=kc, kc_h_list=None, kn_list=kn, kn_h_list=None, vc_list=vc, vc_h_list=None, vn_list=vn, vn_h_list=None,
        num_head_q=Hq, num_head_kv=Hkv, seq_len_m=L, T=T)
    return a


def test_attention_brute_force():
    a = _attn_case()
    out = fo.fourier_attn(**a)
    B, Hq, Hkv, D, L, nf, T = 2, 6, 2, 8, 11, 3, 23
    G = Hq // Hkv
    for b in range(B):
        # explicit K/V rows, element by element
        km = np.zeros((L, Hkv * D)); vm = np.zeros((L, Hkv * D))
        for l in range(L):
            for jj, dim in enumerate(a["kc_list"]):
                s = sum(math.cos(2 * math.pi * n * l / T) * a["k_mc"][b, n, jj] + math.sin(2 * math.pi * n * l / T) * a["k_mc"][b, nf + n, jj] for n in range(nf)) / nf
                km[l, dim] = (s - a["avg_k_d"][b, jj]) * a["scale_k"][b, jj] + a["avg_k_u"][b, jj]
            for jj, dim in enumerate(a["kn_list"]):
                km[l, dim] = a["k_mn"][b, l, jj]
            for jj, dim in enumerate(a["vc_list"]):
                s = sum(math.cos(2 * math.pi * n * l / T) * a["v_mc"][b, n, jj] + math.sin(2 * math.pi * n * l / T) * a["v_mc"][b, nf + n, jj] for n in range(nf)) / nf
                vm[l, dim] = (s - a["avg_v_d"][b, jj]) * a["scale_v"][b, jj] + a["avg_v_u"][b, jj]
            for jj, dim in enumerate(a["vn_list"]):
                vm[l, dim] = a["v_mn"][b, l, jj]
        K = np.concatenate([a["k_il"][b], km]); V = np.concatenate([a["v_il"][b], vm])
        for hq in range(Hq):
            h = hq // G
            qv = a["q"][b, 0, hq * D:(hq + 1) * D]
            s = K[:, h * D:(h + 1) * D] @ qv / math.sqrt(D)
            p = np.exp(s - s.max()); p /= p.sum()
            np.testing.assert_allclose(out[b, hq, 0], p @ V[:, h * D:(h + 1) * D], atol=1e-12)


def test_attention_invariants():
    a = _attn_case(seed=8)
    out = fo.fourier_attn(**a)
    assert out.shape == (2, 6, 1, 8)
    # permuting the sink/local rows (with their values) changes nothing
    perm = np.array([3, 0, 4, 1, 2])
    b = dict(a); b["k_il"] = a["k_il"][:, perm]; b["v_il"] = a["v_il"][:, perm]
    np.testing.assert_allclose(fo.fourier_attn(**b), out, atol=1e-12)
    # identical query heads inside one GQA group give identical rows
    c = dict(a); q = a["q"].copy().reshape(2, 1, 6, 8); q[:, :, 1] = q[:, :, 0]; c["q"] = q.reshape(2, 1, 48)
    o = fo.fourier_attn(**c)
    np.testing.assert_allclose(o[:, 0], o[:, 1], atol=1e-12)
    # explicit sm_scale equal to the default reproduces the default
    d = dict(a); d["sm_scale"] = 1 / math.sqrt(8)
    np.testing.assert_allclose(fo.fourier_attn(**d), out, atol=1e-12)
    # assert on q_len != 1
    e = dict(a); e["q"] = np.concatenate([a["q"], a["q"]], axis=1)
    with pytest.raises(AssertionError):
        fo.fourier_attn(**e)


def test_attention_coefficient_domain_identity():
    """score and output of the compressed dims can be evaluated in the coefficient domain
    (what the GPU kernel does); this pins the algebra on one head."""
    r = rng(9)
    L, nf, T, C = 19, 4, 31, 5
    coefk = r.standard_normal((1, 2 * nf, C)); coefv = r.standard_normal((1, 2 * nf, C))
    au, ad, s = r.standard_normal((1, C)), r.standard_normal((1, C)), r.uniform(0.5, 2, (1, C))
    bu, bd, sv = r.standard_normal((1, C)), r.standard_normal((1, C)), r.uniform(0.5, 2, (1, C))
    q = r.standard_normal(C)
    kt = fo.denormalize(fo.reconstruct(coefk, L, T), ad, s, au)[0]
    vt = fo.denormalize(fo.reconstruct(coefv, L, T), bd, sv, bu)[0]
    score = kt @ q
    l = np.arange(L); n = np.arange(nf)
    ph = 2 * np.pi * np.outer(l, n) / T
    w_c = coefk[0, :nf] @ (q * s[0]); w_s = coefk[0, nf:] @ (q * s[0])
    score2 = (np.cos(ph) @ w_c + np.sin(ph) @ w_s) / nf + q @ (au[0] - ad[0] * s[0])
    np.testing.assert_allclose(score2, score, atol=1e-10)
    p = np.exp(score - score.max())
    g_c = p @ np.cos(ph); g_s = p @ np.sin(ph); P = p.sum()
    o2 = sv[0] * ((g_c @ coefv[0, :nf] + g_s @ coefv[0, nf:]) / nf - bd[0] * P) + bu[0] * P
    np.testing.assert_allclose(o2, p @ vt, atol=1e-10)


# ------------------------------------------------------------------- RoPE ---
def test_rope_is_a_rotation_and_relative():
    D = 8
    cos, sin = fo.rope_tables(np.arange(6), D, base=500000.0)
    x = rng(10).standard_normal((1, 1, 6, D))
    y = fo.apply_rope(x, cos, sin)
    np.testing.assert_allclose(np.linalg.norm(y, axis=-1), np.linalg.norm(x, axis=-1), atol=1e-12)
    np.testing.assert_allclose(y[0, 0, 0], x[0, 0, 0], atol=1e-12)  # position 0 is the identity
    # pair (i, i + D/2) rotates by pos * base^(-2i/D)
    i, pos = 1, 5
    ang = pos * 500000.0 ** (-2 * i / D)
    a, b = x[0, 0, pos, i], x[0, 0, pos, i + D // 2]
    assert abs(y[0, 0, pos, i] - (a * math.cos(ang) - b * math.sin(ang))) < 1e-12
    assert abs(y[0, 0, pos, i + D // 2] - (b * math.cos(ang) + a * math.sin(ang))) < 1e-12
    # q.k depends on the position difference only
    q = rng(11).standard_normal((1, 1, 1, D)); k = rng(12).standard_normal((1, 1, 1, D))
    def dot(pq, pk):
        cq, sq = fo.rope_tables(np.array([pq]), D); ck, sk = fo.rope_tables(np.array([pk]), D)
        return float((fo.apply_rope(q, cq, sq) * fo.apply_rope(k, ck, sk)).sum())
    assert abs(dot(7, 3) - dot(14, 10)) < 1e-9
