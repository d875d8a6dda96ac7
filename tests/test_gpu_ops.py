"""GPU parity of the operator-level entry points against the CPU oracle (through the C ABI)."""
import numpy as np
import pytest
import torch

from oracle import fourier_oracle as fo
from tests import helpers as H

pytestmark = pytest.mark.gpu


def rel_err(a, b):
    a = np.asarray(a, dtype=np.float64); b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,K,Mc,N,T,k0", [(2, 300, 70, 20, 411, 0), (1, 37, 5, 3, 37, 0), (3, 129, 260, 33, 100, 1000)])
def test_mat_fourier(dtype, B, K, Mc, N, T, k0):
    from fourierattention_amd import ops
    r = np.random.default_rng(1)
    x = H.to_dtype_np(r.standard_normal((B, K, Mc)), dtype)
    if k0:   # general phase offset: the sum of K rank-1 terms
        want = np.zeros((B, 2 * N, Mc))
        for k in range(K):
            want = fo.coeff_update(want, x[:, k], k + k0, T)
    else:
        want = fo.compress_prefill(x, N, T)
    got = ops.mat_fourier_triton(H.to_gpu(x, dtype), N, T, k0)
    assert got.dtype == torch.float32 and tuple(got.shape) == (B, 2 * N, Mc)
    assert rel_err(got.cpu().numpy(), want) <= 1e-5  # fp32 accumulation over K rows


def test_mat_fourier_gather_strided_accumulate():
    from fourierattention_amd import ops
    r = np.random.default_rng(2)
    B, S, HD, N, T = 2, 90, 48, 7, 77
    x = H.to_dtype_np(r.standard_normal((B, S, HD)), torch.bfloat16)
    cols = np.sort(r.choice(HD, 19, replace=False))
    xg = H.to_gpu(x, torch.bfloat16)
    view = xg[:, 4:S - 16, :]                         # strided view: rows 4..73 like the sink/window split
    got = ops.mat_fourier(view, N, T, 0, cols=torch.from_numpy(cols).int().cuda())
    want = fo.compress_prefill(x[:, 4:S - 16][:, :, cols], N, T)
    assert rel_err(got.cpu().numpy(), want) <= 1e-5
    base = got.clone()
    ops.mat_fourier(view[:, :1], N, T, 123, cols=torch.from_numpy(cols).int().cuda(), out=got, accumulate=True)
    want2 = fo.coeff_update(want, x[:, 4][:, cols], 123, T)
    assert rel_err(got.cpu().numpy(), want2) <= 1e-5
    assert not torch.equal(base, got)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_stats_original(dtype):
    from fourierattention_amd import ops
    r = np.random.default_rng(3)
    x = H.to_dtype_np(r.standard_normal((2, 777, 45)) * 2 + 0.3, dtype)
    avg, dev = ops.mat_avg_std_triton(H.to_gpu(x, dtype))
    assert avg.dtype == dtype and dev.dtype == dtype and tuple(avg.shape) == (2, 45)
    wa, wd = fo.stats_original(x, H.NP_ROUND[dtype])
    tol = {torch.float32: 2e-6, torch.bfloat16: 8e-3, torch.float16: 1e-3}[dtype]   # one ulp of the output dtype
    np.testing.assert_allclose(avg.float().cpu().numpy(), wa, atol=tol, rtol=tol)
    np.testing.assert_allclose(dev.float().cpu().numpy(), wd, atol=tol, rtol=tol)


def test_stats_reconstructed_and_reconstruction():
    from fourierattention_amd import ops
    r = np.random.default_rng(4)
    B, L, C, N, T = 2, 700, 37, 24, 733
    x = r.standard_normal((B, L, C))
    coef = fo.compress_prefill(x, N, T).astype(np.float32)
    cg = torch.from_numpy(coef).cuda()
    rec = ops.mat_fourier_inv(cg, L, T)
    want = fo.reconstruct(coef, L, T)
    assert rel_err(rec.cpu().numpy(), want) <= 1e-3        # stated tolerance for reconstructed K/V (fp32)
    assert rel_err(rec.cpu().numpy(), want) <= 1e-5        # what fp32 accumulation actually gives
    avg, dev = ops.mat_fourier_avg_std_triton(cg, L, T)
    assert avg.dtype == torch.float16 and dev.dtype == torch.float16
    wa, wd = fo.stats_reconstructed(coef, L, T)
    np.testing.assert_allclose(avg.float().cpu().numpy(), wa, atol=1e-3, rtol=1e-3)   # one fp16 ulp
    np.testing.assert_allclose(dev.float().cpu().numpy(), wd, atol=1e-3, rtol=1e-3)
    # affine form
    au, ad, sc = r.standard_normal((B, C)), r.standard_normal((B, C)), r.uniform(0.5, 2, (B, C))
    rec2 = ops.mat_fourier_inv(cg, L, T, torch.from_numpy(au).cuda(), torch.from_numpy(ad).cuda(), torch.from_numpy(sc).cuda())
    assert rel_err(rec2.cpu().numpy(), fo.denormalize(want, ad.astype(np.float32), sc.astype(np.float32), au.astype(np.float32))) <= 1e-5


def test_hippo_module_contract():
    from fourierattention_amd import ops
    r = np.random.default_rng(5)
    B, L, C, M = 2, 140, 11, 16
    T_x, dt, T_c = fo.periods(93 + 4 + 6, 4, 6)         # a period where int(1/dt) == T_x - 1
    assert (T_x, T_c) == (93, 92)
    hip = ops.MultiDimHiPPO2(N=C * M, input_dim=C, method="legt", dt=dt, T=1)
    x = H.to_dtype_np(r.standard_normal((B, L, C)), torch.bfloat16)
    got = hip(base_input=H.to_gpu(x, torch.bfloat16), token_num=0)
    want = fo.compress_prefill(x, M // 2, T_c)            # L > T_c: the tail is dropped
    assert tuple(got.shape) == (B, M, C) and rel_err(got.cpu().numpy(), want) <= 1e-5
    row = H.to_dtype_np(r.standard_normal((B, 1, C)), torch.bfloat16)
    got2 = hip(got, token_num=L + 1, slice_input=H.to_gpu(row, torch.bfloat16))
    assert rel_err(got2.cpu().numpy(), fo.coeff_update(want, row[:, 0], L + 1, T_c)) <= 1e-5
    assert rel_err(got.cpu().numpy(), want) <= 1e-5       # base_input untouched


CASES = [
    # B, Hq, Hkv, D, n_il, L, n_f, T, k_counts, v_counts
    (2, 8, 2, 64, 37, 300, 16, 411, [32, 20], [40, 64]),
    (1, 6, 2, 128, 5, 700, 24, 733, [0, 128], [128, 1]),          # heads with nothing / everything compressed
    (3, 4, 4, 32, 260, 513, 8, 600, [7, 9, 11, 13], [1, 2, 3, 4]),  # MHA, window longer than one tile
    (2, 24, 8, 128, 20, 130, 40, 1000, [64] * 8, [64] * 8),        # 3:1 grouping
    (2, 4, 2, 64, 9, 150, 3, 200, [10, 50], [33, 64]),             # odd numbers of frequencies: coefficient
    (1, 6, 2, 32, 70, 90, 5, 97, [31, 2], [5, 32]),                # rows that are no multiple of 16 bytes
    (1, 2, 1, 32, 3, 40, 1, 64, [16], [16]),
]


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-4), (torch.bfloat16, 2e-2), (torch.float16, 2e-2)])
@pytest.mark.parametrize("case_id", range(len(CASES)))
def test_decode_attention_matches_oracle(case_id, dtype, tol):
    """max-abs error of the attention output vs the float64 oracle on identical (already rounded)
    operands: <= 2e-2 for 16-bit storage (the stated bound), <= 2e-4 for fp32 storage."""
    from fourierattention_amd import ops
    B, Hq, Hkv, D, n_il, L, n_f, T, kcnt, vcnt = CASES[case_id]
    case = H.attn_case(100 + case_id, B, Hq, Hkv, D, n_il, L, n_f, T, kcnt, vcnt, dtype)
    want = fo.fourier_attn(**case)
    g = H.attn_case_gpu(case, dtype)
    got = ops.triton_fourier_attn(**g)
    assert got.dtype == torch.float32 and tuple(got.shape) == (B, Hq, 1, D)
    err = np.abs(got.cpu().numpy() - want).max()
    assert np.isfinite(got.cpu().numpy()).all()
    assert err <= tol, err
    # the kernels compute in fp32 whatever the storage type: the real error is far below the bound
    assert err <= 5e-4, err


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_function_level_drop_in_repages_long_token_major_inputs(dtype, monkeypatch):
    """``triton_fourier_attn`` with the reference's token-major ``k_mn`` / ``v_mn`` and a long mid: the rows are
    copied into a temporary page store and the matrix-core kernels run; the result must agree with the oracle
    and with the kernels that read the token-major tensors in place."""
    from fourierattention_amd import ops
    B, Hq, Hkv, D, n_il, L, n_f, T = 2, 8, 2, 128, 40, 2500, 128, 2700
    case = H.attn_case(321, B, Hq, Hkv, D, n_il, L, n_f, T, [64, 100], [30, 64], dtype)
    want = fo.fourier_attn(**case)
    g = H.attn_case_gpu(case, dtype)
    got = ops.triton_fourier_attn(**g).cpu().numpy()
    monkeypatch.setattr(ops, "_REPACK_MIN_ROWS", 1 << 30)
    in_place = ops.triton_fourier_attn(**g).cpu().numpy()
    assert np.abs(in_place - want).max() <= 5e-4
    err = np.abs(got - want).max()
    assert err <= 2e-2, err          # the stated bound for 16-bit storage
    assert err <= 5e-3, err          # f16 basis and 16-bit probabilities on the matrix cores
    assert np.abs(got - in_place).max() > 0     # it did take the other kernels


def test_decode_attention_window_only_and_errors():
    from fourierattention_amd import ops, _lib
    case = H.attn_case(7, 2, 8, 2, 64, 300, 0, 4, 50, [10, 10], [10, 10], torch.bfloat16)
    g = H.attn_case_gpu(case, torch.bfloat16)
    want = fo.softmax_attention(case["q"][:, 0], case["k_il"], case["v_il"], 8, 2)
    got = ops.triton_fourier_attn(**g)
    assert np.abs(got.cpu().numpy()[:, :, 0] - want).max() <= 5e-4
    bad = dict(g); bad["q"] = torch.cat([g["q"], g["q"]], dim=1)
    with pytest.raises(AssertionError):
        ops.triton_fourier_attn(**bad)
    with pytest.raises(_lib.FourierAttnError) as ei:
        ops.decode_attn_raw(bad["q"].contiguous(), [(g["k_il"], g["v_il"])], None, None, None, None, None, None,
                            tuple(ops.as_i32(g[k]) for k in ("kc_list", "kc_h_list", "kn_list", "kn_h_list", "vc_list", "vc_h_list", "vn_list", "vn_h_list")),
                            8, 2, 0, 1)
    assert ei.value.code == -2


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("B,K,Mc,N,T,k0,gather", [
    (2, 1500, 96, 40, 1501, 0, True),       # ragged everything: last step partly empty, 5 row tiles, 6 column tiles
    (1, 4096, 512, 128, 4096, 0, True),     # whole tiles, several chunks
    (1, 700, 30, 8, 9000, 12345, False),    # phase offset, fewer columns than one workgroup tile
    (2, 1100, 819, 16, 1100, 0, True),      # an odd number of columns (what a searched mask gives), last tile ragged
    (1, 600, 33, 24, 777, 5, False),        # odd again, rows of the result not 16-byte aligned
])
def test_mat_fourier_matrix_cores(dtype, B, K, Mc, N, T, k0, gather):
    """Long 16-bit inputs take the matrix-core kernels (basis in fp16, fp32 accumulation): checked against the
    oracle and against the fp32 vector kernel on the same input.  Bound: the fp16 basis carries a relative
    rounding error of at most 2^-11 per entry, about 1.5e-4 rms, which is what the result inherits."""
    from fourierattention_amd import ops
    r = np.random.default_rng(5)
    width = Mc + 37 if gather else Mc
    x = H.to_dtype_np(r.standard_normal((B, K, width)), dtype)
    cols = np.sort(r.choice(width, Mc, replace=False)) if gather else None
    xs = x[:, :, cols] if gather else x
    xg = H.to_gpu(x, dtype)
    cg = torch.from_numpy(cols).int().cuda() if gather else None
    from fourierattention_amd import _lib
    assert _lib.load().fa_mat_fourier_workspace_bytes(ops.dtype_code(dtype), B, K, Mc, N) > 0   # the shape is for the matrix cores
    got = ops.mat_fourier(xg, N, T, k0, cols=cg)
    ref = ops.mat_fourier(xg, N, T, k0, cols=cg, matrix_cores=False)
    assert rel_err(got.cpu().numpy(), ref.cpu().numpy()) <= 5e-4
    if k0 == 0:
        want = fo.compress_prefill(xs, N, T)
        assert rel_err(got.cpu().numpy(), want) <= 5e-4
    # accumulate adds onto what is there
    got2 = got.clone()
    ops.mat_fourier(xg, N, T, k0, cols=cg, out=got2, accumulate=True)
    assert rel_err(got2.cpu().numpy(), 2 * got.cpu().numpy()) <= 1e-6


@pytest.mark.parametrize("B,L,C,N,T", [
    (2, 1500, 70, 40, 1533),     # most positions beyond T / 2 are taken as mirror images, odd period
    (1, 4100, 128, 128, 4100),   # a whole even period: position T / 2 is its own image, position 0 has none
    (1, 1100, 16, 200, 5000),    # nothing beyond T / 2
    (1, 1202, 16, 64, 1201),     # one position more than the period: position T is the image of position 0
    (1, 1300, 16, 64, 1201),     # longer than the period: every position is computed directly
    (2, 1400, 819, 32, 1500),    # an odd number of columns
])
def test_stats_reconstructed_matrix_cores(B, L, C, N, T):
    """Long reconstructions take the matrix-core kernel (fp16 basis and per-column scaled fp16 coefficients, fp32
    accumulation): statistics against the oracle and against the fp32 vector kernel.  Bound: each operand carries
    up to 2^-11 relative rounding, the results are rounded through fp16 (2^-11 again)."""
    from fourierattention_amd import ops
    r = np.random.default_rng(6)
    x = r.standard_normal((B, L, C)) * r.uniform(0.2, 30.0, (1, 1, C)) + r.uniform(-3, 3, (1, 1, C))   # mixed column ranges
    coef = fo.compress_prefill(x, N, T).astype(np.float32)
    cg = torch.from_numpy(coef).cuda()
    avg, dev = ops.mat_fourier_avg_std(cg, L, T, torch.float16)
    avg0, dev0 = ops.mat_fourier_avg_std(cg, L, T, torch.float16, matrix_cores=False)
    wa, wd = fo.stats_reconstructed(coef, L, T)
    scale = np.abs(wd).max(axis=None)
    for got, ref, want in ((avg, avg0, wa), (dev, dev0, wd)):
        g = got.cpu().numpy()
        # relative to the size of the reconstructed signal of the column (its deviation), not of the value itself
        assert np.max(np.abs(g - want) / (np.abs(wd) + np.abs(wa))) <= 2e-3
        assert np.max(np.abs(g - ref.cpu().numpy()) / (np.abs(wd) + np.abs(wa))) <= 2e-3
