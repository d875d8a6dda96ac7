"""CPU restatement of the reference's Fourier KV-cache arithmetic.

TEST INFRASTRUCTURE ONLY - see ``oracle/__init__.py``.

Everything here is numpy; accumulation is float64 unless ``dtype`` says
otherwise.  Each function cites the reference lines it follows (paths are
relative to the reference repository root, ``TRI`` =
``fourier_attn_triton/fourier_triton_valid4_v2.py``).

Pinning status (what independently checks each function, see
``tests/test_oracle_pins.py``):

* ``compress_prefill``    - equals ``numpy.fft.fft(x, n=T)[:N_f]`` (real, -imag)
  including zero-padding and truncation; brute-force triple loop on tiny shapes.
* ``coeff_update``        - difference of two batch transforms; additivity.
* ``stats_original`` / ``stats_reconstructed`` - explicit array mean/min/max.
* ``reconstruct``         - brute force; Dirichlet-kernel identity when
  ``T_c == T_x``; exact inverse for band-limited signals.
* ``fourier_attn``        - textbook softmax attention on explicitly assembled
  K/V; permutation / GQA-duplication invariants; coefficient-domain identity.
* bit-level behaviour of the reference's Triton/cuFFT/flash-attn kernels
  (tl.cos on unreduced fp32 phases, TF32 dots, fp16 flash-attn) - PARITY
  UNPINNED: not reproducible without a CUDA box; covered by the stated
  tolerances, not by bit-exactness.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence, Tuple

import numpy as np

TWO_PI = 2.0 * math.pi


# ----------------------------------------------------------------------------
# dtype emulation (numpy has no bfloat16)
# ----------------------------------------------------------------------------
def round_bf16(x: np.ndarray) -> np.ndarray:
    """Round float values to the nearest bfloat16 (ties to even); returns float32."""
    a = np.ascontiguousarray(x, dtype=np.float32)
    u = a.view(np.uint32).astype(np.uint64)
    rounding = ((u >> 16) & 1) + 0x7FFF
    r = ((u + rounding) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32).reshape(a.shape)
    nan = np.isnan(a)
    if nan.any():
        out = np.where(nan, a, out)
    return out


def round_fp16(x: np.ndarray) -> np.ndarray:
    with np.errstate(over="ignore"):
        return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def round_to(x: np.ndarray, dtype_name: str) -> np.ndarray:
    """Emulate a torch ``.to(dtype)`` cast; ``dtype_name`` in {'fp32','fp16','bf16','fp64'}."""
    if dtype_name == "bf16":
        return round_bf16(x)
    if dtype_name == "fp16":
        return round_fp16(x)
    if dtype_name == "fp32":
        return np.asarray(x, dtype=np.float32)
    if dtype_name == "fp64":
        return np.asarray(x, dtype=np.float64)
    raise ValueError(dtype_name)


# ----------------------------------------------------------------------------
# periods  (cache_utils_fourier.py:547, 566; TRI:856, 859)
# ----------------------------------------------------------------------------
def periods(maxtokens: int, numinit: int, maxlocal: int) -> Tuple[int, float, int]:
    """Return ``(T_x, dt, T_c)``.

    ``T_x = maxtokens - numinit - maxlocal`` is the exact period used by the
    reconstruction statistics and decode attention
    (cache_utils_fourier.py:566, modeling_llama_fourier.py:660).  ``dt = 1/T_x``
    is a Python float (cache_utils_fourier.py:547) and ``T_c = int(1/dt)``
    (TRI:856, 859) is the period of the prefill transform and of the rank-1
    update; ``T_c`` is ``T_x`` or ``T_x - 1``.
    """
    t_x = int(maxtokens) - int(numinit) - int(maxlocal)
    dt = 1 / t_x
    t_c = int(1 / dt)
    return t_x, dt, t_c


def _phase_matrix(rows: np.ndarray, cols: np.ndarray, period: int) -> np.ndarray:
    """``2*pi*((rows x cols) mod period)/period`` with exact integer reduction."""
    prod = np.multiply.outer(rows.astype(np.int64), cols.astype(np.int64)) % int(period)
    return prod.astype(np.float64) * (TWO_PI / float(period))


_BASIS_CACHE: dict = {}


def _basis(rows: int, n_f: int, period: int) -> np.ndarray:
    """``(rows, 2 n_f)`` float64: ``cos(2 pi l n / period)`` for ``n < n_f`` then the ``sin`` columns, row ``l``
    a position, phases reduced exactly in integers.  Rows do not depend on each other, so the largest table built
    for an ``(n_f, period)`` pair is kept (two pairs at most) and shorter requests are slices of it: building the
    table, not the contraction, dominates the cost of long sequences."""
    key = (int(n_f), int(period))
    have = _BASIS_CACHE.get(key)
    if have is None or have.shape[0] < rows:
        if have is None and len(_BASIS_CACHE) >= 2:
            _BASIS_CACHE.pop(next(iter(_BASIS_CACHE)))
        build = int(rows) if rows < 4096 else int(rows) + 64      # room for a few streaming steps
        have = np.empty((build, 2 * n_f), dtype=np.float64)
        cols = np.arange(n_f)
        for r0 in range(0, build, 8192):
            ph = _phase_matrix(np.arange(r0, min(build, r0 + 8192)), cols, period)
            np.cos(ph, out=have[r0: r0 + ph.shape[0], :n_f])
            np.sin(ph, out=have[r0: r0 + ph.shape[0], n_f:])
        _BASIS_CACHE[key] = have
    return have[:rows]


# ----------------------------------------------------------------------------
# compression  (TRI:840-865 FFT branch == TRI:21-102 with K_start = 0)
# ----------------------------------------------------------------------------
def compress_prefill(x: np.ndarray, n_f: int, t_c: int, dtype=np.float64) -> np.ndarray:
    """Project ``x (B, L, C)`` onto ``n_f`` cos rows then ``n_f`` sin rows.

    ``out[b, n, j]       = sum_{t < min(L, t_c)} x[b, t, j] * cos(2 pi n t / t_c)``
    ``out[b, n_f + n, j] = sum_{t < min(L, t_c)} x[b, t, j] * sin(2 pi n t / t_c)``

    The reference computes this as ``fft(x, n=t_c, dim=1)[:, :n_f]`` keeping
    ``real`` and ``-imag`` (TRI:858-865): the FFT zero-pads when ``L < t_c`` and
    drops the tail when ``L > t_c``.  Result is float32 in the reference.
    """
    x = np.asarray(x, dtype=dtype)
    b, l, c = x.shape
    l_eff = min(l, int(t_c))
    basis = _basis(l_eff, n_f, t_c).astype(dtype, copy=False)  # (l_eff, 2 n_f): the phase n*t is symmetric in n and t
    return np.ascontiguousarray(np.einsum("tn,btc->bnc", basis, x[:, :l_eff, :], optimize=True))


def coeff_update(coef: np.ndarray, evicted: np.ndarray, p: int, t_c: int, dtype=np.float64) -> np.ndarray:
    """Rank-1 coefficient update for one evicted token (TRI:853-856, TRI:21-78 with K = 1).

    ``coef (B, 2 n_f, C)``, ``evicted (B, C)``; the token enters at phase ``p``
    (``K_start = token_num``): ``coef[b, n] += cos(2 pi p n / t_c) * evicted[b]``,
    sin rows likewise.  Returns a new array.
    """
    coef = np.asarray(coef, dtype=dtype)
    n_f = coef.shape[1] // 2
    ph = _phase_matrix(np.arange(n_f), np.array([p]), t_c)[:, 0]
    basis = np.concatenate([np.cos(ph), np.sin(ph)]).astype(dtype)  # (2 n_f,)
    return coef + basis[None, :, None] * np.asarray(evicted, dtype=dtype)[:, None, :]


# ----------------------------------------------------------------------------
# statistics  (TRI:332-461 and TRI:189-326; used at cache_utils_fourier.py:564-569)
# ----------------------------------------------------------------------------
def mean_max_dev(a: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """Per (b, column): mean over axis 1 and ``max(max - mean, mean - min)`` (TRI:417-420)."""
    a = np.asarray(a, dtype=np.float64)
    avg = a.sum(axis=1) / a.shape[1]
    dev = np.maximum(a.max(axis=1) - avg, avg - a.min(axis=1))
    return avg, dev


def stats_original(x: np.ndarray, out_dtype: str = "fp32") -> Tuple[np.ndarray, np.ndarray]:
    """``mat_avg_std_triton`` (TRI:433-461): fp32 accumulate, cast to the input dtype."""
    avg, dev = mean_max_dev(x)
    return round_to(avg, out_dtype), round_to(dev, out_dtype)


def reconstruct(coef: np.ndarray, k: int, t_x: int, dtype=np.float64) -> np.ndarray:
    """``mat_fourier_inv_torch`` (TRI:782-791) / kernel reconstruction (TRI:600-622).

    ``r[b, l, j] = (1/n_f) * sum_n cos(2 pi n l / t_x) coef[b, n, j]
                             + sin(2 pi n l / t_x) coef[b, n_f + n, j]`` for ``l < k``.
    """
    coef = np.asarray(coef, dtype=dtype)
    n_f = coef.shape[1] // 2
    basis = _basis(int(k), n_f, t_x).astype(dtype, copy=False)  # (k, 2 n_f)
    return np.ascontiguousarray(np.einsum("ln,bnc->blc", basis, coef, optimize=True)) / n_f


def stats_reconstructed(coef: np.ndarray, k: int, t_x: int) -> Tuple[np.ndarray, np.ndarray]:
    """``mat_fourier_avg_std_triton`` (TRI:285-326): stats of the reconstruction, cast to fp16."""
    if k == 0:
        raise ValueError("statistics of an empty reconstruction are undefined")
    avg, dev = mean_max_dev(reconstruct(coef, k, t_x))
    return round_fp16(avg), round_fp16(dev)


def prefill_stats(x: np.ndarray, coef: np.ndarray, t_x: int, model_dtype: str = "bf16"):
    """The three per-(b, dim) vectors the cache stores (cache_utils_fourier.py:564-569).

    Returns ``(scale, avg_u, avg_d)`` = ``(u_std / i_std, u_avg, i_avg)`` with the
    reference's dtypes: ``u_*`` in the model dtype (TRI:461), ``i_*`` in fp16
    (TRI:326); the quotient follows torch promotion (fp16/fp16 -> fp16,
    bf16/fp16 -> fp32, fp32/fp16 -> fp32).
    """
    u_avg, u_std = stats_original(x, model_dtype)
    i_avg, i_std = stats_reconstructed(coef, x.shape[1], t_x)
    with np.errstate(divide="ignore", invalid="ignore"):
        if model_dtype == "fp16":
            scale = round_fp16(u_std.astype(np.float32) / i_std.astype(np.float32))
        else:
            scale = (u_std.astype(np.float32) / i_std.astype(np.float32)).astype(np.float32)
    return scale, u_avg, i_avg


def denormalize(r: np.ndarray, avg_d: np.ndarray, scale: np.ndarray, avg_u: np.ndarray) -> np.ndarray:
    """Affine re-normalisation of a reconstruction (TRI:622, 651, 813, 815)."""
    f = np.float64
    return (r - np.asarray(avg_d, f)[:, None, :]) * np.asarray(scale, f)[:, None, :] + np.asarray(avg_u, f)[:, None, :]


# ----------------------------------------------------------------------------
# decode attention  (TRI:794-837 formulation; kernel TRI:464-779)
# ----------------------------------------------------------------------------
def assemble_mid(coef, mid_n, avg_u, avg_d, scale, c_list, n_list, seq_len_m, t_x, hidden):
    """Full-width mid rows ``(B, seq_len_m, hidden)``: reconstructed dims at ``c_list``
    and stored dims at ``n_list`` (TRI:812-822)."""
    b = coef.shape[0] if coef is not None and coef.size else mid_n.shape[0]
    out = np.zeros((b, seq_len_m, hidden), dtype=np.float64)
    c_list = np.asarray(c_list, dtype=np.int64)
    n_list = np.asarray(n_list, dtype=np.int64)
    if c_list.size:
        r = reconstruct(coef, seq_len_m, t_x)
        out[:, :, c_list] = denormalize(r, avg_d, scale, avg_u)
    if n_list.size:
        out[:, :, n_list] = np.asarray(mid_n, dtype=np.float64)[:, :seq_len_m, :]
    return out


def softmax_attention(q, k, v, num_head_q, num_head_kv, sm_scale=None):
    """Exact one-query attention.  ``q (B, Hq*D)``, ``k, v (B, S, Hkv*D)`` -> ``(B, Hq, D)``.

    GQA: query head ``hq`` reads KV head ``hq // (Hq/Hkv)`` (TRI:504).
    """
    q = np.asarray(q, dtype=np.float64)
    k = np.asarray(k, dtype=np.float64)
    v = np.asarray(v, dtype=np.float64)
    b, s, _ = k.shape
    d = q.shape[-1] // num_head_q
    g = num_head_q // num_head_kv
    if sm_scale is None:
        sm_scale = 1.0 / math.sqrt(d)
    qh = q.reshape(b, num_head_kv, g, d)
    kh = k.reshape(b, s, num_head_kv, d)
    vh = v.reshape(b, s, num_head_kv, d)
    scores = np.einsum("bhgd,bshd->bhgs", qh, kh, optimize=True) * sm_scale
    scores -= scores.max(axis=-1, keepdims=True)
    p = np.exp(scores)
    p /= p.sum(axis=-1, keepdims=True)
    o = np.einsum("bhgs,bshd->bhgd", p, vh, optimize=True)
    return o.reshape(b, num_head_q, d)


def fourier_attn(q, k_il, v_il, k_mc, v_mc, k_mn, v_mn,
                 avg_k_u, avg_k_d, scale_k, avg_v_u, avg_v_d, scale_v,
                 kc_list, kc_h_list, kn_list, kn_h_list,
                 vc_list, vc_h_list, vn_list, vn_h_list,
                 num_head_q, num_head_kv, seq_len_m, T, sm_scale=-1):
    """Same signature as ``torch_fourier_attn`` / ``triton_fourier_attn`` (TRI:684-688, 794-798).

    ``q (B, 1, Hq*D)``; keys are ``[k_il ; reconstructed+stored mid rows]`` and the
    single query sees all of them.  Returns ``(B, Hq, 1, D)`` float64.  The
    ``*_h_list`` arguments are accepted for signature parity; the flat index
    lists already determine the assembly (TRI:817-822).
    """
    q = np.asarray(q)
    assert q.ndim == 3 and q.shape[1] == 1, f"q.shape = {q.shape}"  # TRI:692
    b, _, feat = q.shape
    d = feat // num_head_q
    hidden = num_head_kv * d
    scale = None if sm_scale == -1 else sm_scale
    k_m = assemble_mid(k_mc, k_mn, avg_k_u, avg_k_d, scale_k, kc_list, kn_list, seq_len_m, T, hidden)
    v_m = assemble_mid(v_mc, v_mn, avg_v_u, avg_v_d, scale_v, vc_list, vn_list, seq_len_m, T, hidden)
    k_all = np.concatenate([np.asarray(k_il, dtype=np.float64), k_m], axis=1)
    v_all = np.concatenate([np.asarray(v_il, dtype=np.float64), v_m], axis=1)
    o = softmax_attention(q[:, 0, :], k_all, v_all, num_head_q, num_head_kv, scale)
    return o[:, :, None, :]


# ----------------------------------------------------------------------------
# synthetic-input helpers shared by tests (RoPE: modeling_llama_fourier.py:213-244)
# ----------------------------------------------------------------------------
def rope_tables(positions: np.ndarray, head_dim: int, base: float = 500000.0):
    """Plain RoPE tables ``cos, sin (S, D)`` with ``inv_freq = base^(-2i/D)``; HF layout
    (each frequency appears at ``i`` and ``i + D/2``)."""
    inv = base ** (-np.arange(0, head_dim, 2, dtype=np.float64) / head_dim)
    ang = np.multiply.outer(np.asarray(positions, dtype=np.float64), inv)
    emb = np.concatenate([ang, ang], axis=-1)
    return np.cos(emb), np.sin(emb)


def apply_rope(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """``x (B, H, S, D)``; ``x*cos + rotate_half(x)*sin`` with ``rotate_half = cat(-x2, x1)``."""
    half = x.shape[-1] // 2
    rot = np.concatenate([-x[..., half:], x[..., :half]], axis=-1)
    return x * cos[None, None] + rot * sin[None, None]
