"""Shared builders for parity tests (numpy side is the oracle's input, torch side the HIP path's)."""
import numpy as np
import torch

from oracle import fourier_oracle as fo

NP_ROUND = {torch.float32: "fp32", torch.bfloat16: "bf16", torch.float16: "fp16"}


def to_dtype_np(x: np.ndarray, dtype: torch.dtype) -> np.ndarray:
    """Round a float array to `dtype` and return float64 (what the oracle consumes)."""
    return fo.round_to(x, NP_ROUND[dtype]).astype(np.float64)


def to_gpu(x: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dtype).cuda()


def ragged_mask(rng, num_kv_heads, head_dim, counts):
    """Sorted flat compressed dims with the given per-head counts, plus complement and the
    cumulative lists with the leading 0."""
    c = []
    for h, n in enumerate(counts):
        c += sorted((h * head_dim + rng.choice(head_dim, n, replace=False)).tolist())
    c = np.array(c, dtype=np.int64)
    n = np.setdiff1d(np.arange(num_kv_heads * head_dim), c)
    ch = np.array([0] + [int((c < (h + 1) * head_dim).sum()) for h in range(num_kv_heads)], dtype=np.int64)
    nh = np.array([0] + [int((n < (h + 1) * head_dim).sum()) for h in range(num_kv_heads)], dtype=np.int64)
    return c, ch, n, nh


def attn_case(seed, B, Hq, Hkv, D, n_il, L, n_f, T, k_counts, v_counts, dtype):
    """Random decode-attention operands, rounded to `dtype` where the reference stores that dtype."""
    r = np.random.default_rng(seed)
    hid = Hkv * D
    kc, kch, kn, knh = ragged_mask(r, Hkv, D, k_counts)
    vc, vch, vn, vnh = ragged_mask(r, Hkv, D, v_counts)
    rd = lambda a: to_dtype_np(a, dtype)
    case = dict(
        q=rd(r.standard_normal((B, 1, Hq * D))), k_il=rd(r.standard_normal((B, n_il, hid))), v_il=rd(r.standard_normal((B, n_il, hid))),
        k_mc=r.standard_normal((B, 2 * n_f, kc.size)).astype(np.float32).astype(np.float64) * 3.0,
        v_mc=r.standard_normal((B, 2 * n_f, vc.size)).astype(np.float32).astype(np.float64) * 3.0,
        k_mn=rd(r.standard_normal((B, L, kn.size))), v_mn=rd(r.standard_normal((B, L, vn.size))),
        avg_k_u=rd(r.standard_normal((B, kc.size))), avg_k_d=fo.round_fp16(r.standard_normal((B, kc.size))).astype(np.float64),
        scale_k=r.uniform(0.1, 1.5, (B, kc.size)).astype(np.float32).astype(np.float64),
        avg_v_u=rd(r.standard_normal((B, vc.size))), avg_v_d=fo.round_fp16(r.standard_normal((B, vc.size))).astype(np.float64),
        scale_v=r.uniform(0.1, 1.5, (B, vc.size)).astype(np.float32).astype(np.float64),
        kc_list=kc, kc_h_list=kch, kn_list=kn, kn_h_list=knh, vc_list=vc, vc_h_list=vch, vn_list=vn, vn_h_list=vnh,
        num_head_q=Hq, num_head_kv=Hkv, seq_len_m=L, T=T)
    return case


def attn_case_gpu(case, dtype):
    g = {}
    for k in ("q", "k_il", "v_il", "k_mn", "v_mn"):
        g[k] = to_gpu(case[k], dtype)
    for k in ("k_mc", "v_mc", "scale_k", "scale_v"):
        g[k] = to_gpu(case[k], torch.float32)
    for k in ("avg_k_u", "avg_v_u"):
        g[k] = to_gpu(case[k], dtype)
    for k in ("avg_k_d", "avg_v_d"):
        g[k] = to_gpu(case[k], torch.float16)
    for k in ("kc_list", "kc_h_list", "kn_list", "kn_h_list", "vc_list", "vc_h_list", "vn_list", "vn_h_list"):
        g[k] = torch.from_numpy(case[k]).cuda()
    for k in ("num_head_q", "num_head_kv", "seq_len_m", "T"):
        g[k] = case[k]
    return g
