"""Operator-level mirror of the reference's kernel entry points, backed by the HIP library.

Same names, argument meaning and error behaviour as
``fourier_attn_triton/fourier_triton_valid4_v2.py``:

* ``mat_fourier_triton``            (lines 81-102)
* ``mat_avg_std_triton``            (lines 433-461)
* ``mat_fourier_avg_std_triton``    (lines 285-326)
* ``triton_fourier_attn``           (lines 684-779)  - also exported as ``fourier_attn``
* ``mat_fourier_inv_torch``         (lines 782-791)  - as ``mat_fourier_inv``
* ``MultiDimHiPPO2``                (lines 840-865)

The names keep the reference's ``_triton`` suffix so call sites need no edit; nothing
here uses Triton.  Tensors must live on the GPU; PyTorch only provides the memory and
the current stream.
"""
from __future__ import annotations

import ctypes
from typing import Dict, Optional, Tuple

import torch

from . import _lib
from ._lib import FA_BF16, FA_FP16, FA_FP32, DecodeArgs, check

_DTYPE_CODE = {torch.bfloat16: FA_BF16, torch.float16: FA_FP16, torch.float32: FA_FP32}


def dtype_code(dt: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dt]
    except KeyError:
        raise TypeError(f"unsupported dtype {dt}; expected bfloat16, float16 or float32") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(device) -> int:
    """Handle of the stream the caller's tensor work is queued on (torch's current stream of ``device``).  Looked up
    on every call: the caller may switch streams, or capture into a graph, between two operators."""
    if _raw_stream is not None:     # the bare handle, without building a torch.cuda.Stream object around it
        idx = device.index
        return _raw_stream(torch.cuda.current_device() if idx is None else idx)
    return torch.cuda.current_stream(device).cuda_stream


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor: the HIP kernels are the only implementation")


_workspaces: Dict[Tuple[int, str], torch.Tensor] = {}


def workspace(device: torch.device, nbytes: int, tag: str = "default") -> torch.Tensor:
    """A per-device scratch buffer that only grows.  Work that shares a tag must be issued on
    one stream (kernels of consecutive calls then run in order and may reuse it)."""
    key = (device.index if device.index is not None else torch.cuda.current_device(), tag)
    buf = _workspaces.get(key)
    if buf is None or buf.numel() < nbytes:
        buf = torch.empty(max(int(nbytes), 256), dtype=torch.uint8, device=device)
        _workspaces[key] = buf
    return buf


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None or t.numel() == 0 else t.data_ptr()


def as_i32(t: torch.Tensor) -> torch.Tensor:
    return t if t.dtype == torch.int32 else t.to(torch.int32)


# --------------------------------------------------------------------------- K1
def mat_fourier(a: torch.Tensor, N: int, T: int, K_start: int = 0, cols: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None, accumulate: bool = False, K: Optional[int] = None,
                matrix_cores: bool = True) -> torch.Tensor:
    """``c[b, n, m] (+)= sum_k cos(2 pi (k + K_start) n / T) a[b, k, cols[m]]`` and the sin rows.

    ``a (B, K, width)`` may be a strided view as long as its last dim is contiguous; ``cols``
    (int32, GPU) selects columns; ``K`` limits the rows read.  Long 16-bit inputs run on the matrix
    cores (fp16 basis, fp32 accumulation) unless ``matrix_cores`` is false."""
    _require_gpu(a, "a")
    assert a.dim() == 3 and a.stride(2) == 1, "a must be (B, K, M) with a contiguous last dim"
    B, rows, width = a.shape
    K = rows if K is None else min(int(K), rows)
    Mc = width if cols is None else cols.numel()
    if out is None:
        assert not accumulate
        out = torch.empty((B, 2 * N, Mc), device=a.device, dtype=torch.float32)
    assert out.is_contiguous() and out.dtype == torch.float32 and tuple(out.shape) == (B, 2 * N, Mc)
    if Mc == 0 or B == 0:
        return out
    lib = _lib.load()
    ws_bytes = int(lib.fa_mat_fourier_workspace_bytes(dtype_code(a.dtype), B, K, Mc, N)) if matrix_cores else 0
    ws = workspace(a.device, ws_bytes, "spectral") if ws_bytes else None
    check(lib.fa_mat_fourier(a.data_ptr(), dtype_code(a.dtype), a.stride(0), a.stride(1), _ptr(cols), out.data_ptr(), B, K,
                             Mc, N, int(T), int(K_start), int(accumulate), _ptr(ws), ws_bytes, _stream(a.device)))
    return out


def mat_fourier_triton(a: torch.Tensor, N: int, T: int, K_start: int = 0) -> torch.Tensor:
    assert a.is_contiguous(), "Matrix A must be contiguous"  # TRI:82
    return mat_fourier(a, N, T, K_start)


# --------------------------------------------------------------------------- K2
def mat_avg_std(a: torch.Tensor, cols: Optional[torch.Tensor] = None, round_dtype: Optional[torch.dtype] = None):
    """fp32 ``(avg, max_dev)`` of the columns of ``a (B, K, width)``, each rounded through
    ``round_dtype`` when given."""
    _require_gpu(a, "a")
    assert a.dim() == 3 and a.stride(2) == 1
    B, K, width = a.shape
    Mc = width if cols is None else cols.numel()
    avg = torch.empty((B, Mc), device=a.device, dtype=torch.float32)
    dev = torch.empty((B, Mc), device=a.device, dtype=torch.float32)
    if Mc == 0 or B == 0:
        return avg, dev
    lib = _lib.load()
    nbytes = lib.fa_stats_workspace_bytes(B, Mc, K)
    ws = workspace(a.device, nbytes)
    rd = FA_FP32 if round_dtype is None else dtype_code(round_dtype)
    check(lib.fa_mat_avg_std(a.data_ptr(), dtype_code(a.dtype), a.stride(0), a.stride(1), _ptr(cols), avg.data_ptr(),
                             dev.data_ptr(), B, K, Mc, rd, ws.data_ptr(), ws.numel(), _stream(a.device)))
    return avg, dev


def mat_avg_std_triton(a: torch.Tensor):
    assert a.is_cuda and a.is_contiguous(), "Input tensor must be a contiguous CUDA tensor"  # TRI:438
    assert a.dim() == 3, "Input tensor must be 3-dimensional"
    avg, dev = mat_avg_std(a, round_dtype=a.dtype)
    return avg.to(a.dtype), dev.to(a.dtype)  # TRI:461


# --------------------------------------------------------------------------- K3
def mat_fourier_avg_std(c: torch.Tensor, K: int, T: int, round_dtype: Optional[torch.dtype] = torch.float16,
                        matrix_cores: bool = True):
    """Mean and maximum deviation, per column, of the signal reconstructed from ``c`` at positions 0..K-1.
    Long reconstructions run on the matrix cores (fp16 operands, fp32 accumulation) unless
    ``matrix_cores`` is false."""
    _require_gpu(c, "c")
    assert c.is_contiguous() and c.dtype == torch.float32 and c.dim() == 3
    B, N2, Mc = c.shape
    avg = torch.empty((B, Mc), device=c.device, dtype=torch.float32)
    dev = torch.empty((B, Mc), device=c.device, dtype=torch.float32)
    if Mc == 0 or B == 0:
        return avg, dev
    lib = _lib.load()
    if matrix_cores:
        nbytes = lib.fa_mat_fourier_avg_std_workspace_bytes(B, N2 // 2, Mc, int(K))
    else:
        nbytes = lib.fa_stats_workspace_bytes(B, Mc, int(K))
    ws = workspace(c.device, nbytes, "spectral")
    rd = FA_FP32 if round_dtype is None else dtype_code(round_dtype)
    check(lib.fa_mat_fourier_avg_std(c.data_ptr(), avg.data_ptr(), dev.data_ptr(), B, N2 // 2, Mc, int(K), int(T), rd,
                                     ws.data_ptr(), int(nbytes), _stream(c.device)))
    return avg, dev


def mat_fourier_avg_std_triton(c: torch.Tensor, K: int, T: int):
    assert c.is_contiguous(), "Matrix C must be contiguous"  # TRI:286
    avg, dev = mat_fourier_avg_std(c.float() if c.dtype != torch.float32 else c, K, T, torch.float16)
    return avg.to(torch.float16), dev.to(torch.float16)  # TRI:326


# ------------------------------------------------------------------ reconstruction
def mat_fourier_inv(c: torch.Tensor, K: int, T: int, avg_u=None, avg_d=None, scale=None) -> torch.Tensor:
    """``(B, K, Mc)`` fp32 reconstruction (TRI:782-791), optionally through the affine statistics."""
    _require_gpu(c, "c")
    assert c.is_contiguous() and c.dtype == torch.float32 and c.dim() == 3
    B, N2, Mc = c.shape
    r = torch.empty((B, int(K), Mc), device=c.device, dtype=torch.float32)
    if r.numel() == 0:
        return r
    f = lambda t: None if t is None else t.float().contiguous()
    au, ad, sc = f(avg_u), f(avg_d), f(scale)
    check(_lib.load().fa_reconstruct(c.data_ptr(), _ptr(au), _ptr(ad), _ptr(sc), r.data_ptr(), B, N2 // 2, Mc, int(K), int(T),
                                     _stream(c.device)))
    return r


# -------------------------------------------------------------------- rank-1 update
def coeff_update_(c: torch.Tensor, row: torch.Tensor, cols: Optional[torch.Tensor], p: int, T: int) -> torch.Tensor:
    """In place ``c[b, n, j] += cos(2 pi p n / T) row[b, cols[j]]`` (+ sin rows).  ``row (B, width)``
    may be a strided view with a contiguous last dim."""
    _require_gpu(c, "c")
    assert c.is_contiguous() and c.dtype == torch.float32 and c.dim() == 3
    assert row.dim() == 2 and row.stride(1) == 1
    B, N2, Mc = c.shape
    if Mc == 0 or B == 0:
        return c
    check(_lib.load().fa_coeff_update(c.data_ptr(), row.data_ptr(), dtype_code(row.dtype), row.stride(0), _ptr(cols), B,
                                      N2 // 2, Mc, int(p), int(T), _stream(c.device)))
    return c


def stream_update(k_new: torch.Tensor, v_new: torch.Tensor, k_ring: torch.Tensor, v_ring: torch.Tensor, evict_slot: int,
                  write_slot: int, k_coef: torch.Tensor, v_coef: torch.Tensor, kc_list: torch.Tensor, vc_list: torch.Tensor,
                  phase: int, T: int, k_mid, v_mid, mid_pos: int, skip_coef: bool = False) -> None:
    """One streaming step of one layer in one launch (the body of cache_utils_fourier.py:731-748 for K and V):
    the rows in window slot ``evict_slot`` enter the coefficients (rank-1 update at ``phase``) and the page
    stores (at token ``mid_pos``); ``k_new, v_new (B, width)`` are written to window slot ``write_slot``.
    ``k_ring, v_ring (B, slots, width)`` share their strides; ``k_mid, v_mid`` are ``MidStore`` objects.
    ``skip_coef``: leave the coefficients alone; the caller owes them the update (``coeff_update_``, or the
    ``pending`` argument of the layer's next ``decode_attn_raw``) before that window slot is written again."""
    _require_gpu(k_ring, "k_ring")
    assert k_new.dim() == 2 and k_new.stride(1) == 1 and v_new.stride() == k_new.stride()
    assert k_ring.stride(2) == 1 and v_ring.stride() == k_ring.stride() and k_ring.shape == v_ring.shape
    assert evict_slot != write_slot and k_mid.cap_pages == v_mid.cap_pages
    a = _lib.StreamArgs()
    a.k_new, a.v_new, a.new_batch_stride = k_new.data_ptr(), v_new.data_ptr(), k_new.stride(0)
    a.k_ring, a.v_ring = k_ring.data_ptr(), v_ring.data_ptr()
    a.ring_batch_stride, a.ring_row_stride = k_ring.stride(0), k_ring.stride(1)
    a.evict_slot, a.write_slot = int(evict_slot), int(write_slot)
    a.k_coef, a.v_coef = _ptr(k_coef), _ptr(v_coef)
    a.kc_list, a.vc_list = _ptr(kc_list), _ptr(vc_list)
    a.Ck, a.Cv = int(kc_list.numel()), int(vc_list.numel())
    a.N, a.T, a.phase = int(k_coef.shape[1] // 2), int(T), int(phase)
    a.k_mid, a.v_mid = k_mid.data.data_ptr(), v_mid.data.data_ptr()
    a.k_mid_batch_stride, a.v_mid_batch_stride = int(k_mid.batch_stride), int(v_mid.batch_stride)
    a.cap_pages, a.mid_pos = int(k_mid.cap_pages), int(mid_pos)
    a.kn_list, a.kn_h_list, a.k_pad_h_list = _ptr(k_mid.n_list32), k_mid.n_h32.data_ptr(), k_mid.pad_h32.data_ptr()
    a.vn_list, a.vn_h_list, a.v_pad_h_list = _ptr(v_mid.n_list32), v_mid.n_h32.data_ptr(), v_mid.pad_h32.data_ptr()
    a.Cnk, a.Cnv = int(k_mid.Cn), int(v_mid.Cn)
    a.B, a.Hkv, a.width, a.dtype = int(k_ring.shape[0]), int(k_mid.Hkv), int(k_ring.shape[2]), dtype_code(k_ring.dtype)
    a.skip_coef = int(bool(skip_coef))
    import ctypes
    check(_lib.load().fa_stream_update(ctypes.byref(a), _stream(k_ring.device)))


def add_rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float) -> torch.Tensor:
    """``h += delta`` (when given, in place) and ``LlamaRMSNorm`` of the result in one launch
    (modeling_llama_fourier.py:735-750, 87-92).  ``h, delta (..., hidden)`` contiguous."""
    _require_gpu(h, "h")
    assert h.is_contiguous() and weight.is_contiguous() and weight.dtype == h.dtype
    assert delta is None or (delta.is_contiguous() and delta.shape == h.shape and delta.dtype == h.dtype)
    y = torch.empty_like(h)
    hidden = h.shape[-1]
    check(_lib.load().fa_add_rmsnorm(h.data_ptr(), _ptr(delta), weight.data_ptr(), y.data_ptr(), h.numel() // hidden, hidden,
                                     float(eps), dtype_code(h.dtype), _stream(h.device)))
    return y


def _row_sliced(t: torch.Tensor) -> bool:
    """(B, q_len, width) whose rows are evenly spaced slices of wider rows (or dense)."""
    return t.dim() == 3 and t.stride(2) == 1 and (t.shape[1] == 1 or t.stride(0) == t.shape[1] * t.stride(1))


def rope_qk(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, head_dim: int) -> torch.Tensor:
    """Rotary embedding of ``q (B, q_len, Hq*D)`` and ``k (B, q_len, Hkv*D)`` (the projection outputs, possibly
    column slices of one fused projection output); ``cos, sin (B or 1, q_len, D)`` (modeling_llama_fourier.py:213-244).
    ``k`` is rotated in place; the rotated ``q`` is returned densely packed (``q`` itself when it was dense)."""
    _require_gpu(q, "q")
    assert _row_sliced(q) and _row_sliced(k) and q.dtype == k.dtype
    rows = q.shape[0] * q.shape[1]
    if cos.shape[0] != q.shape[0]:
        cos, sin = cos.expand(q.shape[0], -1, -1), sin.expand(q.shape[0], -1, -1)
    cos, sin = cos.to(q.dtype).contiguous(), sin.to(q.dtype).contiguous()
    q_out = q if q.is_contiguous() else torch.empty(q.shape, dtype=q.dtype, device=q.device)
    qs = q.stride(1) if q.shape[1] > 1 else q.stride(0)
    ks = k.stride(1) if k.shape[1] > 1 else k.stride(0)
    if rows == 1:                      # a single row has no spacing, whatever its view reports
        qs, ks = q.shape[2], k.shape[2]
    check(_lib.load().fa_rope_qk(q.data_ptr(), qs, q_out.data_ptr(), k.data_ptr(), ks, cos.data_ptr(), sin.data_ptr(), rows,
                                 q.shape[2] // head_dim, k.shape[2] // head_dim, head_dim, dtype_code(q.dtype),
                                 _stream(q.device)))
    return q_out


def rope_qk_(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, head_dim: int) -> None:
    """``rope_qk`` in place on densely packed ``q`` and ``k``."""
    assert q.is_contiguous() and k.is_contiguous()
    rope_qk(q, k, cos, sin, head_dim)


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` in one launch (modeling_llama_fourier.py:277); ``gate, up (..., cols)`` dense or column
    slices of one fused projection output (rows evenly spaced, the same spacing for both); the result is dense."""
    _require_gpu(gate, "gate")
    assert gate.shape == up.shape and gate.dtype == up.dtype and gate.stride() == up.stride() and gate.stride(-1) == 1
    cols = gate.shape[-1]
    rows = gate.numel() // max(cols, 1)
    stride = gate.stride(-2) if gate.dim() >= 2 and rows > 1 else cols
    assert all(gate.shape[d] == 1 or gate.stride(d) == gate.stride(d + 1) * gate.shape[d + 1] for d in range(gate.dim() - 2)), \
        "rows are not evenly spaced"
    out = torch.empty(gate.shape, dtype=gate.dtype, device=gate.device)
    es = gate.element_size()
    for r0 in range(0, rows, 65535):   # the row index is the launch's second grid dimension
        check(_lib.load().fa_silu_mul(gate.data_ptr() + r0 * stride * es, up.data_ptr() + r0 * stride * es,
                                      out.data_ptr() + r0 * cols * es, min(65535, rows - r0), cols, stride,
                                      dtype_code(gate.dtype), _stream(gate.device)))
    return out


class WeightStamp:
    """Identity and version of the tensors a derived copy was made from: ``changed()`` once any of them has been
    written in place (``load_state_dict``, an optimizer step) or replaced (``.to()``, re-assignment of ``.data``)."""

    def __init__(self, tensors):
        self._refs = list(tensors)
        self._seen = [(t.data_ptr(), t._version) for t in self._refs]

    def changed(self) -> bool:
        return any((t.data_ptr(), t._version) != s for t, s in zip(self._refs, self._seen))


class PackedLinearWeight:
    """A bias-free ``nn.Linear`` weight ``(n_out, K)`` re-laid for ``linear_packed``: the order in which the matrix
    cores take it, so that a decode step (a handful of rows) streams it in contiguous KiB pieces.  ``sources``: the
    parameters the weight was assembled from; ``stale()`` tells when the copy no longer matches them."""

    def __init__(self, weight: torch.Tensor, sources=None):
        self.stamp = WeightStamp(sources if sources is not None else [weight])
        _require_gpu(weight, "weight")
        assert weight.dim() == 2 and weight.is_contiguous() and weight.dtype in (torch.bfloat16, torch.float16)
        self.n_out, self.k = int(weight.shape[0]), int(weight.shape[1])
        self.dtype = weight.dtype
        self._rows_ok = {}     # row count -> whether the kernel takes it (asked once per count)
        self.data = torch.empty_like(weight)
        check(_lib.load().fa_linear_pack(weight.data_ptr(), self.data.data_ptr(), self.n_out, self.k, dtype_code(weight.dtype),
                                         _stream(weight.device)))

    def stale(self) -> bool:
        return self.stamp.changed()

    def covers(self, x: torch.Tensor) -> bool:
        if not (x.is_cuda and x.dtype == self.dtype and x.shape[-1] == self.k and x.stride(-1) == 1):
            return False
        rows = x.numel() // max(self.k, 1)
        ok = self._rows_ok.get(rows)
        if ok is None:
            ok = self._rows_ok[rows] = bool(_lib.load().fa_linear_packed_ok(rows, self.k, self.n_out))
        return ok


def linear_packed(x: torch.Tensor, w: PackedLinearWeight) -> torch.Tensor:
    """``F.linear(x, weight)`` for ``x (..., K)`` of at most 16 rows (fp32 accumulation, result in the storage type)
    on the packed weight; rows must be evenly spaced (dense, or slices of wider rows)."""
    assert w.covers(x), "shape not covered: at most 16 rows, K a multiple of 1024, n_out of 16"
    rows = x.numel() // w.k
    stride = x.stride(-2) if x.dim() >= 2 and rows > 1 else w.k
    assert all(x.shape[d] == 1 or x.stride(d) == x.stride(d + 1) * x.shape[d + 1] for d in range(x.dim() - 2)), \
        "rows are not evenly spaced"
    out = torch.empty(x.shape[:-1] + (w.n_out,), dtype=x.dtype, device=x.device)
    check(_lib.load().fa_linear_packed(x.data_ptr(), stride, w.data.data_ptr(), out.data_ptr(), rows, w.k, w.n_out,
                                       dtype_code(x.dtype), _stream(x.device)))
    return out


def prefill_attention_supported(q: torch.Tensor, k: torch.Tensor, head_dim: int) -> bool:
    """Shapes the matrix-core prompt attention covers: 16-bit GPU tensors, heads of 64 or 128 dims, 16-byte rows."""
    return (q.is_cuda and q.dtype in (torch.bfloat16, torch.float16) and k.dtype == q.dtype and head_dim in (64, 128)
            and q.stride(-1) == 1 and k.stride(-1) == 1 and all(s % 8 == 0 for s in q.stride()[:-1])
            and all(s % 8 == 0 for s in k.stride()[:-1]) and q.data_ptr() % 16 == 0 and k.data_ptr() % 16 == 0)


def prefill_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, num_kv_heads: int, sm_scale: float = -1.0,
                      out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Exact causal attention of the prompt pass (modeling_llama_fourier.py:623-633, ``flash_attn_func(q, k, v,
    causal=True)``).  ``q (B, Hq, q_len, D)`` (any strides with a contiguous last dim), ``k, v (B, S, Hkv*D)``
    token-major with common strides; returns ``(B, q_len, Hq, D)`` in the dtype of ``q``.  Query row ``i`` sees keys
    ``0 .. i + S - q_len``."""
    _require_gpu(q, "q")
    B, Hq, q_len, D = q.shape
    S = k.shape[1]
    assert k.shape == v.shape and k.stride() == v.stride() and k.shape[0] == B and k.shape[2] == num_kv_heads * D
    assert prefill_attention_supported(q, k, D) and v.dtype == q.dtype and v.data_ptr() % 16 == 0, \
        "prefill_attention: 16-bit GPU tensors, head_dim 64 or 128, 16-byte aligned rows"
    if out is None:
        out = torch.empty((B, q_len, Hq, D), dtype=q.dtype, device=q.device)
    assert out.is_contiguous() and tuple(out.shape) == (B, q_len, Hq, D) and out.dtype == q.dtype
    lib = _lib.load()
    nbytes = lib.fa_prefill_attn_workspace_bytes(B, num_kv_heads, D, S)
    ws = workspace(q.device, nbytes, "prefill")
    check(lib.fa_prefill_attn(q.data_ptr(), q.stride(0), q.stride(1), q.stride(2), k.data_ptr(), v.data_ptr(), k.stride(0),
                              k.stride(1), out.data_ptr(), dtype_code(q.dtype), B, Hq, num_kv_heads, D, S, q_len,
                              float(sm_scale), ws.data_ptr(), ws.numel(), _stream(q.device)))
    return out


class MultiDimHiPPO2(torch.nn.Module):
    """Same call contract as the reference class (TRI:840-865): without ``slice_input`` the
    whole ``base_input (B, L, C)`` is projected (period and length ``int(1/dt)``: longer inputs
    are cut, shorter ones behave as zero-padded); with ``slice_input (B, 1, C)`` the result is
    ``base_input + transform(slice_input)`` entering at phase ``token_num``."""

    def __init__(self, N, input_dim, method="legt", dt=1.0, T=1.0, discretization="bilinear", scale=False, c=0.0):
        super().__init__()
        self.method, self.N, self.input_dim, self.dt, self.T, self.c = method, N, input_dim, dt, T, c
        self.base_N = N // input_dim

    def forward(self, base_input, token_num, slice_input=None, fast=False):
        base_N = self.N // self.input_dim // 2
        period = int(1 / self.dt)
        if slice_input is not None:
            out = base_input.clone()
            return coeff_update_(out, slice_input[:, 0, :], None, token_num, period)
        return mat_fourier(base_input, base_N, period, 0, K=period)


# ------------------------------------------------------------------ decode attention
def decode_tables(n_f: int, period: int, device) -> Optional[torch.Tensor]:
    """Constant operand tables of the MFMA decode path for ``(N, T)``; ``None`` when that path
    does not cover ``N`` (the call then takes the generic kernels)."""
    lib = _lib.load()
    nbytes = lib.fa_decode_tables_bytes(int(n_f))
    if nbytes == 0 or n_f not in (128, 256, 512, 1024):
        return None
    buf = torch.empty(nbytes, dtype=torch.uint8, device=device)
    check(lib.fa_decode_tables_build(buf.data_ptr(), nbytes, int(n_f), int(period), _stream(torch.device(device))))
    return buf


def decode_attn_raw(q, il_segments, k_mc, v_mc, k_mn, v_mn, stats_k, stats_v, lists, num_head_q, num_head_kv, seq_len_m,
                    T, sm_scale=-1.0, out=None, tables=None, force_generic=False, timings=None, out_dtype=None,
                    no_alloc=False, balance_heads=True, no_fuse=False, pending=None):
    """Thin call into ``fa_decode_attn``.  The result is float32 like the reference's (TRI:779) unless ``out_dtype``
    names the dtype of ``q``: then the merge launch rounds it to that type itself (the caller's ``.to(dtype)``).

    ``il_segments``: up to two ``(k, v)`` pairs of ``(B, rows, Hkv*D)`` views (last dim contiguous).
    ``k_mn`` / ``v_mn``: token-major ``(B, >=L_m, Cn)`` tensors or ``MidStore`` objects (paged).
    ``stats_*``: ``(avg_u, avg_d, scale)`` fp32 ``(B, C)``.  ``lists``: the eight int32 tensors
    ``kc, kc_h, kn, kn_h, vc, vc_h, vn, vn_h`` (``*_h`` with the leading 0).
    ``no_alloc``: call ``fa_decode_attn_noalloc`` (partial results in the library's own fixed buffer, no workspace
    tensor; pass ``out`` as well and nothing is allocated on the device at all).
    ``balance_heads``: hand the per-head padded dim counts of a paged store over on the host side too, so that heads
    that store more dims get more splits (``False``: every head the same number, for comparison).
    ``no_fuse``: keep the sink/window tiles, the mid rows and the merge as launches of their own where the library
    would run them as one (for comparison); an int is passed on as the bits of ``fa_decode_args.no_fuse`` (2: fused,
    but without the four sub-splits per workgroup that a batch of one sequence otherwise runs).
    ``pending``: ``(k_row, v_row, phase, T_c)``, a rank-1 update the coefficients are still owed (``stream_update``
    with ``skip_coef``): ``k_row, v_row (B, Hkv*D)`` are the rows that left the window (same strides).  The call
    applies it to ``k_mc`` / ``v_mc`` IN PLACE while it streams them, once; pass it to one call only."""
    from .midstore import MidStore
    _require_gpu(q, "q")
    B, q_len, feat = q.shape
    D = feat // num_head_q
    a = DecodeArgs()
    assert q.is_contiguous()
    a.q = q.data_ptr()
    total_il = 0
    for i in range(2):
        if i < len(il_segments) and il_segments[i] is not None and il_segments[i][0].shape[1] > 0:
            k, v = il_segments[i]
            assert k.stride(2) == 1 and v.stride(2) == 1 and k.stride() == v.stride() and k.shape == v.shape
            assert k.dtype == q.dtype and v.dtype == q.dtype
            a.k_il[i], a.v_il[i] = k.data_ptr(), v.data_ptr()
            a.il_rows[i], a.il_batch_stride[i], a.il_row_stride[i] = k.shape[1], k.stride(0), k.stride(1)
            total_il += k.shape[1]
    kc, kc_h, kn, kn_h, vc, vc_h, vn, vn_h = lists
    a.Ck, a.Cnk, a.Cv, a.Cnv = kc.numel(), kn.numel(), vc.numel(), vn.numel()
    N = 0
    if seq_len_m > 0:
        N = (k_mc.shape[1] if a.Ck else v_mc.shape[1]) // 2
        for t in (k_mc, v_mc):
            assert t.dtype == torch.float32 and t.is_contiguous()
        a.k_mc, a.v_mc = _ptr(k_mc), _ptr(v_mc)
        if isinstance(k_mn, MidStore):
            assert isinstance(v_mn, MidStore) and k_mn.dtype == q.dtype and k_mn.cap_pages == v_mn.cap_pages
            a.mid_layout, a.mid_cap_pages = _lib.FA_MID_PAGED, k_mn.cap_pages
            a.k_mn, a.v_mn = k_mn.data.data_ptr(), v_mn.data.data_ptr()
            a.k_mn_batch_stride, a.v_mn_batch_stride = k_mn.batch_stride, v_mn.batch_stride
            a.k_pad_h_list, a.v_pad_h_list = k_mn.pad_h32.data_ptr(), v_mn.pad_h32.data_ptr()
            a.mid_max_k_pad, a.mid_max_v_pad = k_mn.max_pad, v_mn.max_pad
            if balance_heads:
                a.k_pad_h_host = ctypes.cast(k_mn.pad_h_c, ctypes.c_void_p)
                a.v_pad_h_host = ctypes.cast(v_mn.pad_h_c, ctypes.c_void_p)
        else:
            for t in (k_mn, v_mn):
                assert t.stride(2) == 1 and t.dtype == q.dtype
            a.mid_layout = _lib.FA_MID_TOKEN_MAJOR
            a.k_mn, a.v_mn = _ptr(k_mn), _ptr(v_mn)
            a.k_mn_batch_stride, a.k_mn_row_stride = k_mn.stride(0), k_mn.stride(1)
            a.v_mn_batch_stride, a.v_mn_row_stride = v_mn.stride(0), v_mn.stride(1)
        a.avg_k_u, a.avg_k_d, a.scale_k = (_ptr(t) for t in stats_k)
        a.avg_v_u, a.avg_v_d, a.scale_v = (_ptr(t) for t in stats_v)
        for t in (*stats_k, *stats_v):
            assert t.dtype == torch.float32 and t.is_contiguous()
        if tables is not None:
            a.tables = tables.data_ptr()
    if pending is not None:
        uk, uv, phase, t_c = pending
        assert seq_len_m > 0, "a layer without mid rows has no coefficients to update"
        assert uk.dim() == 2 and uk.stride(1) == 1 and uv.stride() == uk.stride() and uk.dtype == q.dtype == uv.dtype
        a.upd_k_row, a.upd_v_row, a.upd_batch_stride = uk.data_ptr(), uv.data_ptr(), uk.stride(0)
        a.upd_phase, a.upd_T = int(phase), int(t_c)
    a.force_generic = int(bool(force_generic))
    a.no_fuse = int(no_fuse)   # False / True, or the bits of fa_decode_args.no_fuse
    if seq_len_m >= _REPACK_MIN_ROWS and not force_generic:
        _warn_if_off_the_matrix_cores(q.dtype, num_head_q, num_head_kv, D, N, isinstance(k_mn, MidStore))
    a.kc_list, a.kc_h_list, a.kn_list, a.kn_h_list = kc.data_ptr(), kc_h.data_ptr(), kn.data_ptr(), kn_h.data_ptr()
    a.vc_list, a.vc_h_list, a.vn_list, a.vn_h_list = vc.data_ptr(), vc_h.data_ptr(), vn.data_ptr(), vn_h.data_ptr()
    if out is None:
        cast = out_dtype is not None and out_dtype != torch.float32
        assert not cast or out_dtype == q.dtype, "out_dtype must be float32 or the dtype of q"
        out = torch.empty((B, num_head_q, 1, D), device=q.device, dtype=q.dtype if cast else torch.float32)
    if out.dtype == torch.float32:
        a.out = out.data_ptr()
    else:
        assert out.dtype == q.dtype and out.is_contiguous()
        a.out_cast = out.data_ptr()
    a.B, a.Hq, a.Hkv, a.D = B, num_head_q, num_head_kv, D
    a.q_len, a.N, a.L_m, a.T = q_len, N, int(seq_len_m), int(T)
    a.sm_scale = float(sm_scale)
    a.dtype = dtype_code(q.dtype)
    lib = _lib.load()
    if no_alloc:
        check(lib.fa_decode_attn_noalloc(ctypes.byref(a), _stream(q.device)))
        return out
    nbytes = lib.fa_decode_attn_workspace_bytes(B, num_head_q, num_head_kv, D, N, total_il, int(seq_len_m))
    ws = workspace(q.device, nbytes, "decode")
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    if timings is not None:   # list to receive [prep, mid, sink/window, merge] milliseconds
        ms = (ctypes.c_float * 4)()
        check(lib.fa_decode_attn_timed(ctypes.byref(a), _stream(q.device), ms))
        timings[:] = list(ms)
    else:
        check(lib.fa_decode_attn(ctypes.byref(a), _stream(q.device)))
    return out


_warned_shapes = set()


def _warn_if_off_the_matrix_cores(dtype, num_head_q, num_head_kv, head_dim, n_f, paged):
    """Long contexts outside the shapes of the matrix-core kernels (16-bit paged storage, 128 / 256 / 512 / 1024
    frequencies, heads of at most 128 dims, at most 8 query heads per KV head) run on vector-ALU kernels that take any
    shape and are far slower (16.2 ms against 0.31 ms per layer at B=4, 131072 tokens, 24 / 8 heads): say so once
    per shape instead of being silently slow."""
    g = num_head_q // max(num_head_kv, 1)
    ok = (dtype in (torch.bfloat16, torch.float16) and paged and n_f in (128, 256, 512, 1024) and head_dim <= 128 and g <= 8)
    key = (dtype, num_head_q, num_head_kv, head_dim, n_f, paged)
    if ok or key in _warned_shapes:
        return
    _warned_shapes.add(key)
    import warnings
    warnings.warn(
        f"fourier decode attention: dtype={dtype}, {num_head_q}/{num_head_kv} heads of {head_dim} dims, {n_f} frequencies, "
        f"{'paged' if paged else 'token-major'} mid rows run on the any-shape vector kernels, roughly 50x slower than the "
        "matrix-core kernels (16-bit paged storage, 128/256/512/1024 frequencies, head_dim <= 128, <= 8 query heads per KV head)",
        RuntimeWarning, stacklevel=3)


def triton_fourier_attn(q, k_il, v_il, k_mc, v_mc, k_mn, v_mn,
                        avg_k_u, avg_k_d, scale_k, avg_v_u, avg_v_d, scale_v,
                        kc_list, kc_h_list, kn_list, kn_h_list,
                        vc_list, vc_h_list, vn_list, vn_h_list,
                        num_head_q, num_head_kv, seq_len_m, T, sm_scale=-1):
    """Drop-in for the reference function of the same name (TRI:684-779): returns
    ``(B, Hq, 1, D)`` float32."""
    batch_size, seq_len_q, feature_dim = q.shape
    assert seq_len_q == 1, f"{q.shape = }"  # TRI:692
    f32 = lambda t: t.float().contiguous()
    lists = tuple(as_i32(t) for t in (kc_list, kc_h_list, kn_list, kn_h_list, vc_list, vc_h_list, vn_list, vn_h_list))
    k_mc = k_mc if k_mc.dtype == torch.float32 else k_mc.float()
    v_mc = v_mc if v_mc.dtype == torch.float32 else v_mc.float()
    k_mn, v_mn = _paged_if_worthwhile(q, k_mn, v_mn, k_mc if kc_list.numel() else v_mc, lists[3], lists[7], num_head_q,
                                      num_head_kv, int(seq_len_m))
    return decode_attn_raw(q.contiguous(), [(k_il, v_il)], k_mc.contiguous(), v_mc.contiguous(), k_mn, v_mn,
                           (f32(avg_k_u), f32(avg_k_d), f32(scale_k)), (f32(avg_v_u), f32(avg_v_d), f32(scale_v)),
                           lists, num_head_q, num_head_kv, seq_len_m, T, sm_scale)


# below this many mid rows the any-layout kernels are quicker than re-paging first
_REPACK_MIN_ROWS = 2048


def _paged_if_worthwhile(q, k_mn, v_mn, coef, kn_h32, vn_h32, num_head_q, num_head_kv, seq_len_m):
    """The reference hands ``k_mn`` / ``v_mn`` over token-major (``torch.cat`` of gathered columns,
    cache_utils_fourier.py:735, 741).  The matrix-core kernels stream pages; for long contexts copying the
    rows into a temporary page store first (two passes over them) and taking those kernels is several times
    faster than the kernels that read the token-major layout in place.  ``DynamicCache`` keeps its rows paged
    and never comes through here."""
    from .midstore import MidStore
    if isinstance(k_mn, MidStore) or seq_len_m < _REPACK_MIN_ROWS or q.dtype not in (torch.bfloat16, torch.float16):
        return k_mn, v_mn
    D = q.shape[2] // num_head_q
    n_f = coef.shape[1] // 2
    if n_f not in (128, 256, 512, 1024) or D > 128 or num_head_q // num_head_kv > 8 or k_mn.dtype != q.dtype:
        return k_mn, v_mn
    stores = []
    for t, n_h, is_v in ((k_mn, kn_h32, False), (v_mn, vn_h32, True)):
        n_h_host = [int(x) for x in n_h.tolist()]
        ident = torch.arange(n_h_host[-1], dtype=torch.int32, device=q.device)   # the columns are gathered already
        st = MidStore(t.shape[0], ident, n_h, n_h_host, num_head_kv, D, seq_len_m, t.dtype, q.device, is_v)
        st.pack(t, 0, seq_len_m)
        stores.append(st)
    return stores[0], stores[1]


fourier_attn = triton_fourier_attn
