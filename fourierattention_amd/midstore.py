"""Paged store of the mid rows' stored ("critical") dims - the HBM layout the decode kernels
stream (documented in ``include/fourier_attn_hip.h``).  Replaces the reference's
``k_uncompressed`` / ``v_uncompressed`` tensors that grow by ``torch.cat``
(cache_utils_fourier.py:735, 741); ``dense()`` gives that tensor back when asked."""
from __future__ import annotations

from typing import List

import ctypes

import torch

from . import _lib
from ._lib import K_DIM_PAD, PAGE_TOKENS, V_DIM_PAD, check
from .ops import _stream, dtype_code


class MidStore:
    def __init__(self, batch: int, n_list32: torch.Tensor, n_h32: torch.Tensor, n_h_host: List[int], num_kv_heads: int,
                 head_dim: int, cap_tokens: int, dtype: torch.dtype, device, is_v: bool):
        self.B, self.Hkv, self.D, self.is_v = batch, num_kv_heads, head_dim, bool(is_v)
        self.n_list32, self.n_h32 = n_list32, n_h32
        self.Cn = int(n_h_host[-1])
        unit = V_DIM_PAD if is_v else K_DIM_PAD
        pad = [0]
        for h in range(num_kv_heads):
            n = n_h_host[h + 1] - n_h_host[h]
            pad.append(pad[-1] + (n + unit - 1) // unit * unit)
        self.pad_h_host = pad
        self.pad_h_c = (ctypes.c_int32 * len(pad))(*pad)   # the same for the C side (kept alive with the store)
        self.max_pad = max([pad[h + 1] - pad[h] for h in range(num_kv_heads)] + [0])
        self.pad_h32 = torch.tensor(pad, dtype=torch.int32, device=device)
        self.dtype, self.device = dtype, torch.device(device)
        self._alloc(cap_tokens)

    def _alloc(self, cap_tokens: int):
        self.cap_pages = max(1, (int(cap_tokens) + PAGE_TOKENS - 1) // PAGE_TOKENS)
        self.batch_stride = self.pad_h_host[-1] * PAGE_TOKENS * self.cap_pages
        # zero-filled: padded dims and unused token slots must read as zero
        self.data = torch.zeros(max(self.B * self.batch_stride, 8), dtype=self.dtype, device=self.device)

    @property
    def cap_tokens(self) -> int:
        return self.cap_pages * PAGE_TOKENS

    def pack(self, src: torch.Tensor, row0: int, rows: int, n_list32=None, head_dims: bool = False) -> None:
        """Store ``src[:, row0:row0+rows, n_list]`` (``src (B, S, width)``, last dim contiguous) from token 0.
        ``head_dims``: ``src`` holds full K/V rows and the list is the reference's ``kn_list`` / ``vn_list`` (flat
        ``h*D + d`` entries, head by head); otherwise the entries are plain column numbers of ``src``."""
        assert src.dim() == 3 and src.stride(2) == 1 and src.dtype == self.dtype and rows <= self.cap_tokens
        if rows == 0 or self.Cn == 0:
            return
        nl = self.n_list32 if n_list32 is None else n_list32
        check(_lib.load().fa_mid_pack(src.data_ptr(), dtype_code(src.dtype), src.stride(0), src.stride(1), int(row0), int(rows),
                                      self.data.data_ptr(), self.batch_stride, self.cap_pages, nl.data_ptr(),
                                      self.n_h32.data_ptr(), self.pad_h32.data_ptr(), self.B, self.Hkv, self.D,
                                      int(self.is_v), _lib.FA_COLS_HEAD_DIMS if head_dims else _lib.FA_COLS_ANY,
                                      _stream(self.device)))

    def pack_and_compress(self, src: torch.Tensor, row0: int, rows: int, fft_rows: int, c_list32: torch.Tensor,
                          c_h32: torch.Tensor, n_freq: int, period: int, round_dtype: torch.dtype):
        """``pack(src, row0, rows, head_dims=True)`` together with, for the compressed dims ``c_list32`` (flat
        ``h*D + d`` entries with per-head offsets ``c_h32``) of the same rows, ``ops.mat_fourier(..., K=fft_rows)``
        and ``ops.mat_avg_std``: one read of the rows (cache_utils_fourier.py:560-565, 578-587).  Returns
        ``(coef, avg, max_dev)``, or ``None`` with nothing written when the shape is for the separate calls."""
        from .ops import workspace
        lib = _lib.load()
        Mc = int(c_list32.numel())
        if (src.dim() != 3 or src.stride(2) != 1 or src.dtype != self.dtype or src.shape[2] != self.Hkv * self.D
                or self.Cn == 0 or Mc == 0 or rows > self.cap_tokens or src.data_ptr() % 16 or src.stride(0) % 8
                or src.stride(1) % 8
                or not lib.fa_prefill_compress_ok(dtype_code(src.dtype), int(rows), int(fft_rows), Mc, int(n_freq), self.D)):
            return None
        B = self.B
        coef = torch.empty((B, 2 * n_freq, Mc), device=self.device, dtype=torch.float32)
        avg = torch.empty((B, Mc), device=self.device, dtype=torch.float32)
        dev = torch.empty((B, Mc), device=self.device, dtype=torch.float32)
        nbytes = int(lib.fa_prefill_compress_workspace_bytes(B, int(rows), int(fft_rows), Mc, int(n_freq)))
        ws = workspace(self.device, nbytes, "spectral")
        check(lib.fa_prefill_compress(src.data_ptr(), dtype_code(src.dtype), src.stride(0), src.stride(1), int(row0), int(rows),
                                      int(fft_rows), self.data.data_ptr(), self.batch_stride, self.cap_pages,
                                      self.n_list32.data_ptr(), self.n_h32.data_ptr(), self.pad_h32.data_ptr(),
                                      c_list32.data_ptr(), c_h32.data_ptr(), Mc, coef.data_ptr(), avg.data_ptr(),
                                      dev.data_ptr(), dtype_code(round_dtype), B, self.Hkv, self.D, int(n_freq), int(period),
                                      int(self.is_v), ws.data_ptr(), ws.numel(), _stream(self.device)))
        return coef, avg, dev

    def append(self, row: torch.Tensor, pos: int) -> None:
        """Store ``row[:, n_list]`` (``row (B, width)`` view) at token position ``pos``."""
        assert row.dim() == 2 and row.stride(1) == 1 and row.dtype == self.dtype
        if self.Cn == 0:
            return
        check(_lib.load().fa_mid_append(row.data_ptr(), dtype_code(row.dtype), row.stride(0), int(pos), self.data.data_ptr(),
                                        self.batch_stride, self.cap_pages, self.n_list32.data_ptr(), self.n_h32.data_ptr(),
                                        self.pad_h32.data_ptr(), self.B, self.Hkv, self.Cn, int(self.is_v),
                                        _stream(self.device)))

    def dense(self, rows: int) -> torch.Tensor:
        """``(B, rows, Cn)`` token-major copy: the reference's ``*_uncompressed`` tensor."""
        out = torch.empty((self.B, int(rows), self.Cn), dtype=self.dtype, device=self.device)
        if out.numel():
            check(_lib.load().fa_mid_unpack(self.data.data_ptr(), dtype_code(self.dtype), self.batch_stride, self.cap_pages,
                                            int(rows), out.data_ptr(), self.n_h32.data_ptr(), self.pad_h32.data_ptr(), self.B,
                                            self.Hkv, self.D, self.Cn, int(self.is_v), _stream(self.device)))
        return out

    def grow(self, rows_in_use: int, new_cap_tokens: int) -> None:
        """Re-page into a larger store (the head regions move when the capacity changes)."""
        dense = self.dense(rows_in_use)
        self._alloc(new_cap_tokens)
        ident = torch.arange(self.Cn, dtype=torch.int32, device=self.device)
        self.pack(dense, 0, rows_in_use, n_list32=ident)
