"""The Fourier KV cache object: drop-in for ``DynamicCache`` of
fourier_attn_triton/cache_utils_fourier.py:363-773 on the decode hot path.

Same constructor argument (an ``extra_config`` attribute bag), same ``update`` /
``get_seq_length`` / ``get_max_cache_shape`` / ``__len__`` / ``to_legacy_cache`` surface and
the same per-layer attribute lists the attention forward reads.  What differs is how the
state lives in HBM:

* the local window is a ring buffer (no ``torch.cat`` / shift per step);
* the stored ("critical") dims of the mid rows sit in a buffer pre-sized for
  ``maxtokens`` (appending an evicted row writes one row instead of copying the store);
* the coefficients are updated in place.

``update`` therefore returns *views*: mapping objects whose values are materialised in the
reference's shapes only when somebody indexes them; the attention forward in
``fourierattention_amd.attention`` reads the underlying buffers directly.
"""
from __future__ import annotations

import json
from collections.abc import Mapping
from typing import Any, Dict, List, Optional, Tuple

import torch

from . import ops
from .bookkeeping import Action, CacheBook
from .midstore import MidStore

_PART_NAMES = ("init", "compressed", "uncompressed", "local")


class ExtraConfig:
    """Attribute bag with the field names the reference passes (models/fourier.py:8-10, 141-153)."""

    def __init__(self, **kwargs):
        self.__dict__.update(kwargs)


class _Tensor:
    """Per-layer state of one of K / V."""

    def __init__(self):
        self.il: Optional[torch.Tensor] = None          # (B, I + W + 1, HD): sink rows, then the window slots
        self.init: Optional[torch.Tensor] = None        # view il[:, :I]
        self.ring: Optional[torch.Tensor] = None        # view il[:, I:] (W + 1 slots) when compressed, else growing (B, cap, HD)
        self.coef: Optional[torch.Tensor] = None        # (B, 2N, C) fp32
        self.mid: Optional[MidStore] = None             # paged store of the stored dims of the mid rows
        self.stats32: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None  # avg_u, avg_d, scale fp32


class _Layer:
    def __init__(self):
        self.k = _Tensor()
        self.v = _Tensor()
        self.compressed = False   # sink / coefficients / mid store exist
        self.window_only = True   # attention reads the window only (short prompt, or the append branch)
        self.growing = True       # the window is a plain growing buffer rather than a ring
        self.spare = 0            # the window slot that holds no row (ring mode: W + 1 slots for W rows)
        self.n_local = 0
        self.n_mid = 0
        self.version = 0        # bumped by every update; lets views detect staleness
        self.owed = None        # (window slot, phase, period): a rank-1 update the coefficients have not taken yet


class CacheParts(Mapping):
    """What ``update`` returns for a compressed layer: behaves like the reference's dict
    (``parts["k_local"]`` etc. give tensors in the reference's shapes) but builds those tensors
    only on access.  Views are valid until the next ``update`` of the same layer."""

    def __init__(self, cache: "DynamicCache", layer_idx: int, tag: str):
        self.cache, self.layer_idx, self.tag = cache, layer_idx, tag
        self._version = cache._layers[layer_idx].version

    def _names(self):
        return [f"{self.tag}_{p}" for p in _PART_NAMES]

    def __iter__(self):
        return iter(self._names())

    def __len__(self):
        return 4

    def __getitem__(self, key: str) -> torch.Tensor:
        if key not in self._names():
            raise KeyError(key)
        layer = self.cache._layers[self.layer_idx]
        if layer.version != self._version:
            raise RuntimeError("cache view used after a later update of the same layer")
        t = layer.k if self.tag == "k" else layer.v
        part = key.split("_", 1)[1]
        if part == "init":
            return t.init
        if part == "compressed":
            self.cache._settle_coefficients(self.layer_idx)
            return t.coef
        if part == "uncompressed":
            return t.mid.dense(layer.n_mid)
        return self.cache._window_in_order(layer, t)


class Cache(torch.nn.Module):
    """Base class of every cache object, as in cache_utils_fourier.py:39-125 (a ``torch.nn.Module`` there too).
    The modified LLaMA imports this name next to ``DynamicCache`` and ``StaticCache``
    (modeling_llama_fourier.py:29) and routes on ``isinstance(past_key_values, Cache)``
    (modeling_llama_fourier.py:946): an object that is not a ``Cache`` is taken for a legacy tuple."""

    def __init__(self) -> None:
        super().__init__()

    def update(self, key_states, value_states, layer_idx, cache_kwargs=None):
        raise NotImplementedError("Make sure to implement `update` in a subclass.")

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        raise NotImplementedError("Make sure to implement `get_seq_length` in a subclass.")

    def get_max_cache_shape(self) -> Optional[int]:
        raise NotImplementedError("Make sure to implement `get_max_cache_shape` in a subclass.")

    def get_max_length(self) -> Optional[int]:
        return self.get_max_cache_shape()

    def get_usable_length(self, new_seq_length: int, layer_idx: Optional[int] = 0) -> int:
        """cache_utils_fourier.py:93-102: everything is usable unless the cache has a capacity."""
        max_length = self.get_max_cache_shape()
        previous_seq_length = self.get_seq_length(layer_idx)
        if max_length is not None and previous_seq_length + new_seq_length > max_length:
            return max_length - new_seq_length
        return previous_seq_length

    @property
    def seen_tokens(self):
        return getattr(self, "_seen_tokens", None)


class StaticCache(Cache):
    """The name the modified LLaMA tests with ``isinstance(past_key_values, StaticCache)``
    (modeling_llama_fourier.py:1052).  The Fourier path never uses a static cache (the reference's own
    class, cache_utils_fourier.py:1386, is the stock one and unrelated to the Fourier cache), so the class exists
    for those tests only and cannot be constructed."""

    def __init__(self, *args, **kwargs) -> None:
        raise NotImplementedError("StaticCache is not part of the Fourier cache path; only DynamicCache is provided")


class DynamicCache(Cache):
    """See module docstring.  ``extra_config`` needs: ``max_new_tokens``, ``maxlocallen``,
    ``maxmidstates``, ``numinittokens``, ``num_key_value_heads``, ``max_position_embeddings``,
    ``non_critical_dims_path`` (cache_utils_fourier.py:394-403).  As an extension,
    ``extra_config.non_critical_dims`` may hold the already-parsed mask dict instead of a path."""

    def __init__(self, extra_config, num_hidden_layers: Optional[int] = None, device=None) -> None:
        super().__init__()
        self._seen_tokens = 0
        self.maxnewtokens = extra_config.max_new_tokens
        self.maxlocallen = extra_config.maxlocallen
        self.maxmidstates = extra_config.maxmidstates
        self.numinittokens = extra_config.numinittokens
        self.maxlen = self.maxlocallen + self.maxmidstates + self.numinittokens
        self.heads = extra_config.num_key_value_heads
        self.maxtokens = extra_config.max_position_embeddings
        self.curr_tokennum: List[int] = []
        masks = getattr(extra_config, "non_critical_dims", None)
        if masks is None:
            with open(extra_config.non_critical_dims_path, "r") as f:
                masks = json.load(f)
        if device is None:
            if not torch.cuda.is_available():
                raise RuntimeError("the Fourier cache needs a GPU: its arithmetic exists only as HIP kernels")
            device = torch.device("cuda", torch.cuda.current_device())
        self.device = torch.device(device)

        self.k_scale, self.v_scale = [], []
        self.k_layer_average, self.v_layer_average = [], []
        self.kd_layer_average, self.vd_layer_average = [], []
        self.k_non_critical_dims, self.k_non_critical_head_dims = [], []
        self.k_critical_dims, self.k_critical_head_dims = [], []
        self.v_non_critical_dims, self.v_non_critical_head_dims = [], []
        self.v_critical_dims, self.v_critical_head_dims = [], []
        self._lists32: List[Tuple[torch.Tensor, ...]] = []
        dev = self.device
        for layer_idx in range(len(masks)):
            self.curr_tokennum.append(0)
            key = f"Layer_{layer_idx}"
            if key not in masks:
                raise ValueError(f"Layer index {layer_idx} not found in non-critical dimensions JSON file.")
            m = masks[key]
            t64 = lambda lst: torch.tensor(lst, dtype=torch.int64, device=dev)
            self.k_non_critical_dims.append(t64(m["kc_list"]))
            self.k_critical_dims.append(t64(m["kn_list"]))
            self.v_non_critical_dims.append(t64(m["vc_list"]))
            self.v_critical_dims.append(t64(m["vn_list"]))
            self.k_non_critical_head_dims.append(t64([0] + list(m["kc_h_list"])))
            self.k_critical_head_dims.append(t64([0] + list(m["kn_h_list"])))
            self.v_non_critical_head_dims.append(t64([0] + list(m["vc_h_list"])))
            self.v_critical_head_dims.append(t64([0] + list(m["vn_h_list"])))
            self._lists32.append(tuple(t.to(torch.int32) for t in (
                self.k_non_critical_dims[-1], self.k_non_critical_head_dims[-1],
                self.k_critical_dims[-1], self.k_critical_head_dims[-1],
                self.v_non_critical_dims[-1], self.v_non_critical_head_dims[-1],
                self.v_critical_dims[-1], self.v_critical_head_dims[-1])))
        self._num_layers = len(masks)
        self._head_lists = [([0] + list(masks[f"Layer_{i}"]["kn_h_list"]), [0] + list(masks[f"Layer_{i}"]["vn_h_list"]))
                            for i in range(self._num_layers)]
        self._tables: Optional[torch.Tensor] = None   # constant operands of the MFMA decode kernels
        self.force_generic = False                     # testing: keep decode attention off the MFMA kernels
        self.balance_heads = True                      # mid rows: more splits for heads that store more dims
        self.fuse_prefill = True                       # prefill: pages, coefficients and statistics from one read
        self.fuse_decode = True                        # decode: the merge inside the mid-row launch where it applies
        self.sub_splits = True                         # ... and a batch of one as four sub-splits per workgroup
        # streaming: leave the rank-1 update of the coefficients to the next decode_attention of the layer, which
        # streams them anyway.  Off: measured, it is no faster than the update launch (whose reads mostly hit the
        # last-level cache behind the attention of the step before), and two launches where the merge has its own
        self.defer_coef_update = False
        self._book = CacheBook(self._num_layers, self.numinittokens, self.maxlocallen, self.maxmidstates,
                               self.maxnewtokens, self.maxtokens)
        self._layers: List[_Layer] = [_Layer() for _ in range(self._num_layers)]
        self.key_cache: List[Any] = []
        self.value_cache: List[Any] = []
        self.hippo: Optional[ops.MultiDimHiPPO2] = None

    # -- reference surface ---------------------------------------------------
    def __len__(self):
        return len(self.key_cache)

    def __getitem__(self, layer_idx: int):  # "no use" in the reference
        return None

    def __iter__(self):
        return iter(())

    def get_seq_length(self, layer_idx: Optional[int] = 0) -> int:
        if len(self.key_cache) <= layer_idx:
            return 0
        return self._book.layers[layer_idx].seq_length

    def get_max_cache_shape(self) -> Optional[int]:
        return None

    def to_legacy_cache(self):
        return tuple((self.key_cache[i], self.value_cache[i]) for i in range(len(self)))

    def _unsupported(self, name):
        raise NotImplementedError(
            f"DynamicCache.{name} is stale in the reference (it indexes parts that no longer exist or "
            "constructs the cache without its required argument) and is not provided")

    def crop(self, max_length: int):
        self._unsupported("crop")

    def batch_split(self, *a, **k):
        self._unsupported("batch_split")

    def batch_select_indices(self, *a, **k):
        self._unsupported("batch_select_indices")

    @classmethod
    def from_legacy_cache(cls, *a, **k):
        raise NotImplementedError("DynamicCache.from_legacy_cache: the reference calls cls() without extra_config")

    @classmethod
    def from_batch_splits(cls, *a, **k):
        raise NotImplementedError("DynamicCache.from_batch_splits: the reference calls cls() without extra_config")

    # -- helpers -----------------------------------------------------------------
    @property
    def period_reconstruct(self) -> int:
        """``T`` handed to decode attention (modeling_llama_fourier.py:660)."""
        return self.maxtokens - self.numinittokens - self.maxlocallen

    def _window_in_order(self, layer: _Layer, t: _Tensor) -> torch.Tensor:
        if layer.growing:
            return t.ring[:, : layer.n_local, :]
        sp = layer.spare      # oldest row sits right after the spare slot
        if sp == t.ring.shape[1] - 1:
            return t.ring[:, :sp, :]
        return torch.cat([t.ring[:, sp + 1:, :], t.ring[:, :sp, :]], dim=1)

    def _window_segments(self, layer: _Layer):
        """The window as (k, v) views whose union is the window (order irrelevant to attention)."""
        return [(layer.k.ring[:, : layer.n_local, :], layer.v.ring[:, : layer.n_local, :])]

    def _il_segments(self, layer: _Layer):
        """Sink + window of a compressed layer as two views of the one buffer: the rows before and the rows
        after the spare window slot."""
        cut = self.numinittokens + layer.spare
        return [(layer.k.il[:, :cut, :], layer.v.il[:, :cut, :]), (layer.k.il[:, cut + 1:, :], layer.v.il[:, cut + 1:, :])]

    def _compress_tensor(self, t: _Tensor, states: torch.Tensor, c32: torch.Tensor, ch32: torch.Tensor, n32: torch.Tensor,
                         nh32: torch.Tensor, nh_host, is_v: bool, L: int, fft_rows: int, n_f: int):
        I, W = self.numinittokens, self.maxlocallen
        B, S, HD = states.shape
        mid = states[:, I: S - W, :]
        t.il = torch.empty((B, I + W + 1, HD), dtype=states.dtype, device=states.device)
        t.init, t.ring = t.il[:, :I, :], t.il[:, I:, :]
        t.init.copy_(states[:, :I, :])
        t.ring[:, :W, :].copy_(states[:, S - W:, :])
        t.ring[:, W, :].zero_()
        cap = max(self._book.t_x, L + int(self.maxnewtokens)) + 1     # room for every row the decode will evict
        t.mid = MidStore(B, n32, nh32, nh_host, self.heads, self.head_dim, cap, states.dtype, states.device, is_v)
        fused = t.mid.pack_and_compress(states, I, L, fft_rows, c32, ch32, n_f, self._book.t_c, states.dtype) \
            if self.fuse_prefill else None
        if fused is not None:   # pages, coefficients and column statistics from one read of the rows
            t.coef, u_avg, u_std = fused
        else:
            t.mid.pack(states, I, L, head_dims=True)
            # spectral compression of the selected columns (gather fused into the kernel)
            t.coef = ops.mat_fourier(mid, n_f, self._book.t_c, 0, cols=c32, K=fft_rows)
            u_avg, u_std = ops.mat_avg_std(mid, cols=c32, round_dtype=states.dtype)
        i_avg, i_std = ops.mat_fourier_avg_std(t.coef, L, self._book.t_x, torch.float16)
        # dtypes as the reference leaves them: u_* in the model dtype, i_* in fp16, quotient promoted
        u_avg_m, u_std_m = u_avg.to(states.dtype), u_std.to(states.dtype)
        i_avg_h, i_std_h = i_avg.to(torch.float16), i_std.to(torch.float16)
        scale = u_std_m / i_std_h
        t.stats32 = (u_avg.contiguous(), i_avg.contiguous(), scale.float().contiguous())
        return scale, u_avg_m, i_avg_h

    # -- update ------------------------------------------------------------------
    def update(self, key_states: torch.Tensor, value_states: torch.Tensor, layer_idx: int,
               cache_kwargs: Optional[Dict[str, Any]] = None):
        """``key_states, value_states (B, Hkv, q_len, D)``.  Returns ``(k_parts, v_parts)``: for a
        prefill call and for layers that only keep a window, plain dicts whose ``*_init``,
        ``*_compressed`` and ``*_uncompressed`` entries are ``None`` (exact attention over
        ``*_local``); otherwise ``CacheParts`` views of the four parts."""
        bsz, heads, q_len, head_dim = key_states.shape
        self.heads, self.head_dim = heads, head_dim
        step = self._book.step(layer_idx, bsz, q_len)
        self._seen_tokens = self._book.seen_tokens
        self.maxtokens = self._book.maxtokens
        if self._book.prefilllen is not None:
            self.prefilllen = self._book.prefilllen
        k = key_states.permute(0, 2, 1, 3).reshape(bsz, q_len, heads * head_dim)
        v = value_states.permute(0, 2, 1, 3).reshape(bsz, q_len, heads * head_dim)
        layer = self._layers[layer_idx]
        lb = self._book.layers[layer_idx]
        if step.action in (Action.PREFILL_COMPRESS, Action.PREFILL_LOCAL):
            layer.owed = None                       # the coefficients are rebuilt from scratch
        else:
            self._settle_coefficients(layer_idx)    # the row they are owed sits in the window slot written next
        local_only = lambda kk, vv: ({"k_init": None, "k_compressed": None, "k_uncompressed": None, "k_local": kk},
                                     {"v_init": None, "v_compressed": None, "v_uncompressed": None, "v_local": vv})

        if step.action in (Action.PREFILL_COMPRESS, Action.PREFILL_LOCAL):
            if layer_idx == 0 and self.hippo is None:
                ck0 = self.k_non_critical_dims[0].shape[0]
                self.hippo = ops.MultiDimHiPPO2(N=ck0 * self.maxmidstates, input_dim=ck0, method="legt",
                                                dt=self._book.dt, T=1)
            while len(self.key_cache) < layer_idx:  # skipped layers
                self.key_cache.append([])
                self.value_cache.append([])
            layer.version += 1
            if step.action is Action.PREFILL_COMPRESS:
                l32 = self._lists32[layer_idx]
                n_f = self.maxmidstates // 2
                hl = self._head_lists[layer_idx]
                ks, ku, kd = self._compress_tensor(layer.k, k, l32[0], l32[1], l32[2], l32[3], hl[0], False, step.mid_rows,
                                                   step.fft_rows, n_f)
                vs, vu, vd = self._compress_tensor(layer.v, v, l32[4], l32[5], l32[6], l32[7], hl[1], True, step.mid_rows,
                                                   step.fft_rows, n_f)
                if self._tables is None and layer_idx == 0:
                    self._tables = ops.decode_tables(n_f, self.period_reconstruct, self.device)
                layer.compressed, layer.window_only, layer.growing, layer.spare = True, False, False, self.maxlocallen
                layer.n_local, layer.n_mid = self.maxlocallen, step.mid_rows
                self._store_stats(layer_idx, ks, ku, kd, vs, vu, vd)
                kview, vview = CacheParts(self, layer_idx, "k"), CacheParts(self, layer_idx, "v")
            else:
                layer.compressed, layer.window_only, layer.growing, layer.spare = False, True, True, 0
                layer.n_local, layer.n_mid = q_len, 0
                cap = q_len + max(int(self.maxnewtokens), 16)
                for t, s in ((layer.k, k), (layer.v, v)):
                    t.ring = torch.empty((bsz, cap, s.shape[2]), dtype=s.dtype, device=s.device)
                    t.ring[:, :q_len, :].copy_(s)
                    t.il, t.init, t.coef, t.mid, t.stats32 = None, None, None, None, None
                kview, vview = self._placeholder_parts(layer_idx, bsz, heads * head_dim)
            if len(self.key_cache) <= layer_idx:
                self.key_cache.append(kview)
                self.value_cache.append(vview)
            else:
                self.key_cache[layer_idx], self.value_cache[layer_idx] = kview, vview
            self.curr_tokennum[layer_idx] = lb.curr_tokennum
            return local_only(k, v)

        if step.action is Action.APPEND_LOCAL:
            layer.version += 1
            if not layer.growing:
                # a compressed layer whose mid is short: the reference concatenates onto k_local and
                # from then on attends to the window only (cache_utils_fourier.py:681-686); keep that
                # by turning the ring into a growing buffer
                for t in (layer.k, layer.v):
                    t.ring = self._window_in_order(layer, t).contiguous()
                layer.spare, layer.growing, layer.window_only = 0, True, True
            for t, s in ((layer.k, k), (layer.v, v)):
                need = layer.n_local + q_len
                if need > t.ring.shape[1]:
                    grown = torch.empty((bsz, max(need, 2 * t.ring.shape[1]), t.ring.shape[2]), dtype=t.ring.dtype,
                                        device=t.ring.device)
                    grown[:, : layer.n_local, :].copy_(t.ring[:, : layer.n_local, :])
                    t.ring = grown
                t.ring[:, layer.n_local: need, :].copy_(s)
            layer.n_local += q_len
            if layer.compressed:
                self.key_cache[layer_idx] = CacheParts(self, layer_idx, "k")
                self.value_cache[layer_idx] = CacheParts(self, layer_idx, "v")
            else:
                self.key_cache[layer_idx], self.value_cache[layer_idx] = self._placeholder_parts(
                    layer_idx, bsz, heads * head_dim)
            return local_only(layer.k.ring[:, : layer.n_local, :], layer.v.ring[:, : layer.n_local, :])

        if step.action is Action.LATE_COMPRESS:
            raise NotImplementedError(
                "this call lands in the reference's late-compression branch (cache_utils_fourier.py:688-729), "
                "which appends a new layer entry instead of updating this one; its result is undefined")

        # ---- streaming: evict the oldest window row, then overwrite its slot with the new token
        layer.version += 1
        self.curr_tokennum[layer_idx] = lb.curr_tokennum
        p = step.phase
        l32 = self._lists32[layer_idx]
        slots = self.maxlocallen + 1
        sp = layer.spare
        oldest = (sp + 1) % slots
        for t in (layer.k, layer.v):
            if layer.n_mid >= t.mid.cap_tokens:
                t.mid.grow(layer.n_mid, 2 * t.mid.cap_tokens)
        # one launch: coefficients and page store take the oldest row, the new token takes the spare slot.  The
        # attention that follows streams the coefficients anyway: where it can, it is left to apply their rank-1
        # update on the way (the evicted row stays in its window slot until the next update of the layer writes there)
        defer = bool(self.defer_coef_update and k.is_cuda and not torch.cuda.is_current_stream_capturing())
        ops.stream_update(k[:, 0, :], v[:, 0, :], layer.k.ring, layer.v.ring, oldest, sp, layer.k.coef, layer.v.coef,
                          l32[0], l32[4], p, self._book.t_c, layer.k.mid, layer.v.mid, layer.n_mid, skip_coef=defer)
        if defer:
            layer.owed = (oldest, int(p), int(self._book.t_c))
        layer.n_mid += 1
        layer.spare = oldest
        kview, vview = CacheParts(self, layer_idx, "k"), CacheParts(self, layer_idx, "v")
        self.key_cache[layer_idx], self.value_cache[layer_idx] = kview, vview
        return kview, vview

    def _settle_coefficients(self, layer_idx: int) -> None:
        """Apply the rank-1 update a streaming ``update`` left to the next ``decode_attention`` of the layer, if it
        is still owed (somebody reads the coefficients, or the layer is updated again, before that call came)."""
        layer = self._layers[layer_idx]
        owed, layer.owed = layer.owed, None
        if owed is None:
            return
        slot, phase, t_c = owed
        l32 = self._lists32[layer_idx]
        for t, cols in ((layer.k, l32[0]), (layer.v, l32[4])):
            if cols.numel():
                ops.coeff_update_(t.coef, t.ring[:, slot, :], cols, phase, t_c)

    def _store_stats(self, layer_idx, ks, ku, kd, vs, vu, vd):
        lists = (self.k_scale, self.k_layer_average, self.kd_layer_average, self.v_scale, self.v_layer_average,
                 self.vd_layer_average)
        for lst, val in zip(lists, (ks, ku, kd, vs, vu, vd)):
            while len(lst) <= layer_idx:
                lst.append(None)
            lst[layer_idx] = val

    def _placeholder_parts(self, layer_idx: int, bsz: int, hidden: int):
        """Parts of a layer that keeps only a window: empty CPU fp32 placeholders for the other three
        (cache_utils_fourier.py:601-611)."""
        layer = self._layers[layer_idx]
        ck, cn = self.k_non_critical_dims[layer_idx].shape[0], self.k_critical_dims[layer_idx].shape[0]
        cv, cnv = self.v_non_critical_dims[layer_idx].shape[0], self.v_critical_dims[layer_idx].shape[0]
        e = lambda n: torch.empty((bsz, 0, n))
        kd = {"k_init": e(hidden), "k_compressed": e(ck), "k_uncompressed": e(cn),
              "k_local": layer.k.ring[:, : layer.n_local, :]}
        vd = {"v_init": e(hidden), "v_compressed": e(cv), "v_uncompressed": e(cnv),
              "v_local": layer.v.ring[:, : layer.n_local, :]}
        return kd, vd

    # -- attention over the cache's own buffers --------------------------------------
    def decode_attention(self, query_states: torch.Tensor, layer_idx: int, num_heads: int, num_kv_heads: int,
                         sm_scale: float = -1.0, timings=None, out_dtype=None, out=None, no_alloc=False) -> torch.Tensor:
        """``query_states (B, Hq, 1, D)`` -> ``(B, Hq, 1, D)`` float32 over the current state of
        ``layer_idx`` (what modeling_llama_fourier.py:641-660 computes from the returned parts); with
        ``out_dtype = query_states.dtype`` the result comes back rounded to that type (the ``.to(dtype)`` of
        modeling_llama_fourier.py:663 done by the last kernel)."""
        layer = self._layers[layer_idx]
        B, Hq, q_len, D = query_states.shape
        q = query_states.transpose(1, 2).reshape(B, q_len, Hq * D).contiguous()
        l32 = self._lists32[layer_idx]
        if layer.window_only:
            return ops.decode_attn_raw(q, self._window_segments(layer), None, None, None, None, None, None, l32, num_heads,
                                       num_kv_heads, 0, 1, sm_scale, timings=timings, out_dtype=out_dtype, out=out,
                                       no_alloc=no_alloc)
        segs = self._il_segments(layer)
        pending = None
        if layer.owed is not None:
            if q.is_cuda and torch.cuda.is_current_stream_capturing():
                raise RuntimeError("a coefficient update is still owed to this layer: call update() inside the capture "
                                   "as well, or settle it before (read the layer's *_compressed part)")
            slot, phase, t_c = layer.owed
            layer.owed = None
            pending = (layer.k.ring[:, slot, :], layer.v.ring[:, slot, :], phase, t_c)
        return ops.decode_attn_raw(q, segs, layer.k.coef, layer.v.coef, layer.k.mid, layer.v.mid, layer.k.stats32,
                                   layer.v.stats32, l32, num_heads, num_kv_heads, layer.n_mid, self.period_reconstruct,
                                   sm_scale, tables=self._tables, force_generic=self.force_generic, timings=timings,
                                   out_dtype=out_dtype, out=out, no_alloc=no_alloc, balance_heads=self.balance_heads,
                                   no_fuse=(0 if self.fuse_decode else 1) | (0 if self.sub_splits else 2), pending=pending)
