"""Integer bookkeeping of the Fourier KV cache: which branch an ``update`` call takes and what
the part lengths and counters are afterwards.  Pure Python, no tensors - the cache object
drives its device work from these decisions, and they can be checked on any machine.

Follows ``DynamicCache.update`` in fourier_attn_triton/cache_utils_fourier.py:494-750.
"""
from __future__ import annotations

import enum
from dataclasses import dataclass, field
from typing import List, Optional


class Action(enum.Enum):
    PREFILL_COMPRESS = "prefill_compress"   # lines 555-597: split sink / mid / window and compress the mid
    PREFILL_LOCAL = "prefill_local"         # lines 598-611: short prompt, everything stays in the window
    APPEND_LOCAL = "append_local"           # lines 681-686: window grows, only the window is attended
    STREAM = "stream"                       # lines 731-748: evict the oldest window row into the mid store
    LATE_COMPRESS = "late_compress"         # lines 688-729: not supported (see DynamicCache.update)


@dataclass
class LayerBook:
    filled: bool = False
    compressed: bool = False
    n_init: int = 0
    n_coef_rows: int = 0     # k_compressed.size(1): 2*N_f when compressed, 0 otherwise
    n_mid: int = 0           # rows of k_uncompressed
    n_local: int = 0
    curr_tokennum: int = 0   # phase counter of the rank-1 update (line 732)

    @property
    def seq_length(self) -> int:  # line 760
        return self.n_init + self.n_mid + self.n_local if self.filled else 0


@dataclass
class Step:
    action: Action
    phase: Optional[int] = None      # p of the rank-1 update (STREAM)
    mid_rows: Optional[int] = None   # L of the prefill split (PREFILL_COMPRESS)
    fft_rows: Optional[int] = None   # rows that enter the transform: min(L, T_c)


def periods(maxtokens: int, numinit: int, maxlocal: int):
    """``(T_x, dt, T_c)``: the exact period, ``dt = 1/T_x`` and ``T_c = int(1/dt)``
    (lines 547 and 566; the transform uses ``int(1/self.dt)``), which is ``T_x`` or ``T_x - 1``."""
    t_x = int(maxtokens) - int(numinit) - int(maxlocal)
    dt = 1 / t_x
    return t_x, dt, int(1 / dt)


class CacheBook:
    def __init__(self, num_layers: int, numinit: int, maxlocal: int, maxmidstates: int, max_new_tokens: int,
                 max_position_embeddings: int):
        self.numinit, self.maxlocal, self.maxmidstates = int(numinit), int(maxlocal), int(maxmidstates)
        self.max_new_tokens = int(max_new_tokens)
        self.maxtokens = int(max_position_embeddings)
        self.maxlen = self.maxlocal + self.maxmidstates + self.numinit  # line 398
        self.seen_tokens = 0
        self.prefilllen: Optional[int] = None
        self.t_x: Optional[int] = None
        self.t_c: Optional[int] = None
        self.dt: Optional[float] = None
        self.layers: List[LayerBook] = [LayerBook() for _ in range(num_layers)]
        self.n_layers_seen = 0  # len(self.key_cache) in the reference

    def step(self, layer_idx: int, bsz: int, q_len: int) -> Step:
        if layer_idx == 0:
            self.seen_tokens += q_len  # lines 520-521
        lb = self.layers[layer_idx]
        new_layer = self.n_layers_seen <= layer_idx
        if new_layer or not lb.filled:
            if self.t_c is None and layer_idx != 0:
                raise RuntimeError("layer 0 must be prefilled before any other layer (it fixes the period)")
            if new_layer:
                if layer_idx == 0:  # lines 540-549
                    self.prefilllen = q_len
                    self.maxtokens = min(self.prefilllen + self.max_new_tokens, self.maxtokens)
                    self.t_x, self.dt, self.t_c = periods(self.maxtokens, self.numinit, self.maxlocal)
                self.n_layers_seen = layer_idx + 1
            lb.filled = True
            if q_len > self.maxlen:  # line 555
                L = q_len - self.numinit - self.maxlocal
                lb.compressed = True
                lb.n_init, lb.n_coef_rows, lb.n_mid, lb.n_local = self.numinit, 2 * (self.maxmidstates // 2), L, self.maxlocal
                lb.curr_tokennum += L  # line 593
                return Step(Action.PREFILL_COMPRESS, mid_rows=L, fft_rows=min(L, self.t_c))
            lb.compressed = False
            lb.n_init, lb.n_coef_rows, lb.n_mid, lb.n_local = 0, 0, 0, q_len
            return Step(Action.PREFILL_LOCAL)
        # line 680: coefficient rows and the batch size take part in the predicate
        pred = lb.n_init + lb.n_coef_rows + lb.n_mid + bsz + 1
        if pred <= self.maxlen:
            lb.n_local += q_len
            return Step(Action.APPEND_LOCAL)
        if pred == self.maxlen + 1:
            return Step(Action.LATE_COMPRESS)
        if q_len != 1:
            raise ValueError(f"streaming update needs exactly one new token, got {q_len}")
        lb.curr_tokennum += 1  # line 732
        lb.n_mid += 1
        return Step(Action.STREAM, phase=lb.curr_tokennum)
