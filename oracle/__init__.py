"""CPU oracle for the Fourier KV-cache hot path.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
directory; only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` do, and there only as the checker.

The modules restate, in plain numpy (float64 by default), the arithmetic of
the reference's PyTorch/Triton path:

* ``fourier_oracle``  - compression, rank-1 update, statistics, reconstruction
  and decode attention (fourier_triton_valid4_v2.py).
* ``cache_oracle``    - the ``DynamicCache.update`` state machine
  (cache_utils_fourier.py:389-765).
* ``masks_oracle``    - compressed-dim index rules
  (cache_utils_fourier.py:403-455, compressed_dim_search.py:321-397).
"""
