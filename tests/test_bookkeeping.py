"""Host logic without a GPU: the integer state machine against the CPU restatement of the
reference cache (shapes and counters after every call), the period pair, and the C ABI's
exports and argument validation (no kernel is launched)."""
import ctypes
import os
import re

import numpy as np
import pytest

from fourierattention_amd import _lib
from fourierattention_amd.bookkeeping import Action, CacheBook, periods
from fourierattention_amd.cache import ExtraConfig
from fourierattention_amd import masks as pm
from oracle import fourier_oracle as fo
from oracle.cache_oracle import OracleCache

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_periods_match_oracle():
    for mt in list(range(30, 3000, 7)) + [131072, 131072 + 512, 32768 + 128]:
        assert periods(mt, 4, 20) == fo.periods(mt, 4, 20)
    assert periods(131072, 4, 1024)[0::2] == (130044, 130043)


TRACES = [
    # I, W, M, max_new, max_pos, B, prompt, steps
    (4, 16, 16, 10, 4096, 2, 103, 8),      # compressed, streaming
    (4, 16, 16, 10, 4096, 2, 30, 12),      # short prompt: window only, forever
    (4, 16, 16, 10, 113, 2, 120, 5),       # maxtokens clamped by max_position_embeddings
    (4, 64, 8, 8, 4096, 1, 88, 4),         # short mid: append branch of a compressed layer
    (4, 512, 256, 64, 131072, 1, 2048, 3),  # BASELINE config 1 geometry
    (0, 8, 4, 4, 4096, 3, 40, 5),          # no sink tokens
]


@pytest.mark.parametrize("I,W,M,max_new,max_pos,B,prompt,steps", TRACES)
def test_state_machine_trace_matches_reference_restatement(I, W, M, max_new, max_pos, B, prompt, steps):
    Hkv, D, layers = 2, 8, 3
    masks = pm.synthetic_masks(layers, Hkv, D, 3, 5, seed=1)
    cfg = ExtraConfig(numinittokens=I, maxlocallen=W, maxmidstates=M, non_critical_dims_path=None, max_position_embeddings=max_pos,
                      num_key_value_heads=Hkv, max_new_tokens=max_new)
    cpu = OracleCache(cfg, masks=masks, model_dtype="fp32")
    book = CacheBook(layers, I, W, M, max_new, max_pos)
    r = np.random.default_rng(0)

    def check(l, step):
        lb = book.layers[l]
        kc = cpu.key_cache[l]
        assert (lb.n_init, lb.n_coef_rows, lb.n_mid, lb.n_local) == (
            kc["k_init"].shape[1], kc["k_compressed"].shape[1], kc["k_uncompressed"].shape[1], kc["k_local"].shape[1])
        assert lb.seq_length == cpu.get_seq_length(l)
        assert lb.curr_tokennum == cpu.curr_tokennum[l]
        assert book.seen_tokens == cpu._seen_tokens and book.maxtokens == cpu.maxtokens
        assert (book.t_x, book.t_c) == (cpu._t_x(), cpu.t_c)

    for l in range(layers):
        k = r.standard_normal((B, Hkv, prompt, D))
        kd, _ = cpu.update(k, k, l)
        st = book.step(l, B, prompt)
        assert st.action in (Action.PREFILL_COMPRESS, Action.PREFILL_LOCAL)
        assert (st.action is Action.PREFILL_COMPRESS) == (cpu.key_cache[l]["k_compressed"].shape[1] > 0)
        if st.action is Action.PREFILL_COMPRESS:
            assert st.mid_rows == cpu.key_cache[l]["k_uncompressed"].shape[1] and st.fft_rows == min(st.mid_rows, cpu.t_c)
        check(l, st)
    for s in range(steps):
        for l in range(layers):
            k = r.standard_normal((B, Hkv, 1, D))
            before = cpu.curr_tokennum[l]
            kd, _ = cpu.update(k, k, l)
            st = book.step(l, B, 1)
            assert (st.action is Action.STREAM) == (kd["k_init"] is not None)
            if st.action is Action.STREAM:
                assert st.phase == before + 1 == cpu.curr_tokennum[l]
                # phase runs one ahead of the row index of the evicted token
                assert st.phase == book.layers[l].n_mid
            check(l, st)


# Literal expectations, derived by hand from cache_utils_fourier.py:494-761 (not from either restatement).
# Each trace: configuration, then per call (layer, q_len) -> what the call returns ("local" = the three other parts
# are None, line 613 / 686; "parts" = all four, line 748) and the state afterwards:
# (k_init rows, k_compressed rows, k_uncompressed rows, k_local rows, curr_tokennum[layer], _seen_tokens, seq length).
LITERAL_TRACES = {
    # prompt 50 > maxlen 36: sink 4, mid 50 - 4 - 16 = 30, window 16, 16 coefficient rows; maxtokens = min(50 + 10, 4096),
    # period 60 - 20 = 40.  Decode: 4 + 16 + 30 + B(2) + 1 = 53 > 37 -> streaming; the counter runs 31, 32, ...
    "stream": dict(cfg=dict(I=4, W=16, M=16, max_new=10, max_pos=4096, B=2), periods=(40, 40), maxtokens=60, calls=[
        ((0, 50), "local", (4, 16, 30, 16, 30, 50, 50)),
        ((1, 50), "local", (4, 16, 30, 16, 30, 50, 50)),     # _seen_tokens moves at layer 0 only (line 520)
        ((0, 1), "parts", (4, 16, 31, 16, 31, 51, 51)),
        ((1, 1), "parts", (4, 16, 31, 16, 31, 51, 51)),
        ((0, 1), "parts", (4, 16, 32, 16, 32, 52, 52)),
    ]),
    # prompt 30 <= maxlen 36: everything stays in the window, the other parts are empty (lines 598-611); decode:
    # 0 + 0 + 0 + B + 1 <= 36 for ever -> the window grows and the layer is never compressed
    "window_only": dict(cfg=dict(I=4, W=16, M=16, max_new=10, max_pos=4096, B=2), periods=(20, 20), maxtokens=40, calls=[
        ((0, 30), "local", (0, 0, 0, 30, 0, 30, 30)),
        ((0, 1), "local", (0, 0, 0, 31, 0, 31, 31)),
        ((0, 1), "local", (0, 0, 0, 32, 0, 32, 32)),
    ]),
    # maxlen 76, prompt 128 -> mid 60, compressed (8 coefficient rows).  Batch 1: 4 + 8 + 60 + 1 + 1 = 74 <= 76 -> the
    # append branch of a COMPRESSED layer (line 681): the window grows, the caller sees the window only, the
    # counter and the mid rows stand still; the predicate does not depend on the window length, so it never ends
    "append_batch1": dict(cfg=dict(I=4, W=64, M=8, max_new=8, max_pos=4096, B=1), periods=(68, 68), maxtokens=136, calls=[
        ((0, 128), "local", (4, 8, 60, 64, 60, 128, 128)),
        ((0, 1), "local", (4, 8, 60, 65, 60, 129, 129)),
        ((0, 1), "local", (4, 8, 60, 66, 60, 130, 130)),
    ]),
    # the same cache and prompt with batch 5: 4 + 8 + 60 + 5 + 1 = 78 > 77 -> streaming.  Only k_local.size(0), the
    # batch size, differs from the trace above (line 680)
    "stream_batch5": dict(cfg=dict(I=4, W=64, M=8, max_new=8, max_pos=4096, B=5), periods=(68, 68), maxtokens=136, calls=[
        ((0, 128), "local", (4, 8, 60, 64, 60, 128, 128)),
        ((0, 1), "parts", (4, 8, 61, 64, 61, 129, 129)),
        ((0, 1), "parts", (4, 8, 62, 64, 62, 130, 130)),
    ]),
    # maxtokens clamped by max_position_embeddings (line 542): min(120 + 10, 113) = 113, period 93, and
    # int(1 / (1 / 93)) = 92; the mid (100 rows) is longer than that period
    "clamped": dict(cfg=dict(I=4, W=16, M=16, max_new=10, max_pos=113, B=2), periods=(93, 92), maxtokens=113, calls=[
        ((0, 120), "local", (4, 16, 100, 16, 100, 120, 120)),
        ((0, 1), "parts", (4, 16, 101, 16, 101, 121, 121)),
    ]),
}


@pytest.mark.parametrize("name", sorted(LITERAL_TRACES))
def test_literal_trace_table(name):
    """Both restatements of the state machine against hand-derived numbers, the oracle first."""
    tr = LITERAL_TRACES[name]
    c = tr["cfg"]
    Hkv, D, layers = 2, 8, 2
    masks = pm.synthetic_masks(layers, Hkv, D, 3, 5, seed=1)
    cfg = ExtraConfig(numinittokens=c["I"], maxlocallen=c["W"], maxmidstates=c["M"], non_critical_dims_path=None,
                      max_position_embeddings=c["max_pos"], num_key_value_heads=Hkv, max_new_tokens=c["max_new"])
    cpu = OracleCache(cfg, masks=masks, model_dtype="fp32")
    book = CacheBook(layers, c["I"], c["W"], c["M"], c["max_new"], c["max_pos"])
    r = np.random.default_rng(0)
    for (layer, q_len), returned, want in tr["calls"]:
        x = r.standard_normal((c["B"], Hkv, q_len, D))
        kd, vd = cpu.update(x, x, layer)
        st = book.step(layer, c["B"], q_len)
        none_pattern = [kd[k] is None for k in ("k_init", "k_compressed", "k_uncompressed")]
        assert none_pattern == [returned == "local"] * 3 and kd["k_local"] is not None and vd["v_local"] is not None
        assert (st.action is Action.STREAM) == (returned == "parts")
        kc = cpu.key_cache[layer]
        got = (kc["k_init"].shape[1], kc["k_compressed"].shape[1], kc["k_uncompressed"].shape[1], kc["k_local"].shape[1],
               cpu.curr_tokennum[layer], cpu._seen_tokens, cpu.get_seq_length(layer))
        assert got == want, (name, layer, q_len, got)
        assert kd["k_local"].shape[1] == (q_len if q_len > 1 else want[3])      # prefill returns the whole prompt
        lb = book.layers[layer]
        assert (lb.n_init, lb.n_coef_rows, lb.n_mid, lb.n_local, lb.curr_tokennum, book.seen_tokens, lb.seq_length) == want
        assert cpu.maxtokens == book.maxtokens == tr["maxtokens"]
        assert (cpu._t_x(), cpu.t_c) == (book.t_x, book.t_c) == tr["periods"]
    assert len(cpu) == 1 + max(l for (l, _), _, _ in tr["calls"])


def test_batch_size_alone_can_land_in_the_unsupported_late_compression_branch():
    """Between the two batch sizes of the traces above: 4 + 8 + 60 + 4 + 1 = 77 = maxlen + 1 (line 688)."""
    masks = pm.synthetic_masks(1, 2, 8, 3, 5, seed=1)
    cfg = ExtraConfig(numinittokens=4, maxlocallen=64, maxmidstates=8, non_critical_dims_path=None,
                      max_position_embeddings=4096, num_key_value_heads=2, max_new_tokens=8)
    cpu, book = OracleCache(cfg, masks=masks, model_dtype="fp32"), CacheBook(1, 4, 64, 8, 8, 4096)
    x = np.zeros((4, 2, 128, 8))
    cpu.update(x, x, 0)
    book.step(0, 4, 128)
    with pytest.raises(NotImplementedError):
        cpu.update(x[:, :, :1], x[:, :, :1], 0)
    assert book.step(0, 4, 1).action is Action.LATE_COMPRESS


def test_layer_zero_must_come_first_and_stream_needs_one_token():
    book = CacheBook(2, 4, 16, 16, 10, 4096)
    with pytest.raises(RuntimeError):
        book.step(1, 1, 100)
    book.step(0, 1, 100)
    book.step(1, 1, 100)
    with pytest.raises(ValueError):
        book.step(0, 1, 2)


def test_missing_layer_key_raises_value_error():
    masks = pm.synthetic_masks(3, 2, 8, 3)
    del masks["Layer_1"]
    masks["Layer_7"] = masks["Layer_0"]
    cfg = ExtraConfig(numinittokens=4, maxlocallen=16, maxmidstates=16, non_critical_dims_path=None, non_critical_dims=masks,
                      max_position_embeddings=4096, num_key_value_heads=2, max_new_tokens=4)
    with pytest.raises(ValueError):
        OracleCache(cfg, masks=masks)
    from fourierattention_amd import DynamicCache
    with pytest.raises(ValueError):
        DynamicCache(cfg, device="cpu")


# ----------------------------------------------------------------- C ABI ------
def _declared_functions():
    text = open(os.path.join(ROOT, "include", "fourier_attn_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    declared = _declared_functions()
    assert len(declared) >= 10
    for name in declared:
        assert hasattr(lib, name), name
    assert set(declared) == set(_lib.EXPORTED), set(declared) ^ set(_lib.EXPORTED)
    assert lib.fa_abi_version() >= 1
    assert lib.fa_decode_args_size() == ctypes.sizeof(_lib.DecodeArgs)


def test_argument_validation_returns_codes_without_a_gpu():
    lib = _lib.load()
    assert lib.fa_decode_attn(None, None) == -1
    a = _lib.DecodeArgs()
    a.q_len = 2
    assert lib.fa_decode_attn(ctypes.byref(a), None) == -2 and b"q_len" in lib.fa_last_error_string()
    a.q_len, a.B, a.Hq, a.Hkv, a.D = 1, 1, 6, 4, 64
    assert lib.fa_decode_attn(ctypes.byref(a), None) == -2          # Hq not a multiple of Hkv
    a.Hq, a.Hkv = 8, 2
    a.il_rows[0] = 4
    assert lib.fa_decode_attn(ctypes.byref(a), None) == -1          # q / out null
    buf = ctypes.create_string_buffer(1 << 16)
    p = ctypes.addressof(buf)
    a.q = a.out = p
    assert lib.fa_decode_attn(ctypes.byref(a), None) == -1          # il segment null
    a.k_il[0] = a.v_il[0] = p
    a.dtype = 9
    assert lib.fa_decode_attn(ctypes.byref(a), None) == -3
    a.dtype = 0
    assert lib.fa_decode_attn(ctypes.byref(a), None) == -4          # workspace missing
    a.Hq, a.Hkv = 64, 2
    assert lib.fa_decode_attn(ctypes.byref(a), None) == -5          # 32 query heads per KV head
    assert lib.fa_mat_fourier(None, 0, 0, 0, None, None, 1, 1, 1, 1, 1, 0, 0, None, 0, None) == -1
    assert lib.fa_mat_fourier(p, 0, 0, 0, None, p, 1, 1, 1, 0, 1, 0, 0, None, 0, None) == -2
    assert lib.fa_mat_fourier(p, 7, 0, 0, None, p, 1, 1, 1, 1, 1, 0, 0, None, 0, None) == -3
    assert lib.fa_mat_avg_std(p, 0, 0, 0, None, p, p, 1, 4, 4, 2, None, 0, None) == -4
    assert lib.fa_coeff_update(p, None, 0, 0, None, 1, 1, 1, 0, 1, None) == -1
    # the decoder-side elementwise entry points and the streaming update
    assert lib.fa_add_rmsnorm(None, None, p, p, 1, 64, 1e-5, 0, None) == -1
    assert lib.fa_add_rmsnorm(p, None, p, p, 1, 9000, 1e-5, 0, None) == -2     # rows longer than 8192
    assert lib.fa_add_rmsnorm(p, None, p, p, 1, 64, 1e-5, 5, None) == -3
    assert lib.fa_add_rmsnorm(p, None, p, p, 0, 64, 1e-5, 0, None) == 0         # nothing to do
    assert lib.fa_rope_qk(p, 256, p, None, 128, p, p, 1, 4, 2, 64, 0, None) == -1
    assert lib.fa_rope_qk(p, 252, p, p, 126, p, p, 1, 4, 2, 63, 0, None) == -2    # odd head_dim
    assert lib.fa_rope_qk(p, 255, p, p, 128, p, p, 1, 4, 2, 64, 0, None) == -2    # stride shorter than a row
    assert lib.fa_rope_qk(p, 512, p, p, 128, p, p, 2, 4, 2, 64, 0, None) == -2    # in place on sliced rows (more than one)
    assert lib.fa_silu_mul(p, p, None, 1, 8, 8, 0, None) == -1
    assert lib.fa_silu_mul(p, p, p, -1, 8, 8, 0, None) == -2
    assert lib.fa_silu_mul(p, p, p, 2, 8, 4, 0, None) == -2                        # stride shorter than a row
    assert lib.fa_linear_pack(None, p, 16, 1024, 0, None) == -1
    assert lib.fa_linear_pack(p, p, 24, 1024, 0, None) == -2                       # output features not a multiple of 16
    assert lib.fa_linear_pack(p, p, 16, 1024, 2, None) == -3                       # float32 storage
    assert lib.fa_linear_packed(p, 1024, p, None, 1, 1024, 16, 0, None) == -1
    assert lib.fa_linear_packed(p, 1024, p, p, 17, 1024, 16, 0, None) == -5        # more than 16 rows: the GEMM library's
    assert lib.fa_linear_packed(p, 1536, p, p, 1, 1536, 16, 0, None) == -5         # K not a multiple of 1024
    assert lib.fa_linear_packed(p, 1000, p, p, 2, 1024, 16, 0, None) == -7         # rows of x closer than K
    assert lib.fa_linear_packed_ok(16, 4096, 6144) == 1 and lib.fa_linear_packed_ok(0, 4096, 6144) == 0
    # the one-pass prefill: (src, dtype, bs, rs, row0, L, K_fft, store, st_bs, cap_pages, n_list, n_h, pad_h, c_list, c_h, Mc,
    #                        coef, avg, dev, round_dtype, B, Hkv, D, N, T, is_v, workspace, bytes, stream)
    pc = lambda *a: lib.fa_prefill_compress(*a)
    ok_args = [p, 0, 1 << 20, 1024, 4, 1000, 1000, p, 1 << 20, 40, p, p, p, p, p, 512, p, p, p, 0, 1, 8, 128, 64, 4096, 0, p, 1 << 30, None]
    names = {n: i for i, n in enumerate("src dtype bs rs row0 L K_fft store st_bs cap n_list n_h pad_h c_list c_h Mc coef avg dev rd B Hkv D N T is_v ws ws_bytes stream".split())}
    arg = lambda **kw: [kw.get(n, ok_args[i]) for n, i in names.items()]
    assert pc(*arg(src=None)) == -1
    assert pc(*arg(L=0)) == -2
    assert pc(*arg(cap=10)) == -2                                     # 1000 rows do not fit 10 pages
    assert pc(*arg(dtype=2)) == -5                                    # float32 rows: the separate calls
    assert pc(*arg(L=100, K_fft=100, cap=40)) == -5                   # too short for the matrix-core transform
    assert pc(*arg(K_fft=1001)) == -5                                 # more rows into the transform than there are
    assert pc(*arg(D=130)) == -5
    assert pc(*arg(rs=1000)) == -7                                    # rows shorter than Hkv * D
    assert pc(*arg(ws_bytes=1024)) == -4
    assert b"workspace" in lib.fa_last_error_string()
    assert lib.fa_prefill_compress_ok(0, 1000, 1000, 819, 64, 128) == 1 and lib.fa_prefill_compress_ok(2, 1000, 1000, 512, 64, 128) == 0
    need = lib.fa_prefill_compress_workspace_bytes(1, 1000, 1000, 512, 64)
    assert need > lib.fa_mat_fourier_workspace_bytes(0, 1, 1000, 512, 64) > 0       # + the partials of the column statistics
    assert lib.fa_mat_fourier_workspace_bytes(0, 1, 1000, 819, 64) > 0               # an odd number of columns is fine
    assert lib.fa_stream_update(None, None) == -1
    sa = _lib.StreamArgs()
    assert lib.fa_stream_update(ctypes.byref(sa), None) == -2                  # empty shape
    assert lib.fa_stats_workspace_bytes(2, 10, 1000) == 3 * 2 * 4 * 10 * 4
    assert lib.fa_decode_attn_workspace_bytes(8, 32, 8, 128, 512, 1028, 31740) > 0


def test_split_plan_of_the_mid_rows():
    """``fa_decode_split_plan`` (host-side arithmetic of the launch, runs without a GPU): how the mid rows of each KV
    head are cut into splits.  Same count for every head without the per-head lists or with a uniform mask; with a
    ragged mask the total stays the same, nobody gets more than the workspace query leaves room for, nobody gets
    none, and the head with the widest pages gets more than the even share.  Where the merge may run inside the
    mid-row launch (this geometry), the workgroups of a (batch group, KV head) must fill the dies of the device
    exactly: heads are shared out in bins (here pairs, two heads per die and batch group) that keep their total."""
    import ctypes
    from fourierattention_amd import _lib
    lib = _lib.load()

    def plan(L_m, kpads, vpads, B=8, Hq=32, Hkv=8, N=512):
        out, room = (ctypes.c_int32 * Hkv)(), ctypes.c_int32()
        cum = lambda p: (ctypes.c_int32 * (Hkv + 1))(*([0] + list(np.cumsum(p)))) if p is not None else None
        k, v = cum(kpads), cum(vpads)
        rc = lib.fa_decode_split_plan(B, Hq, Hkv, 128, N, 1028, L_m, k, v, out, ctypes.byref(room))
        assert rc == 0, lib.fa_last_error_string()
        return list(out), room.value

    even, room = plan(31740, None, None)
    assert len(set(even)) == 1 and even[0] >= 1 and room == -(-3 * even[0] // 2)
    assert plan(31740, [64] * 8, [64] * 8)[0] == even                    # a uniform mask changes nothing
    # padded per-head counts of layers 15 and 31 of the reference's Llama-3.1-8B mask
    for kp, vp in (([64, 32, 32, 32, 32, 64, 32, 64], [16, 0, 32, 32, 128, 16, 0, 48]),
                   ([96, 64, 96, 96, 64, 64, 64, 64], [48, 16, 16, 80, 16, 128, 48, 16])):
        got, room2 = plan(31740, kp, vp)
        assert room2 == room and sum(got) == sum(even)
        assert min(got) >= 1 and max(got) <= room
        # the heads pair up into bins of twice the even share: B = 8 makes two batch groups of eight teams, sixteen
        # teams on eight dies
        left = sorted(got)
        while left:
            big = left.pop()
            assert 2 * even[0] - big in left, (got, big)
            left.remove(2 * even[0] - big)
        assert got[vp.index(max(vp))] > even[0]                          # the head with the widest V pages gets more
    # one batch group (B <= 4): a team per die, nothing to share out
    assert plan(31740, [96, 64, 96, 96, 64, 64, 64, 64], [48, 16, 16, 80, 16, 128, 48, 16], B=4)[0] == [32] * 8
    # a geometry the fused merge does not take (eight query heads per KV head): shared out freely, dominated heads
    # never get more (beyond one of rounding)
    kp, vp = [96, 64, 96, 96, 64, 64, 64, 64], [48, 16, 16, 80, 16, 128, 48, 16]
    got, _ = plan(31740, kp, vp, B=8, Hq=64)
    assert len(set(got)) > 1
    for a in range(8):
        for b in range(8):
            if kp[a] >= kp[b] and vp[a] >= vp[b]:
                assert got[a] + 1 >= got[b], (a, b, got)                 # (single splits move: equal heads may differ by one)
    # fewer pages than workgroups: one page per split for everybody
    short, _ = plan(200, [96, 64, 96, 96, 64, 64, 64, 64], [48, 16, 16, 80, 16, 128, 48, 16])
    assert short == [7] * 8
    assert lib.fa_decode_split_plan(8, 32, 8, 128, 100, 0, 5000, None, None, (ctypes.c_int32 * 8)(), None) == -5   # N not covered
