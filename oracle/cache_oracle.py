"""CPU restatement of the reference's Fourier ``DynamicCache`` state machine.

TEST INFRASTRUCTURE ONLY - see ``oracle/__init__.py``.

Follows cache_utils_fourier.py:389-765 branch by branch, including the
behaviours that look accidental but decide shapes and counters:

* the period pair ``T_x`` / ``T_c = int(1/dt)`` (lines 547, 566; TRI:856-859);
* the evicted token's phase starts at ``L + 1`` while its row index is ``L``
  (lines 732-735);
* the decode branch predicate adds the coefficient ROW count and the BATCH size
  (line 680: ``k_compressed.size(1)`` and ``k_local.size(0)``);
* layers whose prompt is not longer than ``maxlen`` keep everything in
  ``k_local`` and never compress later (lines 598-611, 681-686);
* ``_seen_tokens`` moves only at layer 0; ``maxtokens`` is clamped at layer-0
  prefill (lines 520-521, 541-542).

Arrays are numpy float64 holding values already rounded to the model dtype by
the caller; the statistics carry the reference's dtype casts.
"""
from __future__ import annotations

import json
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import fourier_oracle as fo


class OracleCache:
    def __init__(self, extra_config, masks: Optional[dict] = None, model_dtype: str = "bf16"):
        # cache_utils_fourier.py:391-403
        self._seen_tokens = 0
        self.key_cache: List[Dict[str, np.ndarray]] = []
        self.value_cache: List[Dict[str, np.ndarray]] = []
        self.maxnewtokens = extra_config.max_new_tokens
        self.maxlocallen = extra_config.maxlocallen
        self.maxmidstates = extra_config.maxmidstates
        self.numinittokens = extra_config.numinittokens
        self.maxlen = self.maxlocallen + self.maxmidstates + self.numinittokens
        self.heads = extra_config.num_key_value_heads
        self.maxtokens = extra_config.max_position_embeddings
        self.curr_tokennum: List[int] = []
        self.model_dtype = model_dtype
        if masks is None:
            with open(extra_config.non_critical_dims_path, "r") as f:
                masks = json.load(f)
        self.k_scale, self.v_scale = [], []
        self.k_layer_average, self.v_layer_average = [], []
        self.kd_layer_average, self.vd_layer_average = [], []
        self.k_non_critical_dims, self.k_non_critical_head_dims = [], []
        self.k_critical_dims, self.k_critical_head_dims = [], []
        self.v_non_critical_dims, self.v_non_critical_head_dims = [], []
        self.v_critical_dims, self.v_critical_head_dims = [], []
        i64 = np.int64
        for layer_idx in range(len(masks)):  # :433
            self.curr_tokennum.append(0)
            key = f"Layer_{layer_idx}"
            if key not in masks:
                raise ValueError(f"Layer index {layer_idx} not found in non-critical dimensions JSON file.")  # :455
            m = masks[key]
            self.k_non_critical_dims.append(np.asarray(m["kc_list"], dtype=i64))
            self.k_critical_dims.append(np.asarray(m["kn_list"], dtype=i64))
            self.v_non_critical_dims.append(np.asarray(m["vc_list"], dtype=i64))
            self.v_critical_dims.append(np.asarray(m["vn_list"], dtype=i64))
            self.k_non_critical_head_dims.append(np.asarray([0] + list(m["kc_h_list"]), dtype=i64))  # :449
            self.k_critical_head_dims.append(np.asarray([0] + list(m["kn_h_list"]), dtype=i64))
            self.v_non_critical_head_dims.append(np.asarray([0] + list(m["vc_h_list"]), dtype=i64))
            self.v_critical_head_dims.append(np.asarray([0] + list(m["vn_h_list"]), dtype=i64))

    def __len__(self):
        return len(self.key_cache)

    # -- helpers ---------------------------------------------------------------
    def _t_x(self) -> int:
        return self.maxtokens - self.numinittokens - self.maxlocallen

    def _compress_part(self, states, c_dims, n_dims):
        """Lines 556-569 for one tensor: split, gather, compress, statistics."""
        init = states[:, : self.numinittokens, :]
        local = states[:, -self.maxlocallen:, :]
        mid = states[:, self.numinittokens: -self.maxlocallen, :]
        unc = mid[:, :, n_dims]
        toc = mid[:, :, c_dims]
        coef = fo.compress_prefill(toc, self.n_f, self.t_c)
        scale, u_avg, i_avg = fo.prefill_stats(toc, coef, self._t_x(), self.model_dtype)
        return init, coef, unc, local, scale, u_avg, i_avg

    # -- update ----------------------------------------------------------------
    def update(self, key_states: np.ndarray, value_states: np.ndarray, layer_idx: int,
               cache_kwargs=None) -> Tuple[dict, dict]:
        """``key_states (B, Hkv, q, D)`` like the reference; returns ``(k_dict, v_dict)``."""
        if layer_idx == 0:
            self._seen_tokens += key_states.shape[-2]  # :520-521
        self.heads = key_states.shape[1]
        self.head_dim = key_states.shape[-1]
        bsz, q_len = key_states.shape[0], key_states.shape[-2]
        key_states = np.transpose(key_states, (0, 2, 1, 3)).reshape(bsz, q_len, -1)  # :529-534
        value_states = np.transpose(value_states, (0, 2, 1, 3)).reshape(bsz, q_len, -1)
        none3 = lambda t, loc: {f"{t}_init": None, f"{t}_compressed": None, f"{t}_uncompressed": None, f"{t}_local": loc}

        if len(self.key_cache) <= layer_idx:  # prefill of a new layer, :538
            if layer_idx == 0:  # :540-549
                self.prefilllen = q_len
                self.maxtokens = min(self.prefilllen + self.maxnewtokens, self.maxtokens)
                _, self.dt, self.t_c = fo.periods(self.maxtokens, self.numinittokens, self.maxlocallen)
                ck0 = self.k_non_critical_dims[0].shape[0]
                self.n_f = (ck0 * self.maxmidstates) // ck0 // 2  # TRI:854
            for _ in range(len(self.key_cache), layer_idx):  # skipped layers, :552-554
                self.key_cache.append([])
                self.value_cache.append([])
            self._prefill_layer(key_states, value_states, layer_idx, append=True)
            return none3("k", key_states), none3("v", value_states)  # :613

        if len(self.key_cache[layer_idx]) == 0:  # a previously skipped layer, :616
            self._prefill_layer(key_states, value_states, layer_idx, append=False)
            return none3("k", key_states), none3("v", value_states)

        kc, vc = self.key_cache[layer_idx], self.value_cache[layer_idx]
        k_init, k_comp, k_unc, k_local = kc["k_init"], kc["k_compressed"], kc["k_uncompressed"], kc["k_local"]
        v_init, v_comp, v_unc, v_local = vc["v_init"], vc["v_compressed"], vc["v_uncompressed"], vc["v_local"]
        # :680 - coefficient rows and batch size enter the predicate
        q_len = k_init.shape[1] + k_comp.shape[1] + k_unc.shape[1] + k_local.shape[0] + 1
        if q_len <= self.maxlen:  # :681-686
            k_local = np.concatenate([k_local, key_states], axis=1)
            v_local = np.concatenate([v_local, value_states], axis=1)
            kc["k_local"], vc["v_local"] = k_local, v_local
            return none3("k", k_local), none3("v", v_local)
        if q_len == self.maxlen + 1:  # :688-729
            raise NotImplementedError(
                "late-compression branch (cache_utils_fourier.py:688-729) appends a new layer entry "
                "instead of replacing this one; its behaviour is undefined and not restated")
        # streaming branch, :731-748
        self.curr_tokennum[layer_idx] += 1
        p = self.curr_tokennum[layer_idx]
        kcd, knd = self.k_non_critical_dims[layer_idx], self.k_critical_dims[layer_idx]
        vcd, vnd = self.v_non_critical_dims[layer_idx], self.v_critical_dims[layer_idx]
        k_comp = fo.coeff_update(k_comp, k_local[:, 0, :][:, kcd], p, self.t_c)
        k_unc = np.concatenate([k_unc, k_local[:, 0:1, :][:, :, knd]], axis=1)
        k_local = np.concatenate([k_local, key_states], axis=1)[:, 1:, :]
        v_comp = fo.coeff_update(v_comp, v_local[:, 0, :][:, vcd], p, self.t_c)
        v_unc = np.concatenate([v_unc, v_local[:, 0:1, :][:, :, vnd]], axis=1)
        v_local = np.concatenate([v_local, value_states], axis=1)[:, 1:, :]
        self.key_cache[layer_idx] = {"k_init": k_init, "k_compressed": k_comp, "k_uncompressed": k_unc, "k_local": k_local}
        self.value_cache[layer_idx] = {"v_init": v_init, "v_compressed": v_comp, "v_uncompressed": v_unc, "v_local": v_local}
        return dict(self.key_cache[layer_idx]), dict(self.value_cache[layer_idx])

    def _prefill_layer(self, key_states, value_states, layer_idx, append: bool):
        bsz, q_len, hidden = key_states.shape
        kcd, knd = self.k_non_critical_dims[layer_idx], self.k_critical_dims[layer_idx]
        vcd, vnd = self.v_non_critical_dims[layer_idx], self.v_critical_dims[layer_idx]
        if q_len > self.maxlen:  # :555
            k_init, k_comp, k_unc, k_local, ks, ku, kd = self._compress_part(key_states, kcd, knd)
            v_init, v_comp, v_unc, v_local, vs, vu, vd = self._compress_part(value_states, vcd, vnd)
            if append:
                self.k_scale.append(ks); self.k_layer_average.append(ku); self.kd_layer_average.append(kd)
                self.v_scale.append(vs); self.v_layer_average.append(vu); self.vd_layer_average.append(vd)
            else:
                self.k_scale[layer_idx] = ks; self.k_layer_average[layer_idx] = ku; self.kd_layer_average[layer_idx] = kd
                self.v_scale[layer_idx] = vs; self.v_layer_average[layer_idx] = vu; self.vd_layer_average[layer_idx] = vd
            self.curr_tokennum[layer_idx] += k_unc.shape[1]  # :593
        else:  # :598-611 - everything stays local, the other parts are empty placeholders
            e = lambda n: np.empty((bsz, 0, n), dtype=np.float32)
            k_init, k_comp, k_unc, k_local = e(hidden), e(kcd.shape[0]), e(knd.shape[0]), key_states
            v_init, v_comp, v_unc, v_local = e(hidden), e(vcd.shape[0]), e(vnd.shape[0]), value_states
        kd_ = {"k_init": k_init, "k_compressed": k_comp, "k_uncompressed": k_unc, "k_local": k_local}
        vd_ = {"v_init": v_init, "v_compressed": v_comp, "v_uncompressed": v_unc, "v_local": v_local}
        if append:
            self.key_cache.append(kd_); self.value_cache.append(vd_)
        else:
            self.key_cache[layer_idx] = kd_; self.value_cache[layer_idx] = vd_

    # -- bookkeeping surface (cache_utils_fourier.py:752-773) -----------------
    def get_seq_length(self, layer_idx: int = 0) -> int:
        empty = len(self.key_cache) == 0 or len(self.key_cache) <= layer_idx or len(self.key_cache[layer_idx]) == 0
        if empty:
            return 0
        c = self.key_cache[layer_idx]
        return c["k_init"].shape[-2] + c["k_uncompressed"].shape[-2] + c["k_local"].shape[-2]

    def get_max_cache_shape(self):
        return None

    def to_legacy_cache(self):
        return tuple((self.key_cache[i], self.value_cache[i]) for i in range(len(self)))

    # -- attention over the returned dicts (modeling_llama_fourier.py:623-661) --
    def attend(self, q, k_dict, v_dict, layer_idx, num_head_q, num_head_kv):
        """``q (B, Hq, 1, D)`` -> ``(B, Hq, 1, D)`` float64, dispatching like the attention forward:
        exact attention over ``k_local`` when the other three parts are ``None``."""
        b, hq, ql, d = q.shape
        if k_dict["k_init"] is None and k_dict["k_compressed"] is None and k_dict["k_uncompressed"] is None:
            assert ql == 1
            o = fo.softmax_attention(np.transpose(q, (0, 2, 1, 3)).reshape(b, hq * d), k_dict["k_local"],
                                     v_dict["v_local"], num_head_q, num_head_kv)
            return o[:, :, None, :]
        qf = np.transpose(q, (0, 2, 1, 3)).reshape(b, ql, hq * d)
        return fo.fourier_attn(
            qf, np.concatenate([k_dict["k_init"], k_dict["k_local"]], axis=1),
            np.concatenate([v_dict["v_init"], v_dict["v_local"]], axis=1),
            k_dict["k_compressed"], v_dict["v_compressed"], k_dict["k_uncompressed"], v_dict["v_uncompressed"],
            self.k_layer_average[layer_idx], self.kd_layer_average[layer_idx], self.k_scale[layer_idx],
            self.v_layer_average[layer_idx], self.vd_layer_average[layer_idx], self.v_scale[layer_idx],
            self.k_non_critical_dims[layer_idx], self.k_non_critical_head_dims[layer_idx],
            self.k_critical_dims[layer_idx], self.k_critical_head_dims[layer_idx],
            self.v_non_critical_dims[layer_idx], self.v_non_critical_head_dims[layer_idx],
            self.v_critical_dims[layer_idx], self.v_critical_head_dims[layer_idx],
            num_head_q, num_head_kv, k_dict["k_uncompressed"].shape[1], self._t_x())
