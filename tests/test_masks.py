"""Index-list rules: bit-exact against the mask data the reference ships."""
import glob
import hashlib
import json
import os

import pytest

from fourierattention_amd import masks as pm
from oracle import masks_oracle as mo

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference/compressed_dims_file"


def _extract():
    return json.load(open(os.path.join(HERE, "golden", "masks_extract.json")))


def test_golden_extract_rule_oracle_and_product():
    ex = _extract()
    n = 0
    for stem, blob in ex.items():
        for key, pair in blob["layers"].items():
            raw, split = pair["raw"], pair["splithead"]
            want = {k: split[k] for k in pm.LAYER_KEYS}
            got_o = mo.splithead_layer(raw["self_attn.k_proj"], raw["self_attn.v_proj"], 8, 128)
            got_p = pm.layer_from_compressed(raw["self_attn.k_proj"], raw["self_attn.v_proj"], 8, 128)
            assert got_o == want and got_p == want, (stem, key)
            pm.validate_layer(split, 8, 128)
            n += 1
    assert n == 5


def test_percent_schedule_matches_list_lengths():
    ex = _extract()
    blob = ex["llama3.2-3b-fourier/compressed_dims_4k_fourier"]["layers"]
    for key, pair in blob.items():
        layer = int(key.split("_")[1])
        assert len(pair["raw"]["self_attn.k_proj"]) == int(mo.percent_schedule(layer, "k") * 1024)
        assert len(pair["raw"]["self_attn.v_proj"]) == int(mo.percent_schedule(layer, "v") * 1024)
    # every layer of that file, both band edges (3 | 4 and 19 | 20) and the 0.8 band between them
    lengths = ex["llama3.2-3b-fourier/compressed_dims_4k_fourier"]["raw_lengths"]
    assert len(lengths) == 28
    for key, (nk, nv) in lengths.items():
        layer = int(key.split("_")[1])
        assert (nk, nv) == (int(mo.percent_schedule(layer, "k") * 1024), int(mo.percent_schedule(layer, "v") * 1024)), key
    assert lengths["Layer_3"] == [921, 972] and lengths["Layer_4"] == [819, 819]
    assert lengths["Layer_19"] == [819, 819] and lengths["Layer_20"] == [512, 716]


def test_selection_rule():
    mse = [0.5, -0.1, 0.3, 0.05, -0.7, 0.2, 0.0, 0.9, 0.4, 0.6]
    assert mo.select_noncritical(mse, 0.5) == [6, 3, 1, 5, 2]
    assert mo.select_noncritical(mse, 0.95) == [6, 3, 1, 5, 2, 8, 0, 9, 4]


def test_synthetic_masks_are_valid_and_seeded():
    a = pm.synthetic_masks(3, 8, 128, 64, seed=0)
    b = pm.synthetic_masks(3, 8, 128, 64, seed=0)
    c = pm.synthetic_masks(3, 8, 128, 64, seed=1)
    assert a == b and a != c
    for key, entry in a.items():
        pm.validate_layer(entry, 8, 128)
        assert entry["kc_h_list"] == [64 * (h + 1) for h in range(8)]
        assert len(entry["kc_list"]) == 512 and len(entry["vn_list"]) == 512
    r = pm.synthetic_masks(1, 4, 16, 0, 16)["Layer_0"]
    assert r["kc_list"] == [] and r["kn_h_list"] == [16, 32, 48, 64] and r["vn_list"] == []
    # one count per head (masks whose heads differ, like the reference's own)
    e = pm.synthetic_masks(1, 4, 16, [3, 0, 16, 7], [16, 1, 2, 0], seed=2)["Layer_0"]
    pm.validate_layer(e, 4, 16)
    assert e["kc_h_list"] == [3, 3, 19, 26] and e["vc_h_list"] == [16, 17, 19, 19]
    with pytest.raises(ValueError):
        pm.synthetic_masks(1, 4, 16, [3, 0, 16])


def test_validate_rejects_inconsistent():
    e = pm.synthetic_masks(1, 2, 8, 4)["Layer_0"]
    bad = dict(e); bad["kc_h_list"] = [1, 2]
    with pytest.raises(ValueError):
        pm.validate_layer(bad, 2, 8)
    bad = dict(e); bad["kn_list"] = e["kn_list"][:-1]
    with pytest.raises(ValueError):
        pm.validate_layer(bad, 2, 8)


@pytest.mark.skipif(not os.path.isdir(REF), reason="reference tree not mounted")
def test_every_reference_pair():
    """All raw/splithead pairs in the reference obey the rule, except the one whose
    splithead file is a byte copy of another configuration's."""
    pairs = 0
    for split_path in sorted(glob.glob(os.path.join(REF, "*", "*_splithead.json"))):
        raw_path = split_path.replace("_splithead", "")
        split = json.load(open(split_path)); raw = json.load(open(raw_path))
        conv = pm.splithead_from_raw(raw, 8, 128)
        same = all({k: split[key][k] for k in pm.LAYER_KEYS} == conv[key] for key in conv)
        if split_path.endswith("32k_2048states_splithead.json"):
            twin = split_path.replace("2048states", "512states")
            assert hashlib.sha256(open(split_path, "rb").read()).digest() == hashlib.sha256(open(twin, "rb").read()).digest()
            assert not same
        else:
            assert same, split_path
        for key in split:
            pm.validate_layer(split[key], 8, 128)
        pairs += 1
    assert pairs == 8
