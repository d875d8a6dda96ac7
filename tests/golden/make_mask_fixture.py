"""Writes tests/golden/masks_extract.json: a few layers of the reference's mask data
files (raw search output next to its splithead form).  Data only; run in the build
container where the reference tree is mounted:

    python tests/golden/make_mask_fixture.py
"""
import json
import os

SRC = "/root/reference/compressed_dims_file"
HERE = os.path.dirname(os.path.abspath(__file__))
PICK = {
    "llama3.1-8b-fourier/compressed_dims_32k_1024states": [0, 15, 31],
    "llama3.2-3b-fourier/compressed_dims_4k_fourier": [0, 27],
}


def main():
    out = {}
    for stem, layers in PICK.items():
        raw = json.load(open(os.path.join(SRC, stem + ".json")))
        split = json.load(open(os.path.join(SRC, stem + "_splithead.json")))
        # lengths of the raw lists of every layer: they pin the per-layer fraction schedule of the search
        lengths = {k: [len(raw[k]["self_attn.k_proj"]), len(raw[k]["self_attn.v_proj"])] for k in sorted(raw, key=lambda s: int(s.split("_")[1]))}
        out[stem] = {"num_layers": len(split), "raw_lengths": lengths, "layers": {}}
        for l in layers:
            key = f"Layer_{l}"
            out[stem]["layers"][key] = {"raw": raw[key], "splithead": split[key]}
    with open(os.path.join(HERE, "masks_extract.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))


if __name__ == "__main__":
    main()
