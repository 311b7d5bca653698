"""Extract golden vectors from outputs stored in the reference's notebooks.

Reads the notebooks as JSON text (nothing from the reference is imported or
run) and writes ``notebook_vectors.json`` next to this script:

* ``sample/router/generate_indices.ipynb`` cells 0-2: a 16x4 hot mask, its
  seat ("dst") indices, the 0-based tag ("src") list printed by an older kernel
  build, a row-shuffled seat matrix with its converted tag list, and the loads;
* same notebook, cell 4: a ``throttle_hotmask`` case (mask, prefix, threshold,
  throttled mask, returned prefix);
* ``sample/cpp/dispatch.ipynb`` cell 0: the printed loads for T=2048, E=4,
  top-2 routing with capacities [64..2048] and capacity padding.

Usage: python tests/golden/extract_notebook_vectors.py [/root/reference]
"""
import json
import os
import re
import sys


def tensors_in(text):
    """All integer tensors printed in ``text`` as nested lists."""
    out = []
    for m in re.finditer(r"tensor\((\[.*?\])(?:,\s*(?:device|dtype)=[^)]*)*\)", text, re.S):
        body = m.group(1)
        if "..." in body:
            out.append(None)
            continue
        out.append(json.loads(body))
    return out


def cell_text(cell):
    chunks = []
    for o in cell.get("outputs", []):
        if "text" in o:
            chunks.append("".join(o["text"]))
    return "\n".join(chunks)


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    nb = json.load(open(os.path.join(ref, "sample/router/generate_indices.ipynb")))
    cells = nb["cells"]
    (mask,) = tensors_in(cell_text(cells[0]))
    seat, tag0 = tensors_in(cell_text(cells[1]))
    shuffled_seat, loads, shuffled_tag0 = tensors_in(cell_text(cells[2]))
    t4 = tensors_in(cell_text(cells[4]))
    thr_mask, thr_colsum, throttled, throttled_colsum, new_prefix = t4
    src4 = "".join(cells[4]["source"])
    prefix = json.loads(re.search(r"prefix = torch.tensor\((\[.*?\])", src4).group(1))
    threshold = json.loads(re.search(r"threshold = torch.tensor\((\[.*?\])", src4).group(1))

    nb2 = json.load(open(os.path.join(ref, "sample/cpp/dispatch.ipynb")))
    t0 = tensors_in(cell_text(nb2["cells"][0]))
    dispatch_loads = [t for t in t0 if t is not None][-1]
    caps = [int(float(v)) for v in re.search(
        r"supported_capacities = torch.Tensor\(\[(.*?)\]\)", "".join(nb2["cells"][0]["source"])
    ).group(1).split(",")]

    out = {
        "source": {
            "generate_indices": "sample/router/generate_indices.ipynb (cells 0,1,2,4, stored outputs)",
            "dispatch": "sample/cpp/dispatch.ipynb (cell 0, stored outputs)",
        },
        "generate_indices": {
            "mask": mask,
            "seat_indices": seat,
            "tag_indices_zero_based_legacy": tag0,
            "loads": loads,
            "shuffled_seat_indices": shuffled_seat,
            "shuffled_tag_indices_zero_based_legacy": shuffled_tag0,
        },
        "throttle": {
            "mask": thr_mask,
            "mask_colsum": thr_colsum,
            "prefix": prefix,
            "threshold": threshold,
            "throttled": throttled,
            "throttled_colsum": throttled_colsum,
            "new_prefix": new_prefix,
        },
        "dispatch_loads": {
            "T": 2048, "E": 4, "top_k": 2,
            "supported_capacities": caps,
            "capacity_padding": True,
            "padded_loads": dispatch_loads,
        },
    }
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "notebook_vectors.json")
    with open(dst, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", dst)


if __name__ == "__main__":
    main()
