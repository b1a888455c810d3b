"""Extract the integer golden vectors held by the reference's hand-run C++ test.

Source: layers/test.cpp:89-164 of the reference (one 4096-token sequence, n=64
blocks, 12 heads, 160 CTAs): the BigBird to-block CSR the kernel test feeds and
the LPT work plan `from_select_index(_position)`.  Only the numbers are taken
(data, not code); the output is `layers_test_n64_h12_cta160.json` beside this
script.  Run in the authoring container only:

    python tests/golden/extract_layers_test_vectors.py /root/reference
"""
import json
import os
import re
import sys


def grab(text, name):
    m = re.search(r"std::vector<int>\s+" + name + r"\s*=\s*\{([^}]*)\}", text)
    if m is None:
        raise SystemExit("vector %s not found" % name)
    return [int(t) for t in re.findall(r"-?\d+", m.group(1))]


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    with open(os.path.join(root, "layers", "test.cpp")) as f:
        lines = f.read().split("\n")
    text = "\n".join(lines[84:170])          # the live test_sparse_attention() literals only
    out = {
        "source": "layers/test.cpp:89-164",
        "n_blocks": 64, "heads": 12, "n_cta": 160,
        "to_select_index_position": grab(text, "to_select_index_position"),
        "to_select_index": grab(text, "to_select_index"),
        "from_select_index_position": grab(text, "from_select_index_position"),
        "from_select_index": grab(text, "from_select_index"),
    }
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "layers_test_n64_h12_cta160.json"), "w") as f:
        json.dump(out, f, separators=(",", ":"))
    print({k: (len(v) if isinstance(v, list) else v) for k, v in out.items()})


if __name__ == "__main__":
    main()
