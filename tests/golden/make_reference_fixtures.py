"""Re-type the data tables that the reference's own tests hold for this path into
tests/golden/reference_fixtures.json.  The reference files are read as TEXT (the
numbers between the brackets are parsed with a regex); nothing is imported or run.

    python tests/golden/make_reference_fixtures.py [/root/reference]

Tables taken:
  SELECTED_EXPERTS_B8_E256 / SELECTED_EXPERTS_B22_E256  python/test/fused_moe.py:30-62
  err_data (256-value permutation)  python/regression/test_llm/test_noaux_tc_topk.py:116-138
"""
import json
import os
import re
import sys


def grab(text, name, closing):
    start = text.index(name)
    start = text.index("[", start)
    end = text.index(closing, start)
    return [float(v) for v in re.findall(r"-?\d+\.?\d*", text[start:end])]


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    moe = open(os.path.join(root, "python/test/fused_moe.py")).read()
    topk = open(os.path.join(root, "python/regression/test_llm/test_noaux_tc_topk.py")).read()
    b8 = [int(v) for v in grab(moe, "SELECTED_EXPERTS_B8_E256", "dtype")]
    b22 = [int(v) for v in grab(moe, "SELECTED_EXPERTS_B22_E256", "dtype")]
    err = grab(topk, "err_data = ", "]")
    assert len(b8) == 8 * 8 and len(b22) == 22 * 8 and len(err) == 256
    out = {
        "SELECTED_EXPERTS_B8_E256": [b8[i * 8:(i + 1) * 8] for i in range(8)],
        "SELECTED_EXPERTS_B22_E256": [b22[i * 8:(i + 1) * 8] for i in range(22)],
        "noaux_tc_topk_err_data": err,
        "moe_shapes_T_H_I_E_K": [[1, 7168, 256, 1, 1], [1, 7168, 256, 2, 2], [1, 7168, 256, 16, 8],
                                 [1, 7168, 256, 256, 8], [8, 7168, 256, 256, 8], [256, 7168, 256, 256, 8]],
        "noaux_tc_topk_cases_batch_groups_topkgroups_topk": [[1, 8, 4, 8], [8, 8, 4, 8], [16, 8, 4, 8],
                                                             [64, 8, 4, 8], [128, 8, 4, 8]],
    }
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_fixtures.json")
    with open(path, "w") as f:
        json.dump(out, f, indent=1)
    print("wrote", path)


if __name__ == "__main__":
    main()
