"""Writes ``mace_symmetric_contraction.json`` next to this script.

The vectors are the ones the reference's own test holds
(``cuequivariance_torch/tests/operations/symmetric_contraction_test.py:77-124``): an input, the weights and
the output of the ORIGINAL MACE implementation of the symmetric contraction (``4x(0e+1o+2e) -> 4x(0e+1o)``,
correlation 3, 2 elements, e3nn conventions), base64 of float32.  The reference file is read as text and
only the data strings are kept.
"""

import json
import re
from pathlib import Path

SRC = Path("/root/reference/cuequivariance_torch/tests/operations/symmetric_contraction_test.py")


def main():
    text = SRC.read_text()
    blobs = re.findall(r'"([A-Za-z0-9+/=]{40,})"', text)
    assert len(blobs) == 3
    out = {
        "source": "cuequivariance_torch/tests/operations/symmetric_contraction_test.py:77-124",
        "mul": 4,
        "irreps_in": "0e + 1o + 2e",
        "irreps_out": "0e + 1o",
        "contraction_degree": 3,
        "num_elements": 2,
        "layout_in": "ir_mul",
        "layout_out": "mul_ir",
        "indices": [0, 1, 0],
        "x": {"shape": [3, 36], "float32_base64": blobs[0]},
        "expected_output": {"shape": [3, 16], "float32_base64": blobs[1]},
        "weight": {"shape": [2, 41, 4], "float32_base64": blobs[2]},
        "atol": 1e-5,
        "rtol": 1e-5,
    }
    (Path(__file__).parent / "mace_symmetric_contraction.json").write_text(json.dumps(out, indent=1) + "\n")


if __name__ == "__main__":
    main()
