"""Writes tests/golden/lenet_asymu8.npz: the trained parameter blob and the 28x28 input
image that the reference's LeNet sample carries as C arrays (samples/lenet/
lenet_asymu8_weights.h:24 `lenet_weights[432820]`, samples/lenet/lenet_asymu8.cc:41
`input_data`). Only the numbers are taken, parsed from the text; nothing is compiled or run.
The sample holds no expected output (it prints a top-5), so the fixture has none either.

Usage: python tests/golden/make_lenet_fixture.py [/root/reference]
"""
import os
import re
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def numbers_after(text, marker):
    start = text.index(marker)
    body = text[text.index("{", start) + 1:text.index("};", start)]
    return [int(tok, 0) for tok in re.findall(r"0x[0-9a-fA-F]+|\d+", body)]


def main():
    ref = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    w = numbers_after(open(os.path.join(ref, "samples/lenet/lenet_asymu8_weights.h")).read(),
                      "lenet_weights[")
    x = numbers_after(open(os.path.join(ref, "samples/lenet/lenet_asymu8.cc")).read(),
                      "input_data =")
    assert len(w) == 432820 and len(x) == 28 * 28, (len(w), len(x))
    np.savez_compressed(os.path.join(HERE, "lenet_asymu8.npz"),
                        weights=np.array(w, dtype=np.uint8), input=np.array(x, dtype=np.uint8))
    print("wrote lenet_asymu8.npz: weights", len(w), "input", len(x))


if __name__ == "__main__":
    main()
