"""Writes tests/golden/ir/<kernel>.ir from spoc_amd.reference_kernels (the Sarek IR of the
reference's benchmark kernels; each file is pinned by tests/golden/generated/<kernel>.cuda.txt,
which the HIP lowering of the IR has to reproduce).

    python tests/golden/make_ir.py
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from spoc_amd.reference_kernels import KERNELS  # noqa: E402

OUT = os.path.join(HERE, "ir")


def main():
    os.makedirs(OUT, exist_ok=True)
    for name, fn in KERNELS.items():
        with open(os.path.join(OUT, name + ".ir"), "w") as f:
            f.write(fn())
        print("wrote", name)


if __name__ == "__main__":
    main()
