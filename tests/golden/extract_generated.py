"""Copies the CUDA section of the reference's golden generated-kernel files
(benchmarks/descriptions/generated/*_generated.md, kept current by the reference's CI job
`check-generated-code`) into tests/golden/generated/<kernel>.cuda.txt.

These are expected OUTPUTS of the reference's IR->source lowering, used as fixtures: for
kernels that use no warp-level construct the HIP lowering must emit the same text.
Run in the build container only (the reference tree is not present on the GPU box):
    python tests/golden/extract_generated.py
"""
import glob
import os
import re

REF = "/root/reference/benchmarks/descriptions/generated"
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "generated")


def main():
    os.makedirs(OUT, exist_ok=True)
    for path in sorted(glob.glob(os.path.join(REF, "*_generated.md"))):
        text = open(path).read()
        m = re.search(r"## CUDA C\s*```cuda\n(.*?)```", text, flags=re.S)
        if not m:
            continue
        name = os.path.basename(path)[: -len("_generated.md")]
        with open(os.path.join(OUT, name + ".cuda.txt"), "w") as f:
            f.write(m.group(1))
        print("wrote", name)


if __name__ == "__main__":
    main()
