"""Writes tests/golden/io/*.bin with the reference's own converter
(tools/read_convert_mm.cpp, built by `make -C oracle ref` into oracle/_ref/conv2bin)
from the small MatrixMarket files next to them.  The .mtx files are this
repository's own test inputs; the .bin files are the reference's outputs for
them.  Run in the build container only:

    python tests/golden/make_golden_io.py
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
IO = os.path.join(HERE, "io")
CONV = os.path.join(os.path.dirname(os.path.dirname(HERE)), "oracle", "_ref", "conv2bin")

FILES = {
    "general.mtx": """%%MatrixMarket matrix coordinate real general
% 6 x 5, 9 entries, unsorted, one repeated position
6 5 9
1 2 1.5
2 1 -2.25
2 5 3.0
3 3 4.125
4 4 5e-3
5 2 6.0
6 1 7.0
6 5 -8.5
3 3 9.0
""",
    "symmetric.mtx": """%%MatrixMarket matrix coordinate real symmetric
%
% lower triangle with two diagonal entries
5 5 6
1 1 2.0
2 1 -1.0
3 2 0.5
4 4 3.0
5 1 1e10
5 4 -0.125
""",
    "pattern_symmetric.mtx": """%%MatrixMarket matrix coordinate pattern symmetric
4 4 4
2 1
3 1
4 3
4 4
""",
    "complex.mtx": """%%MatrixMarket matrix coordinate complex general
3 4 3
1 4 1.0 2.0
2 2 -3.5 0.25
3 1 0.0 -1.0
""",
    "integer.mtx": """%%MatrixMarket matrix coordinate integer general
2 3 2
1 3 7
2 1 -4
""",
}


def main():
    assert os.path.exists(CONV), "build it first: make -C oracle ref"
    os.makedirs(IO, exist_ok=True)
    for name, text in FILES.items():
        path = os.path.join(IO, name)
        with open(path, "w") as f:
            f.write(text)
        out = path[:-4] + ".bin"
        subprocess.run([CONV, "-o", out, path], check=True)
        print(name, "->", os.path.basename(out), os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
