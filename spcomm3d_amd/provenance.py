"""Which device code a measurement was taken on.

``source_hash()`` is a digest of the sources the HIP library is built from
(``spcomm3d_amd/csrc``: ``*.hip``, ``*.cpp``, ``*.h`` and the Makefile).  Profile
summaries record it in their header; ``bench.py`` quotes figures from a summary only
while the digest still matches, and a test compares the two.

``python3 -m spcomm3d_amd.provenance`` prints the digest.
"""
import hashlib
import os

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
SUFFIXES = (".hip", ".cpp", ".h")
MARK = "Source hash:"


def source_files():
    names = sorted(n for n in os.listdir(CSRC) if n.endswith(SUFFIXES) or n == "Makefile")
    return [os.path.join(CSRC, n) for n in names]


def source_hash() -> str:
    h = hashlib.sha256()
    for path in source_files():
        h.update(os.path.basename(path).encode() + b"\0")
        with open(path, "rb") as f:
            h.update(f.read())
        h.update(b"\0")
    return h.hexdigest()[:16]


def recorded_hash(profile_path: str):
    """The digest a profile summary names in its header, or None."""
    try:
        with open(profile_path) as f:
            for line in f:
                if MARK in line:
                    return line.split(MARK, 1)[1].strip().strip("`. ").split("`")[0].split()[0]
    except OSError:
        pass
    return None


if __name__ == "__main__":
    print(source_hash())
