"""Writes tests/golden/small.tiny (megcc_amd.tiny.write_model on tests/tiny_cases.small_model) and
tests/golden/small.tiny.txt = what the REFERENCE's generated reader
(runtime/src/cheader/model_reader.h, through oracle/_ref/ref_tiny_dump) sees in that file. Needs
`make -C oracle ref`, i.e. the reference tree.

    python tests/golden/make_tiny.py
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))

from megcc_amd import tiny  # noqa: E402
from oracle import ref  # noqa: E402
import tiny_cases  # noqa: E402


def main():
    path = os.path.join(HERE, "small.tiny")
    with open(path, "wb") as f:
        f.write(tiny.write_model(tiny_cases.small_model()))
    text = ref.tiny_dump(path)
    with open(path + ".txt", "w") as f:
        f.write(text)
    print("%s: %d bytes, %d lines" % (path, os.path.getsize(path), text.count("\n")))


if __name__ == "__main__":
    main()
