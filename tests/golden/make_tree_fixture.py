"""Writes tests/golden/array_tree_first24.txt: the first 24 of the 1101 sentiment trees that the reference's evaluation
ships as data (src/out/PLDI19evaluation/treelstm/lantern/array_tree.txt: tree count, then per tree its size and the four
arrays scores / words / left child / right child), in the same text format.  Run where /root/reference exists:

    python tests/golden/make_tree_fixture.py
"""
import os

SRC = "/root/reference/src/out/PLDI19evaluation/treelstm/lantern/array_tree.txt"
DST = os.path.join(os.path.dirname(os.path.abspath(__file__)), "array_tree_first24.txt")
KEEP = 24


def main():
    lines = open(SRC).read().split("\n")
    assert int(lines[0]) >= KEEP
    out, pos = [str(KEEP)], 1
    for _ in range(KEEP):
        out.extend(lines[pos:pos + 5])          # size line + four arrays
        pos += 5
    open(DST, "w").write("\n".join(out) + "\n")
    print("wrote", DST, "with", KEEP, "trees")


if __name__ == "__main__":
    main()
