#!/usr/bin/env python3
"""Copies the data files the data-feed tests need from the reference's test data into
tests/golden/molgrid_data: the example lists, the type maps, the ligand cache and the
pre-typed structure files that the first lines of the lists name.  Data only; run once:

    python tests/golden/make_provider_fixtures.py /root/reference/test/data
"""
import os
import shutil
import sys

LISTS = {"small.types": 120, "ligonly.types": 60, "grouped.types": None, "multilig.types": None}
PLAIN = ["recmap", "emap", "gnina35.recmap", "gnina35.ligmap", "lig.molcache2"]


def main(src):
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "molgrid_data")
    os.makedirs(os.path.join(dst, "structs"), exist_ok=True)
    needed = set()
    for name, lines in LISTS.items():
        shutil.copyfile(os.path.join(src, name), os.path.join(dst, name))
        with open(os.path.join(src, name)) as f:
            for i, line in enumerate(f):
                if lines is not None and i >= lines:
                    break
                needed.update(tok for tok in line.split() if tok.endswith(".gninatypes"))
    for name in PLAIN:
        shutil.copyfile(os.path.join(src, name), os.path.join(dst, name))
    for rel in sorted(needed):
        out = os.path.join(dst, "structs", rel)
        os.makedirs(os.path.dirname(out), exist_ok=True)
        shutil.copyfile(os.path.join(src, "structs", rel), out)
    print("copied %d structure files" % len(needed))


if __name__ == "__main__":
    main(sys.argv[1])
