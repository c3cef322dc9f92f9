"""TEST INFRASTRUCTURE: __graft_entry__.smoke() on the fake device of fake_cuda.py."""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, HERE)

import fake_cuda  # noqa: E402

fake_cuda.activate()
import __graft_entry__  # noqa: E402

__graft_entry__.smoke()
print("smoke dry run: passed")
