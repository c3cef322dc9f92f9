"""TEST INFRASTRUCTURE: bench.py from argument parsing to its JSON line on the fake device of
fake_cuda.py (emulated kernels, host clock for events, no graph capture) with a batch of one
example.  The figures mean nothing; what this checks is that every code path of the benchmark runs
and that its JSON line has the fields the driver reads.  Takes several minutes.
    python tests/emu/bench_dry_run.py [extra bench.py flags, e.g. --small-extras or --no-extras --no-cpu]"""
import io
import json
import os
import sys
from contextlib import redirect_stdout

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))
sys.path.insert(0, HERE)

import fake_cuda  # noqa: E402

fake_cuda.activate()
import bench  # noqa: E402

if "--candidates" in sys.argv:          # started by bench.py itself: its child process, same device
    sys.argv = ["bench.py"] + sys.argv[1:]
    bench.main()
    sys.exit(0)
bench.CANDIDATE_COMMAND = [sys.executable, os.path.abspath(__file__)]
sys.argv = ["bench.py", "--batch", "1", "--steps", "1", "--warmup", "0"] + sys.argv[1:]
buf = io.StringIO()
with redirect_stdout(buf):
    bench.main()
line = buf.getvalue().strip().splitlines()[-1]
d = json.loads(line)
for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
            "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "parity",
            "enqueue_ms_per_step", "step_variants", "forward_write_out", "kernels"):
    assert key in d, key
for key in ("bound", "achieved", "peak", "unit", "frac", "traffic"):
    assert key in d["roofline"], key
print(json.dumps({k: d[k] for k in ("value", "ms_per_step", "launch", "step_variants", "forward_write_out", "kernels")}, indent=1))
print("bench dry run: JSON line complete")
