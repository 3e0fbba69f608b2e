"""Writes tests/golden/fast_builds_vs_strict.json on a machine with an MI355X: every speed build bench.py times outside
the config 4 chain (config 5 decode, plain and row-scaled; config 5 row-scaled prefill; the config 2 dequantising
pair) against its strict build at the benchmark's size, over all outputs (tests/fast_builds.py).

    python tests/golden/make_fast_builds_report.py [output.json]
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import x17ai_amd as X
from tests import fast_builds


def main():
	out_path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(ROOT, "tests", "golden", "fast_builds_vs_strict.json")
	dev = X.Device(0)
	rep = {"device": dev.name, "fast_vs_strict": fast_builds.report(dev)}
	with open(out_path, "w") as f:
		json.dump(rep, f, indent=1)
		f.write("\n")
	print(json.dumps(rep))


if __name__ == "__main__":
	main()
