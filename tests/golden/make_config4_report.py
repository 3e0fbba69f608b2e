"""Writes tests/golden/config4_fast_vs_strict.json on a machine with an MI355X: benchmark config 4 as one chain
(tests/config4_chain.py), the strict builds checked against the CPU oracle, then per stage the speed build against
the strict one -- mismatch histogram, max-abs and relative-L2 difference over the whole tensors.

    python tests/golden/make_config4_report.py [output.json]
"""
import json
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

import x17ai_amd as X
from tests import config4_chain as C


def main():
	out_path = sys.argv[1] if len(sys.argv) > 1 else os.path.join(ROOT, "tests", "golden", "config4_fast_vs_strict.json")
	dev = X.Device(0)
	inp = C.inputs()
	got = C.run_strict(dev, inp)
	checked = C.check_strict(inp, got)
	rep = {"workload": f"config 4: {C.B} x {C.T} tokens, d_model {C.D}, {C.H} heads x {C.HD}, window {C.W}, d_ff {C.F}",
	       "device": dev.name, "strict_vs_oracle": checked, "fast_vs_strict": C.fast_vs_strict(dev, inp, got)}
	with open(out_path, "w") as f:
		json.dump(rep, f, indent=1)
		f.write("\n")
	print(json.dumps(rep))


if __name__ == "__main__":
	main()
