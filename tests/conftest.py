import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
	sys.path.insert(0, ROOT)


def pytest_configure(config):
	config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
	config.addinivalue_line("markers", "slow: minutes of CPU work; set X17_SLOW=1 to run")


def pytest_collection_modifyitems(config, items):
	if os.environ.get("X17_SLOW") == "1":
		return
	skip = pytest.mark.skip(reason="slow golden run; set X17_SLOW=1")
	for item in items:
		if "slow" in item.keywords:
			item.add_marker(skip)
