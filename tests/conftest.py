import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "jax-flash-attn2_amd"), os.path.join(ROOT, "oracle"), ROOT):
	if p not in sys.path:
		sys.path.insert(0, p)


def pytest_configure(config):
	config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
