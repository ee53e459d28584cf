import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run on the GPU box)")

# torch first: it brings its own HIP runtime, and the engine library must share that copy rather
# than load a second one into the process.
try:
    import torch  # noqa: F401,E402
except Exception:  # pragma: no cover - CPU-only environments without torch
    torch = None
