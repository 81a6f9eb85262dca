"""pytest configuration: the ``gpu`` marker and import paths.

Tests marked ``gpu`` need an MI355X and the built HIP library; everything else runs
on the CPU (oracle pins, host logic, C-ABI symbol checks)."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (gfx950) and the built HIP library")
