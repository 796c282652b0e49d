import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionstart(session):
    """The tests load what is built; they build only when nothing is (a fresh
    checkout: the libraries are build products and not in the repository)."""
    built = [os.path.join(ROOT, "tfjs_amd", "lib", "libtfjs_hip.so"), os.path.join(ROOT, "oracle", "liboracle.so")]
    if not all(os.path.exists(p) for p in built):
        import __graft_entry__
        __graft_entry__.build()
