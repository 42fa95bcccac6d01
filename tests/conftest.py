import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_sessionfinish(session, exitstatus):
    """A proof of an unseen statement over large tables starts a compilation of its kernels in the background; the
    session waits for the last of them, so that the process ends in the ordinary way."""
    lib = sys.modules.get("sable_amd.lib")
    if lib is not None and getattr(lib, "_lib", None) is not None:
        lib._lib.exh_stmt_generate_idle(1)


@pytest.fixture(scope="session")
def vectors():
    """The reference's golden vectors (tests/vectors.sexp converted by tests/golden/make_vectors.py)."""
    with open(os.path.join(ROOT, "tests", "golden", "vectors.json")) as f:
        data = json.load(f)

    def of(kind):
        out = [v for v in data if v["kind"] == kind]
        assert out, f"no test vectors of kind {kind}"
        return out

    return of


def launch_names(step):
    """The names of the launches `step` makes, from the library's own launch timing (GPU tests)."""
    import ctypes as C

    import sable_amd as sa
    lib = sa.load()
    sa.check(lib.exh_profile_enable(1))
    try:
        step()
        names = []
        for i in range(lib.exh_profile_count()):
            name = C.create_string_buffer(64)
            rnd, ms, nbytes = C.c_int(), C.c_float(), C.c_uint64()
            sa.check(lib.exh_profile_entry(i, name, 64, C.byref(rnd), C.byref(ms), C.byref(nbytes)))
            names.append(name.value.decode())
    finally:
        sa.check(lib.exh_profile_enable(0))
    return names
