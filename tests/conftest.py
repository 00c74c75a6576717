import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line('markers', 'gpu: needs a real MI355X (run with -m gpu)')


@pytest.fixture(scope='session')
def pack_oracle_c():
    """The C restatement of the reference pack/unpack kernels, built on demand."""
    import subprocess
    so = os.path.join(ROOT, 'oracle', 'libpack_oracle.so')
    if not os.path.exists(so):
        subprocess.check_call(['make', '-C', os.path.join(ROOT, 'oracle')])
    from oracle import pack_oracle
    return pack_oracle
