"""The C ABI called from a plain C program (tests/native/c_abi_check.c, built by __graft_entry__.build()):
hipMalloc'd buffers, a user stream, results checked inside the program against a scalar restatement."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, 'native', 'c_abi_check')


def test_c_program_calls_the_library():
    if not os.path.exists(BINARY):
        pytest.skip('tests/native/c_abi_check has not been built (python -c "import __graft_entry__ as g; g.build()")')
    lib_dir = os.path.join(os.path.dirname(HERE), 'lava-dl_amd', 'slayer')
    env = dict(os.environ, LD_LIBRARY_PATH=lib_dir + ':/opt/rocm/lib:' + os.environ.get('LD_LIBRARY_PATH', ''))
    run = subprocess.run([BINARY], env=env, capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stdout + run.stderr
    assert 'c abi ok' in run.stdout
