"""The C ABI driven by a plain C++ program (tests/cabi_consumer.cpp: no Python, no torch,
its own hipMalloc'd buffers) and checked inside that program against the C oracle."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cabi_consumer")


def _binary():
    if not os.path.exists(BINARY):
        subprocess.check_call(["make", "-C", HERE])
    return BINARY


@pytest.mark.gpu
def test_cabi_consumer_matches_oracle():
    r = subprocess.run([_binary()], capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "cabi consumer ok" in r.stdout, r.stdout[-4000:] + r.stderr[-2000:]


def test_cabi_consumer_links_and_reports_a_missing_gpu():
    """Without a GPU the program must get as far as asking for one: that proves that it links
    against every entry point it uses and that nothing in the library runs at load time."""
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present; the GPU test covers the program")
    r = subprocess.run([_binary()], capture_output=True, text=True, timeout=110)
    assert r.returncode == 2 and "no GPU" in r.stdout, r.stdout[-2000:] + r.stderr[-2000:]
