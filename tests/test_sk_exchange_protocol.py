"""The arrival-flag protocol of the in-launch split-K exchange, run on CPU threads.

``juliavision_amd/csrc/sk_exchange.hpp`` is instantiated twice: by the HIP kernel over agent-scope atomics, and by
``tests/sk_exchange_host_test.cpp`` over host atomics with one thread per wave.  The host program covers what a GPU
test must not provoke: a partner that arrives after the bound (the waiters report it and release nothing, the bank
stays dirty until the host zeroes it), a partner on another XCD, replays that carry the same epoch, the 28-bit wrap.
"""
import os
import subprocess
import tempfile

HERE = os.path.dirname(os.path.abspath(__file__))


def test_protocol_on_host_threads():
    src = os.path.join(HERE, "sk_exchange_host_test.cpp")
    with tempfile.TemporaryDirectory() as tmp:
        exe = os.path.join(tmp, "sk_exchange_host_test")
        subprocess.run(["g++", "-O1", "-std=c++17", "-pthread", src, "-o", exe], check=True)
        r = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    lines = r.stdout.strip().splitlines()
    assert len(lines) == 8 and all(l.endswith("ok") for l in lines), r.stdout
