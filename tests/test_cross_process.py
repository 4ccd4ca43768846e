"""Two agents in two processes on the same GPU: the initiator maps the target's VRAM through
the IPC handle in the target's published metadata, WRITEs and READs it, and its notification
arrives through the target's shared-memory mailbox after the bytes.  The two sides are fresh
child programs (tests/xproc_peer.py)."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))


def test_write_read_and_notify_between_two_processes(cuda, tmp_path):
    env = dict(os.environ, HSA_ENABLE_IPC_MODE_LEGACY="0")
    peer = os.path.join(HERE, "xproc_peer.py")
    target = subprocess.Popen([sys.executable, "-u", peer, "target", str(tmp_path)], stdout=subprocess.PIPE,
                              stderr=subprocess.STDOUT, text=True, env=env)
    initiator = subprocess.Popen([sys.executable, "-u", peer, "initiator", str(tmp_path)], stdout=subprocess.PIPE,
                                 stderr=subprocess.STDOUT, text=True, env=env)
    try:
        out_i, _ = initiator.communicate(timeout=150)
        out_t, _ = target.communicate(timeout=60)
    finally:
        for p in (target, initiator):
            if p.poll() is None:
                p.kill()
    assert initiator.returncode == 0 and "initiator OK" in out_i, out_i
    # the forged blob was turned down for the right reason (the backend's own error line)
    assert "forged blob refused" in out_i and "does not fit the allocation it names" in out_i, out_i
    assert target.returncode == 0 and "target OK" in out_t, out_t
