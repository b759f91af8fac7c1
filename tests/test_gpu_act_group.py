"""RQ_ACT_GROUP = 128 / 256 (reference patch lines 2623-2631): the variable is read once per process, so each width
runs in a child process (a plain script, one GPU process at a time)."""
import os
import subprocess
import sys

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


@pytest.mark.gpu
@pytest.mark.parametrize("G", [128, 256])
def test_activation_groups_wider_than_64(G):
    env = dict(os.environ)
    env["RQ_ACT_GROUP"] = str(G)
    out = subprocess.run([sys.executable, "-u", os.path.join(HERE, "act_group_case.py")], env=env,
                         capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and "ALL OK" in out.stdout, out.stdout[-3000:] + out.stderr[-2000:]
