"""Every JITNN_HIP_* environment switch the library reads selects a code path of the product: each gets a slice of the
parity checks with the switch set, in a fresh child process (the switches are read once, at jitnn_hip_init), one child at
a time.  The list below is checked against the getenv calls of the library's source, so a switch cannot be added without
a test."""
import os
import re
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
KNOBS = {"JITNN_HIP_GEMV_MAX_ROWS": "8", "JITNN_HIP_GEMV_I8": "0", "JITNN_HIP_TRANSCODE": "0"}


def test_every_switch_of_the_source_is_listed():
    src = "".join(p.read_text() for p in (ROOT / "jitnn_amd" / "csrc").glob("*.h*"))
    assert set(re.findall(r'getenv\("(JITNN_HIP_[A-Z0-9_]+)"\)', src)) == set(KNOBS)


@pytest.mark.gpu
@pytest.mark.parametrize("knob", sorted(KNOBS))
def test_switch_in_a_fresh_process(knob):
    env = dict(os.environ)
    for k in KNOBS:
        env.pop(k, None)
    env[knob] = KNOBS[knob]
    r = subprocess.run([sys.executable, str(ROOT / "tests" / "knob_child.py"), knob], env=env, capture_output=True, text=True, timeout=110)
    assert r.returncode == 0 and "knob ok" in r.stdout, (r.stdout[-2000:], r.stderr[-4000:])
