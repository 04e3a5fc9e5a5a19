"""The first launch of a kernel variant may happen while a stream is being captured: esp_attn_init has
already raised every variant's dynamic LDS limit, so nothing but launches is recorded."""
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu


def test_first_launch_of_a_variant_inside_a_capture():
    script = os.path.join(os.path.dirname(os.path.abspath(__file__)), "capture_first_launch.py")
    print("starting capture_first_launch.py in a process of its own", flush=True)
    r = subprocess.run([sys.executable, "-u", script], capture_output=True, text=True, timeout=300)
    print(r.stdout[-2000:], r.stderr[-2000:], flush=True)
    assert r.returncode == 0 and "capture_first_launch: ok" in r.stdout
