"""The build's compiler flags do what they are there for (CPU only: hipcc cross-compiles without a GPU)."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

from neuralattentionsearch_amd import build as nats_build

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# float2 arithmetic that hipcc -O3 turns into packed fp32 instructions when it is allowed to
SOURCE = r"""
#include <hip/hip_runtime.h>
__global__ void k(float2* a, const float2* b) {
  const int i = threadIdx.x;
  float2 x = a[i], y = b[i];
  x.x = x.x * y.x + 1.f;
  x.y = x.y * y.y + 1.f;
  a[i] = x;
}
"""


def device_isa(flags):
    with tempfile.TemporaryDirectory() as d:
        src, out = os.path.join(d, "k.hip"), os.path.join(d, "k.s")
        with open(src, "w") as f:
            f.write(SOURCE)
        subprocess.run([HIPCC, *flags, "--cuda-device-only", "-S", src, "-o", out], check=True, stderr=subprocess.DEVNULL)
        with open(out) as f:
            return f.read()


@pytest.mark.skipif(shutil.which(HIPCC) is None, reason="no hipcc")
def test_the_device_pass_takes_the_packed_fp32_switch():
    """The switch is handed to hipcc with -Xclang, which its x86 host pass answers with a note that it does not know
    the feature (build.py drops that one line).  The gfx950 pass does take it: the same source gives packed fp32
    instructions without the switch and none with it."""
    packed = re.compile(r"\bv_pk_(add|mul|fma)_f32\b")
    base = [f for f in nats_build.HIPCC_FLAGS if f not in ("-fPIC",)]
    assert not packed.search(device_isa(base))
    plain = [f for f in base if f not in ("-Xclang", "-target-feature", "-packed-fp32-ops")]
    assert packed.search(device_isa(plain)), "the probe kernel no longer forms packed instructions: it proves nothing"
