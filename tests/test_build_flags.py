"""The build's ``-packed-fp32-ops`` target feature is a device-pass flag: hipcc's host pass (x86) prints "not a
recognized feature" for it, the gfx950 pass honours it.  Compiled for the device only, a float2 multiply-add becomes a
packed instruction without the flag and scalar ones with it."""
import importlib.util
import os
import re
import subprocess
import tempfile

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
spec = importlib.util.spec_from_file_location("mfsdp_build", os.path.join(ROOT, "matrix-fsdp_amd", "csrc", "build.py"))
build = importlib.util.module_from_spec(spec)
spec.loader.exec_module(build)

SOURCE = """
#include <hip/hip_runtime.h>
__global__ void k(float2* a, const float2* b, float s) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  float2 x = a[i], y = b[i];
  x.x = x.x * s + y.x;
  x.y = x.y * s + y.y;
  a[i] = x;
}
"""
PACKED = re.compile(r"\bv_pk_(fma|mul|add)_f32\b")


@pytest.mark.skipif(not os.path.exists(build.HIPCC), reason="hipcc not installed")
def test_packed_fp32_feature_is_honoured_by_the_device_pass():
    feature = ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
    assert all(f in build.FLAGS for f in feature)
    with tempfile.TemporaryDirectory() as tmp:
        src = os.path.join(tmp, "probe.hip")
        with open(src, "w") as f:
            f.write(SOURCE)

        def assembly(flags):
            out = os.path.join(tmp, "probe.s")
            subprocess.run([build.HIPCC, "--offload-arch=gfx950", "-O3", "-S", "--offload-device-only", *flags, src, "-o", out],
                           check=True, stdout=subprocess.PIPE, stderr=subprocess.STDOUT)
            return open(out).read()

        assert PACKED.search(assembly([])), "the probe no longer compiles to a packed op without the flag: it proves nothing"
        assert not PACKED.search(assembly(feature))
