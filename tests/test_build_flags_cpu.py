"""The device code must hold no packed fp32 arithmetic (v_pk_add_f32, v_pk_mul_f32, v_pk_fma_f32): the
build switches the feature off with a target-feature flag, whose effect is checked here on a probe that
the compiler does pack when left alone.  hipcc cross-compiles for gfx950 without a GPU."""
import os
import re
import subprocess
import tempfile

from fastmax_amd import build

PROBE = """
#include <hip/hip_runtime.h>
__global__ void probe(const float2* a, const float2* b, float2* c, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) { float2 x = a[i], y = b[i]; c[i] = make_float2(x.x * y.x + 1.5f, x.y * y.y + 1.5f); }
}
"""


def _packed_ops(flags):
    with tempfile.TemporaryDirectory() as tmp:
        src, out = os.path.join(tmp, "probe.hip"), os.path.join(tmp, "probe.s")
        with open(src, "w") as f:
            f.write(PROBE)
        subprocess.run([build.HIPCC, "--offload-arch=gfx950", "-O3", "--cuda-device-only", "-S", src, "-o", out, *flags],
                       check=True, capture_output=True)
        return len(re.findall(r"\bv_pk_(?:add|mul|fma)_f32\b", open(out).read()))


def test_packed_fp32_is_switched_off_in_device_code():
    feature = [f for f in build.HIP_FLAGS if f in ("-Xclang", "-target-feature", "-packed-fp32-ops")]
    assert feature == ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
    assert _packed_ops([]) > 0          # the probe is one the compiler packs when allowed to
    assert _packed_ops(feature) == 0    # and does not with the library's flags
