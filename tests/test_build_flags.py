"""The device-side compiler flags of megray_amd/build.py do what the build relies on (no GPU needed: hipcc
cross-compiles gfx950 and the checks read the generated device assembly of a probe kernel)."""
import os
import re
import subprocess

from megray_amd import build

PROBE = r"""
#include <hip/hip_runtime.h>
__global__ void probe(float2* a, const float2* b, const float2* c) {
    int i = threadIdx.x;
    float2 x = a[i], y = b[i], z = c[i];
    x.x += y.x; x.y += y.y;
    x.x *= z.x; x.y *= z.y;
    x.x = x.x * y.x + z.x; x.y = x.y * y.y + z.y;
    a[i] = x;
}
"""

PACKED = re.compile(r"\bv_pk_(add|mul|fma)_f32\b")
FUSED = re.compile(r"\bv_(fma|fmac|mad|mac)_f32\b|\bv_pk_fma_f32\b")


def device_asm(tmp_path, flags):
    src = tmp_path / "probe.hip"
    src.write_text(PROBE)
    out = tmp_path / "probe.s"
    cmd = [build.HIPCC, "-x", "hip", "-O3", "-S", "--cuda-device-only", f"--offload-arch={build.ARCH}", str(src), "-o", str(out)] + flags
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr
    return out.read_text()


def test_packed_fp32_flag_acts_on_device_code(tmp_path):
    """Without the feature flag hipcc -O3 turns the float2 arithmetic into packed fp32 instructions; with the
    flags the library is built with it emits none (the host pass's "not a recognized feature" is about the host
    target only)."""
    device_flags = [f for f in build.DEVICE_FLAGS if not f.startswith("--offload-arch")]
    assert "-packed-fp32-ops" in device_flags
    plain = device_asm(tmp_path, [])
    assert PACKED.search(plain), "the probe no longer provokes packed fp32 code: the test proves nothing"
    guarded = device_asm(tmp_path, device_flags)
    assert not PACKED.search(guarded)


def test_contraction_is_off(tmp_path):
    """A fold is a chain of single IEEE operations: a * b + c must stay a multiply and an add."""
    assert "-ffp-contract=off" in build.COMMON_FLAGS
    device_flags = [f for f in build.DEVICE_FLAGS if not f.startswith("--offload-arch")]
    plain = device_asm(tmp_path, device_flags)
    assert FUSED.search(plain), "the probe no longer provokes a fused multiply-add: the test proves nothing"
    guarded = device_asm(tmp_path, device_flags + ["-ffp-contract=off"])
    assert not FUSED.search(guarded)
