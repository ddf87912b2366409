"""What the compiler made of the MFMA kernels, read on the host (no GPU): no MFMA instruction may
stand where the wave can arrive with an EXEC mask of zeros.

The compiler lowers a branch whose condition it cannot prove to be the same for the whole wave
into a mask: ``s_and_saveexec`` switches the lanes off for which the condition is false, and for
a short block it leaves out the jump over it (``s_cbranch_execz``), because instructions without
active lanes do nothing. MFMA is the exception: it does not look at EXEC. A wave for which the
condition is false then runs the product anyway, on operands whose loads were masked off. This
has happened here (an accumulator met registers never loaded and a NaN now and then); the cure is
conditions the compiler knows to be uniform (``uniform_wave_number`` in ``common.h``). The scan
below finds the pattern in the assembly of every MFMA source at two head sizes.
"""

import re
import shutil
import subprocess

import pytest

from qwen3_runtime_amd.ops import build

HIPCC = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"


def mfma_under_empty_mask(assembly: str):
    """(kernel, line) of every MFMA that follows a ``saveexec`` with no label, no jump on EXEC and
    no restoring of EXEC in between: the wave may arrive there with no lane switched on."""
    kernel, unguarded, hits = None, False, []
    for number, line in enumerate(assembly.splitlines(), 1):
        text = line.strip()
        if re.match(r"^_Z\w+:", text):
            kernel, unguarded = text.rstrip(":"), False
        if "saveexec" in text:
            unguarded = True
        elif text.startswith(".LBB") or "s_cbranch_exec" in text or re.search(r"s_(or|mov)_b64 exec", text):
            unguarded = False
        elif "v_mfma" in text and unguarded:
            hits.append((kernel, number))
    return hits


def test_the_scan_sees_the_pattern():
    bad = """
_Z6kernelv:
    s_and_saveexec_b64 s[0:1], s[24:25]
; %bb.61:
    v_mfma_f32_16x16x32_bf16 v[22:25], v[58:61], v[34:37], v[22:25]
    s_or_b64 exec, exec, s[0:1]
"""
    good = bad.replace("; %bb.61:", "    s_cbranch_execz .LBB0_2\n; %bb.61:")
    assert mfma_under_empty_mask(bad) == [("_Z6kernelv", 5)]
    assert mfma_under_empty_mask(good) == []


@pytest.mark.parametrize("source,defines", [
    ("attention_bf16.hip", ["-DQRT_HEAD_DIM=16"]),
    ("attention_bf16.hip", ["-DQRT_HEAD_DIM=128"]),
    ("gemm_bf16.hip", []),
])
def test_no_mfma_where_exec_may_be_zero(source, defines, tmp_path):
    out = tmp_path / "device.s"
    flags = [f for f in build.FLAGS if f != "-fPIC"]
    cmd = [HIPCC, *flags, f"-I{build.CSRC}", *defines, "--cuda-device-only", "-S", str(build.CSRC / source), "-o", str(out)]
    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assembly = out.read_text()
    assert "v_mfma" in assembly
    assert mfma_under_empty_mask(assembly) == []
