"""What the compiler made of the decode-batch kernel's loop, read from its assembly (compiled
here for gfx950; no GPU needed).  The kernel keeps two buffers of weight loads in flight and
waits for them one by one (``s_waitcnt vmcnt(7)`` down to ``vmcnt(4)`` with four loads a
buffer).  A load that ends up inside a branch, or a select of two addresses that the compiler
turns into one, makes it wait for every load in flight before each product instead
(``vmcnt(0)``): the results stay right and the kernel takes a microsecond more, which no test of
its numbers shows.  This test does."""

import os
import re
import shutil
import subprocess
import tempfile

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "..", "kllm_amd", "csrc")


def _hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    return None


def _kernels(asm: str):
    """(mangled name, instructions) of every kernel of the decode-batch template."""
    lines = asm.split("\n")
    for i, line in enumerate(lines):
        if line.startswith("_ZN4kllm19fused_linear_kernel") and ": ; @" in line:
            body = []
            for l in lines[i + 1:]:
                body.append(l.strip())
                if "s_endpgm" in l:
                    break
            yield line.split(":")[0], body


def test_the_decode_batch_kernel_keeps_its_loads_in_flight():
    hipcc = _hipcc()
    if hipcc is None:
        pytest.skip("hipcc is not here")
    from kllm_amd.csrc.build import FLAGS
    flags = [f for f in FLAGS if f != "-fPIC"]
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "fused_linear.s")
        env = dict(os.environ, TMPDIR=tmp)
        p = subprocess.run([hipcc, *flags, "-I", CSRC, "-S", "--cuda-device-only",
                            os.path.join(CSRC, "fused_linear.hip"), "-o", out],
                           capture_output=True, text=True, env=env, timeout=600)
        assert p.returncode == 0, p.stderr[-2000:]
        asm = open(out).read()
    seen = 0
    for name, body in _kernels(asm):
        seen += 1
        waits, last = [], None
        for ins in body:
            m = re.match(r"s_waitcnt .*vmcnt\((\d+)\)", ins)
            if m:
                last = int(m.group(1))
            if ins.startswith("v_mfma"):
                if last is not None:
                    waits.append(last)
                last = None
        assert waits, name
        # every product waits for its own buffer's loads only: four to seven others stay in flight
        assert min(waits) >= 4, f"{name}: the loop waits for all loads in flight (vmcnt {sorted(set(waits))})"
    assert seen >= 24          # rows in one or two tiles x four epilogues (two of them also scaled) x one pass or several
