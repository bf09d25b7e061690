"""Static check of the one hazard the compiler cannot see.

The dK/dV kernel emits its S / dP MFMAs by hand (accumulators pinned to the architectural VGPRs), so
the compiler's hazard recogniser does not insert the wait states an 8-pass MFMA needs before the
vector ALU may touch its result.  The kernel is structured so that at least two further MFMAs are
issued first; this test compiles the library to assembly and verifies that for every such MFMA."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

from flame_amd import build as fb

SRC = os.path.join(fb.CSRC, "flame_attn.hip")


def _regs(tok):
    m = re.match(r"v\[(\d+):(\d+)\]", tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", tok)
    return {int(m.group(1))} if m else set()


@pytest.mark.skipif(shutil.which(fb.HIPCC) is None and not os.path.exists(fb.HIPCC), reason="hipcc not available")
def test_hand_emitted_mfma_results_are_not_touched_too_early():
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "flame_attn.s")
        flags = [f for f in fb.FLAGS if f not in ("-shared", "-fPIC")]
        subprocess.run([fb.HIPCC, *flags, "-S", "--cuda-device-only", SRC, "-o", out], check=True,
                       stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        text = open(out).read()
    kernels = re.findall(r"^(_ZN5fattn15bwd_dkdv_kernel\w+):.*?\.end_amdhsa_kernel", text, re.S | re.M)
    assert len(kernels) >= 4
    checked = 0
    for name in kernels:
        body = re.search(r"^%s:.*?\.end_amdhsa_kernel" % re.escape(name), text, re.S | re.M).group(0)
        ins = [l.strip() for l in body.split("\n") if re.match(r"^\s+[a-z]", l)]
        for idx, l in enumerate(ins):
            if not l.startswith("v_mfma"):
                continue
            ops = [t.strip() for t in l.split(None, 1)[1].split(",")]
            if not ops[0].startswith("v["):        # accumulator in the accumulation registers: compiler-managed
                continue
            checked += 1
            dst = _regs(ops[0])
            later_mfma = 0
            for l2 in ins[idx + 1:]:
                if l2.startswith("v_mfma"):
                    later_mfma += 1
                    if later_mfma >= 2:
                        break
                    continue
                if l2.startswith("s_") or l2.startswith("ds_read") or l2.startswith("global_load_lds"):
                    continue                        # scalar, or vector registers used as addresses / LDS destinations only
                used = set()
                for t in re.findall(r"v\[\d+:\d+\]|v\d+", l2):
                    used |= _regs(t)
                assert not (used & dst), f"{name}: `{l2}` touches the result of `{l}` before two more MFMAs"
    assert checked >= 4 * 96
