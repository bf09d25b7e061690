"""Static checks of the hazards the compiler cannot see, on the library compiled to assembly.

1. The dK/dV kernel and the 256-query forward and dQ kernels emit their logit MFMAs by hand (accumulators
   pinned to the architectural VGPRs),
   so the compiler's hazard recogniser does not insert the wait states an 8-pass MFMA needs before
   anything else may touch its result.  The kernels are structured so that at least two further MFMAs
   (or, off the hot paths, 11 wait states of s_nop) are issued first.
2. The LDS-DMA copies are emitted by hand as well and take their LDS destination from M0: every one of
   them must find, in its own basic block, an s_mov_b32 to M0 with at least one instruction in between
   (the wait state between a scalar write of M0 and an LDS-DMA that reads it)."""
import os
import re
import shutil
import subprocess
import tempfile

import pytest

from flame_amd import build as fb

SRC = os.path.join(fb.CSRC, "flame_attn.hip")


def _regs(tok, file="v"):
    m = re.match(r"%s\[(\d+):(\d+)\]" % file, tok)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"%s(\d+)$" % file, tok)
    return {int(m.group(1))} if m else set()


@pytest.fixture(scope="module")
def text():
    if shutil.which(fb.HIPCC) is None and not os.path.exists(fb.HIPCC):
        pytest.skip("hipcc not available")
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "flame_attn.s")
        flags = [f for f in fb.FLAGS if f not in ("-shared", "-fPIC")]     # the flags the library is built with
        subprocess.run([fb.HIPCC, *flags, "-S", "--cuda-device-only", SRC, "-o", out], check=True,
                       stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        return open(out).read()


def test_checks_run_on_the_compiler_that_built_the_library():
    """The assembly inspected here comes from this machine's hipcc; the shipped library records the hipcc
    that built it.  The checks say nothing about the library unless the two are the same compiler."""
    import ctypes
    lib_path = fb.LIB_PATH
    if not os.path.exists(lib_path):
        pytest.skip("library not built")
    if shutil.which(fb.HIPCC) is None and not os.path.exists(fb.HIPCC):
        pytest.skip("hipcc not available")
    lib = ctypes.CDLL(lib_path)
    lib.flame_attn_version.restype = ctypes.c_char_p
    built_with = lib.flame_attn_version().decode()
    assert f"(hipcc {fb.hipcc_version()})" in built_with, (built_with, fb.hipcc_version())


def test_hand_emitted_mfma_results_are_not_touched_too_early(text):
    """The result of a hand-emitted MFMA (architectural accumulator, or the big-head-dim forward's pinned accumulation
    tuples) may be touched only after two more MFMAs or 11 wait states of s_nop.  Followed along the control flow:
    an unconditional branch to its target, a conditional one both ways."""
    kernels = re.findall(r"^(_ZN5fattn(?:15bwd_dkdv_kernel|18bwd_dq_wide_kernel|15fwd_wide_kernel|20sage_fwd_wide_kernel|15fwd_bigd_kernel)\w+):.*?\.end_amdhsa_kernel", text, re.S | re.M)
    assert len(kernels) >= 9
    checked = 0
    for name in kernels:
        body = re.search(r"^%s:.*?\.end_amdhsa_kernel" % re.escape(name), text, re.S | re.M).group(0)
        # instructions and labels, in order
        ins = [l.strip() for l in body.split("\n") if re.match(r"^\s+[a-z]", l) or re.match(r"^\.LBB\S+:", l)]
        label_at = {re.match(r"(\.LBB\w+):", l).group(1): i for i, l in enumerate(ins) if l.startswith(".LBB")}
        for idx, l in enumerate(ins):
            if not l.startswith("v_mfma"):
                continue
            ops = [t.strip() for t in l.split(None, 1)[1].split(",")]
            # an accumulator in the accumulation registers is the compiler's own MFMA form, which it guards itself,
            # except in the big-head-dim forward, which emits its O^T MFMAs by hand into pinned a[0:127]
            by_hand_acc = "fwd_bigd_kernel" in name and ops[0].startswith("a[")
            if not ops[0].startswith("v[") and not by_hand_acc:
                continue
            checked += 1
            dst = _regs(ops[0], "a" if by_hand_acc else "v")
            todo = [(idx + 1, 0, 0)]                    # (position, MFMAs since, wait states spent in s_nop since)
            seen = set()
            while todo:
                pos, later_mfma, idle = todo.pop()
                while pos < len(ins) and pos not in seen:
                    seen.add(pos)
                    l2 = ins[pos]
                    pos += 1
                    if l2.startswith(".LBB"):
                        continue
                    if l2.startswith("v_mfma"):
                        later_mfma += 1
                        if later_mfma >= 2:
                            break
                        continue
                    m = re.match(r"s_nop\s+(\d+)", l2)
                    if m:
                        idle += int(m.group(1)) + 1
                        if idle >= 11:                  # an 8-pass result is visible 11 wait states after issue
                            break
                        continue
                    if l2.startswith("s_endpgm"):
                        break
                    m = re.match(r"s_(c?)branch\w*\s+(\.LBB\S+)", l2)
                    if m:
                        if m.group(1):
                            todo.append((label_at[m.group(2)], later_mfma, idle))     # taken; not taken goes on below
                            continue
                        pos = label_at[m.group(2)]
                        continue
                    if l2.startswith("s_") or l2.startswith("global_load_lds"):
                        continue                        # scalar, or vector registers used as addresses only
                    if by_hand_acc:
                        used = set()
                        for t in re.findall(r"\ba\[\d+:\d+\]|\ba\d+\b", l2):
                            used |= _regs(t, "a")
                    else:
                        toks = re.findall(r"v\[\d+:\d+\]|v\d+", l2)
                        if l2.startswith("ds_read"):
                            toks = toks[:1]             # the destination; the other register is an address
                        used = set()
                        for t in toks:
                            used |= _regs(t)
                    assert not (used & dst), f"{name}: `{l2}` touches the result of `{l}` before two more MFMAs"
    assert checked >= 4 * 96


def test_operands_of_hand_emitted_mfmas_are_not_written_just_before(text):
    """An MFMA may read a register the vector ALU wrote two wait states later at the earliest.  The compiler keeps
    that distance for its own MFMAs; for the hand-emitted ones (architectural accumulator, or the big-head-dim
    forward's pinned accumulation tuples) it must come from the statement itself (an s_nop in front) or from where
    the operands live (pinned registers that nothing moves).  Checked on every MFMA of every kernel: no vector-ALU
    instruction within the two wait states in front of it writes one of its source registers."""
    kernels = re.findall(r"^(_ZN5fattn\w+):.*?\.end_amdhsa_kernel", text, re.S | re.M)      # every kernel of the library
    checked = 0
    for name in kernels:
        body = re.search(r"^%s:.*?\.end_amdhsa_kernel" % re.escape(name), text, re.S | re.M).group(0)
        ins = [l.strip() for l in body.split("\n") if re.match(r"^\s+[a-z]", l)]
        for idx, l in enumerate(ins):
            if not l.startswith("v_mfma"):
                continue
            ops = [t.strip() for t in l.split(None, 1)[1].split(",")]      # the compiler's own MFMAs pass by construction
            checked += 1
            src_v, src_a = set(), set()
            for t in ops[1:4]:
                src_v |= _regs(t, "v")
                src_a |= _regs(t, "a")
            states = 0
            for l2 in reversed(ins[max(0, idx - 4):idx]):
                m = re.match(r"s_nop\s+(\d+)", l2)
                if m:
                    states += int(m.group(1)) + 1
                elif l2.startswith("v_") and not l2.startswith("v_mfma"):
                    dst = l2.split(None, 1)[1].split(",")[0].strip()
                    wrote = (_regs(dst, "v") & src_v) | (_regs(dst, "a") & src_a)
                    assert not wrote, f"{name}: `{l2}` writes an operand of `{l}` {states} wait states before it"
                    states += 1
                else:
                    states += 1
                if states >= 2:
                    break
    assert checked >= 4 * 96


def test_every_lds_dma_finds_its_destination_in_m0(text):
    kernels = re.findall(r"^(_ZN5fattn\w+):.*?\.end_amdhsa_kernel", text, re.S | re.M)
    assert kernels
    checked = 0
    for name in kernels:
        body = re.search(r"^%s:.*?\.end_amdhsa_kernel" % re.escape(name), text, re.S | re.M).group(0)
        # instructions and labels, in order
        ins = [l.strip() for l in body.split("\n") if re.match(r"^\s+[a-z]", l) or re.match(r"^\.LBB\S+:", l)]
        for idx, l in enumerate(ins):
            if not l.startswith("global_load_lds"):
                continue
            checked += 1
            between = 0
            for l2 in reversed(ins[:idx]):
                assert not l2.startswith(".LBB"), f"{name}: `{l}` has no M0 write in its basic block"
                if re.match(r"s_mov_b32\s+m0,", l2):
                    break
                assert "m0" not in l2.split(";")[0], f"{name}: `{l2}` uses M0 between its write and `{l}`"
                between += 1
            else:
                raise AssertionError(f"{name}: `{l}` has no M0 write before it")
            assert between >= 1, f"{name}: `{l}` follows its M0 write without a wait state"
    assert checked >= 100
