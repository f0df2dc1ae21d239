"""The streamed TernGrad encode requests rows of its register ring with hand-written loads whose destination the
compiler believes to be written at once (ring_request / ring_wait in csrc/hpx_terngrad.hip).  That is only sound
if, in the code the compiler made, nothing touches a row's registers between the request and the wait for it, and
if no part of the ring was spilled.  This test reads the device assembly of the library's own build flags and checks
both, for every width and rounding mode.  CPU only: hipcc cross-compiles."""
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "torch-hipress-extension_amd", "csrc")


def _regs(text):
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", text):
        if m.group(1):
            out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


@pytest.fixture(scope="module")
def isa():
    target = os.path.join(CSRC, "build", "hpx_terngrad.s")
    r = subprocess.run(["make", "-C", CSRC, target], capture_output=True, text=True)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    return open(target).read()


def _kernels(isa):
    return re.findall(r"^(_ZN\S*terngrad_resident_kernel\S*):[^\n]*\n(.*?)^\.Lfunc_end", isa, re.S | re.M)


def test_ring_rows_are_left_alone_between_request_and_wait(isa):
    streamed = 0
    for name, body in _kernels(isa):
        pending = {}
        requests = waits = 0
        for i, line in enumerate(body.split("\n")):
            code = line.split(";")[0].strip()
            if "ring request" in line:
                dst = re.search(r"global_load_dwordx4 (v\[\d+:\d+\])", line).group(1)
                sources = _regs(code.split(",", 1)[1])
                assert not (sources & set(pending)), (name, i, line)
                for r in _regs(dst):
                    pending[r] = i
                requests += 1
            elif "ring wait" in line:
                for r in _regs(re.search(r"ring wait (v\[\d+:\d+\])", line).group(1)):
                    pending.pop(r, None)
                waits += 1
            elif code.startswith("s_waitcnt vmcnt(0)"):
                pending.clear()
            elif code and not code.endswith(":") and not code.startswith("."):
                hit = _regs(code) & set(pending)
                assert not hit, f"{name}: line {i} `{code}` names registers {sorted(hit)} of a row that is still on its way"
        if requests:
            streamed += 1
            # every ring row: one request in the first trip, one in the loop; one wait in the loop, one at the end
            assert requests == waits and requests % 2 == 0, (name, requests, waits)
            assert not pending, (name, pending)
    assert streamed == 8, streamed  # 1, 2, 4, 8 bits x both rounding modes


def test_no_streamed_kernel_spills_in_its_loop(isa):
    """Spilled registers are legal, but a spill of a ring row between request and wait would store what is not there
    yet: the streamed kernels are allowed scratch only outside the ring's life (the 8-bit stochastic one keeps a few
    addresses there during the first trip)."""
    for name, body in _kernels(isa):
        if "ring request" not in body:
            continue
        lines = body.split("\n")
        loop_requests = [i for i, l in enumerate(lines) if "ring request" in l]
        # the loop's requests are the second half (the first trip comes first in program order)
        first_loop_request = loop_requests[len(loop_requests) // 2]
        scratch_in_loop = [l for l in lines[first_loop_request:] if re.search(r"\bscratch_(load|store)", l)]
        # reloads of values spilled before the loop are harmless; stores inside it would be ring-adjacent pressure
        assert not [l for l in scratch_in_loop if "scratch_store" in l], (name, scratch_in_loop[:4])
