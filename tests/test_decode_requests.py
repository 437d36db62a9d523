"""The fused decode kernel requests its K rows with load instructions the compiler
does not track (pluto_amd/csrc/gqa_decode.hip: request_rows / wait_for_rows) and
waits for them with hand-counted vmcnt values.  The hardware delivers such a
load whenever it arrives: an instruction that touches the destination registers
before the matching wait (a copy the register allocator thought harmless, a
spill) would read or overwrite them half-way.  The source ties every use to the
wait; this test checks what the compiler made of it, without a GPU: it
compiles the file to gfx950 assembly with the library's own flags and walks
every instantiation of the kernel, keeping the queue of outstanding vector
memory operations as s_waitcnt vmcnt(n) sees it (operations complete in order;
loads, stores and LDS fills share the counter).

The walk is linear: it follows the text, not the branches.  The request/wait
pairs sit in straight-line, fully unrolled code, which is what makes that
good enough; a violation inside it cannot be hidden by a branch elsewhere."""
import os
import re
import shutil
import subprocess

import pytest

from pluto_amd import build

SOURCE = os.path.join(build.CSRC, "gqa_decode.hip")
VMEM = ("global_load", "global_store", "global_atomic", "buffer_load", "buffer_store",
        "buffer_atomic", "scratch_", "flat_")


def registers(token):
    for pattern, base in ((r"v\[(\d+):(\d+)\]", 0), (r"a\[(\d+):(\d+)\]", 1000)):
        m = re.fullmatch(pattern, token)
        if m:
            return {base + r for r in range(int(m.group(1)), int(m.group(2)) + 1)}
    for pattern, base in ((r"v(\d+)", 0), (r"a(\d+)", 1000)):
        m = re.fullmatch(pattern, token)
        if m:
            return {base + int(m.group(1))}
    return set()


def walk(lines, start):
    """Returns (explicit requests seen, [(line number, text)] of instructions that
    touch a requested register before its wait) for the function at `start`."""
    in_asm, queue, requests, problems = False, [], 0, []
    for number in range(start + 1, len(lines)):
        text = lines[number].strip()
        if text.startswith(".Lfunc_end"):
            break
        if text.startswith(";;#ASMSTART"):
            in_asm = True
            continue
        if text.startswith(";;#ASMEND"):
            in_asm = False
            continue
        code = text.split(";")[0].strip()
        if not code or code.startswith(".") or code.endswith(":"):
            continue
        op, _, rest = code.partition(" ")
        if op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", code)
            if m and len(queue) > int(m.group(1)):
                queue = queue[len(queue) - int(m.group(1)):]
            continue
        tokens = [t.strip().split(" ")[0] for t in rest.split(",")] if rest else []
        used = set().union(*[registers(t) for t in tokens]) if tokens else set()
        pending = set().union(*[r for r in queue]) if queue else set()
        if used & pending:
            problems.append((number + 1, code))
        if op.startswith(VMEM):
            explicit = in_asm and op == "global_load_dwordx4"
            requests += explicit
            queue.append(registers(tokens[0]) if explicit else set())
    return requests, problems


@pytest.mark.skipif(shutil.which(build.HIPCC) is None and not os.path.exists(build.HIPCC),
                    reason="needs hipcc")
def test_no_instruction_touches_a_requested_register_before_its_wait(tmp_path):
    listing = tmp_path / "gqa_decode.s"
    flags = [f for f in build.DEVICE_FLAGS if f != "-fPIC"]
    done = subprocess.run([build.HIPCC] + flags + ["-S", "--cuda-device-only", SOURCE, "-o",
                                                   str(listing)],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert done.returncode == 0, done.stdout[-2000:]
    lines = listing.read_text().split("\n")
    kernels = [i for i, l in enumerate(lines)
               if re.match(r"^_ZN9pluto_hip.*decode_fused_kernelILi\d+ELi\d+EEE.*:\s*;", l)]
    # three head widths x five group sizes
    assert len(kernels) == 15
    total = 0
    for start in kernels:
        requests, problems = walk(lines, start)
        name = lines[start].split(":")[0]
        assert not problems, (name, problems[:5])
        # a compile-time block size takes the explicit requests (both variants of the
        # block, with and without the appended row): 8 or 16 groups of D / 32 loads
        assert requests > 0, name
        total += requests
    # widths 64 and 128: 8 groups x (2 or 4) loads x 2 variants; width 256: 16 x 8 x 2
    assert total == 5 * (8 * 2 * 2 + 8 * 4 * 2 + 16 * 8 * 2)
