"""Static check of the matrix-core convolution's machine code (no GPU needed).

The kernel starts its vector memory loads by hand and waits for them later with s_waitcnt
vmcnt(N).  Between the load and the wait that covers it, the destination registers hold stale
data and the hardware will still write them: any other instruction that reads or writes such a
register in that window is a bug the compiler cannot see (it takes the inline-asm load for an
ordinary definition), and the symptom is a wrong result or a wild address on the GPU.  The test
compiles the kernel file to ISA and walks every path of every kernel's control flow graph with
the queue of loads in flight."""
import os
import re
import subprocess

import pytest

from xnor_nn_amd import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE = os.path.join(ROOT, "xnor_nn_amd", "csrc", "kernels_conv_mfma.hip")

# Variants the host never launches because they do not fit the register file (pick_ps in the
# kernel file): 4 pixel blocks with 16 steps per tap, or with tap pairing over 5 words.  Their
# spill code moves registers around while loads are in flight.
NEVER_LAUNCHED = re.compile(r"conv_mfma_fp4_kernelILi(16ELi4ELb[01]ELb0|5ELi4ELb[01]ELb1)E")


def vgprs(token):
    token = token.strip().rstrip(",")
    m = re.match(r"v\[(\d+):(\d+)\]$", token)
    if m:
        return frozenset(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", token)
    return frozenset({int(m.group(1))}) if m else frozenset()


def parse(body):
    """One tuple per line: (kind, registers touched, load destination, vmcnt, branch target)."""
    label_at = {l[:-1]: i for i, l in enumerate(body) if l.startswith(".LBB")}
    out = []
    for line in body:
        if line.startswith(".LBB"):
            out.append(("label", None, None, None, None))
            continue
        op = line.split()[0]
        ops = [o for o in re.split(r"[ ,]+", line)[1:] if o]
        if op == "s_endpgm":
            out.append(("end", None, None, None, None))
        elif op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", line)
            out.append(("wait", None, None, int(m.group(1)) if m else None, None))
        elif op.startswith("s_cbranch") or op == "s_branch":
            out.append(("jump" if op == "s_branch" else "branch", None, None, None,
                        label_at.get(ops[-1])))
        elif op.startswith("s_"):
            out.append(("scalar", None, None, None, None))
        else:
            touched = frozenset().union(*[vgprs(o) for o in ops]) if ops else frozenset()
            dst = None
            if re.match(r"(buffer|global|scratch)_load", op):
                dst = vgprs(ops[0])
            elif re.match(r"(buffer|global|scratch)_store", op):
                dst = frozenset()  # stores count in vmcnt as well
            out.append(("vector", touched, dst, None, None))
    return out


def hazards_of(body):
    """body: instructions and .LBB labels of one kernel, in layout order."""
    first = next((i for i, l in enumerate(body) if l.startswith("buffer_load_dwordx4")), None)
    if first is None:
        return None
    code = parse(body)
    seen, work, bad = set(), [(first, ())], set()
    while work:
        pc, queue = work.pop()  # queue: destination registers of the loads in flight, oldest first
        in_flight = frozenset().union(*queue) if queue else frozenset()
        while pc < len(code):
            kind, touched, dst, vm, target = code[pc]
            if kind == "label":
                if (pc, queue) in seen:
                    break
                seen.add((pc, queue))
            elif kind == "end":
                break
            elif kind == "wait":
                if vm is not None and len(queue) > vm:
                    queue = queue[len(queue) - vm:] if vm else ()
                    in_flight = frozenset().union(*queue) if queue else frozenset()
            elif kind in ("branch", "jump"):
                if target is not None:
                    work.append((target, queue))
                if kind == "jump":
                    break
            elif kind == "vector":
                if touched & in_flight:
                    bad.add((pc, body[pc]))
                if dst is not None:
                    queue = queue + (dst,)
                    in_flight = in_flight | dst
            pc += 1
    return sorted(bad)


@pytest.fixture(scope="module")
def isa(tmp_path_factory):
    out = tmp_path_factory.mktemp("isa") / "kernels_conv_mfma.s"
    cmd = [build.hipcc()] + [f for f in build.FLAGS if f not in ("-shared", "-fPIC")] + [
        "-S", "--cuda-device-only", "-I" + os.path.join(ROOT, "include"),
        "-I" + os.path.dirname(SOURCE), SOURCE, "-o", str(out)]
    subprocess.check_call(cmd, stderr=subprocess.DEVNULL)
    return out.read_text().split("\n")


def test_no_register_is_touched_while_its_load_is_in_flight(isa):
    starts = [i for i, l in enumerate(isa) if re.match(r"^_ZN\S*conv_mfma_fp4_kernel\S*:", l)]
    assert len(starts) >= 90
    checked = 0
    for st in starts:
        if NEVER_LAUNCHED.search(isa[st]):
            continue
        end = next(i for i in range(st, len(isa)) if ".end_amdhsa_kernel" in isa[i])
        body = [l.strip().split(";")[0].rstrip() for l in isa[st:end]]
        body = [l for l in body if l and (not l.startswith(".") or l.startswith(".LBB"))]
        bad = hazards_of(body)
        assert bad is not None, "no fragment loads found in " + isa[st]
        assert not bad, "%s: %d instructions touch a register whose load is in flight, " \
            "first: %s" % (isa[st][:90], len(bad), bad[0][1])
        checked += 1
    assert checked >= 80
