"""Static check of hand-scheduled machine code (no GPU needed).

The matrix-core convolution starts its vector memory loads and its LDS reads by hand and waits
for them later with s_waitcnt vmcnt(N) / lgkmcnt(N).  Between a load and the wait that covers
it, the destination registers hold stale data and the hardware will still write them: any
other instruction that reads or writes such a register in that window is a bug the compiler
cannot see (it takes the inline-asm load for an ordinary definition), and the symptom is a
wrong result or a wild address on the GPU.  The test compiles the kernel files to ISA and
walks every path of every kernel's control flow graph with the queues of loads in flight:
vector memory (loads and stores, which return in order and share vmcnt) and LDS (reads and
writes; LDS operations complete in order among themselves, so after lgkmcnt(N) all but the
newest N of them are done whatever scalar memory loads share the counter).

What is tracked are the loads the source issues by hand: the instructions between the
compiler's ";;#ASMSTART" and ";;#ASMEND" markers.  Loads that the compiler issues itself
(builtins, ordinary pointer reads) are covered by its own wait insertion, which knows their
destinations; they are not tracked, but they are counted, because every operation in a queue
ages the ones ahead of it.  (Tracking them as well reports paths that cannot be taken: the
compiler guards a load and the wait that covers it with the same lane mask, and a walk that
knows nothing about branch conditions takes the load and skips the wait.  The same goes for a
kernel made of two inlined tile bodies, where falling from the first body into the second is
a path the hardware never takes.)  Every kernel is walked from its first instruction, so a
kernel with several tile bodies, or a loop over tiles around one body, is covered whole.

Only the matrix-core kernel is walked.  The streaming kernels of stages 1 and 2 issue their
buffer loads through compiler builtins only."""
import os
import re
import subprocess

import pytest

from xnor_nn_amd import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "xnor_nn_amd", "csrc")
VM_MAX, LGKM_MAX = 64, 16
ASM_BEGIN, ASM_END = "#ASMSTART", "#ASMEND"
EXPECTED_VARIANTS = 141  # kernels the matrix-core file instantiates (9 of them persistent)


def vgprs(token):
    token = token.strip().rstrip(",")
    m = re.match(r"v\[(\d+):(\d+)\]$", token)
    if m:
        return frozenset(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", token)
    return frozenset({int(m.group(1))}) if m else frozenset()


def parse(body):
    """One tuple per line: (kind, registers touched, vector-memory destination, LDS
    destination, (vmcnt, lgkmcnt), branch target); a destination of frozenset() is an
    operation that counts without writing a register (a store, an LDS write)."""
    body = [l for l in body]
    label_at, n = {}, 0
    for l in body:  # index of every label among the parsed entries (markers produce none)
        if l in (ASM_BEGIN, ASM_END):
            continue
        if l.startswith(".LBB"):
            label_at[l[:-1]] = n
        n += 1
    out = []
    by_hand = False
    for line in body:
        if line in (ASM_BEGIN, ASM_END):
            by_hand = line == ASM_BEGIN
            continue
        if line.startswith(".LBB"):
            out.append(("label", None, None, None, None, None))
            continue
        op = line.split()[0]
        ops = [o for o in re.split(r"[ ,]+", line)[1:] if o]
        if op == "s_endpgm":
            out.append(("end", None, None, None, None, None))
        elif op == "s_waitcnt":
            vm = re.search(r"vmcnt\((\d+)\)", line)
            lg = re.search(r"lgkmcnt\((\d+)\)", line)
            out.append(("wait", None, None, None,
                        (int(vm.group(1)) if vm else None, int(lg.group(1)) if lg else None),
                        None))
        elif op.startswith("s_cbranch") or op == "s_branch":
            out.append(("jump" if op == "s_branch" else "branch", None, None, None, None,
                        label_at.get(ops[-1])))
        elif op.startswith("s_"):
            out.append(("scalar", None, None, None, None, None))
        else:
            touched = frozenset().union(*[vgprs(o) for o in ops]) if ops else frozenset()
            vdst = ldst = None
            if re.match(r"(buffer|global)_load_lds_", op) or \
                    (re.match(r"buffer_load", op) and "lds" in ops):
                vdst = frozenset()  # LDS-direct: counts in vmcnt, writes no register
            elif re.match(r"(buffer|global|scratch|flat)_load", op):
                vdst = vgprs(ops[0])
                if op.startswith("flat"):
                    ldst = vdst  # a flat load counts in both
            elif re.match(r"(buffer|global|scratch|flat)_(store|atomic)", op):
                vdst = frozenset()  # stores count in vmcnt as well
            elif op.startswith("ds_"):
                ldst = frozenset() if re.match(r"ds_(write|add|sub|min|max|and|or|xor)", op) \
                    and "_rtn" not in op else vgprs(ops[0])
            if not by_hand:  # the compiler's own: counted, not tracked
                vdst = frozenset() if vdst is not None else None
                ldst = frozenset() if ldst is not None else None
            out.append(("vector", touched, vdst, ldst, None, None))
    return out


def instructions(body):
    """The lines of a body that parse() turns into entries, in the same order."""
    return [l for l in body if l not in (ASM_BEGIN, ASM_END)]


def hazards_of(body, first=0):
    """body: instructions and .LBB labels of one kernel, in layout order; the walk starts at
    instruction `first` with nothing in flight.

    State: for every register with a load on the way, how many operations of the same queue
    have been issued since (its age).  s_waitcnt with count N completes everything of age >= N;
    the counters have 6 and 4 bits, so the hardware itself holds an instruction back until
    fewer than 64 vector memory / 16 LDS operations are in flight, and whatever is older has
    completed.  Where paths meet (labels), a register keeps the smaller of its ages: the walk
    is a fixed-point iteration over the control flow graph, conservative where paths differ."""
    code = parse(body)
    body = instructions(body)
    at_label, work, bad = {}, [(first, {}, {})], set()

    def issue(ages, dst, limit):
        ages = {r: a + 1 for r, a in ages.items() if a + 1 < limit}
        for r in dst:
            ages[r] = 0
        return ages

    def join(old, new):
        out = dict(old)
        for r, a in new.items():
            out[r] = min(a, out.get(r, a))
        return out

    while work:
        pc, vm_age, lds_age = work.pop()
        while pc < len(code):
            kind, touched, vdst, ldst, counts, target = code[pc]
            if kind == "label":
                if pc in at_label:
                    merged = (join(at_label[pc][0], vm_age), join(at_label[pc][1], lds_age))
                    if merged == at_label[pc]:
                        break
                    at_label[pc] = merged
                    vm_age, lds_age = merged
                else:
                    at_label[pc] = (dict(vm_age), dict(lds_age))
            elif kind == "end":
                break
            elif kind == "wait":
                vm, lg = counts
                if vm is not None:
                    vm_age = {r: a for r, a in vm_age.items() if a < vm}
                if lg is not None:
                    lds_age = {r: a for r, a in lds_age.items() if a < lg}
            elif kind in ("branch", "jump"):
                if target is not None:
                    work.append((target, dict(vm_age), dict(lds_age)))
                if kind == "jump":
                    break
            elif kind == "vector":
                if any(r in vm_age or r in lds_age for r in touched):
                    bad.add((pc, body[pc]))
                if vdst is not None:
                    vm_age = issue(vm_age, vdst, VM_MAX)
                if ldst is not None:
                    lds_age = issue(lds_age, ldst, LGKM_MAX)
            pc += 1
    return sorted(bad)


def compile_to_isa(tmp, name):
    out = tmp / (name + ".s")
    source = os.path.join(CSRC, name + ".hip")
    cmd = [build.hipcc()] + [f for f in build.FLAGS if f not in ("-shared", "-fPIC")] + [
        "-S", "--cuda-device-only", "-I" + os.path.join(ROOT, "include"), "-I" + CSRC, source,
        "-o", str(out)]
    subprocess.check_call(cmd, stderr=subprocess.DEVNULL)
    return out.read_text().split("\n")


def kernels_of(isa, pattern):
    """(mangled name, instructions and labels) of every kernel whose symbol matches."""
    for st in [i for i, l in enumerate(isa) if re.match(pattern, l)]:
        end = next(i for i in range(st, len(isa)) if ".end_amdhsa_kernel" in isa[i])
        body = []
        for l in isa[st:end]:
            l = l.strip()
            if l.startswith(";;" + ASM_BEGIN) or l.startswith(";;" + ASM_END):
                body.append(l[2:].split()[0])
                continue
            l = l.split(";")[0].rstrip()
            if l and (not l.startswith(".") or l.startswith(".LBB")):
                body.append(l)
        yield isa[st], body


def m0_outside_asm(body):
    """Instructions that name M0 outside the hand-written asm statements."""
    out, by_hand_now = [], False
    for line in body:
        if line in (ASM_BEGIN, ASM_END):
            by_hand_now = line == ASM_BEGIN
        elif not by_hand_now and re.search(r"\bm0\b", line):
            out.append(line)
    return out


def by_hand(*lines):
    """The lines as the compiler prints an inline-asm statement."""
    return [ASM_BEGIN] + list(lines) + [ASM_END]


@pytest.fixture(scope="module")
def conv_isa(tmp_path_factory):
    """The matrix-core kernels as the compiler prints them (one compilation for the module)."""
    return compile_to_isa(tmp_path_factory.mktemp("isa"), "kernels_conv_mfma")


def test_no_register_is_touched_while_its_load_is_in_flight(conv_isa):
    """Every variant of the matrix-core kernel that the library holds (all of them can be
    launched), from its first instruction to the end."""
    isa = conv_isa
    checked = 0
    for name, body in kernels_of(isa, r"^_ZN\S*conv_mfma_fp4\S*kernel\S*:"):
        lines = instructions(body)
        code = parse(body)
        tracked = sum(1 for c in code if c[0] == "vector" and (c[2] or c[3]))
        assert tracked >= 4, "no hand-issued loads found in " + name
        assert len(code) == len(lines)
        bad = hazards_of(body)
        assert not bad, "%s: %d instructions touch a register whose load is in flight, " \
            "first: %s" % (name[:90], len(bad), bad[0][1])
        # the LDS-direct loads of the persistent kernels set M0 by hand; that is only safe as
        # long as the compiler keeps nothing of its own in M0 in these kernels
        assert not m0_outside_asm(body), "%s: the compiler uses M0: %s" % (
            name[:90], m0_outside_asm(body)[0])
        checked += 1
    assert checked >= EXPECTED_VARIANTS, checked


def test_the_walker_sees_a_planted_hazard():
    """The checker itself: a register read one instruction before the wait that covers its
    load, for a vector memory load and for an LDS read, and the same code with the wait in
    place."""
    load = "buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen"
    read = "ds_read_b128 v[8:11], v2"
    use = "v_add_u32_e32 v3, v4, v8"
    ok = by_hand(load) + by_hand(read) + ["s_waitcnt vmcnt(0) lgkmcnt(0)", use, "s_endpgm"]
    assert hazards_of(ok) == []
    early_vm = by_hand(load) + by_hand(read) + ["s_waitcnt lgkmcnt(0)", use, "s_endpgm"]
    assert [b[1] for b in hazards_of(early_vm)] == [use]
    early_lds = by_hand(load) + by_hand(read) + ["s_waitcnt vmcnt(0)", use, "s_endpgm"]
    assert [b[1] for b in hazards_of(early_lds)] == [use]
    # in-order return: with one operation allowed in flight the older of two is done
    two = by_hand("ds_read_b128 v[4:7], v2", "ds_read_b128 v[8:11], v2 offset:16") + [
        "s_waitcnt lgkmcnt(1)", "v_mov_b32_e32 v0, v4", "v_mov_b32_e32 v1, v8", "s_endpgm"]
    assert [b[1] for b in hazards_of(two)] == ["v_mov_b32_e32 v1, v8"]
    # a wait inside the asm statement itself (wait, then start the next reads) is seen
    fused = by_hand(read) + by_hand("s_waitcnt lgkmcnt(0)", "ds_read_b128 v[12:15], v2") + [
        "v_mov_b32_e32 v0, v8", "v_mov_b32_e32 v1, v12", "s_endpgm"]
    assert [b[1] for b in hazards_of(fused)] == ["v_mov_b32_e32 v1, v12"]


def test_the_compilers_own_loads_are_counted_but_not_tracked():
    """A load outside the asm markers is the compiler's: its destination is not followed
    (the compiler waits for it itself), but it ages what is in flight ahead of it."""
    load = "buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen"
    own = "global_load_dword v29, v[30:31], off"
    # the compiler's load and its guarded wait: taking the load and skipping the wait is a
    # path of the walk that the hardware never takes, and nothing is reported for it
    guarded = [own, "s_and_saveexec_b64 s[4:5], vcc", "s_cbranch_execz .LBB0_2", ".LBB0_1:",
               "s_waitcnt vmcnt(0)", "ds_write_b32 v2, v29", ".LBB0_2:", own, "s_endpgm"]
    assert hazards_of(guarded) == []
    # ... but one load by hand followed by one of the compiler's: vmcnt(1) covers the first
    aged = by_hand(load) + [own, "s_waitcnt vmcnt(1)", "v_mov_b32_e32 v0, v4", "s_endpgm"]
    assert hazards_of(aged) == []
    not_aged = by_hand(load) + ["s_waitcnt vmcnt(1)", "v_mov_b32_e32 v0, v4", "s_endpgm"]
    assert [b[1] for b in hazards_of(not_aged)] == ["v_mov_b32_e32 v0, v4"]


def test_a_hazard_in_a_second_body_is_seen():
    """A kernel of two inlined tile bodies, as the compiler lays out `if (big) body1 else
    body2` with a uniform skip over the second body (s_mov_b64 sX, 0 / s_andn2_b64 vcc, exec,
    sX / s_cbranch_vccnz): the first body is clean, the second touches a fragment register
    ahead of its wait.  Both the entry branch and the fall-through reach the second body."""
    load = "buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen"
    body1 = by_hand(load) + ["s_waitcnt vmcnt(0)", "v_mov_b32_e32 v0, v4"]
    skip = ["s_mov_b64 s[0:1], 0", "s_andn2_b64 vcc, exec, s[0:1]", "s_cbranch_vccnz .LBB0_3"]
    body2_bad = [".LBB0_2:"] + by_hand(load) + ["v_mov_b32_e32 v0, v5", "s_waitcnt vmcnt(0)"]
    body2_ok = [".LBB0_2:"] + by_hand(load) + ["s_waitcnt vmcnt(0)", "v_mov_b32_e32 v0, v5"]
    head = ["s_cmp_lt_u32 s8, s9", "s_cbranch_scc0 .LBB0_2"]
    tail = [".LBB0_3:", "s_endpgm"]
    assert [b[1] for b in hazards_of(head + body1 + skip + body2_bad + tail)] \
        == ["v_mov_b32_e32 v0, v5"]
    assert hazards_of(head + body1 + skip + body2_ok + tail) == []
    # a loop over tiles around one body: a load left in flight at the back edge is seen at
    # the top of the next round
    loop = [".LBB0_1:", "v_mov_b32_e32 v0, v4"] + by_hand(load) + [
        "s_cmp_lt_u32 s8, s9", "s_cbranch_scc1 .LBB0_1", "s_waitcnt vmcnt(0)", "s_endpgm"]
    # (and so is the second load into registers whose first load has not arrived)
    assert [b[1] for b in hazards_of(loop)] == ["v_mov_b32_e32 v0, v4", load]


def test_lds_direct_loads_count_but_write_no_register():
    """A load that goes straight to LDS (global_load_lds_dword, buffer_load ... lds) takes a
    place in the vector memory queue and has no destination register: the address register
    it names is free at once, and the loads ahead of it are one operation older."""
    load = "buffer_load_dwordx4 v[4:7], v1, s[0:3], 0 offen"
    to_lds = ["s_mov_b32 m0, s7", "s_nop 0", "global_load_lds_dword v2, s[4:5]"]
    ok = by_hand(load) + by_hand(*to_lds) + ["v_add_u32_e32 v2, 0x400, v2",
                                              "s_waitcnt vmcnt(1)", "v_mov_b32_e32 v0, v4",
                                              "s_endpgm"]
    assert hazards_of(ok) == []
    assert m0_outside_asm(ok) == []
    assert m0_outside_asm(ok + ["s_mov_b32 m0, s8"]) == ["s_mov_b32 m0, s8"]


def resident_by_registers(ks, ps):
    """The register half of resident_workgroups() in kernels_conv_mfma.hip, restated."""
    if ps == 3:
        return 3 if ks == 1 else 2
    if ps == 2:
        return 4 if ks == 1 else 3 if (ks <= 4 or ks == 12) else 2
    if ps == 1:
        return 4 if (ks <= 4 or ks >= 12) else 3 if ks <= 6 else 2
    return 2


def test_the_tile_model_counts_resident_workgroups_as_the_registers_allow(conv_isa):
    """The tile-size model prices a tile by how many workgroups fit a compute unit together.
    Its register rule is held against the compiler's own counts (.vgpr_count of the kernel
    metadata, 512 registers per SIMD lane in granules of 8) for every forward variant with
    one tile size: the rule never promises a workgroup that does not fit, and is exact for all
    but a few variants."""
    counts, name = {}, None
    for line in conv_isa:
        line = line.strip()
        if line.startswith(".name:"):
            name = line.split()[1]
        elif line.startswith(".vgpr_count:") and name:
            counts[name] = int(line.split()[1])
    plain = subprocess.run(["c++filt"], input="\n".join(counts), capture_output=True, text=True,
                           check=True).stdout.split("\n")
    seen = exact = 0
    for mangled, text in zip(counts, plain):
        m = re.search(r"conv_mfma_fp4_kernel<(\d+), (\d+), (\d+), (\w+), (\w+), (\w+)>", text)
        if not m or m[3] != "0" or m[4] == "true":  # two tile sizes, raw accumulators
            continue
        ks, ps = int(m[1]), int(m[2])
        fit = min(4, 512 // ((counts[mangled] + 7) // 8 * 8))
        rule = resident_by_registers(ks, ps)
        assert rule <= fit, "%s: %d registers hold %d workgroups, the model counts %d" % (
            text[:60], counts[mangled], fit, rule)
        seen += 1
        exact += rule == fit
    assert seen >= 40, seen
    assert seen - exact <= 2, (seen, exact)
