"""Build-time check of the prefill kernels' hand-issued loads.

tk_gemm_kernel and tk_gemm32_kernel issue their weight loads as inline asm and wait for them with
explicit `s_waitcnt vmcnt(N)` several hundred instructions later (the compiler's own wait insertion
drains the whole counter when LDS-DMA and register loads are pending together). The compiler does
not know that the destination registers of such an asm are still in flight: under register pressure
it may split their live range and copy one (`v_mov_b32 v5, v66` ... `v_mov_b32 v66, v5`) before the
wait, which reads a register the load has not written yet. Nothing in the source can forbid that,
so the generated code is checked instead: between a vector-memory load and the wait that covers it,
no other instruction may name one of its destination registers.

    python -m tritium_amd.check_isa <file.s>      # exit status 1 and a report when a hazard is found
"""
import re
import sys

_VREG_RANGE = re.compile(r"\bv\[(\d+):(\d+)\]")
_VREG_ONE = re.compile(r"\bv(\d+)\b")
_VMCNT = re.compile(r"vmcnt\((\d+)\)")
_LGKMCNT = re.compile(r"lgkmcnt\((\d+)\)")


def _vregs(text):
    regs = set()
    for lo, hi in _VREG_RANGE.findall(text):
        regs.update(range(int(lo), int(hi) + 1))
    for r in _VREG_ONE.findall(_VREG_RANGE.sub(" ", text)):
        regs.add(int(r))
    return regs


def check_function(name, lines):
    """Scan of one function in layout order: returns a list of (line number, instruction, register)
    hazards. Control flow is followed as far as forward branches go: a label entered only by jumps
    starts from the loads that were in flight at the first jump to it, a label entered by falling
    through keeps the state of the code above it; backward branches (loops) are not re-walked, which
    is enough here because every iteration of the pipelined loops ends in the same wait."""
    pending = []  # issue order: (destination registers, line) of every vector-memory operation
    lds = []      # the same for LDS and scalar-memory operations (one counter, lgkmcnt); LDS returns in order
    at_label = {}  # label -> loads in flight at the first forward jump to it
    reachable = True
    hazards = []
    for no, raw in lines:
        ins = raw.split(";")[0].strip()
        if not ins or ins.startswith("."):
            if ins.endswith(":"):  # a local label
                label = ins[:-1]
                if not reachable:
                    pending, lds = (list(x) for x in at_label.get(label, ([], [])))
                reachable = True
            continue
        if ins.endswith(":"):
            continue
        if not reachable:
            continue
        op = ins.split()[0]
        if op.startswith("s_cbranch") or op == "s_branch":
            at_label.setdefault(ins.split()[-1], (list(pending), list(lds)))
            if op == "s_branch":
                reachable = False
            continue
        if op == "s_endpgm":
            reachable = False
            continue
        if op == "s_waitcnt":
            m = _VMCNT.search(ins)
            if m:
                keep = int(m.group(1))
                pending = pending[len(pending) - keep:] if keep else []
            m = _LGKMCNT.search(ins)
            if m:
                keep = int(m.group(1))
                lds = lds[len(lds) - keep:] if keep else []
            continue
        in_flight = set().union(*(p[0] for p in pending + lds)) if pending or lds else set()
        if op.startswith(("ds_", "s_load", "s_buffer_load")):
            # the prefill kernels read their A pieces one k step ahead and wait with lgkmcnt(N > 0)
            operands = ins[len(op):].split(",")
            is_read = op.startswith(("ds_read", "ds_load"))
            dest = _vregs(operands[0]) if is_read else set()
            used = _vregs(",".join(operands[1:])) if is_read else _vregs(ins)
            for r in sorted((used | dest) & in_flight):
                hazards.append((no, ins, r))
            lds.append((dest, no))
            continue
        if op.startswith("global_load_lds"):  # LDS-DMA: counted by vmcnt, no destination register
            used = _vregs(ins)
            dest = set()
        elif op.startswith(("global_load", "buffer_load", "flat_load", "scratch_load")):
            operands = ins[len(op):].split(",")
            dest = _vregs(operands[0])
            used = _vregs(",".join(operands[1:]))
        elif op.startswith(("global_store", "buffer_store", "flat_store", "scratch_store", "global_atomic")):
            used = _vregs(ins)
            dest = set()
        else:
            used = _vregs(ins)
            dest = None
        for r in sorted(used & in_flight):
            hazards.append((no, ins, r))
        if dest is not None:
            for r in sorted(dest & in_flight):
                hazards.append((no, ins, r))
            pending.append((dest, no))
    return hazards


def check_text(text, only=("tk_gemm",)):
    """Checks every function whose (mangled) name contains one of `only`. Returns {name: hazards}."""
    found = {}
    name, body = None, []
    for no, line in enumerate(text.splitlines(), 1):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            name, body = m.group(1), []
            continue
        if name is None:
            continue
        if line.startswith(".Lfunc_end"):
            if any(s in name for s in only):
                hz = check_function(name, body)
                if hz:
                    found[name] = hz
            name = None
            continue
        body.append((no, line))
    return found


# Register budgets of the bandwidth kernels: (template arguments of the kernel, vector registers at most).
# A CU runs floor(512 / registers) waves per SIMD, in steps of 8 registers: 128 -> 4, 168 -> 3, 256 -> 2. The
# decode kernels' rate follows the bytes their waves keep in flight, so a change that pushes one of these
# forms over its step (a few registers are enough) costs a third or a quarter of the rate without any test
# noticing. The build fails instead.
REGISTER_BUDGETS = (
    ("tk_flow_kernelILi1ELi1ELi1ELi4ELb1ELb0ELb0E", 128),   # one plane, one run per wave: a single operand row
    ("tk_flow_kernelILi1ELi1ELi2ELi4ELb1ELb0ELb0E", 128),   # one plane, two runs per wave: 2..16 rows
    ("tk_flow_kernelILi2ELi1ELi1ELi4ELb1ELb0ELb0E", 128),   # two planes, up to 8 rows
    ("tk_flow_kernelILi2ELi1ELi1ELi2ELb1ELb0ELb0E", 96),    # ... on a ring of two (eight K blocks or fewer, 4 rows): five waves per SIMD
    ("tk_flow_kernelILi2ELi1ELi2ELi2ELb1ELb0ELb0E", 128),   # two planes, 9..16 rows on a ring of two: four waves per SIMD
    ("tk_flow_kernelILi2ELi1ELi2ELi4ELb1ELb0ELb0E", 168),   # two planes, 9..16 rows
    ("tk_flow32_kernelILi2ELi1ELi4ELb1ELb0ELb0E", 168), # two planes, 25..32 rows, four-wave workgroups
    ("tk_flow32_kernelILi2ELi1ELi2ELb1ELb0ELb0E", 168), # ... eight-wave workgroups (from 53 KiB of rows on) on a ring of two
    ("tk_flow32_kernelILi2ELi1ELi2ELb1ELb0ELb1E", 168), # ... weights first (int8 contract; sixteen scales per plane held over a pair of tiles)
    ("tk_flow_kernelILi2ELi4ELi2ELi2ELb1ELb0ELb0E", 256),   # two planes, 33..64 rows
    ("tk_flow_kernelILi1ELi2ELi2ELi2ELb1ELb0ELb1E", 128),   # weights first, two row tiles on a ring of two: the forms of 1024 threads
    ("tk_flow_kernelILi2ELi2ELi1ELi2ELb1ELb0ELb1E", 128),   # (sixteen waves per workgroup; no spills)
    ("tk_flow_kernelILi1ELi2ELi2ELi2ELb1ELb0ELb0E", 128),   # ... activations first, from a problem table
    ("tk_flow_kernelILi2ELi2ELi1ELi2ELb1ELb0ELb0E", 128),
    ("tk_gemm32_kernelILi1ELi2ELb0ELb0E", 168),     # prefill, one plane (three waves per SIMD by design)
    ("tk_gemm32_kernelILi1ELi4ELb0ELb0E", 168),
    ("tk_gemm32_kernelILi3ELi2ELb0ELb0E", 256),     # prefill, three planes (two waves per SIMD)
    ("tk_gemm128_kernel", 128),                     # prefill, 128 x 256 form (four waves per SIMD)
    ("tk_gemm256_kernelILi0E", 512),                # prefill, 256 x 224 form, four waves (one per SIMD)
    ("tk_gemm256_kernelILi1E", 256),                # ... eight waves (two per SIMD)
    ("tk_gemm256_kernelILi2E", 256),                # ... four waves over 128 | 96 outputs, two workgroups per CU
) + tuple(  # the 32x32x32 flow forms that consult the zero-chunk maps, in both operand orders: present, no spills
    (f"tk_flow32_kernelILi{p}ELi{rt2}ELi{dr}ELb{t}ELb1ELb{sw}E", 256)
    for p in (1, 2) for rt2 in (1, 2) for dr in (2, 3, 4) for t in (0, 1) for sw in (0, 1)
)


def check_budgets(text, budgets=REGISTER_BUDGETS):
    """[(kernel, registers used, budget)] for every budgeted kernel over its budget, or that spills, or that
    the assembly does not contain (a renamed kernel must not drop out of the check silently)."""
    used, spills, name = {}, {}, None
    for line in text.splitlines():
        m = re.match(r"[\s-]+\.name:\s+(\S+)", line)
        if m:
            name = m.group(1)
        m = re.match(r"[\s-]+\.vgpr_count:\s+(\d+)", line)
        if m and name:
            used[name] = int(m.group(1))
        m = re.match(r"[\s-]+\.vgpr_spill_count:\s+(\d+)", line)
        if m and name:
            spills[name] = int(m.group(1))
    bad = []
    for key, budget in budgets:
        names = [n for n in used if key in n]
        if not names:
            bad.append((key, None, budget))
        for n in names:
            if used[n] > budget or spills.get(n, 0):
                bad.append((n, used[n] + (10000 if spills.get(n, 0) else 0), budget))
    return bad


# Kernels that build raw LDS addresses from offsets into their dynamic array and therefore need that array to
# start at LDS address 0: no static LDS in front of it (the base-3 flow kernel's decode-table lookup is one
# v_perm_b32 of the byte and the lane offset, with no add of a base).
NO_STATIC_LDS = ("tk_flow3_kernel",)


def check_static_lds(text, kernels=NO_STATIC_LDS):
    """[(kernel, static LDS bytes)] for every listed kernel whose fixed LDS segment is not empty, and
    (key, None) for a listed kernel the assembly does not contain."""
    # one metadata entry per kernel ("  - .agpr_count: ..." starts it); its keys come in alphabetical order, so
    # the fixed LDS size precedes the name
    fixed, size = {}, None
    for line in text.splitlines():
        if re.match(r"\s+- \.\w+:", line):
            size = None
        m = re.match(r"[\s-]+\.group_segment_fixed_size:\s+(\d+)", line)
        if m:
            size = int(m.group(1))
        m = re.match(r"[\s-]+\.name:\s+(\S+)", line)
        if m and size is not None:
            fixed[m.group(1)] = size
    bad = []
    for key in kernels:
        names = [n for n in fixed if key in n]
        if not names:
            bad.append((key, None))
        bad += [(n, fixed[n]) for n in names if fixed[n]]
    return bad


def report(found):
    out = []
    for name, hz in found.items():
        out.append(f"{name}: {len(hz)} use(s) of a register whose load is still in flight")
        for no, ins, r in hz[:8]:
            out.append(f"  line {no}: v{r} in `{ins}`")
    return "\n".join(out)


if __name__ == "__main__":
    bad = check_text(open(sys.argv[1]).read())
    if bad:
        print(report(bad))
        sys.exit(1)
    print("no in-flight register is touched before its wait")
