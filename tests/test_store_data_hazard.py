"""Generated code of every kernel: no 12- or 16-byte buffer store is followed too closely by a
vector instruction that overwrites its data registers.

A buffer store of more than 8 bytes reads its data registers for some cycles after it has
issued.  The compiler keeps such a vector write two wait states away, but only when the store's
scalar offset is not a register; with the offset in a scalar register it inserts nothing, and on
gfx950 a write stream built that way stored a few vectors in 100 000 with their successor's
contents.  This test compiles the library's kernels (and the test programs whose kernels inline
the device API) to assembly and looks for the pattern; it runs without a GPU."""
import os
import re
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
WAIT_STATES = 3          # instructions (or s_nop cycles) that must separate the store from the write

STORE = re.compile(r"^\s*buffer_store_dwordx([34])\s+v\[(\d+):(\d+)\],\s*(\S+),\s*s\[\d+:\d+\],\s*([^\s,]+)")


def vector_destination(line):
    """VGPRs a vector-ALU instruction writes, or None."""
    m = re.match(r"^\s*(v_\w+)\s+([^,]+)", line)
    if not m:
        return None
    op, dst = m.group(1), m.group(2).strip()
    if op.startswith(("v_cmp", "v_readfirstlane", "v_readlane")):
        return None
    m = re.match(r"v\[(\d+):(\d+)\]$", dst)
    if m:
        return set(range(int(m.group(1)), int(m.group(2)) + 1))
    m = re.match(r"v(\d+)$", dst)
    return {int(m.group(1))} if m else None


def hazards(text):
    """[(function, store line, overwriting line, instructions between)] in one assembly text."""
    lines = [l for l in text.splitlines() if l.strip() and not l.lstrip().startswith(";")]
    found, func = [], None
    for n, line in enumerate(lines):
        if re.match(r"^[_A-Za-z][\w$.]*:", line) and not line.startswith(".L"):
            func = line.split(":")[0]
        m = STORE.match(line)
        if not m or not re.match(r"(s\d+|s\[|m0)", m.group(5)):
            continue       # a literal scalar offset: the compiler inserts the wait itself
        data = set(range(int(m.group(2)), int(m.group(3)) + 1))
        between, j = 0, n + 1
        while between < WAIT_STATES and j < len(lines):
            nxt = lines[j]
            j += 1
            if re.match(r"^\s*\.", nxt) or re.match(r"^[\w.$]+:", nxt):
                continue                      # directives and labels take no time
            nop = re.match(r"^\s*s_nop\s+(\d+)", nxt)
            if nop:
                between += int(nop.group(1)) + 1
                continue
            dst = vector_destination(nxt)
            if dst and dst & data:
                found.append((func, line.strip(), nxt.strip(), between))
                break
            between += 1
    return found


def test_the_scan_sees_the_pattern_and_only_the_pattern():
    exposed = """
kernel_a:
	buffer_store_dwordx4 v[2:5], v10, s[8:11], s20 offen nt sc1
	v_lshl_add_u64 v[2:3], s[18:19], 0, v[0:1]
"""
    assert [(f, k) for f, _, _, k in hazards(exposed)] == [("kernel_a", 0)]
    covered = """
kernel_b:
	buffer_store_dwordx4 v[2:5], v10, s[8:11], 0 offen nt sc1
	s_nop 1
	v_lshl_add_u64 v[2:3], s[18:19], 0, v[0:1]
	buffer_store_dwordx4 v[2:5], v10, s[8:11], s20 offen
	s_add_u32 s18, s24, s22
	s_addc_u32 s19, s25, 0
	s_lshr_b64 s[18:19], s[18:19], 4
	v_lshl_add_u64 v[2:3], s[18:19], 0, v[0:1]
	buffer_store_dwordx4 v[6:9], v10, s[8:11], s20 offen
	v_mov_b32_e32 v10, 0
	v_mov_b32_e32 v11, v6
	buffer_store_dwordx2 v[2:3], v10, s[8:11], s20 offen
	v_mov_b32_e32 v2, 0
"""
    assert hazards(covered) == []
    nop_counts = """
kernel_c:
	buffer_store_dwordx3 v[2:4], v10, s[8:11], s20 offen
	s_nop 0
	v_mov_b32_e32 v4, 0
"""
    assert [(f, k) for f, _, _, k in hazards(nop_counts)] == [("kernel_c", 1)]


def test_no_kernel_overwrites_store_data_behind_a_store():
    jobs = [(os.path.join(ROOT, "roc_shmem_amd", "csrc"), "-j8", os.path.join("build", "isa")),
            (os.path.join(ROOT, "tests", "cxx"), "-j2", "isa")]
    files = []
    for where, parallel, out in jobs:
        run = subprocess.run(["make", "-s", parallel, "-C", where, "isa"], capture_output=True, text=True)
        assert run.returncode == 0, run.stdout[-2000:] + run.stderr[-2000:]
        folder = os.path.join(where, out)
        files += [os.path.join(folder, f) for f in sorted(os.listdir(folder)) if f.endswith(".s")]
    assert len(files) >= 7, files
    stores = 0
    for path in files:
        with open(path) as f:
            text = f.read()
        stores += len(re.findall(r"buffer_store_dwordx[34]", text))
        found = hazards(text)
        assert not found, (path, len(found), found[:3])
    assert stores > 1000, stores      # the scan did read the kernels' stores
