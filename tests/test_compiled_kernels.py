"""Checks of the compiled kernels, on the CPU.

1. No kernel uses scratch memory: a spilled register means that the compiler ran out of them somewhere a source change can
help (the prefill attention kernel kept two lane coordinates across its tile loop that its epilogue can take again).

2. No workgroup barrier may be reachable with an LDS store of the same wavefront still unwaited.

An LDS store is visible to the wavefronts that a following `s_barrier` releases only if the storing wavefront has waited
for it (`s_waitcnt lgkmcnt(0)`).  The compiler puts that wait before a `__syncthreads()`; it has been seen to leave it out
where the barrier is the first instruction of a loop and the store sits at the end of the previous trip, and the kernel then
reads the previous trip's value now and then, under load only.  So every csrc/*.hip is compiled to gfx950 assembly here and
every function is walked: a forward data flow over its basic blocks (pending = an LDS store since the last full
`lgkmcnt(0)` wait, OR over predecessors) that reports each `s_barrier` reached while pending.  Hand-written barriers in the
sources carry their own `s_waitcnt lgkmcnt(0)` and pass the same check.

3. The prefill attention kernel waits for its LDS fragment reads by count.  While a direct-to-LDS load that the compiler knows of
is outstanding it closes every LDS wait with `lgkmcnt(0)`; that kernel always has such loads in flight, which is why it issues
them as inline assembly.  A kernel of it without a single partial wait has fallen back into that habit (10 % slower)."""
import glob
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

CSRC = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "qwen-tailor_amd", "csrc")
LDS_STORE = re.compile(r"^(ds_write|ds_add|ds_sub|ds_max|ds_min|ds_or|ds_and|ds_xor|ds_inc|ds_dec|ds_cmpst|ds_wrxchg|flat_store|flat_atomic)")
ENDS_BLOCK = ("s_cbranch", "s_branch", "s_endpgm", "s_setpc")


def unwaited_barriers(asm: str):
    """[(function, line within the function)] of every s_barrier that an unwaited LDS store can reach"""
    lines = asm.split("\n")
    funcs, cur = [], None
    for i, l in enumerate(lines):
        m = re.match(r"^([A-Za-z_][\w.$]*):", l)
        if m and not m.group(1).startswith(".L"):
            cur = [m.group(1), i]
        if l.startswith(".Lfunc_end") and cur:
            funcs.append((cur[0], cur[1], i))
            cur = None
    found = []
    for name, a, b in funcs:
        labels, starts = {}, {a + 1}
        for i in range(a + 1, b):
            s = lines[i].strip()
            m = re.match(r"^(\.LBB\d+_\d+):", s)
            if m:
                labels[m.group(1)] = i
                starts.add(i)
            if s.startswith(ENDS_BLOCK):
                starts.add(i + 1)
        starts = sorted(x for x in starts if x < b)
        index = {st: k for k, st in enumerate(starts)}
        blocks = [(st, starts[k + 1] if k + 1 < len(starts) else b) for k, st in enumerate(starts)]
        succ = []
        for k, (st, en) in enumerate(blocks):
            code = [lines[i].strip() for i in range(st, en)]
            code = [s for s in code if s and not s.startswith((";", "."))]
            nxt, falls = [], True
            if code:
                m = re.match(r"^s_c?branch\w*\s+(\.LBB\d+_\d+)", code[-1])
                if m and m.group(1) in labels:
                    nxt.append(index[labels[m.group(1)]])
                if code[-1].startswith(("s_branch", "s_endpgm", "s_setpc")):
                    falls = False
            if falls and k + 1 < len(blocks):
                nxt.append(k + 1)
            succ.append(nxt)

        def walk(k, pending, report):
            st, en = blocks[k]
            for i in range(st, en):
                s = lines[i].strip()
                if LDS_STORE.match(s):
                    pending = True
                elif s.startswith("s_waitcnt"):
                    m = re.search(r"lgkmcnt\((\d+)\)", s)
                    if m and m.group(1) == "0":
                        pending = False
                elif s.startswith("s_barrier") and pending and report is not None:
                    report.append((name, i - a))
            return pending

        entry = [False] * len(blocks)
        changed = True
        while changed:
            changed = False
            for k in range(len(blocks)):
                if walk(k, entry[k], None):
                    for s2 in succ[k]:
                        if not entry[s2]:
                            entry[s2] = changed = True
        for k in range(len(blocks)):
            walk(k, entry[k], found)
    return found


def scratch_users(asm: str):
    """[(kernel, scratch bytes, spilled vector registers)] from the code object metadata, for kernels that have either"""
    out = []
    for blk in asm.split("  - .agpr_count:")[1:]:
        name = re.search(r"\.name:\s+(\S+)", blk)
        priv = re.search(r"\.private_segment_fixed_size:\s+(\d+)", blk)
        spill = re.search(r"\.vgpr_spill_count:\s+(\d+)", blk)
        if name and priv and spill and (int(priv.group(1)) or int(spill.group(1))):
            out.append((name.group(1), int(priv.group(1)), int(spill.group(1))))
    return out


def partial_lds_waits(asm: str, kernel: str):
    """number of `s_waitcnt lgkmcnt(N)`, N > 0, in the functions whose name contains `kernel`"""
    n, inside = 0, False
    for l in asm.split("\n"):
        m = re.match(r"^([A-Za-z_][\w.$]*):", l)
        if m and not m.group(1).startswith(".L"):
            inside = kernel in m.group(1)
        if inside:
            w = re.search(r"s_waitcnt.*lgkmcnt\((\d+)\)", l)
            n += bool(w and int(w.group(1)) > 0)
    return n


def test_scratch_users_reads_the_metadata():
    meta = "  - .agpr_count:     0\n    .name:           k1\n    .private_segment_fixed_size: 12\n    .vgpr_spill_count: 2\n" \
           "  - .agpr_count:     0\n    .name:           k2\n    .private_segment_fixed_size: 0\n    .vgpr_spill_count: 0\n"
    assert scratch_users(meta) == [("k1", 12, 2)]


LOOP_WITH_THE_WAIT = """
kern:
\ts_branch .LBB0_2
.LBB0_1:
\tds_write_b32 v1, v2
.LBB0_2:
\t%s
\ts_barrier
\tds_read_b32 v3, v1
\ts_waitcnt lgkmcnt(0)
\ts_barrier
\tv_readfirstlane_b32 s4, v3
\ts_cmp_lt_i32 s4, s5
\ts_cbranch_scc1 .LBB0_1
\ts_endpgm
.Lfunc_end0:
"""


def test_the_walk_finds_a_store_that_reaches_a_loop_header_barrier_through_the_back_edge():
    assert unwaited_barriers(LOOP_WITH_THE_WAIT % "s_nop 0") == [("kern", 6)]
    assert unwaited_barriers(LOOP_WITH_THE_WAIT % "s_waitcnt lgkmcnt(0)") == []
    assert unwaited_barriers(LOOP_WITH_THE_WAIT % "s_waitcnt vmcnt(0) lgkmcnt(1)") == [("kern", 6)]


def test_partial_lds_waits_counts_per_kernel():
    asm = "k_a:\n\ts_waitcnt lgkmcnt(0)\n\ts_waitcnt vmcnt(2) lgkmcnt(3)\n.Lfunc_end0:\nk_b:\n\ts_waitcnt lgkmcnt(1)\n"
    assert partial_lds_waits(asm, "k_a") == 1 and partial_lds_waits(asm, "k_") == 2 and partial_lds_waits(asm, "k_c") == 0


def test_no_kernel_spills_or_reaches_a_barrier_with_an_unwaited_lds_store(tmp_path):
    hipcc = next((c for c in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")) if c and os.path.exists(c)), None)
    if hipcc is None:
        pytest.skip("hipcc not found")
    import qwen_tailor_amd._build as B
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    assert srcs

    def one(src):
        out = os.path.join(tmp_path, os.path.basename(src)[:-4] + ".s")
        r = subprocess.run([hipcc, *[f for f in B.FLAGS if f != "-fPIC"], "--cuda-device-only", "-S", src, "-o", out],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
        with open(out) as f:
            asm = f.read()
        if os.path.basename(src) == "gqa_prefill.hip":
            for kernel in ("attn_prefill_kernelILi1E", "attn_prefill_kernelILi2E"):
                assert partial_lds_waits(asm, kernel) >= 50, f"{kernel}: the tile loop waits for every LDS read in full"
        return os.path.basename(src), asm.count("s_barrier"), unwaited_barriers(asm), scratch_users(asm)

    with ThreadPoolExecutor(max_workers=8) as ex:
        results = list(ex.map(one, srcs))
    assert sum(n for _, n, _, _ in results) > 100       # the kernels were seen (they hold a few hundred barriers)
    bad = [(f, hits) for f, _, hits, _ in results if hits]
    assert not bad, bad
    spilling = [(f, k) for f, _, _, ks in results for k in ks]
    assert not spilling, spilling
