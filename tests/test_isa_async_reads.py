"""Static check of the compiled kernels that read LDS through inline asm (csrc/gemm.hip).

An inline-asm `ds_read` hands the compiler an output register that the hardware fills LATER, when the read returns;
the kernel's own `s_waitcnt lgkmcnt(n)` says when.  The compiler knows nothing of this: once the C++ value is dead it
may reuse the register at once -- e.g. at a loop exit, for the epilogue's column index, ahead of the wait -- and the
late return then overwrites the new contents (an index far outside the buffers: a GPU memory fault that shows only
when LDS is slow, such as with two kernels sharing a CU).  This test compiles such sources to ISA for gfx950 and
walks every kernel: between an inline-asm read and the `s_waitcnt` that retires it, no other instruction may read
or write its destination registers.  No GPU needed.
"""
import glob
import os
import re
import shutil
import subprocess

import pytest

from chatrwkv_amd import build as _build

ASM_READ = re.compile(r'asm volatile\(\s*"(ds_read|global_load|buffer_load)')
VREG = re.compile(r'\bv\[(\d+):(\d+)\]|\bv(\d+)\b')
LABEL = re.compile(r'^(\.LBB\d+_\d+):')


def _vregs(text):
    out = set()
    for a, b, c in VREG.findall(text):
        out |= set(range(int(a), int(b) + 1)) if a else {int(c)}
    return out


def _kernels(lines):
    """(name, first line, last line) of every function in the ISA listing"""
    i = 0
    while i < len(lines):
        m = re.match(r'^(\w+):\s*; @(\w+)', lines[i])
        if m and m.group(1) == m.group(2):
            j = i
            while not lines[j].startswith('.Lfunc_end'):
                j += 1
            yield m.group(1), i, j
            i = j
        i += 1


def find_hazards(lines, first, last):
    """Instructions of lines[first:last] that touch a register an inline-asm LDS read may still be writing."""
    labels = {LABEL.match(lines[j]).group(1): j for j in range(first, last) if LABEL.match(lines[j])}
    # the walk: straight through, and every loop (backward branch) a second time, so that what is in flight at the
    # back edge meets the top of the body
    order, j = [], first
    replayed = set()
    while j < last:
        order.append(j)
        t = lines[j].split()
        if t and t[0].startswith(('s_cbranch', 's_branch')) and t[-1] in labels and labels[t[-1]] <= j and j not in replayed:
            replayed.add(j)
            order.extend(range(labels[t[-1]], j + 1))
        j += 1
    # queue: destination registers of the outstanding LDS operations, oldest first.  LDS operations return in order,
    # so after `s_waitcnt lgkmcnt(n)` at most the newest n are outstanding (scalar loads share the counter and
    # return in any order: one of them outstanding only makes the wait stricter)
    queue, hazards, in_asm = [], [], False
    for j in order:
        l = lines[j].strip()
        if l.startswith(';;#ASMSTART'):
            in_asm = True
            continue
        if l.startswith(';;#ASMEND'):
            in_asm = False
            continue
        if not l or l.startswith((';', '.')) or l.endswith(':'):
            continue
        op = l.split()[0]
        if op == 's_waitcnt':
            m = re.search(r'lgkmcnt\((\d+)\)', l)
            if m:
                n = int(m.group(1))
                del queue[:max(0, len(queue) - n)]
            continue
        inflight = set().union(*queue) if queue else set()
        body = l.split(';')[0]
        if _vregs(body) & inflight:
            hazards.append((j - first, l, sorted(_vregs(body) & inflight)))
        if op.startswith('ds_'):
            queue.append(_vregs(body.split(',')[0]) if (in_asm and op.startswith('ds_read')) else set())
    return hazards


def test_checker_sees_a_reused_register():
    isa = """k: ; @k
\t;;#ASMSTART
\tds_read_b128 v[4:7], v9
\t;;#ASMEND
.LBB0_1:
\ts_waitcnt lgkmcnt(0)
\tv_mfma_f32_32x32x16_f16 v[10:25], v[4:7], v[34:37], v[10:25]
\t;;#ASMSTART
\tds_read_b128 v[4:7], v9
\t;;#ASMEND
\ts_cbranch_scc0 .LBB0_1
\tv_or_b32_e32 v5, s2, v1
\ts_waitcnt vmcnt(0) lgkmcnt(0)
\tv_or_b32_e32 v6, s2, v1
\ts_endpgm
.Lfunc_end0:
""".split('\n')
    (name, a, b), = list(_kernels(isa))
    hz = find_hazards(isa, a, b)
    assert [h[2] for h in hz] == [[5]], hz
    ok = [l for l in isa if 'v_or_b32_e32 v5' not in l]
    (name, a, b), = list(_kernels(ok))
    assert find_hazards(ok, a, b) == []


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="hipcc not installed")
def test_no_register_is_reused_under_an_inline_asm_read(tmp_path):
    srcs = [s for s in sorted(glob.glob(os.path.join(_build.CSRC, "*.hip"))) if ASM_READ.search(open(s).read())]
    assert srcs, "csrc/gemm.hip reads its MFMA fragments through inline asm"
    for src in srcs:
        out = tmp_path / (os.path.basename(src) + ".s")
        r = subprocess.run(["hipcc", *_build.FLAGS, "--cuda-device-only", "-S", "-o", str(out), src],
                           capture_output=True, text=True)
        assert r.returncode == 0, r.stderr
        lines = out.read_text().split('\n')
        checked = 0
        for name, a, b in _kernels(lines):
            if not any('ASMSTART' in lines[j] for j in range(a, b)):
                continue
            checked += 1
            hz = find_hazards(lines, a, b)
            assert not hz, f"{os.path.basename(src)}: {name}: " + "; ".join(f"+{o}: {l} (in flight: v{r})" for o, l, r in hz[:5])
        assert checked >= 16, checked   # the eight direct-to-LDS kernels and their grouped forms
