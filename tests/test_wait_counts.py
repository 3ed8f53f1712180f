"""Static check of the hand-written wait counts in the MFMA kernels' machine code.

The tiled and the mid-M kernel stream their activation tiles global -> LDS with LDS-direct loads and wait for a tile
with an inline `s_waitcnt vmcnt(N)`, N > 0: vector-memory operations complete in order, so "at most N outstanding"
means the tile has landed only if the wave has issued at least N vector-memory instructions behind the tile's last
LDS-direct load.  N is written by hand next to the loads it counts (gptq4_gemm.hip, gptq4_kslice.hip); a compiler that
merged, dropped or hoisted one of those loads above the LDS-direct loads would make the wait return early and the MFMAs
read a tile that is still in flight - with results that are wrong only sometimes.  This test compiles the two files to
gfx950 assembly and follows every path of every kernel variant from the kernel's entry and from each such wait to the
next one: behind the first group of LDS-direct loads on the path (the tile that the next wait is for) it counts the
vector-memory instructions, and the count must reach the N of the wait the path ends in.
"""
import importlib.util
import re
import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
CSRC = ROOT / "gptq-triton_amd" / "csrc"

VMEM = re.compile(r"^(buffer|global|flat|scratch)_(load|store|atomic)")
WAIT = re.compile(r"^s_waitcnt\b.*\bvmcnt\((\d+)\)")
LABEL = re.compile(r"^(\.LBB\d+_\d+):")
BRANCH = re.compile(r"^(s_c?branch\w*)\s+(\.LBB\d+_\d+)")
CAP = 64  # counts beyond any wait's N are all the same


def _build_flags():
    spec = importlib.util.spec_from_file_location("_gptq4_build", ROOT / "gptq-triton_amd" / "build.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod._hipcc(), [f for f in mod.HIPCC_FLAGS if f != "-fPIC"]


def _assembly(source: Path, tmp: Path) -> str:
    hipcc, flags = _build_flags()
    out = tmp / (source.stem + ".s")
    res = subprocess.run([hipcc, *flags, "-w", "-S", "--cuda-device-only", str(source), "-o", str(out)],
                         stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert res.returncode == 0, res.stdout[-2000:]
    return out.read_text()


def _kernels(asm: str):
    """(name, [(line, inline)]) per kernel function: instruction and label lines without comments; inline = the line
    stands between the markers the compiler puts around an asm statement of the source."""
    for m in re.finditer(r"^(_Z\w*gptq4_\w+_kernel\w*):.*$", asm, re.M):
        end = asm.index(".Lfunc_end", m.end())
        lines, inline = [], False
        for raw in asm[m.end():end].splitlines():
            if "#ASMSTART" in raw:
                inline = True
            elif "#ASMEND" in raw:
                inline = False
            line = raw.split(";")[0].strip()
            if line:
                lines.append((line, inline))
        yield m.group(1), lines


def _paths_to_waits(lines):
    """[(N, vector-memory instructions behind the first group of LDS-direct loads, index of the wait)] over all paths
    from the entry and from every hand-written wait to the next hand-written wait."""
    text = [l for l, _ in lines]
    label_at = {m.group(1): i for i, l in enumerate(text) if (m := LABEL.match(l))}
    hand = {i: int(m.group(1)) for i, (l, inline) in enumerate(lines) if inline and (m := WAIT.match(l)) and int(m.group(1)) > 0}
    results, seen = [], set()
    # state: (index, phase, count); phase 0 = no LDS-direct load yet, 1 = inside the first group, 2 = behind it
    stack = [(0, 0, 0)] + [(w + 1, 0, 0) for w in hand]
    while stack:
        i, phase, count = stack.pop()
        while i < len(text):
            if (i, phase, count) in seen:
                break
            seen.add((i, phase, count))
            cur = text[i]
            if i in hand:
                if phase:
                    results.append((hand[i], count, i))
                break
            if VMEM.match(cur):
                direct = cur.split()[-1] == "lds"
                if direct and phase == 0:
                    phase = 1
                elif not direct and phase == 1:
                    phase, count = 2, 1
                elif phase == 2:
                    count = min(count + 1, CAP)
            if cur.startswith(("s_endpgm", "s_setpc")):
                break
            b = BRANCH.match(cur)
            if b:
                stack.append((label_at[b.group(2)], phase, count))
                if b.group(1) == "s_branch":
                    break
            i += 1
    return results


@pytest.fixture(scope="module")
def assemblies(tmp_path_factory):
    if shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists():
        pytest.skip("hipcc not available")
    tmp = tmp_path_factory.mktemp("isa")
    return {name: _assembly(CSRC / name, tmp) for name in ("gptq4_gemm.hip", "gptq4_kslice.hip")}


@pytest.mark.parametrize("source,variants", [("gptq4_gemm.hip", 9), ("gptq4_kslice.hip", 19)])
def test_hand_written_wait_counts_match_the_loads_behind_the_lds_direct_loads(assemblies, source, variants):
    with_waits = 0
    for name, lines in _kernels(assemblies[source]):
        found = _paths_to_waits(lines)
        for n, behind, at in found:
            assert behind >= n, (f"{name}: a path reaches `{lines[at][0]}` with only {behind} vector-memory instructions "
                                 f"behind the activation tile's LDS-direct loads: the tile may not have landed")
        with_waits += bool(found)
    # (the act-order variants of the tiled kernel stage their tiles through registers and have no such wait)
    assert with_waits >= variants, f"only {with_waits} kernel variants of {source} show such waits: the scan no longer sees them"


def test_the_scan_sees_a_missing_load():
    """The checker itself: a tile requested before the loop and at the top of every pass, the wait at the top."""
    def prog(loads_in_loop):
        body = [("buffer_load_dwordx4 v1, s[0:3], s4 offen lds", False)] + [("global_load_dword v9, v[4:5], off", False)] * 5
        body += [(".LBB0_1:", False), ("s_waitcnt vmcnt(4) lgkmcnt(0)", True), ("s_barrier", True),
                 ("buffer_load_dwordx4 v1, s[0:3], s4 offen lds", False), ("buffer_load_dwordx4 v2, s[0:3], s4 offen lds", False)]
        body += [("global_load_dword v6, v[4:5], off", False)] * loads_in_loop
        body += [("v_mfma_f32_32x32x16_f16 a[0:15], v[0:3], v[4:7], a[0:15]", False), ("s_cbranch_scc1 .LBB0_1", False), ("s_endpgm", False)]
        return body
    assert sorted(_paths_to_waits(prog(4))) == [(4, 4, 7), (4, 5, 7)]
    assert sorted(_paths_to_waits(prog(3))) == [(4, 3, 7), (4, 5, 7)]
    # a wait of the compiler's own (not between the asm markers) is not a checkpoint
    assert _paths_to_waits([(l, False) for l, _ in prog(3)]) == []
