"""Host-side check of the device code of the MX GEMM kernels: the K loop of a persistent kernel
must not contain a vector-memory wait that the compiler added on its own.

The kernels wait for their direct-to-LDS copies with hand-written ``s_waitcnt vmcnt(N)``
instructions inside ``asm`` statements, which leave copies of later slabs in flight. The
compiler's own wait-count bookkeeping does not see those; if it believes that a vector load of
the epilogue may still be outstanding when the K loop of the next tile begins (a load and its use
in two separately guarded blocks are enough), it puts an ``s_waitcnt vmcnt(0)`` in front of the
first instruction of the loop that overwrites the load's register -- and every slab then begins by
waiting for all copies in flight (dense MXFP8 16384^3: 3.2 -> 3.7 ms). The test compiles three
translation units to assembly (no GPU needed) and looks at the MFMA loops of their kernels."""

import re
import subprocess
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT / "primus-turbo_amd"))


def _functions(lines):
    cur = None
    for i, line in enumerate(lines):
        m = re.match(r"^(_Z\w+):", line)
        if m:
            cur = [m.group(1), i, None]
        elif cur is not None and line.startswith(".Lfunc_end"):
            cur[2] = i
            yield tuple(cur)
            cur = None


def _innermost_mfma_loops(body):
    labels = {m.group(1): i for i, l in enumerate(body) if (m := re.match(r"^(\.LBB\d+_\d+):", l))}
    loops = []
    for i, l in enumerate(body):
        m = re.match(r"\s+s_cbranch_\w+ (\.LBB\d+_\d+)", l)
        if m and labels.get(m.group(1), i) < i:
            loops.append((labels[m.group(1)], i))
    with_mfma = [(s, e) for s, e in loops if sum("v_mfma" in x for x in body[s:e]) >= 16]
    return [(s, e) for s, e in with_mfma if not any(s < s2 and e2 < e for s2, e2 in with_mfma)]


def _compiler_vmcnt_waits(seg):
    """``s_waitcnt`` instructions with a vmcnt field outside the kernel's own asm statements."""
    out, in_asm = [], False
    for x in seg:
        if "#ASMSTART" in x:
            in_asm = True
        elif "#ASMEND" in x:
            in_asm = False
        elif not in_asm and "s_waitcnt" in x and "vmcnt" in x:
            out.append(x.strip())
    return out


def test_scanner_sees_a_compiler_wait():
    body = [".LBB0_1:"] + ["\tv_mfma_f32 a, b, c"] * 16 + ["\t;;#ASMSTART", "\ts_waitcnt vmcnt(3)", "\t;;#ASMEND",
                                                          "\ts_waitcnt vmcnt(0)", "\ts_cbranch_scc0 .LBB0_1"]
    (s, e), = _innermost_mfma_loops(body)
    assert _compiler_vmcnt_waits(body[s:e]) == ["s_waitcnt vmcnt(0)"]


# translation unit -> which of its kernels are looked at: the dense MX kernels (gemm_mx8_kernel and
# gemm_fp8_nt_kernel<TM, TN, 2 = MX, ...>), the block-scaled eight-wavefront kernel of the
# headline workload (the four-wavefront block kernels of that unit load their scales into
# registers inside the loop and wait for them legitimately) and the grouped vector-scale kernels
UNITS = {
    "gemm_mx.hip": (lambda n: "gemm_mx8_kernel" in n or re.search(r"gemm_fp8_nt_kernelILi\dELi\dELi2E", n), 8),
    "gemm_fp8_block.hip": (lambda n: "gemm_fp8_block8_kernel" in n, 4),
    # vector scales (tensorwise / rowwise), row groups and variable K: the epilogue loads its scales
    "gemm_fp8_grouped_vec.hip": (lambda n: re.search(r"gemm_fp8_nt_kernelILi\dELi\dELi0E", n), 8),
}


@pytest.fixture(scope="module")
def assembly(tmp_path_factory):
    """Device assembly of the units, compiled side by side (about two minutes of hipcc)."""
    from concurrent.futures import ThreadPoolExecutor

    import build_native

    try:
        hipcc = build_native.hipcc_path()
    except RuntimeError:
        pytest.skip("hipcc not found")
    out = tmp_path_factory.mktemp("asm")
    flags = [f for f in build_native.HIPCC_FLAGS if f != "-fPIC"]

    def one(unit):
        src = build_native.CSRC / unit
        asm = out / (src.stem + ".s")
        cmd = [hipcc, *flags, *build_native._extra_flags(src), "-S", "--cuda-device-only", "-o", str(asm), str(src)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        assert res.returncode == 0, res.stderr[-2000:]
        return unit, asm.read_text().split("\n")

    with ThreadPoolExecutor(max_workers=len(UNITS)) as ex:
        return dict(ex.map(one, UNITS))


@pytest.mark.parametrize("unit", sorted(UNITS))
def test_mfma_loops_have_no_compiler_inserted_vmcnt_wait(assembly, unit):
    lines = assembly[unit]
    wanted, least = UNITS[unit]
    seen, bad = 0, []
    for name, a, b in _functions(lines):
        if not wanted(name):
            continue
        body = lines[a:b]
        for s, e in _innermost_mfma_loops(body):
            seen += 1
            waits = _compiler_vmcnt_waits(body[s:e])
            if waits:
                bad.append((name, waits))
    assert seen >= least, f"only {seen} MFMA loops found: the scanner no longer matches the compiler's output"
    assert not bad, bad
