"""Build-time properties of the hand-scheduled kernels that no numerical test can be relied on to catch.

The rules themselves live in bergson_amd/isa_checks.py, and `build_ext.build()` applies them to every library it
links; this file runs them on a fresh compilation and checks that they do report violations.

The kernel issues its LDS fragment reads and its matrix instructions as inline assembly and waits for the reads
itself; to the compiler the value of a read is there as soon as the statement is.  Should the register allocator
run out of registers inside the tile loop (the kernel uses all 512 of a wave), it would store such a value to
scratch memory before the read has arrived, or reuse a register that a read in flight is still going to write
-- wrong rows in the first case, a wild address in the second.  So the compiled code is inspected: from the first
fragment read to the end of the tile loop there must be no scratch instruction, and the loop must be one copy
(one loop header).  The other kernels that read their fragments this way (`scan_direct_kernel`,
`adam_fused_direct_kernel`) have registers to spare; for them the check is that they use no scratch memory at all.
`adam_fused_wide_kernel` runs one wave per SIMD like the wide scan kernel, with several copies of its tile code;
it ends every k-step with a wait for its reads, so that no read is in flight where the copies meet, and the checks
are: no scratch memory, no wait for all vector-memory loads between the first and the last matrix instruction (a
scratch access or a table the compiler keeps in memory would bring one, and it would drain the load pipeline
every tile), the accumulators never moved between the register files, and two wait states in front of every
matrix instruction that reads what vector instructions have just written.
hipcc cross-compiles without a GPU; the two compilations run side by side and take about a minute.
"""
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def isa(tmp_path_factory):
    """{source name: compiled device code as text} for scan.hip and adam.hip."""
    from concurrent.futures import ThreadPoolExecutor

    from bergson_amd import build_ext

    tmp = tmp_path_factory.mktemp("isa")

    def compile_one(src):
        out = tmp / (src + ".s")
        cmd = [build_ext.HIPCC, *build_ext.FLAGS, "--cuda-device-only", "-S", str(build_ext.CSRC / src), "-o", str(out)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        assert res.returncode == 0, res.stderr[-2000:]
        return out.read_text()

    with ThreadPoolExecutor(max_workers=2) as ex:
        texts = list(ex.map(compile_one, ["scan.hip", "adam.hip"]))
    return {"scan.hip": texts[0], "adam.hip": texts[1]}


@pytest.mark.parametrize("norms_given", [0, 1])
@pytest.mark.parametrize("elem", ["5f16_t", "6bf16_t"])
def test_wide_scan_kernel_keeps_its_fragments_in_registers(isa, elem, norms_given):
    from bergson_amd import isa_checks

    assert isa_checks.wide_scan_kernel(isa["scan.hip"], elem, norms_given) == []


@pytest.mark.parametrize("source,pattern", [
    ("scan.hip", r"_ZN3bgx18scan_direct_kernelI\S*"),
    ("adam.hip", r"_ZN3bgx24adam_fused_direct_kernelI\S*"),
])
def test_direct_to_lds_kernels_use_no_scratch(isa, source, pattern):
    """Every instantiation: no scratch instruction anywhere and a private segment of zero bytes."""
    from bergson_amd import isa_checks

    assert isa_checks.no_scratch(isa[source], pattern) == []


@pytest.mark.parametrize("elem", ["5f16_t", "6bf16_t"])
def test_wide_adam_kernel_keeps_its_pipeline(isa, elem):
    from bergson_amd import isa_checks

    assert isa_checks.wide_adam_kernel(isa["adam.hip"], elem) == []


def test_the_checks_see_a_violation(isa):
    """The inspection is not vacuous: a scratch store planted in the tile loop, a dropped wait state and a
    missing kernel are each reported."""
    from bergson_amd import isa_checks

    text = isa["scan.hip"]
    name = "_ZN3bgx16scan_wide_kernelINS_5f16_tELb0EEEvNS_8ScanArgsE"
    start = text.index(f"\n{name}:")
    at = text.index("v_mfma_f32_32x32x16", text.index("Loop Header", text.index("ds_read_b128", start)))
    planted = text[:at] + "scratch_store_dword off, v0, off\n\t" + text[at:]
    assert any("scratch" in v for v in isa_checks.wide_scan_kernel(planted, "5f16_t", 0))
    adam = isa["adam.hip"].replace("s_nop 1", "s_nop 0")
    assert any("s_nop" in v for v in isa_checks.wide_adam_kernel(adam, "6bf16_t"))
    assert isa_checks.wide_scan_kernel("", "5f16_t", 0) and isa_checks.no_scratch("", "_ZN3bgx18scan_direct_kernelI\\S*")


def test_build_refuses_a_library_that_breaks_the_rules(monkeypatch):
    """build() runs the same inspection before it links (here with the inspection made to fail, and the
    compile and link steps left out)."""
    from bergson_amd import build_ext, isa_checks

    monkeypatch.setattr(build_ext, "_compile", lambda src, verbose, temps=None: build_ext.CSRC / "x.o")
    monkeypatch.setattr(build_ext, "device_assembly", lambda temps, src: "")
    monkeypatch.setattr(build_ext.Path, "unlink", lambda self, missing_ok=False: None)
    with pytest.raises(RuntimeError, match="scheduling rules"):
        build_ext.build(verbose=False)
    assert isa_checks.all_violations({"scan.hip": "", "adam.hip": ""})
