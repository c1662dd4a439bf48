"""Build-time properties of the hand-scheduled kernels that no numerical test can be relied on to catch.

The kernel issues its LDS fragment reads and its matrix instructions as inline assembly and waits for the reads
itself; to the compiler the value of a read is there as soon as the statement is.  Should the register allocator
run out of registers inside the tile loop (the kernel uses all 512 of a wave), it would store such a value to
scratch memory before the read has arrived, or reuse a register that a read in flight is still going to write
-- wrong rows in the first case, a wild address in the second.  So the compiled code is inspected: from the first
fragment read to the end of the tile loop there must be no scratch instruction, and the loop must be one copy
(one loop header).  The other kernels that read their fragments this way (`scan_direct_kernel`,
`adam_fused_direct_kernel`) have registers to spare; for them the check is that they use no scratch memory at all.
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


@pytest.fixture(scope="module")
def scan_isa(isa):
    return isa["scan.hip"]


@pytest.mark.parametrize("norms_given", [0, 1])
@pytest.mark.parametrize("elem", ["5f16_t", "6bf16_t"])
def test_wide_scan_kernel_keeps_its_fragments_in_registers(scan_isa, elem, norms_given):
    name = f"_ZN3bgx16scan_wide_kernelINS_{elem}ELb{norms_given}EEEvNS_8ScanArgsE"
    m = re.search(rf"^{name}:[^\n]*\n(.*?)\n\s*s_endpgm", scan_isa, re.S | re.M)
    assert m, f"{name} not found in the compiled code"
    lines = m.group(1).splitlines()
    reads = [i for i, l in enumerate(lines) if "ds_read_b128" in l]
    headers = [i for i, l in enumerate(lines) if "Loop Header" in l and i > reads[0]]
    back = [i for i, l in enumerate(lines) if re.search(r"s_cbranch_scc\d\s+\.LBB", l) and i > headers[0]]
    assert reads and headers and back
    loop_end = back[0]
    body = lines[reads[0]:loop_end + 1]
    assert sum("v_mfma_f32_32x32x16" in l for l in lines[headers[0]:loop_end]) == 96, "one copy of the tile code"
    scratch = [l.strip() for l in body if "scratch_" in l]
    assert not scratch, f"scratch traffic between the first fragment read and the end of the tile loop: {scratch[:4]}"
    assert not any(re.search(r"\bs_load|s_buffer_load", l) for l in lines[headers[0]:loop_end]), \
        "scalar loads inside the loop share the counter the fragment waits count on"


@pytest.mark.parametrize("source,pattern", [
    ("scan.hip", r"_ZN3bgx18scan_direct_kernelI\S*"),
    ("adam.hip", r"_ZN3bgx24adam_fused_direct_kernelI\S*"),
])
def test_direct_to_lds_kernels_use_no_scratch(isa, source, pattern):
    """Every instantiation: no scratch instruction anywhere and a private segment of zero bytes."""
    text = isa[source]
    names = sorted(set(re.findall(rf"^({pattern}):", text, re.M)))
    assert names, f"no kernel matching {pattern} in {source}"
    for name in names:
        m = re.search(rf"^{re.escape(name)}:[^\n]*\n(.*?)\n\s*s_endpgm", text, re.S | re.M)
        assert m, name
        assert "scratch_" not in m.group(1), f"{name} spills"
        meta = re.search(rf"\.amdhsa_kernel {re.escape(name)}\n(.*?)\.end_amdhsa_kernel", text, re.S)
        assert meta and re.search(r"\.amdhsa_private_segment_fixed_size 0\b", meta.group(1)), name
