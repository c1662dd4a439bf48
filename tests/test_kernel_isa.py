"""A build-time property of `scan_wide_kernel` that no numerical test can be relied on to catch.

The kernel issues its LDS fragment reads and its matrix instructions as inline assembly and waits for the reads
itself; to the compiler the value of a read is there as soon as the statement is.  Should the register allocator
run out of registers inside the tile loop (the kernel uses all 512 of a wave), it would store such a value to
scratch memory before the read has arrived, or reuse a register that a read in flight is still going to write
-- wrong rows in the first case, a wild address in the second.  So the compiled code is inspected: from the first
fragment read to the end of the tile loop there must be no scratch instruction, and the loop must be one copy
(one loop header).  hipcc cross-compiles without a GPU; the test takes about a minute.
"""
import re
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def scan_isa(tmp_path_factory):
    from bergson_amd import build_ext

    out = tmp_path_factory.mktemp("isa") / "scan.s"
    cmd = [build_ext.HIPCC, *build_ext.FLAGS, "--cuda-device-only", "-S", str(build_ext.CSRC / "scan.hip"), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    return out.read_text()


@pytest.mark.parametrize("elem", ["5f16_t", "6bf16_t"])
def test_wide_scan_kernel_keeps_its_fragments_in_registers(scan_isa, elem):
    name = f"_ZN3bgx16scan_wide_kernelINS_{elem}EEEvNS_8ScanArgsE"
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
