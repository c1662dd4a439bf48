"""Build-time properties of the hand-scheduled kernels that no numerical test can be relied on to catch.

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


@pytest.mark.parametrize("elem", ["5f16_t", "6bf16_t"])
def test_wide_adam_kernel_keeps_its_pipeline(isa, elem):
    name = f"_ZN3bgx22adam_fused_wide_kernelINS_{elem}EEEvNS_9FusedArgsE"
    text = isa["adam.hip"]
    m = re.search(rf"^{name}:[^\n]*\n(.*?)\n\s*s_endpgm", text, re.S | re.M)
    assert m, f"{name} not found in the compiled code"
    meta = re.search(rf"\.amdhsa_kernel {re.escape(name)}\n(.*?)\.end_amdhsa_kernel", text, re.S)
    assert meta and re.search(r"\.amdhsa_private_segment_fixed_size 0\b", meta.group(1))
    lines = [l.strip() for l in m.group(1).splitlines()]
    lines = [l for l in lines if l and not l.startswith(";")]
    assert not any("scratch_" in l for l in lines), "spills"
    mfma = [i for i, l in enumerate(lines) if l.startswith("v_mfma_f32_32x32x16")]
    body = lines[mfma[0]:mfma[-1] + 1]
    # five copies of the K tile (64 each) and four g slices (8 each)
    assert len(mfma) == 5 * 64 + 4 * 8
    assert not any(re.match(r"s_waitcnt.*vmcnt\(0\)", l) for l in body), "a wait for every load inside the pipeline"
    assert not any(re.search(r"\bs_load|s_buffer_load|flat_load|global_load_dword", l) for l in body), \
        "memory reads other than the direct-to-LDS loads inside the pipeline"
    assert not any(l.startswith(("v_accvgpr_write", "v_accvgpr_mov")) for l in body), "accumulators moved between the files"
    # 256 accumulators are read once per chunk, 64 per slice
    assert sum(l.startswith("v_accvgpr_read") for l in body) == 256
    # the second pass's MFMAs (ordinary registers as destination) follow an s_nop 1
    second = [i for i in mfma if re.match(r"v_mfma\S+ v\[", lines[i])]
    assert len(second) == 32
    for i in second:
        assert lines[i - 1] == "s_nop 1", (lines[i - 2:i + 1])
