"""Build-time properties of the hand-scheduled kernels, checked on the compiled device code.

`scan_wide_kernel` and `adam_fused_wide_kernel` issue their LDS fragment reads and matrix instructions as
inline assembly and wait for the reads themselves; to the compiler the value of such a read is there as soon
as the statement ends.  Should the register allocator run out of registers inside the tile loop (the kernels
use all 512 of a wave) it would store such a value to scratch memory before the read has arrived, or reuse a
register a read in flight is still going to write -- wrong results in the first case, a wild address in the
second, and no numerical test can be relied on to catch either.  So the text of the compiled code is
inspected; `build_ext.build()` refuses to link a library whose kernels break one of these rules, and
tests/test_kernel_isa.py runs the same functions.

Each function takes the device assembly of one source file and returns a list of violations (empty = fine).
"""
from __future__ import annotations

import re

WIDE_SCAN_MFMAS_PER_TILE = 96
WIDE_ADAM_TILE_COPIES = 5  # copies of the 64-MFMA K tile in the unrolled chunk
WIDE_ADAM_SLICES = 4  # g slices per chunk, 8 MFMAs each


def _body(text: str, name: str) -> list[str] | None:
    m = re.search(rf"^{re.escape(name)}:[^\n]*\n(.*?)\n\s*s_endpgm", text, re.S | re.M)
    return None if m is None else m.group(1).splitlines()


def _private_segment_is_empty(text: str, name: str) -> bool:
    meta = re.search(rf"\.amdhsa_kernel {re.escape(name)}\n(.*?)\.end_amdhsa_kernel", text, re.S)
    return bool(meta and re.search(r"\.amdhsa_private_segment_fixed_size 0\b", meta.group(1)))


def wide_scan_kernel(text: str, elem: str, norms_given: int) -> list[str]:
    """From the first fragment read to the end of the tile loop: no scratch instruction, no scalar load (they
    share the counter the fragment waits count on), and one copy of the tile code."""
    name = f"_ZN3bgx16scan_wide_kernelINS_{elem}ELb{norms_given}EEEvNS_8ScanArgsE"
    lines = _body(text, name)
    if lines is None:
        return [f"{name} not found in the compiled code"]
    reads = [i for i, l in enumerate(lines) if "ds_read_b128" in l]
    if not reads:
        return [f"{name}: no fragment reads"]
    headers = [i for i, l in enumerate(lines) if "Loop Header" in l and i > reads[0]]
    back = [i for i, l in enumerate(lines) if headers and re.search(r"s_cbranch_scc\d\s+\.LBB", l) and i > headers[0]]
    if not headers or not back:
        return [f"{name}: tile loop not found"]
    loop = lines[headers[0]:back[0]]
    bad = []
    n = sum("v_mfma_f32_32x32x16" in l for l in loop)
    if n != WIDE_SCAN_MFMAS_PER_TILE:
        bad.append(f"{name}: {n} matrix instructions in the tile loop, expected one copy of {WIDE_SCAN_MFMAS_PER_TILE}")
    scratch = [l.strip() for l in lines[reads[0]:back[0] + 1] if "scratch_" in l]
    if scratch:
        bad.append(f"{name}: scratch traffic between the first fragment read and the end of the tile loop: {scratch[:4]}")
    if any(re.search(r"\bs_load|s_buffer_load", l) for l in loop):
        bad.append(f"{name}: scalar loads inside the tile loop")
    return bad


def no_scratch(text: str, pattern: str) -> list[str]:
    """Every kernel whose mangled name matches `pattern`: no scratch instruction, a private segment of 0 bytes."""
    names = sorted(set(re.findall(rf"^({pattern}):", text, re.M)))
    if not names:
        return [f"no kernel matching {pattern}"]
    bad = []
    for name in names:
        lines = _body(text, name)
        if lines is None or any("scratch_" in l for l in lines) or not _private_segment_is_empty(text, name):
            bad.append(f"{name} spills")
    return bad


def wide_adam_kernel(text: str, elem: str) -> list[str]:
    """No scratch memory; between the first and the last matrix instruction no wait for all vector-memory
    loads and no memory read other than the direct-to-LDS loads (either would drain the load pipeline every
    tile); the accumulators never moved between the register files; two wait states in front of every matrix
    instruction that reads what vector instructions have just written (the hardware does not interlock an
    MFMA written as an instruction against the VALU result it reads)."""
    name = f"_ZN3bgx22adam_fused_wide_kernelINS_{elem}EEEvNS_9FusedArgsE"
    raw = _body(text, name)
    if raw is None:
        return [f"{name} not found in the compiled code"]
    bad = []
    if not _private_segment_is_empty(text, name):
        bad.append(f"{name}: private segment is not empty")
    lines = [l.strip() for l in raw]
    lines = [l for l in lines if l and not l.startswith(";")]
    if any("scratch_" in l for l in lines):
        bad.append(f"{name} spills")
    mfma = [i for i, l in enumerate(lines) if l.startswith("v_mfma_f32_32x32x16")]
    want = WIDE_ADAM_TILE_COPIES * 64 + WIDE_ADAM_SLICES * 8
    if len(mfma) != want:
        return bad + [f"{name}: {len(mfma)} matrix instructions, expected {want}"]
    body = lines[mfma[0]:mfma[-1] + 1]
    if any(re.match(r"s_waitcnt.*vmcnt\(0\)", l) for l in body):
        bad.append(f"{name}: a wait for every load inside the pipeline")
    if any(re.search(r"\bs_load|s_buffer_load|flat_load|global_load_dword", l) for l in body):
        bad.append(f"{name}: memory reads other than the direct-to-LDS loads inside the pipeline")
    if any(l.startswith(("v_accvgpr_write", "v_accvgpr_mov")) for l in body):
        bad.append(f"{name}: accumulators moved between the register files")
    n_read = sum(l.startswith("v_accvgpr_read") for l in body)
    if n_read != 256:
        bad.append(f"{name}: {n_read} accumulator reads per chunk, expected 256")
    second = [i for i in mfma if re.match(r"v_mfma\S+ v\[", lines[i])]
    if len(second) != WIDE_ADAM_SLICES * 8:
        bad.append(f"{name}: {len(second)} second-pass matrix instructions, expected {WIDE_ADAM_SLICES * 8}")
    for i in second:
        if lines[i - 1] != "s_nop 1":
            bad.append(f"{name}: no s_nop 1 in front of {lines[i]!r} (after {lines[i - 1]!r})")
            break
    return bad


def all_violations(texts: dict[str, str]) -> list[str]:
    """`texts`: {"scan.hip": device assembly, "adam.hip": device assembly}."""
    bad = []
    for elem in ("5f16_t", "6bf16_t"):
        for norms_given in (0, 1):
            bad += wide_scan_kernel(texts["scan.hip"], elem, norms_given)
        bad += wide_adam_kernel(texts["adam.hip"], elem)
    bad += no_scratch(texts["scan.hip"], r"_ZN3bgx18scan_direct_kernelI\S*")
    bad += no_scratch(texts["adam.hip"], r"_ZN3bgx24adam_fused_direct_kernelI\S*")
    return bad
