"""`bgx_collect_seq_static`, the entry point that allocates nothing: its rows must equal `bgx_collect_seq`'s bit
for bit (same kernels, the workspace being the library's static scratch array instead of a caller's buffer,
the tables arriving as kernel arguments instead of a host-to-device copy) and the oracle's within the
collection tolerance; on two calls in a row, the second smaller than the first, so that what the first call
left in the array would show.  Collected last, so that it also runs after every other test has used the GPU.
"""
import ctypes as C

import pytest
import torch

from helpers import TOL, rel_l2
from oracle import hooks as ohooks
from oracle.projection import module_projections

pytestmark = pytest.mark.gpu


def _case(N, S, shapes, p, dtype, seed, lengths):
    gen = torch.Generator().manual_seed(seed)
    mods = []
    for k, (I, O) in enumerate(shapes):
        a = torch.randn(N, S, I, generator=gen).to(dtype)
        g = (torch.randn(N, S, O, generator=gen) * 0.1).to(dtype)
        for n, l in enumerate(lengths):
            g[n, l - 1:] = 0
        left, right = module_projections(f"layers.{k}.mlp.dense_h_to_4h", p, O, I, dtype)
        norm = ohooks.Adafactor(row=torch.rand(O, generator=gen) * 1e-4 + 1e-8,
                                col=torch.rand(I, generator=gen) * 1e-4 + 1e-8) if k % 2 == 0 else None
        mods.append((a, g, left, right, norm))
    return mods


def _run(device, mods, p, lengths, out_rows, n_rows, out_dtype, static):
    from bergson_amd import ops

    inputs = []
    for k, (a, g, left, right, norm) in enumerate(mods):
        row_scale = col_scale = None
        if norm is not None:
            row_scale, col_scale = ops.adafactor_scales(norm.row.to(device), norm.col.to(device), a.dtype)
        inputs.append(ops.ModuleInput(a=a.to(device), g=g.to(device), r_in=right.to(device), r_out=left.to(device),
                                      out_col=k * p * p, col_scale=col_scale, row_scale=row_scale))
    out = torch.zeros(n_rows, len(mods) * p * p, dtype=out_dtype, device=device)
    ldev = torch.tensor(lengths, dtype=torch.int32, device=device)
    rdev = torch.tensor(out_rows, dtype=torch.int64, device=device)
    fn = ops.collect_seq_static if static else ops.collect_seq
    fn(inputs, p, out, lengths=ldev, out_rows=rdev, lo=torch.finfo(out_dtype).min, hi=torch.finfo(out_dtype).max)
    torch.cuda.synchronize()
    return out.cpu()


@pytest.mark.parametrize("dtype,out_dtype", [(torch.bfloat16, torch.float16), (torch.float32, torch.float32)])
def test_static_scratch_entry_equals_the_workspace_entry(device, dtype, out_dtype):
    p = 16
    # first call: 5 modules, a wide one among them, ragged lengths; second call: fewer, smaller, other shapes
    calls = [
        (3, 300, [(128, 384), (512, 128), (128, 128), (256, 1024), (96, 160)], [300, 41, 177], [4, 0, 2], 5),
        (2, 70, [(64, 96), (128, 64)], [70, 33], [1, 0], 2),
    ]
    for seed, (N, S, shapes, lengths, out_rows, n_rows) in enumerate(calls):
        mods = _case(N, S, shapes, p, dtype, 80 + seed, lengths)
        got = _run(device, mods, p, lengths, out_rows, n_rows, out_dtype, static=True)
        ref = _run(device, mods, p, lengths, out_rows, n_rows, out_dtype, static=False)
        assert torch.equal(got, ref), f"call {seed}"
        lo, hi = torch.finfo(out_dtype).min, torch.finfo(out_dtype).max
        want = torch.cat([ohooks.module_gradient(a, g, norm, left, right).float().clamp(lo, hi)
                          for a, g, left, right, norm in mods], dim=1)
        assert rel_l2(got[out_rows], want) <= TOL[dtype], f"call {seed}"
        untouched = [r for r in range(n_rows) if r not in out_rows]
        assert got[untouched].abs().sum() == 0


def test_static_scratch_entry_allocates_no_device_memory(device):
    """The property the entry point is named for: a call (after the first on the device, which looks up the
    array's address) leaves the device's free memory and torch's allocator exactly where they were."""
    from bergson_amd import ops

    p, N, S, lengths = 16, 2, 200, [200, 77]
    mods = _case(N, S, [(128, 256), (256, 128)], p, torch.bfloat16, 90, lengths)
    inputs = [ops.ModuleInput(a=a.to(device), g=g.to(device), r_in=right.to(device), r_out=left.to(device),
                              out_col=k * p * p) for k, (a, g, left, right, _norm) in enumerate(mods)]
    out = torch.zeros(N, len(mods) * p * p, dtype=torch.float16, device=device)
    ldev = torch.tensor(lengths, dtype=torch.int32, device=device)
    ops.collect_seq_static(inputs, p, out, lengths=ldev)   # warm-up: first use on this device
    torch.cuda.synchronize()
    first = out.clone()
    free0, _ = torch.cuda.mem_get_info()
    held0, reserved0 = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    for _ in range(3):
        ops.collect_seq_static(inputs, p, out, lengths=ldev)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == held0 and torch.cuda.memory_reserved() == reserved0
    assert torch.cuda.mem_get_info()[0] == free0
    assert torch.equal(out, first)


def test_static_scratch_entry_refuses_what_does_not_fit(device):
    from bergson_amd import _lib

    lib = _lib.load()
    n_modules, N, S, p = 48, 64, 4096, 16
    assert lib.bgx_collect_workspace_bytes(n_modules, N, S, p) > _lib.STATIC_SCRATCH_BYTES
    descs = (_lib.ModuleDesc * n_modules)()
    rc = lib.bgx_collect_seq_static(descs, n_modules, N, S, p, _lib.BGX_BF16, None, None, C.c_void_p(256), 48 * 256,
                                    _lib.BGX_F16, 0.0, 0.0, None)
    assert rc == -4 and b"static" in lib.bgx_last_error()
