"""Dense preconditioner on the GPU against the CPU oracle (oracle/hessians.py): the fused per-module
`g @ H` launch, the Gram accumulation, and the classes that call them (Builder, InMemoryCollector,
Attributor, create_scorer's split transform).

Tolerance: the kernels work in fp32 like the reference (`g.float() @ H`, `P.float().T @ P.float()`):
relative L2 <= 1e-5 against the float64 oracle on the same (already rounded) inputs.
"""
import numpy as np
import pytest
import torch

from helpers import rel_l2
from oracle import hessians as oh
from oracle import loop as oloop
from oracle import scan as oscan

pytestmark = pytest.mark.gpu


def _rows(n, width, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    return torch.randn(n, width, generator=gen).to(dtype)


def _mats(dims, seed):
    gen = torch.Generator().manual_seed(seed)
    return [torch.randn(d, d, generator=gen) / d ** 0.5 for d in dims]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [1, 130, 1000])
def test_block_gemm_against_oracle(device, dtype, n):
    from bergson_amd import ops

    dims = [256, 64, 128, 256]
    cols = [0, 256, 320, 448]
    rows = _rows(n, sum(dims), dtype, 1)
    mats = _mats(dims, 2)
    out = ops.block_gemm(rows.to(device), [(m.to(device), c) for m, c in zip(mats, cols)])
    torch.cuda.synchronize()
    assert out.dtype == torch.float32 and out.shape == rows.shape
    want = np.concatenate([rows[:, c:c + d].double().numpy() @ m.double().numpy()
                           for m, c, d in zip(mats, cols, dims)], axis=1)
    assert rel_l2(out, torch.from_numpy(want)) <= 1e-5


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_block_gemm_odd_sizes_gaps_and_strides(device, dtype):
    """Block sizes that are no multiple of anything (p = 5 -> 25, 13 -> 169), a module without a matrix in the
    middle (copied through), a row block that is a column slice of a wider buffer, a 16-bit output."""
    from bergson_amd import ops

    dims = [25, 169, 40, 1030]
    cols = [0, 25, 194, 234]
    width = sum(dims)
    wide = _rows(77, width + 3, dtype, 3)
    rows = wide[:, 3:]                                  # unaligned first column, stride != width
    mats = _mats(dims, 4)
    blocks = [(mats[i].to(device), cols[i]) for i in (0, 1, 3)]   # dims[2] has no matrix
    out = ops.block_gemm(wide.to(device)[:, 3:], blocks)
    torch.cuda.synchronize()
    want = rows.double().clone()
    for i in (0, 1, 3):
        want[:, cols[i]:cols[i] + dims[i]] = rows[:, cols[i]:cols[i] + dims[i]].double() @ mats[i].double()
    assert rel_l2(out, want) <= 1e-5
    assert torch.equal(out[:, 194:234].cpu(), rows[:, 194:234].float())
    out16 = ops.block_gemm(wide.to(device)[:, 3:], blocks, out_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    assert out16.dtype == torch.bfloat16 and rel_l2(out16, want) <= 1e-2


def test_block_gemm_rejects_bad_arguments(device):
    from bergson_amd import ops

    rows = torch.zeros(4, 32, device=device)
    with pytest.raises(ValueError):
        ops.block_gemm(rows, [(torch.zeros(16, 16, device=device), 20)])       # runs past the row
    with pytest.raises(ValueError):
        ops.block_gemm(rows, [(torch.zeros(16, 8, device=device), 0)])         # not square
    with pytest.raises(ValueError):
        ops.block_gemm(rows, [(torch.zeros(32, 32, device=device), 0)], out=rows)  # in place
    with pytest.raises(RuntimeError):
        ops.block_gemm(rows.cpu(), [(torch.zeros(32, 32, device=device), 0)])  # no CPU path


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
def test_gram_accumulate_against_oracle(device, dtype):
    from bergson_amd import ops

    dims = [256, 25, 64, 300]
    cols = [0, 256, 281, 345]
    width = sum(dims)
    batches = [_rows(n, width, dtype, 10 + n) for n in (7, 130, 1, 48)]
    hs = [torch.zeros(d, d, device=device) for d in dims]
    for b in batches:
        ops.gram_accumulate(b.to(device), list(zip(hs, cols)))
    torch.cuda.synchronize()
    for h, c, d in zip(hs, cols, dims):
        want = oh.gram([b[:, c:c + d].double().numpy() for b in batches], 1)
        assert rel_l2(h, torch.from_numpy(want)) <= 1e-5
        assert torch.equal(h, h.T)  # every (i, j) and (j, i) pair is the same sum in the same order


def _save_hessians(path, names, dims, seed):
    """A processor directory holding a random s.p.d. Gram per module; returns the Grams."""
    from bergson_amd import GradientProcessor

    gen = torch.Generator().manual_seed(seed)
    hess = {}
    for name, d in zip(names, dims):
        A = torch.randn(d, 2 * d, generator=gen)
        hess[name] = (A @ A.T / (2 * d)) * 1e-2
    proc = GradientProcessor(projection_dim=16, projection_type="normal")
    proc.hessians = hess
    proc.save(path)
    return hess


@pytest.mark.parametrize("unit_normalize", [False, True])
def test_builder_preconditions_rows(device, tmp_path, unit_normalize):
    """Builder with preprocess_cfg.hessian_path: rows @ H^-1 (or H^-1/2, then unit norm) land in the store."""
    from bergson_amd import Builder, InversionConfig, PreprocessConfig
    from bergson_amd.synthetic import ListDataset

    names, dims = ["m0", "m1", "m2"], [256, 64, 256]
    hess = _save_hessians(tmp_path / "hess", names, dims, 5)
    cfg = PreprocessConfig(unit_normalize=unit_normalize, hessian_path=str(tmp_path / "hess"),
                           inversion_cfg=InversionConfig("damped_inverse", 0.2))
    data = ListDataset([[1, 2, 3]] * 9)
    b = Builder(data, dict(zip(names, dims)), torch.float32, cfg, device=torch.device(device))
    assert not b.direct
    rows = _rows(9, sum(dims), torch.float32, 6) * 0.1
    mod = {n: rows[:, lo:lo + d].to(device) for n, lo, d in zip(names, [0, 256, 320], dims)}
    b(list(range(9)), mod)
    b.teardown()
    power = -0.5 if unit_normalize else -1.0
    want = np.concatenate([rows[:, lo:lo + d].double().numpy() @ oh.invert_psd(hess[n].numpy(), "damped_inverse", 0.2, power)
                           for n, lo, d in zip(names, [0, 256, 320], dims)], axis=1)
    if unit_normalize:
        want = want / np.linalg.norm(want, axis=1, keepdims=True)
    assert rel_l2(torch.from_numpy(np.array(b.grad_buffer)), torch.from_numpy(want)) <= 2e-5


def test_in_memory_collector_fits_the_autocorrelation(device, tmp_path):
    """skip_hessians=False: processor.hessians[name] = sum over documents of P^T P / num documents, where P are
    the rows the collector produced; eigendecompositions attached; the saved processor loads as a
    preconditioner."""
    from bergson_amd import GradientProcessor, IndexConfig, InMemoryCollector, allocate_batches, load_preconditioner
    from bergson_amd.collector import CollectorComputer
    from bergson_amd.synthetic import ListDataset, make_gpt_neox, random_docs

    lengths = [40, 22, 31, 17, 48, 9]
    docs = random_docs(lengths, seed=12)
    data = ListDataset(docs)
    batches = allocate_batches(lengths, 96)
    assert len(batches) > 1
    cpu = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=0, layers=2)
    gpu = make_gpt_neox("pythia-14m", torch.float32, device, seed=0, layers=2)
    want_rows, _ = oloop.collect(cpu, cpu.base_model, docs, batches, p=16)
    proc = GradientProcessor(projection_dim=16, projection_type="normal")
    cfg = IndexConfig(projection_dim=16, projection_type="normal")
    col = InMemoryCollector(model=gpu.base_model, cfg=cfg, data=data, processor=proc, skip_hessians=False)
    CollectorComputer(model=gpu, data=data, collector=col, batches=batches, cfg=cfg).run_with_collector_hooks()
    names = list(col.gradients)
    assert set(proc.hessians) == set(names) and set(proc.hessians_eigen) == set(names)
    for i, name in enumerate(names):
        P = want_rows[:, i * 256:(i + 1) * 256].double().numpy()
        want = oh.gram([P], len(lengths))
        got = proc.hessians[name]
        assert got.device.type == "cpu" and got.dtype == torch.float32
        assert rel_l2(got, torch.from_numpy(want)) <= 1e-4
        lam, vec = proc.hessians_eigen[name]
        assert rel_l2((vec * lam) @ vec.T, got) <= 1e-4
    proc.save(tmp_path / "fit")
    pre = load_preconditioner(tmp_path / "fit", power=-1.0, device=device)
    assert set(pre.h_inv) == set(names) and all(h.is_cuda and h.dtype == torch.float32 for h in pre.h_inv.values())


@pytest.mark.parametrize("unit_norm", [False, True])
def test_attributor_with_hessian(device, tmp_path, unit_norm):
    """Preconditioned search: scores are q H^-1 g (one-sided) or the cosine of H^-1/2 q and H^-1/2 g."""
    from bergson_amd import Attributor, GradientProcessor, create_index

    names, dims = ["a", "b"], [256, 64]
    n, Q, k = 300, 5, 7
    hess = _save_hessians(tmp_path / "hess", names, dims, 7)
    rows = _rows(n, 320, torch.float32, 8) * 0.1
    idx = tmp_path / "index"
    buf = create_index(idx, num_grads=n, grad_sizes=dict(zip(names, dims)), dtype="float32")
    buf[:] = rows.numpy()
    buf.flush()
    GradientProcessor(projection_dim=16, projection_type="normal").save(idx)
    q = _rows(Q, 320, torch.float32, 9)
    attr = Attributor(idx, device=device, unit_norm=unit_norm, hessian_path=tmp_path / "hess")
    assert attr.precondition == ("two-sided" if unit_norm else "one-sided")
    vals, inds = attr.search({"a": q[:, :256], "b": q[:, 256:]}, k=k)
    power = -0.5 if unit_norm else -1.0
    hinv = [oh.invert_psd(hess[nm].numpy(), "damped_inverse", 0.1, power) for nm in names]

    def transform(x):
        x = x.double().numpy()
        return np.concatenate([x[:, :256] @ hinv[0], x[:, 256:] @ hinv[1]], axis=1)

    qt = transform(q)
    if unit_norm:
        gt = transform(rows)
        scores = (qt / np.linalg.norm(qt, axis=1, keepdims=True)) @ (gt / np.linalg.norm(gt, axis=1, keepdims=True)).T
        tol = 1e-3
    else:
        scores = qt @ rows.double().numpy().T
        tol = 1e-3 * np.abs(scores).max()
    want_idx = np.argsort(-scores, axis=1)[:, :k]
    got_scores = np.take_along_axis(scores, inds.cpu().numpy(), axis=1)
    assert np.abs(got_scores - vals.cpu().double().numpy()).max() <= tol          # values are the scores of those rows
    assert np.abs(np.take_along_axis(scores, want_idx, axis=1) - got_scores).max() <= tol   # and they are the top k


def test_split_transform_of_create_scorer(device, tmp_path):
    """make_split_hessian: the per-batch index transform is rows @ H^-1/2 per module, as a row block the
    Scorer takes without another concatenation."""
    from bergson_amd.builder import RowBlock
    from bergson_amd.hessians import load_preconditioner, make_split_hessian

    names, dims = ["x", "y"], [64, 256]
    hess = _save_hessians(tmp_path / "hess", names, dims, 11)
    pre = load_preconditioner(tmp_path / "hess", power=-0.5, device=device)
    tr = make_split_hessian(pre.h_inv, names, torch.device(device), torch.float32)
    rows = _rows(33, 320, torch.bfloat16, 12)
    out = tr({"x": rows[:, :64].to(device), "y": rows[:, 64:].to(device)})
    assert isinstance(out, RowBlock) and list(out) == names and out.rows.shape == (33, 320)
    want = np.concatenate([rows[:, :64].double().numpy() @ oh.invert_psd(hess["x"].numpy(), "damped_inverse", 0.1, -0.5),
                           rows[:, 64:].double().numpy() @ oh.invert_psd(hess["y"].numpy(), "damped_inverse", 0.1, -0.5)], 1)
    assert rel_l2(out.rows, torch.from_numpy(want)) <= 2e-5
