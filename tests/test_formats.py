"""Byte-level layout of the gradient and score stores, product writers against the oracle's layout
description and against the literal values the reference's tests hold.

  * tests/test_score_writer_dist.py:61-74 of the reference writes the fp32 single-score record as
    {"score_0": "<f4" @ 0, "written_0": "?" @ 4, itemsize 8};
  * tests/test_attribute_tokens.py:37-178: num_token_grads = max(len - 1, 0), offsets = cumsum, empty
    documents own no rows;
  * tests/test_data.py: flat row-major round trip.
"""
import json

import numpy as np
import pytest
import torch

from oracle import store as ostore


class _Docs:
    def __init__(self, lengths):
        self.lengths = lengths
        self.column_names = ["length"]

    def __len__(self):
        return len(self.lengths)

    def __getitem__(self, k):
        assert k == "length"
        return self.lengths


def test_score_record_literals():
    from bergson_amd.score_writer import _score_struct_dtype

    spec, js = _score_struct_dtype(1, "float32")
    assert js == {"names": ["score_0", "written_0"], "formats": ["float32", "bool"], "offsets": [0, 4], "itemsize": 8}
    assert np.dtype(spec) == np.dtype({"names": ["score_0", "written_0"], "formats": ["<f4", "?"],
                                       "offsets": [0, 4], "itemsize": 8})
    # 16-bit scores: pairs of 4 bytes, record padded to 8
    _, js16 = _score_struct_dtype(3, "bfloat16")
    assert js16["offsets"] == [0, 2, 4, 6, 8, 10] and js16["itemsize"] == 16
    assert js16["formats"] == ["bfloat16", "bool"] * 3
    for n, name, size in [(1, "float32", 4), (5, "float32", 4), (3, "float16", 2), (2, "float64", 8)]:
        _, got = _score_struct_dtype(n, name)
        assert got == ostore.score_struct_dtype(n, size, name)


def test_token_offsets_known_answers():
    from bergson_amd.data import compute_num_token_grads

    lengths = [5, 1, 0, 2, 9]
    assert compute_num_token_grads(_Docs(lengths)).tolist() == [4, 0, 0, 1, 8]
    assert ostore.num_token_grads(lengths).tolist() == [4, 0, 0, 1, 8]
    assert ostore.token_offsets(lengths).tolist() == [0, 4, 4, 4, 5, 13]


@pytest.mark.parametrize("dtype", ["float16", "float32", "bfloat16"])
def test_create_index_bytes(tmp_path, dtype):
    from bergson_amd.data import column_offsets, create_index, load_gradients, load_module_gradients

    sizes = {"layers.0.a": 4, "layers.0.b": 6}
    mm = create_index(tmp_path, 3, sizes, dtype)
    assert mm.shape == (3, 10)
    itemsize = 4 if dtype == "float32" else 2
    assert (tmp_path / "gradients.bin").stat().st_size == 3 * 10 * itemsize
    assert not np.asarray(mm).any()  # created by truncate: all zero
    vals = torch.arange(30, dtype=torch.float32).reshape(3, 10) / 4
    tdt = {"float16": torch.float16, "float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    t = vals.to(tdt)
    mm[:] = t.view(torch.uint16).numpy() if dtype == "bfloat16" else t.numpy()
    mm.flush()
    info = json.loads((tmp_path / "info.json").read_text())
    assert info == ostore.index_info(3, 3, sizes, dtype, False)
    assert list(info["grad_sizes"]) == ["layers.0.a", "layers.0.b"]
    oinfo, raw = ostore.read_store_bytes(tmp_path)
    assert raw.shape == (3, 10 * itemsize)
    # row-major little-endian: element (r, c) sits at byte (r * 10 + c) * itemsize
    flat = np.frombuffer(raw.tobytes(), dtype=np.uint16 if itemsize == 2 else np.float32)
    back = torch.from_numpy(flat.copy()).view(tdt).reshape(3, 10) if itemsize == 2 else torch.from_numpy(flat.copy()).reshape(3, 10)
    assert torch.equal(back, t)
    assert np.array_equal(np.asarray(load_gradients(tmp_path)), np.asarray(mm))
    mg = load_module_gradients(tmp_path)
    assert column_offsets(sizes) == ostore.column_offsets(sizes) == {"layers.0.a": (0, 4), "layers.0.b": (4, 10)}
    assert mg["layers.0.b"].shape == (3, 6) and len(mg) == 3 and list(mg) == list(sizes)


def test_create_token_index_ragged(tmp_path):
    from bergson_amd.data import TokenGradients, create_token_index, load_token_gradients

    counts = np.array([4, 0, 1, 8], dtype=np.int64)
    mm, offsets = create_token_index(tmp_path, counts, {"m": 3}, "float32")
    assert offsets.tolist() == [0, 4, 4, 5, 13] and mm.shape == (13, 3)
    mm[:] = np.arange(39, dtype=np.float32).reshape(13, 3)
    mm.flush()
    info = json.loads((tmp_path / "info.json").read_text())
    assert info == ostore.index_info(4, 13, {"m": 3}, "float32", True)
    assert np.load(tmp_path / "offsets.npy").dtype == np.int64
    m2, n2, o2 = load_token_gradients(tmp_path)
    assert n2.tolist() == counts.tolist() and o2.tolist() == offsets.tolist()
    tg = TokenGradients(tmp_path)
    assert len(tg) == 4 and tg[1].shape == (0, 3) and tg[3].shape == (8, 3)
    assert tg[2][0].tolist() == [12.0, 13.0, 14.0]


def test_legacy_store_without_base_dtype(tmp_path):
    from bergson_amd.data import create_index, load_gradients

    create_index(tmp_path, 2, {"m": 4}, "float16")
    info = json.loads((tmp_path / "info.json").read_text())
    del info["base_dtype"]
    info["dtype"] = {"names": ["m"], "formats": ["('<f2', (4,))"], "offsets": [0], "itemsize": 8}
    info["dtype"]["formats"] = ["<f2"]
    (tmp_path / "info.json").write_text(json.dumps(info))
    assert load_gradients(tmp_path).dtype == np.float16


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_sequence_score_writer_columns_and_resume(tmp_path, dtype):
    from bergson_amd.data import load_scores
    from bergson_amd.score_writer import MemmapSequenceScoreWriter

    w = MemmapSequenceScoreWriter(tmp_path, 5, 3, dtype=dtype)
    w([4, 1], torch.tensor([[1.0, 2.0], [3.0, 4.0]]), query_offset=1)
    w.flush()
    sc = load_scores(tmp_path)
    assert len(sc) == 5 and sc.num_scores == 3 and not sc.is_written()
    rec = sc.mmap
    assert rec["written_1"].tolist() == [False, True, False, False, True]
    assert rec["written_0"].tolist() == [False] * 5
    if dtype != torch.bfloat16:
        assert rec["score_2"].tolist() == [0, 4.0, 0, 0, 2.0]
    else:
        bits = rec["score_2"].view(np.uint16)
        assert torch.from_numpy(bits.copy()).view(torch.bfloat16).tolist() == [0, 4.0, 0, 0, 2.0]
    # reopening keeps what was written (resume); further passes fill other columns
    w2 = MemmapSequenceScoreWriter(tmp_path, 5, 3, dtype=dtype)
    w2([0, 1, 2, 3, 4], torch.ones(5, 1), query_offset=0)
    w2([0, 2, 3], torch.ones(3, 2), query_offset=1)
    w2.flush()
    sc = load_scores(tmp_path)
    assert sc.is_written()
    info = json.loads((tmp_path / "info.json").read_text())
    assert info["num_rows"] == 5 and info["attribute_tokens"] is False
    size = 2 if dtype != torch.float32 else 4
    assert info["dtype"] == ostore.score_struct_dtype(3, size, {torch.float32: "float32", torch.float16: "float16",
                                                                  torch.bfloat16: "bfloat16"}[dtype])
    assert (tmp_path / "scores.bin").stat().st_size == 5 * info["dtype"]["itemsize"]


def test_token_score_writer(tmp_path):
    from bergson_amd.data import load_scores
    from bergson_amd.score_writer import MemmapTokenScoreWriter

    w = MemmapTokenScoreWriter(tmp_path, np.array([2, 0, 3]), 2)
    w([2, 0], torch.arange(10, dtype=torch.float32).reshape(5, 2))
    w.flush()
    sc = load_scores(tmp_path)
    assert sc.offsets.tolist() == [0, 2, 2, 5]
    assert sc[2:5].tolist() == [[0, 1], [2, 3], [4, 5]] and sc[0:2].tolist() == [[6, 7], [8, 9]]
    grid = sc.to_grid()
    assert grid.shape == (3, 4, 2) and grid[2, 1].tolist() == [2, 3] and grid[1].abs().sum() == 0
