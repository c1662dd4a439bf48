"""CPU restatement of the reference's algorithm for the collection and scoring path.

TEST INFRASTRUCTURE ONLY.  Nothing under ``bergson_amd/`` imports this package;
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` do, and only as the checker / the timed CPU baseline.

The reference (EleutherAI/bergson v0.26.1) is pure Python on PyTorch, so the
restatement is the same op sequence on PyTorch CPU tensors, written from the
reference's source (each function cites the file:line it follows) and pinned,
in ``tests/test_oracle_*.py``, by autograd identities, closed forms, fp64
brute force and the literal values the reference's own tests hold.  Every
function below has at least one such check; none is "parity unpinned".
"""
