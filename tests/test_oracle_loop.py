"""Pins the oracle's loop (`oracle.loop.collect`, `losses_and_backward`) and `oracle.store.preprocess` on the CPU.

What fixes them, independent of the oracle's own code:
  * a document alone: the row of module m equals L @ W_m.grad @ R^T, where W_m.grad is what autograd leaves in
    the parameter after a plain `model(x)` and a next-token cross entropy written out here from log-softmax
    (sum or mean over the supervised positions, with and without label smoothing) -- the identity the
    reference's tests/test_gradients.py:196-206 and tests/test_attribute_tokens.py:924-1070 rest on;
  * the same document inside a padded batch gives the same row (tests/test_batch_size_invariance.py);
  * prompt-masked labels: the row is the gradient of the completion-only loss, prompt positions included, and
    the per-token rows sum to it;
  * the advantage column scales loss and row;
  * unit normalisation written out in float64: g / max(||g||, eps_fp32), a zero row stays zero.
"""
import numpy as np
import pytest
import torch

from bergson_amd.synthetic import make_gpt_neox, random_docs
from oracle import loop as oloop
from oracle import store as ostore
from oracle.projection import module_projections

VOCAB = 384
P = 4


@pytest.fixture(scope="module")
def model():
    m = make_gpt_neox("pythia-14m", torch.float32, "cpu", seed=3, layers=2, vocab=VOCAB, max_positions=64)
    return m


def _hand_loss(model, ids, labels, reduction, smoothing):
    """Next-token loss of ONE document written from log-softmax: position t predicts labels[t+1]."""
    x = torch.tensor([ids])
    logp = torch.log_softmax(model(x).logits[0].double(), dim=-1)  # [S, V]
    total = torch.zeros((), dtype=torch.float64)
    count = 0
    for t in range(len(ids) - 1):
        tgt = labels[t + 1]
        if tgt == -100:
            continue
        nll = -logp[t, tgt]
        uniform = -logp[t].mean()
        total = total + (1.0 - smoothing) * nll + smoothing * uniform
        count += 1
    return total / count if reduction == "mean" else total


def _autograd_rows(model, ids, labels, reduction, smoothing, scale=1.0):
    """Per module: L @ W.grad @ R^T from a plain backward pass with every parameter trainable."""
    model.requires_grad_(True)
    model.zero_grad()
    loss = _hand_loss(model, ids, labels, reduction, smoothing) * scale
    loss.backward()
    rows = []
    for name, mod in oloop.target_linears(model.base_model).items():
        left, right = module_projections(name, P, mod.out_features, mod.in_features, torch.float32)
        rows.append((left.double() @ mod.weight.grad.double() @ right.double().T).flatten())
    model.zero_grad()
    model.requires_grad_(False)
    model.get_input_embeddings().requires_grad_(True)
    return torch.cat(rows), float(loss.detach())


@pytest.mark.parametrize("reduction", ["sum", "mean"])
@pytest.mark.parametrize("smoothing", [0.0, 0.1])
def test_single_document_row_is_the_projected_autograd_gradient(model, reduction, smoothing):
    ids = random_docs([13], vocab=VOCAB, seed=5)[0]
    want, loss = _autograd_rows(model, ids, ids, reduction, smoothing)
    rows, losses = oloop.collect(model, model.base_model, [ids], [[0]], p=P, loss_reduction=reduction,
                                 label_smoothing=smoothing)
    assert rows.shape == (1, 8 * P * P)
    assert abs(float(losses[0]) - loss) <= 1e-4 * abs(loss)
    err = ((rows[0].double() - want).norm() / want.norm()).item()
    assert err <= 1e-4, err
    # a dropped shift (position t scored against its own token) or a wrong denominator would not pass:
    if reduction == "mean":
        total, _ = _autograd_rows(model, ids, ids, "sum", smoothing)
        assert ((rows[0].double() * (len(ids) - 1) - total).norm() / total.norm()).item() <= 1e-4


@pytest.mark.parametrize("reduction", ["sum", "mean"])
def test_row_does_not_depend_on_the_batch_it_is_padded_into(model, reduction):
    lengths = [13, 7, 20, 2, 9]
    docs = random_docs(lengths, vocab=VOCAB, seed=6)
    alone, l_alone = oloop.collect(model, model.base_model, docs, [[i] for i in range(len(docs))], p=P,
                                   loss_reduction=reduction, label_smoothing=0.1)
    batched, l_batched = oloop.collect(model, model.base_model, docs, [[2, 0, 3], [4, 1]], p=P,
                                       loss_reduction=reduction, label_smoothing=0.1)
    assert ((alone - batched).norm() / alone.norm()).item() <= 1e-4
    assert torch.allclose(l_alone, l_batched, rtol=1e-4)
    for i in (0, 3):  # and each row is the autograd one, so the agreement is not two equal mistakes
        want, _ = _autograd_rows(model, docs[i], docs[i], reduction, 0.1)
        assert ((batched[i].double() - want).norm() / want.norm()).item() <= 1e-4


def test_prompt_masked_labels(model):
    ids = random_docs([12], vocab=VOCAB, seed=7)[0]
    labels = [-100] * 7 + ids[7:]
    for reduction in ("sum", "mean"):
        want, loss = _autograd_rows(model, ids, labels, reduction, 0.0)
        rows, losses = oloop.collect(model, model.base_model, [ids], [[0]], p=P, labels=[labels],
                                     loss_reduction=reduction)
        assert abs(float(losses[0]) - loss) <= 1e-4 * abs(loss)
        assert ((rows[0].double() - want).norm() / want.norm()).item() <= 1e-4
    # masking changes the gradient (the unmasked one is another vector) ...
    unmasked, _ = _autograd_rows(model, ids, ids, "sum", 0.0)
    want, _ = _autograd_rows(model, ids, labels, "sum", 0.0)
    assert ((unmasked - want).norm() / want.norm()).item() > 0.1
    # ... and the per-token rows cover all len - 1 positions and sum to the per-document row
    tok, _ = oloop.collect(model, model.base_model, [ids], [[0]], p=P, labels=[labels], attribute_tokens=True)
    assert tok.shape[0] == len(ids) - 1
    assert ((tok.double().sum(0) - want).norm() / want.norm()).item() <= 1e-4


def test_advantage_scales_loss_and_row(model):
    docs = random_docs([9, 6], vocab=VOCAB, seed=8)
    adv = [0.5, -2.0]
    rows, losses = oloop.collect(model, model.base_model, docs, [[0, 1]], p=P, advantages=adv)
    for i in range(2):
        want, loss = _autograd_rows(model, docs[i], docs[i], "sum", 0.0, scale=adv[i])
        assert abs(float(losses[i]) - loss) <= 1e-4 * abs(loss)
        assert ((rows[i].double() - want).norm() / want.norm()).item() <= 1e-4


def test_losses_and_backward_clears_gradients(model):
    x, y, _ = oloop.pad_and_tensor(random_docs([5, 8], vocab=VOCAB, seed=9))
    losses = oloop.losses_and_backward(model, x, y, "mean", 0.0)
    assert losses.shape == (2,) and all(q.grad is None for q in model.parameters())


def test_pad_and_tensor_masks():
    x, y, mask = oloop.pad_and_tensor([[5, 6, 7], [8]], [[-100, 6, 7], [8]])
    assert x.tolist() == [[5, 6, 7], [8, 0, 0]]
    assert y.tolist() == [[-100, 6, 7], [8, -100, -100]]
    assert mask.tolist() == [[True, True, False], [False, False, False]]


def test_preprocess_concatenates_in_grad_sizes_order_and_unit_normalises():
    gen = torch.Generator().manual_seed(0)
    a = torch.randn(4, 6, generator=gen)
    b = torch.randn(4, 3, generator=gen)
    a[2] = 0
    b[2] = 0
    a[3] *= 1e-9  # norm below eps_fp32: divided by eps, not by its norm
    b[3] *= 1e-9
    sizes = {"b": 3, "a": 6}  # deliberately not the dict order of mod_grads
    got = ostore.preprocess({"a": a, "b": b}, sizes, unit_normalize=False)
    assert torch.equal(got, torch.cat([b, a], dim=1))
    got = ostore.preprocess({"a": a, "b": b}, sizes, unit_normalize=True)
    cat = np.concatenate([b.numpy(), a.numpy()], axis=1).astype(np.float64)
    eps = float(np.finfo(np.float32).eps)
    want = cat / np.maximum(np.sqrt((cat ** 2).sum(1, keepdims=True)), eps)
    assert np.allclose(got.double().numpy(), want, rtol=1e-5, atol=0)
    assert np.allclose(np.linalg.norm(got[:2].double().numpy(), axis=1), 1.0, rtol=1e-5)
    assert not got[2].any()
    assert np.linalg.norm(got[3].double().numpy()) < 0.1  # the clamp, not a unit vector
