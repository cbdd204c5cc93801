"""Pins oracle/handoff_oracle.py against torch's masked_scatter (the call of python/ray/text.py:913) and its autograd."""

import numpy as np
import pytest
import torch

from oracle import handoff_oracle as ho

IMG = ho.IMAGE_TOKEN_ID


def _case(seed, B, T, frac, hidden):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, 1000, (B, T), generator=g)
    ids[torch.rand(B, T, generator=g) < frac] = IMG
    n = int((ids == IMG).sum())
    return ids, torch.randn(B, T, hidden, generator=g), torch.randn(n, hidden, generator=g), torch.randn(B, T, hidden, generator=g)


@pytest.mark.parametrize("B,T,frac,hidden", [(1, 50, 0.3, 8), (3, 17, 0.5, 5), (2, 64, 1.0, 4), (1, 9, 0.15, 16)])
def test_merge_matches_masked_scatter_and_its_autograd(B, T, frac, hidden):
    ids, emb, vis, gout = _case(0, B, T, frac, hidden)
    if int((ids == IMG).sum()) == 0:
        ids[0, 0] = IMG
        vis = torch.randn(1, hidden)
    e = emb.clone().requires_grad_(True)
    v = vis.clone().unsqueeze(0).requires_grad_(True)  # [1, M, O] as the reference holds it
    mask = (ids == IMG).unsqueeze(-1).expand_as(e)
    ref = e.masked_scatter(mask, v.reshape(-1, hidden))
    ref.backward(gout)
    got = ho.merge(emb.numpy(), ids.numpy(), v.detach().numpy())
    assert np.array_equal(got, ref.detach().numpy())
    d_e, d_v = ho.merge_backward(gout.numpy(), ids.numpy())
    assert np.array_equal(d_e, e.grad.numpy()) and np.array_equal(d_v, v.grad.reshape(-1, hidden).numpy())


def test_hand_example_and_guards():
    ids = np.array([[7, IMG, 3, IMG]])
    emb = np.arange(8, dtype=np.float32).reshape(1, 4, 2)
    vis = np.array([[100.0, 101.0], [200.0, 201.0]], dtype=np.float32)
    out = ho.merge(emb, ids, vis, labels=np.array([[5, -100, 6, -100]]))
    assert out.tolist() == [[[0, 1], [100, 101], [4, 5], [200, 201]]]
    assert ho.placeholder_positions(ids).tolist() == [1, 3]
    with pytest.raises(RuntimeError, match="No <image> tokens"):
        ho.merge(emb, np.array([[1, 2, 3, 4]]), vis)
    with pytest.raises(RuntimeError, match="Mismatch: 2 vision embeddings but 1"):
        ho.merge(emb, np.array([[1, IMG, 3, 4]]), vis)
    with pytest.raises(RuntimeError, match="Labels should be -100"):
        ho.merge(emb, ids, vis, labels=np.array([[5, -100, 6, 9]]))
