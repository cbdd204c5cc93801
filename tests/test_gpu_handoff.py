"""Parity of the vision -> text hand-off kernels (through the C ABI) against the CPU oracle: index / copy work,
bit-exact; error behaviour as python/ray/text.py:883-910 and :1000-1007."""

import numpy as np
import pytest
import torch

from oracle import handoff_oracle as ho

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
IMG = ho.IMAGE_TOKEN_ID


def _announce(msg):
    print(f"[case] {msg}", flush=True)


def _case(seed, B, T, frac, hidden, dtype):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, 1000, (B, T), generator=g)
    ids[torch.rand(B, T, generator=g) < frac] = IMG
    if int((ids == IMG).sum()) == 0:
        ids[0, T // 2] = IMG
    n = int((ids == IMG).sum())
    mk = lambda *s: torch.randn(*s, generator=g).to(dtype)
    return ids, mk(B, T, hidden), mk(n, hidden), mk(B, T, hidden)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("B,T,frac,hidden", [(1, 4096, 0.6, 3584), (3, 1000, 0.3, 256), (2, 77, 1.0, 40), (1, 5000, 0.001, 64),
                                             (1, 1, 1.0, 8), (2, 1500, 0.5, 6), (1, 333, 0.4, 7)])
def test_merge_and_backward_bit_exact(dtype, B, T, frac, hidden):
    from mi355_vit.handoff import extract_vision_grad, merge_vision_embeddings, prepare_vision_embeddings

    _announce(f"handoff {dtype} B={B} T={T} frac={frac} hidden={hidden}")
    ids, emb, vis, gout = _case(1, B, T, frac, hidden, dtype)
    labels = torch.randint(0, 1000, (B, T))
    labels[ids == IMG] = -100
    e = emb.to(DEV).requires_grad_(True)
    leaf = prepare_vision_embeddings(vis.to(DEV))
    assert leaf.shape == (1, vis.shape[0], hidden) and leaf.is_leaf and leaf.requires_grad
    out = merge_vision_embeddings(e, ids.to(DEV), leaf, labels.to(DEV))
    out.backward(gout.to(DEV))
    as_np = lambda t: t.detach().cpu().float().numpy()
    assert np.array_equal(as_np(out), ho.merge(as_np(emb), ids.numpy(), as_np(vis), labels.numpy()))
    d_e, d_v = ho.merge_backward(as_np(gout), ids.numpy())
    assert np.array_equal(as_np(e.grad), d_e)
    sent = extract_vision_grad(leaf)
    assert sent.shape == (vis.shape[0], hidden) and sent.dtype == dtype and np.array_equal(as_np(sent), d_v)
    # and against the reference's own call on the same device
    ref = emb.to(DEV).masked_scatter((ids.to(DEV) == IMG).unsqueeze(-1).expand(B, T, hidden), vis.to(DEV))
    assert torch.equal(out.detach(), ref)


def test_guards_raise_like_the_reference():
    from mi355_vit.handoff import extract_vision_grad, merge_vision_embeddings

    ids = torch.tensor([[7, IMG, 3, IMG]], device=DEV)
    emb = torch.zeros(1, 4, 8, device=DEV)
    vis = torch.ones(2, 8, device=DEV)
    with pytest.raises(RuntimeError, match=r"\[r2\] No <image> tokens \(ID=151655\) found in input_ids!"):
        merge_vision_embeddings(emb, torch.tensor([[1, 2, 3, 4]], device=DEV), vis, rank=2)
    with pytest.raises(RuntimeError, match=r"Mismatch: 3 vision embeddings but 2 <image> tokens in input_ids!"):
        merge_vision_embeddings(emb, ids, torch.ones(3, 8, device=DEV))
    with pytest.raises(RuntimeError, match=r"Labels should be -100 at <image> positions, but found 1 positions"):
        merge_vision_embeddings(emb, ids, vis, labels=torch.tensor([[5, -100, 6, 9]], device=DEV))
    with pytest.raises(RuntimeError, match="vision_embeddings or its gradient is None"):
        extract_vision_grad(None)
    with pytest.raises(RuntimeError, match="no CPU path"):
        merge_vision_embeddings(emb.cpu(), ids.cpu(), vis.cpu())
    out = merge_vision_embeddings(emb, ids, vis, labels=torch.tensor([[5, -100, 6, -100]], device=DEV))
    assert out[0, :, 0].tolist() == [0.0, 1.0, 0.0, 1.0]


def test_tower_output_feeds_the_handoff():
    """End of the path: the tower's [M, O] output goes into the placeholders and its gradient comes back unchanged
    in shape and order (the vision actor's backward_step accepts the 2-D gradient)."""
    from mi355_vit.config import Qwen2_5_VLVisionConfig
    from mi355_vit.handoff import extract_vision_grad, merge_vision_embeddings, prepare_vision_embeddings
    from mi355_vit.modeling import Qwen2_5_VisionTransformerPretrainedModel

    torch.manual_seed(0)
    kw = dict(depth=2, hidden_size=256, intermediate_size=300, num_heads=8, out_hidden_size=128, window_size=56, fullatt_block_indexes=[1])
    model = Qwen2_5_VisionTransformerPretrainedModel(Qwen2_5_VLVisionConfig(**kw)).to(torch.bfloat16).to(DEV).train()
    grid = torch.tensor([[1, 16, 16], [1, 8, 24]])
    S = int((grid[:, 0] * grid[:, 1] * grid[:, 2]).sum())
    emb = model(torch.randn(S, 1176, device=DEV, dtype=torch.bfloat16), grid.to(DEV))
    M = S // 4
    ids = torch.full((1, M + 20), 11, device=DEV)
    ids[0, 5 : 5 + M] = IMG
    leaf = prepare_vision_embeddings(emb)
    text = torch.randn(1, M + 20, 128, device=DEV, dtype=torch.bfloat16)
    merged = merge_vision_embeddings(text, ids, leaf)
    assert torch.equal(merged[0, 5 : 5 + M], emb.detach()) and torch.equal(merged[0, :5], text[0, :5])
    (merged.float() ** 2).sum().backward()
    g = extract_vision_grad(leaf)
    assert g.shape == emb.shape and torch.equal(g, (2 * emb.detach().float()).to(torch.bfloat16))
    emb.backward(g)
    assert all(p.grad is not None for p in model.parameters())
