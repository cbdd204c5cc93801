"""Vision -> text hand-off on the GPU: the vision actor's embeddings are written into the ``<image>`` slots of
the text embeddings, and the gradient of those slots is handed back.

Mirrors the text actor's side of the exchange in the reference, python/ray/text.py:
  * ``prepare_vision_embeddings``  text.py:860-872  (batch dimension, detached leaf that collects ``.grad``)
  * ``merge_vision_embeddings``    text.py:883-913  (placeholder mask, the three count / label guards with their
                                                     error messages, ``masked_scatter``)
  * ``extract_vision_grad``        text.py:1000-1019 (gradient of the leaf, batch dimension removed, detached copy)

One ranking kernel and one row-merge kernel replace the expanded boolean mask, three reductions with host
read-backs and ``masked_scatter``; the backward is one row gather and one zero-filling merge.
"""

from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .ops import _stream, gather_rows

IMAGE_TOKEN_ID = 151655  # text.py:884


def _ranks(input_ids: torch.Tensor, labels: Optional[torch.Tensor], image_token_id: int):
    ids = input_ids.reshape(-1)
    if ids.dtype != torch.int64 or not ids.is_contiguous():
        ids = ids.to(torch.int64).contiguous()
    lab = None
    if labels is not None:
        lab = labels.reshape(-1)
        if lab.numel() != ids.numel():
            raise ValueError("labels and input_ids differ in size")
        if lab.dtype != torch.int64 or not lab.is_contiguous():
            lab = lab.to(torch.int64).contiguous()
    n = ids.numel()
    rank = torch.empty(n, dtype=torch.int32, device=ids.device)
    positions = torch.empty(n, dtype=torch.int64, device=ids.device)
    counts = torch.empty(2, dtype=torch.int64, device=ids.device)
    rc = _lib.load().mvit_image_token_ranks(ids.data_ptr(), None if lab is None else lab.data_ptr(), n, image_token_id, -100,
                                            rank.data_ptr(), positions.data_ptr(), counts.data_ptr(), _stream(ids))
    _lib.check(rc, "mvit_image_token_ranks")
    n_image, n_bad_labels = counts.tolist()  # the one host read-back (the reference has three)
    return rank, positions[:n_image], n_image, n_bad_labels


def _merge(embeds2d: torch.Tensor, vision2d: Optional[torch.Tensor], rank: torch.Tensor, n_vision: int) -> torch.Tensor:
    out = torch.empty_like(embeds2d)
    rc = _lib.load().mvit_merge_rows(embeds2d.data_ptr(), None if vision2d is None else vision2d.data_ptr(), rank.data_ptr(),
                                     out.data_ptr(), embeds2d.shape[0], n_vision, embeds2d.shape[1] * embeds2d.element_size(),
                                     _stream(embeds2d))
    _lib.check(rc, "mvit_merge_rows")
    return out


class _MergeRowsFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, embeds2d, vision2d, rank, positions):
        ctx.save_for_backward(rank, positions)
        ctx.n_vision = vision2d.shape[0]
        return _merge(embeds2d, vision2d, rank, vision2d.shape[0])

    @staticmethod
    def backward(ctx, grad):
        rank, positions = ctx.saved_tensors
        grad = grad.contiguous()
        d_embeds = _merge(grad, None, rank, ctx.n_vision) if ctx.needs_input_grad[0] else None
        d_vision = gather_rows(grad, positions, 1) if ctx.needs_input_grad[1] else None
        return d_embeds, d_vision, None, None


def prepare_vision_embeddings(vision_embeddings: torch.Tensor) -> torch.Tensor:
    """[M, O] or [B, M, O] from the vision actor -> a detached leaf [B, M, O] that collects ``.grad`` (text.py:860-872)."""
    if vision_embeddings.dim() == 2:
        vision_embeddings = vision_embeddings.unsqueeze(0)
    vision_embeddings = vision_embeddings.detach().clone().requires_grad_(True)
    vision_embeddings.retain_grad()
    return vision_embeddings


def merge_vision_embeddings(inputs_embeds: torch.Tensor, input_ids: torch.Tensor, vision_embeddings: torch.Tensor,
                            labels: Optional[torch.Tensor] = None, image_token_id: int = IMAGE_TOKEN_ID, rank: int = 0) -> torch.Tensor:
    """``inputs_embeds`` [B, T, O] with the rows at ``input_ids == image_token_id`` replaced, in order, by the rows of
    ``vision_embeddings`` ([*, O]); differentiable in both.  Raises the reference's RuntimeErrors when there is no
    placeholder, when the counts differ, or when a placeholder position carries a label other than -100."""
    if not inputs_embeds.is_cuda:
        raise RuntimeError("merge_vision_embeddings needs tensors on the GPU; there is no CPU path")
    if tuple(inputs_embeds.shape[:-1]) != tuple(input_ids.shape):
        raise ValueError(f"inputs_embeds {tuple(inputs_embeds.shape)} does not match input_ids {tuple(input_ids.shape)}")
    hidden = inputs_embeds.shape[-1]
    vision_flat = vision_embeddings.reshape(-1, vision_embeddings.shape[-1])
    if vision_flat.shape[1] != hidden or vision_flat.dtype != inputs_embeds.dtype or vision_flat.device != inputs_embeds.device:
        raise ValueError("vision embeddings must share hidden size, dtype and device with inputs_embeds")
    ranks, positions, n_image, n_bad = _ranks(input_ids, labels, image_token_id)
    if n_image == 0:
        raise RuntimeError(
            f"[r{rank}] No <image> tokens (ID={image_token_id}) found in input_ids! "
            f"This likely means modality filter is wrong. input_ids shape: {input_ids.shape}")
    if vision_flat.shape[0] != n_image:
        raise RuntimeError(
            f"[r{rank}] Mismatch: {vision_flat.shape[0]} vision embeddings but "
            f"{n_image} <image> tokens in input_ids! "
            f"Vision and text trainers are out of sync.")
    if n_bad:
        raise RuntimeError(
            f"[r{rank}] Labels should be -100 at <image> positions, but found {n_bad} "
            f"positions with other values. This indicates incorrect label preprocessing.")
    merged = _MergeRowsFn.apply(inputs_embeds.reshape(-1, hidden).contiguous(), vision_flat.contiguous(), ranks, positions)
    return merged.view(inputs_embeds.shape)


def extract_vision_grad(vision_embeddings: Optional[torch.Tensor], rank: int = 0) -> torch.Tensor:
    """The gradient to send back to the vision actor (text.py:1000-1019): ``.grad`` of the leaf made by
    ``prepare_vision_embeddings``, without a batch dimension of one, as a detached copy."""
    if vision_embeddings is None or vision_embeddings.grad is None:
        raise RuntimeError(
            f"[r{rank}] vision_embeddings or its gradient is None! "
            f"This should not happen - check that vision_embeddings.requires_grad=True in forward.")
    grad = vision_embeddings.grad
    if grad.dim() == 3 and grad.shape[0] == 1:
        grad = grad.squeeze(0)
    return grad.detach().clone()
