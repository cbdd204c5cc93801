"""CPU restatement of the vision -> text hand-off (the text actor's side of the exchange).

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  ``text`` below is the reference file
``python/ray/text.py``.

``merge`` restates text:883-913: rows of the text embedding at ``input_ids == image_token_id`` are replaced, in
order, by the vision rows (``masked_scatter`` with the mask expanded over the hidden dimension), after the guards
of text:886-910.  ``merge_backward`` restates what autograd derives for it and text:1000-1019: the text rows'
gradient is the incoming gradient with the placeholder rows zeroed, the vision gradient is the incoming gradient's
placeholder rows in order.  Index / copy work: the product must agree bit for bit.

Pins (tests/test_oracle_handoff.py): ``torch.Tensor.masked_scatter`` and its autograd on the CPU (the library
routine the reference calls), a hand-worked example, and the three error cases.
"""

from __future__ import annotations

from typing import Optional, Tuple

import numpy as np

IMAGE_TOKEN_ID = 151655


def placeholder_positions(input_ids: np.ndarray, image_token_id: int = IMAGE_TOKEN_ID) -> np.ndarray:
    """Flat token indices of the placeholders, ascending (row-major over [B, T])."""
    return np.flatnonzero(np.asarray(input_ids).reshape(-1) == image_token_id)


def merge(inputs_embeds: np.ndarray, input_ids: np.ndarray, vision: np.ndarray, labels: Optional[np.ndarray] = None,
          image_token_id: int = IMAGE_TOKEN_ID) -> np.ndarray:
    hidden = inputs_embeds.shape[-1]
    pos = placeholder_positions(input_ids, image_token_id)
    if pos.size == 0:
        raise RuntimeError("No <image> tokens")
    vision_flat = vision.reshape(-1, vision.shape[-1])
    if vision_flat.shape[0] != pos.size:
        raise RuntimeError(f"Mismatch: {vision_flat.shape[0]} vision embeddings but {pos.size} <image> tokens")
    if labels is not None and np.any(np.asarray(labels).reshape(-1)[pos] != -100):
        raise RuntimeError("Labels should be -100 at <image> positions")
    out = inputs_embeds.reshape(-1, hidden).copy()
    out[pos] = vision_flat
    return out.reshape(inputs_embeds.shape)


def merge_backward(grad: np.ndarray, input_ids: np.ndarray, image_token_id: int = IMAGE_TOKEN_ID) -> Tuple[np.ndarray, np.ndarray]:
    """(gradient of inputs_embeds, gradient of the flat vision rows)."""
    hidden = grad.shape[-1]
    pos = placeholder_positions(input_ids, image_token_id)
    g2 = grad.reshape(-1, hidden)
    d_embeds = g2.copy()
    d_embeds[pos] = 0
    return d_embeds.reshape(grad.shape), g2[pos].copy()
