"""Softmax cross-entropy loss and accuracy (mirror of src/loss.rs)."""
from __future__ import annotations

from .array import Array, DualArray


def softmax_cross_entropy_loss(z: DualArray, y) -> DualArray:
    """z: logits [m, n]; y: labels [m, 1] holding class ids as f32.
    Gradient is the fused (softmax - onehot) * dloss (src/loss.rs:4-23)."""
    z, dz = z.next_colour().into_inner()
    y = z._lift(y)
    t = (z - z.reduce_max(-1, True)).exp()
    p = t / t.reduce_sum(-1, True)
    loss, dloss = y.select_eq(p.coord(-1), -p.log(), 0.0).reduce_sum(-1, True).with_empty_grad()
    dz.accumulate((p - y.one_hot(p.shape[-1])) * dloss)
    return DualArray(loss, dloss)


def softmax_cross_entropy_accuracy(z: DualArray, y) -> Array:
    """1.0 where argmax(z) == y else 0.0 (src/loss.rs:25-34)."""
    z = z.value()
    y = z._lift(y)
    return z.argmax(-1, True).select_eq(y, 1.0, 0.0)
