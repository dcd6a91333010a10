"""Pieces of the training step that sit next to the scoring path (smore/training/train_process.py)."""
from .sample_loss import sample_loss  # noqa: F401
