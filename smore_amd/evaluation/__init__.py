"""Evaluation against all entities (the test_all branch of smore/training/train_process.py)."""
from .ranking import filtered_ranks, ranking_metrics  # noqa: F401
