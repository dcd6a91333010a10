"""Evaluation against all entities (the test_all branch of smore/training/train_process.py)."""
from .ranking import candidate_ranks, filtered_ranks, ranking_metrics  # noqa: F401
