from .interface import BatchMeta, GroupMeta, Ops, ScoreExtras

__all__ = ["BatchMeta", "GroupMeta", "Ops", "ScoreExtras"]
