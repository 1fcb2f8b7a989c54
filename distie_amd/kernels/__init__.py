from .interface import BatchMeta, GroupMeta, Ops

__all__ = ["BatchMeta", "GroupMeta", "Ops"]
