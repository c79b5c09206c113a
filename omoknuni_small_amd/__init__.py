"""MI355X-native tree-search hot path: device-resident forest, batched PUCT selection with
virtual loss, value backup and leaf gather behind a C ABI (include/omk_forest.h)."""
from .forest import Forest, Batch, TranspositionTable, SelectParams, OmkError, library_path, load_library, compact_legal  # noqa: F401

__all__ = ["Forest", "Batch", "TranspositionTable", "SelectParams", "OmkError", "library_path", "load_library", "compact_legal"]
