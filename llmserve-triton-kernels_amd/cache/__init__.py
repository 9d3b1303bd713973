"""Cache manager: pages, block tables, groups of layers, state slots."""

from .allocator import BlockAllocator, OutOfBlocks
from .manager import CacheGroup, CacheManager, StepLayout, group_layers

__all__ = ["BlockAllocator", "OutOfBlocks", "CacheGroup", "CacheManager", "StepLayout", "group_layers"]
