from .allocator import HOLE, AllocResult, AllocStatus, BlockAllocator, BlockTable
from .manager import CacheGroup, CacheManager, PagedSpec, StateSlots, StateSpec
