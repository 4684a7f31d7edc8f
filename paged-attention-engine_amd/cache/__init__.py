from .allocator import HOLE, AllocResult, AllocStatus, BlockAllocator, BlockTable
from .manager import (PAGE, CacheGroup, CacheManager, PagedSpec, PagedTensor, StateSlots, StateSpec, attention_pages,
                      bytes_of_one_page_everywhere)
