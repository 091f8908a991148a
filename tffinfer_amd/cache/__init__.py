from .block_pool import BlockPool, OutOfPages
from .manager import CacheGroup, CacheManager
from .state_slots import OutOfSlots, StateSlots
from .sizing import min_window_pages, plan_pages, window_pool_pages
