from .block_pool import BlockPool, OutOfPages
from .manager import CacheGroup, CacheManager
from .state_slots import OutOfSlots, StateSlots
