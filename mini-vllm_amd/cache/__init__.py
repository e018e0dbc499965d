from .page_pool import OutOfPages, PagePool, page_hash
from .state_slots import OutOfSlots, StateSlots
from .manager import CacheManager, GroupSpec, SequenceCache, groups_from_needs
