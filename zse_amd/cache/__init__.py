from .manager import CacheManager, GroupInfo, group_needs
from .pages import OutOfPages, PagePool
from .slots import OutOfSlots, StateSlots
