from mini_infer_amd.cache.manager import RELEASED, CacheManager, PageGroup, StepIndex
from mini_infer_amd.cache.page_pool import PagePool
from mini_infer_amd.cache.state_slots import StateSlots

__all__ = ["RELEASED", "CacheManager", "PageGroup", "PagePool", "StateSlots", "StepIndex"]
