from .manager import (
    CacheGroupSpec,
    CacheManager,
    KVLayerView,
    OutOfPages,
    OutOfSlots,
    PagePool,
    StateSlotSpec,
    StateView,
    group_layers,
)

__all__ = [
    "CacheGroupSpec",
    "CacheManager",
    "KVLayerView",
    "OutOfPages",
    "OutOfSlots",
    "PagePool",
    "StateSlotSpec",
    "StateView",
    "group_layers",
]
