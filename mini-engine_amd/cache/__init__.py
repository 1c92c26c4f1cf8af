from .block_manager import ROOT_HASH, BlockManager, GroupSpec, PagePool, StateSlots, hash_block

__all__ = ["ROOT_HASH", "BlockManager", "GroupSpec", "PagePool", "StateSlots", "hash_block"]
