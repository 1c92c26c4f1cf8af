from .block_manager import ROOT_HASH, BlockManager, GroupSpec, PoolView, SlotsView, hash_block

__all__ = ["ROOT_HASH", "BlockManager", "GroupSpec", "PoolView", "SlotsView", "hash_block"]
