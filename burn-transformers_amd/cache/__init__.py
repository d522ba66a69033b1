from .ledger import BLOCK, CacheFull, CacheLedger, FreeList

__all__ = ["BLOCK", "CacheFull", "CacheLedger", "FreeList", "KVSpec", "StateSpec", "Cache"]


def __getattr__(name):
    # the storage needs torch and the kernel bindings; the ledger alone does not
    if name in ("KVSpec", "StateSpec", "Cache", "KVGroup", "StateGroup"):
        from . import storage
        return getattr(storage, name)
    raise AttributeError(name)
