from tileccl_amd.memory.bump import BumpAllocator

__all__ = ["BumpAllocator", "SymmetricHeap"]


def __getattr__(name: str):
    if name == "SymmetricHeap":
        from tileccl_amd.memory.symmetric_heap import SymmetricHeap

        return SymmetricHeap
    raise AttributeError(name)
