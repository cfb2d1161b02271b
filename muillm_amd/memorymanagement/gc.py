"""trigger_gc -- muillm/memorymanagement/gc.py:1-14 of the reference: free what a layer
replacement just orphaned (host garbage, then the caching allocator's unused blocks)."""
import gc

import torch


def trigger_gc() -> None:
    if torch.cuda.is_available():
        torch.cuda.synchronize()
    gc.collect()
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
