from .pages import (PagePool, CacheGroup, CacheManager, PagedSpec, PagedArray, PAGE, kv_spec, FixedSpec, FixedArray, StateSpec,
                    OutOfPages, CacheError)
