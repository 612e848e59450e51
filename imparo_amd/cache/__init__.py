from .pages import (PagePool, CacheGroup, CacheManager, PagedSpec, PagedArray, PAGE, kv_spec, FixedSpec, StateSpec,
                    OutOfPages, CacheError)
