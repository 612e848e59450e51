from .pages import (PagePool, CacheGroup, CacheManager, PagedSpec, FixedSpec, StateSpec,
                    OutOfPages, CacheError)
