from .pages import (PagePool, CacheGroup, CacheManager, PagedSpec, PagedArray, PAGE, kv_spec, FixedSpec, FixedArray, StateSpec, fixed_part, with_fixed_arrays,
                    OutOfPages, CacheError)
