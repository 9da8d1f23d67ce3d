"""MI355X-native bucketed key-value hash table (HierarchicalKV semantics).

The product is the HIP library libhkv.so behind the C ABI of
include/hkv_c_api.h and the C++ drop-in header include/merlin_hashtable.hpp.
This package is the thin Python host layer used by the tests and the benchmark.
"""
from .table import (EvictStrategy, HashTable, HipException, MerlinException,
                    Predicate, ValueKind, default_options)

__all__ = ["EvictStrategy", "HashTable", "HipException", "MerlinException",
           "Predicate", "ValueKind", "default_options"]
