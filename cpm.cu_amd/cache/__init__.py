from .paged import CacheError, CacheNeeds, CacheView, SequenceCache, StateSpec, StreamSpec
