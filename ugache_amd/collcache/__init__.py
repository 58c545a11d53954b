"""`collcache` package of the reference (python/collcache/__init__.py), backed by libcoll_cache.so."""
