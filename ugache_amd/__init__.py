"""MI355X-native embedding-extraction path with the interface of SJTU-IPADS/ugache (coll_cache).

  ugache_amd.hip        ctypes binding of the HIP kernel C-ABI (include/ugache_hip.h)
  ugache_amd.collcache  Python package with the reference's `collcache` surface (collcache.common / collcache.torch);
                        put this directory on sys.path to `import collcache.torch as co` unchanged
  ugache_amd.build      builds the two native libraries in-tree
"""
import os

PACKAGE_DIR = os.path.dirname(os.path.abspath(__file__))
__version__ = "0.1.0"
