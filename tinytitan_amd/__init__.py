"""MI355X-native KV-cache attention path behind the CTinyTitanHIP C ABI.

``capi`` loads the in-tree shared library; ``engine`` mirrors the reference's
operator interface (KVCacheManager / Attention / PrefillAttention) over it;
``synthetic`` draws the seeded benchmark inputs.  Importing this package does
not touch the GPU and does not load the library.
"""
__all__ = ["capi", "engine", "synthetic", "build"]
