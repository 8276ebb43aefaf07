from nha_amd.cache import NHACache

__all__ = ["NHACache"]
