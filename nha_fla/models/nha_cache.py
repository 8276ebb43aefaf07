from nha_amd.cache import NHARingCache as NHACache

__all__ = ["NHACache"]
