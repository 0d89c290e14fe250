from .backend import (MAX_KV_SPLITS, AttnBackend, AttnMetadata, BaseAttnMetadata,
                      DecodeMetadata, PrefillMetadata)
from .gdn_backend import GDNBackend

__all__ = ["GDNBackend", "AttnBackend", "AttnMetadata", "BaseAttnMetadata", "DecodeMetadata",
           "PrefillMetadata", "MAX_KV_SPLITS"]
