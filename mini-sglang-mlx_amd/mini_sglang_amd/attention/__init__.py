from .backend import (MAX_KV_SPLITS, AttnBackend, AttnMetadata, BaseAttnMetadata,
                      DecodeMetadata, PrefillMetadata)

__all__ = ["AttnBackend", "AttnMetadata", "BaseAttnMetadata", "DecodeMetadata",
           "PrefillMetadata", "MAX_KV_SPLITS"]
