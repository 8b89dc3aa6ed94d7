"""Parts of a layer.  Importing the package registers the standard kinds."""
from .base import (CacheTensor, LayerCache, ParamRequest, Part, PositionPart, Rotary, Runtime,  # noqa: F401
                   StateRequest, TokenCacheRequest, kv_cache_request)
from . import standard  # noqa: F401
