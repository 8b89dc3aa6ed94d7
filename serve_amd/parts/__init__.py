"""Parts of a layer.  Importing the package registers the standard kinds."""
from .base import KVCacheRequest, LayerCache, ParamRequest, Part, Runtime, StateRequest  # noqa: F401
from . import standard  # noqa: F401
