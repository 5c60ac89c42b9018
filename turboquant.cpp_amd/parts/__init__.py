"""Parts of a layer, chosen by kind from registries.  Importing this package registers the built-in ones."""
from .base import (CacheNeed, ParamSpec, Part, StateNeed, build_part, known_parts, register_part,
                   unregister_part)
from . import attention, block, ffn, norm, rope  # noqa: F401
