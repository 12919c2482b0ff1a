"""Drop-in name for flashserve/PAT's `prefix_attn` package: everything is served by
`pat_amd` (MI355X). `import prefix_attn` code written against the reference keeps
working unchanged, including `prefix_attn._prefix_attn` and the submodules."""
import sys as _sys

import pat_amd as _impl
from pat_amd import *  # noqa: F401,F403
from pat_amd import (_prefix_attn, async_tree, block_scheduler, data_class, prefix_tree,  # noqa: F401
                     utils)

__all__ = list(_impl.__all__)
for _name in ("_prefix_attn", "async_tree", "block_scheduler", "data_class", "prefix_tree", "utils"):
    _sys.modules[f"{__name__}.{_name}"] = getattr(_impl, _name)
