"""`import torch_dist_ext` -- the name callers of the reference package use -- resolves to this build.

The reference's package derives its library path from its own directory name (torch_dist_ext/__init__.py:8-12:
`<parent of the package>/libtorch_dist_ext.so`); this directory has that name and the build puts the operator
library at that path.  The implementation lives in `torch_dist_ext_amd`; this module replaces itself with it, so
both names are one module object: the same `CommWorkspace`, `allreduce_rms_fusion_impl`, `CommProcess`,
`setup_env`, `get_workspace`, `allreduce_rms`, and the same module-level `comm` / `world_size_` that `setup_env`
sets (torch_dist_ext/__init__.py:37-46 of the reference).
"""
import sys

import torch_dist_ext_amd

sys.modules[__name__] = torch_dist_ext_amd
