"""kerops_amd: MI355X (gfx950) implementation of the channels-last 3D depthwise-conv
path of neuro-ml/kerops.  `kerops_amd.ops` and `kerops_amd.settings` mirror the module
layout and function names of `kerops.ops` / `kerops.settings`; every op launches a
hand-written HIP kernel through the C ABI in include/kerops_hip.h."""
from .__version__ import __version__  # noqa: F401
