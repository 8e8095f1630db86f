"""Launch-configuration mechanism of the ops (same public names as kerops.settings).

Mirrors kerops/settings/__init__.py:1-3 of the reference: `configure`, `confexc`,
`ConfigurableArg`, `CongiguratorError` (the reference's spelling, kept because it
is exported API) and `get_l1_cache`.  The tables that the ops feed through this
mechanism hold gfx950 tile / workgroup choices instead of RTX-3090 ones.
"""
from .hardware_conf import get_l1_cache
from .utils import ConfigurableArg, CongiguratorError
from .wrapper import confexc, configure

__all__ = ['get_l1_cache', 'ConfigurableArg', 'CongiguratorError', 'confexc', 'configure']
