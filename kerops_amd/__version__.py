"""Version of the kerops_amd package (the HIP library reports its own through kerops_hip_version())."""
__version__ = '0.1.0'
