"""Hardware constants the launch configurators read.

`L1_CACHE_BYTES` with `get_l1_cache` / `set_l1_cache` keeps the reference's knob
(kerops/settings/hardware_conf.py:1-11): there it sizes every 1-D stream block; here
the stream kernels are persistent grid-stride loops and the value only bounds the
contract checks that the reference derives from it (e.g. the AvgPoolCeilStats row
limit at kerops/ops/avgpool.py:20).  The MI355X facts below size the grids.
"""
L1_CACHE_BYTES = 65536

# MI355X (gfx950 / CDNA4)
NUM_CUS = 256
NUM_XCDS = 8
WAVEFRONT = 64
LDS_BYTES_PER_CU = 160 * 1024
HBM_PEAK_BYTES_PER_S = 8.0e12


def get_l1_cache():
    return L1_CACHE_BYTES


def set_l1_cache(new_cache):
    global L1_CACHE_BYTES
    L1_CACHE_BYTES = new_cache


def stream_blocks(waves_per_cu=8):
    """Default workgroup count of a persistent 256-thread stream kernel."""
    return NUM_CUS * max(1, waves_per_cu // 4)
