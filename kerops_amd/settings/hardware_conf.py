"""The reference's one global hardware knob (kerops/settings/hardware_conf.py:1-11).

`L1_CACHE_BYTES` with `get_l1_cache` / `set_l1_cache`: in the reference it sizes every 1-D stream block; here the
stream kernels are persistent loops whose launch shapes come from `stream_table`, and the value only bounds the
contract checks that the reference derives from it (the AvgPoolCeilStats row limit at kerops/ops/avgpool.py:20).
"""
L1_CACHE_BYTES = 65536


def get_l1_cache():
    return L1_CACHE_BYTES


def set_l1_cache(new_cache):
    global L1_CACHE_BYTES
    L1_CACHE_BYTES = new_cache
