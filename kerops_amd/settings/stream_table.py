"""Launch shapes of the flat stream ops, one entry per op: (blocks, num_warps, segment).

    blocks     workgroups of the persistent loop
    num_warps  64-wide wavefronts per workgroup (4, 8 or 16); the reference's knob of the same name
               (e.g. kerops/ops/bnrelu.py:11) counted 32-wide warps of a Triton program
    segment    1 = the 16-byte chunks of a workgroup are interleaved with the other workgroups',
               4 or 8 = every step of a workgroup covers one contiguous run of that many chunks per thread

The table lives in stream_shapes.json beside this file; `python -m kerops_amd.tune --streams --write` measures
every built shape on the GPU at hand and rewrites it.  An op missing from the table, or a value of 0, leaves the
choice to the library's built-in default.  The ops read the table through zero-argument configurators, so a
change made with `set_stream_shape` (or `tune.apply_streams`) takes effect on the next call.
"""
import json
import os

TABLE_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'stream_shapes.json')
KEYS = ('blocks', 'num_warps', 'segment')

_table = {}


def load(path=TABLE_PATH):
    """(Re)reads the table file; a missing file means built-in defaults everywhere."""
    global _table
    _table = {}
    if os.path.exists(path):
        with open(path) as f:
            raw = json.load(f)
        for op, entry in raw.get('shapes', {}).items():
            _table[op] = {k: int(entry.get(k, 0)) for k in KEYS}
    return _table


def save(path=TABLE_PATH, note=''):
    with open(path, 'w') as f:
        json.dump({'note': note, 'shapes': _table}, f, indent=1, sort_keys=True)
        f.write('\n')


def stream_shape(op):
    return dict(_table.get(op, dict.fromkeys(KEYS, 0)))


def set_stream_shape(op, blocks=0, num_warps=0, segment=0):
    _table[op] = {'blocks': int(blocks), 'num_warps': int(num_warps), 'segment': int(segment)}


def stream_knob(op, key):
    """Zero-argument configurator for `@configure`: the live table value of `key` for `op`."""
    assert key in KEYS

    def knob():
        entry = _table.get(op)
        return entry[key] if entry else 0

    knob.__name__ = f'{op}_{key}'
    return knob


load()
