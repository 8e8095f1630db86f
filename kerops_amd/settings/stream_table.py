"""Launch shapes of the flat stream ops: (blocks, num_warps, segment) per op and channel count.

    blocks     workgroups of the persistent loop
    num_warps  64-wide wavefronts per workgroup (4, 8 or 16); the reference's knob of the same name
               (e.g. kerops/ops/bnrelu.py:11) counted 32-wide warps of a Triton program
    segment    1 = the 16-byte chunks of a workgroup are interleaved with the other workgroups',
               4 or 8 = every step of a workgroup covers one contiguous run of that many chunks per thread

The reference keys its launch tables by channel count (kerops/ops/conv/dwconv.py:10-17); so does this one.  An op's
entry maps a key to a shape:

    "8", "16", ...   the channel count of the tensor (measured at (1, C, 350, 350, 128))
    "small"          tensors below SMALL_BYTES, whatever their channel count: they do not fill the grids that the
                     large tensors want
    "default"        every other case (channel counts without an entry, tensors that are not 5-D)

The table lives in stream_shapes.json beside this file; `python -m kerops_amd.tune --streams --all --write` measures
every built shape on the GPU at hand and rewrites it.  An op missing from the table, or a value of 0, leaves the
choice to the library's built-in default.  The ops read the table through configurators that receive the op's
tensor, so a change made with `set_stream_shape` (or `tune.apply_streams`) takes effect on the next call.
"""
import inspect
import json
import os

TABLE_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'stream_shapes.json')
KEYS = ('blocks', 'num_warps', 'segment')
SMALL_BYTES = 64 << 20

_table = {}


def _entry(raw):
    return {k: int(raw.get(k, 0)) for k in KEYS}


def load(path=TABLE_PATH):
    """(Re)reads the table file; a missing file means built-in defaults everywhere.  An op entry that holds a
    shape directly (the one-shape-per-op form of earlier files) becomes its "default"."""
    global _table
    _table = {}
    if os.path.exists(path):
        with open(path) as f:
            raw = json.load(f)
        for op, entry in raw.get('shapes', {}).items():
            if any(k in entry for k in KEYS):
                _table[op] = {'default': _entry(entry)}
            else:
                _table[op] = {str(key): _entry(shape) for key, shape in entry.items()}
    return _table


def save(path=TABLE_PATH, note=''):
    with open(path, 'w') as f:
        json.dump({'note': note, 'shapes': _table}, f, indent=1, sort_keys=True)
        f.write('\n')


def table_key(channels=None, nbytes=None):
    """The key a tensor of that channel count and size looks for first."""
    if nbytes is not None and nbytes < SMALL_BYTES:
        return 'small'
    return str(int(channels)) if channels else 'default'


def stream_shape(op, channels=None, nbytes=None):
    """The shape an op would use for a tensor with `channels` channels and `nbytes` bytes (zeros = built-in)."""
    entry = _table.get(op)
    if entry:
        for key in (table_key(channels, nbytes), str(int(channels)) if channels else 'default', 'default'):
            if key in entry:
                return dict(entry[key])
    return dict.fromkeys(KEYS, 0)


def set_stream_shape(op, blocks=0, num_warps=0, segment=0, key='default'):
    _table.setdefault(op, {})[str(key)] = {'blocks': int(blocks), 'num_warps': int(num_warps), 'segment': int(segment)}


def stream_knob(op, key, arg='x'):
    """Configurator for `@configure`: the live table value of `key` for `op`, looked up with the channel count and
    size of the op's positional argument `arg` (a tensor)."""
    assert key in KEYS

    def knob(*args, **kwargs):
        t = args[0] if args else kwargs.get(arg)
        if t is None or not hasattr(t, 'shape'):
            return stream_shape(op)[key]
        channels = t.shape[1] if t.ndim == 5 else None
        return stream_shape(op, channels, t.numel() * t.element_size())[key]

    knob.__name__ = f'{op}_{key}'
    # `configure` hands a configurator the positional arguments named by its own parameters
    knob.__signature__ = inspect.Signature([inspect.Parameter(arg, inspect.Parameter.POSITIONAL_OR_KEYWORD)])
    return knob


load()
