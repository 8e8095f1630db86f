"""CPU tests of the configuration mechanism (same rules as kerops/settings of the reference)."""
import pytest

from kerops_amd.settings import ConfigurableArg, CongiguratorError, confexc, configure, get_l1_cache
from kerops_amd.settings import hardware_conf
from kerops_amd.settings.wrapper import ConfiguredFunction


@confexc(KeyError)
def table(channels):
    return {8: 1, 16: 2}[channels]


class FakeTensor:
    def __init__(self, c):
        self.shape = (1, c, 4, 4, 4)


@configure(a=lambda x: table(x.shape[1]), b=7)
def op(x, y=3, *, a: ConfigurableArg, b: ConfigurableArg):
    return x.shape[1], y, a, b


def test_configurators_fill_missing_kwargs():
    assert isinstance(op, ConfiguredFunction)
    assert op(FakeTensor(8)) == (8, 3, 1, 7)
    assert op(FakeTensor(16), 5) == (16, 5, 2, 7)
    assert op.__name__ == 'op'


def test_explicit_kwargs_win():
    assert op(FakeTensor(8), a=99) == (8, 3, 99, 7)
    assert op(FakeTensor(8), b=0, a=None) == (8, 3, None, 0)
    # an explicit value means the configurator is not even consulted
    assert op(FakeTensor(5), a=1) == (5, 3, 1, 7)


def test_unsupported_key_raises_configurator_error():
    with pytest.raises(CongiguratorError):
        op(FakeTensor(5))
    assert op.can_be_configured(x=FakeTensor(8)) is True
    assert op.can_be_configured(x=FakeTensor(5)) is False


def test_configurator_receives_arguments_by_name():
    @configure(k=lambda second, first: (first, second))
    def f(first, second, *, k: ConfigurableArg):
        return k

    assert f(1, 2) == (1, 2)
    assert f(second=2, first=1) == (1, 2)


def test_signature_rules():
    with pytest.raises(RuntimeError, match='ConfigurableArg must be keyword-only'):
        @configure(a=1)
        def bad1(x, a: ConfigurableArg):
            return a

    with pytest.raises(RuntimeError, match='non-ConfigurableArg must not be keyword-only'):
        @configure(a=1)
        def bad2(x, *, a: ConfigurableArg, stray=2):
            return a

    with pytest.raises(RuntimeError, match='Configuration mismatch'):
        @configure(a=1, zzz=2)
        def bad3(x, *, a: ConfigurableArg):
            return a

    with pytest.raises(RuntimeError, match='Configuration mismatch'):
        @configure()
        def bad4(x, *, a: ConfigurableArg):
            return a


def test_reconfigure_and_repr():
    @configure(a=1, b=lambda x: x + 1)
    def f(x, *, a: ConfigurableArg, b: ConfigurableArg):
        return a, b

    assert f(1) == (1, 2)
    f.reconfigure(a=10, b=20)
    assert f(1) == (10, 20)
    with pytest.raises(RuntimeError, match='Configuration mismatch'):
        f.reconfigure(a=1)
    f.reconfigure(a=1, b=lambda x: x * 2)
    text = repr(f)
    assert text.splitlines()[0].startswith('f(x, *, a')
    assert 'a: 1' in text and 'b: Configurator(x)' in text


def test_l1_cache_knob():
    assert get_l1_cache() == 65536
    hardware_conf.set_l1_cache(1024)
    try:
        assert get_l1_cache() == 1024
    finally:
        hardware_conf.set_l1_cache(65536)


def test_confexc_passes_other_exceptions():
    @confexc(KeyError)
    def c(v):
        raise ValueError('x')

    with pytest.raises(ValueError):
        c(1)


def test_tuner_apply_installs_and_falls_back():
    """kerops_amd.tune.apply reconfigures the conv ops through the settings mechanism; channel counts that were
    not measured keep the built-in tables (no GPU needed: only the configurators are evaluated)."""
    import torch

    from kerops_amd import tune
    from kerops_amd.ops.conv import DWConv, DWConvWGRAD
    from kerops_amd.ops.conv.variants import FWD_VARIANTS, WGRAD_VARIANTS, threads_per_workgroup

    saved = dict(DWConv.configurators), dict(DWConvWGRAD.configurators)
    try:
        tune.apply({'DWConv': {64: (4, 8, 16, 88, 0.9)}, 'DWConvWGRAD': {64: (4, 16, 2, 0, 0.9)}})
        x64, x32 = torch.empty(1, 64, 2, 2, 2), torch.empty(1, 32, 2, 2, 2)
        got = {k: (c(x64) if callable(c) else c) for k, c in DWConv.configurators.items()}
        assert (got['W_block'], got['D_block'], got['lane_channels'], got['H_chunk'], got['num_warps']) == (4, 8, 16, 88, 4)
        got = {k: (c(x32) if callable(c) else c) for k, c in DWConv.configurators.items()}
        assert (got['W_block'], got['D_block'], got['lane_channels'], got['H_chunk']) == (8, 16, 16, 0)
        got = {k: (c(x64) if callable(c) else c) for k, c in DWConvWGRAD.configurators.items()}
        assert (got['W_block'], got['D_block'], got['lane_channels'], got['num_warps']) == (4, 16, 2, 4)
    finally:
        DWConv.reconfigure(**saved[0])
        DWConvWGRAD.reconfigure(**saved[1])
    # the built-in defaults are entries of the variant tables, with the workgroup size the library uses
    for c in (8, 16, 32, 64, 128):
        x = torch.empty(1, c, 2, 2, 2)
        for op, table in ((DWConv, FWD_VARIANTS), (DWConvWGRAD, WGRAD_VARIANTS)):
            conf = {k: (f(x) if callable(f) else f) for k, f in op.configurators.items()}
            shape = (conf['W_block'], conf['D_block'], conf['lane_channels'])
            assert shape in table[c], (op, c, shape)
            assert conf['num_warps'] * 64 == threads_per_workgroup(c, *shape)


def test_stream_table_feeds_the_stream_ops_live():
    """The launch shapes of the stream ops come from settings/stream_shapes.json, keyed by op and channel count like
    the reference's tables (kerops/ops/conv/dwconv.py:10-17), through configurators that receive the op's tensor:
    the ops see a changed table on their next call; a channel count without an entry gets the op's default, small
    tensors their own class, an op missing from the table zeros (the library's built-in choice)."""
    from kerops_amd.ops.addition import AddStatsBackward
    from kerops_amd.ops.bnrelu import ApplyBNReLU
    from kerops_amd.settings import stream_table

    table = stream_table.load()
    assert 'default' in table['ApplyBNReLU']
    for op, entry in table.items():
        for key, shape in entry.items():
            assert key in ('default', 'small') or int(key) in (2, 4, 8, 16, 32, 64, 128, 256), (op, key)
            assert set(shape) == {'blocks', 'num_warps', 'segment'}
            assert shape['num_warps'] in (0, 4, 8, 16) and shape['segment'] in (0, 1, 2, 4, 8)
            assert 0 <= shape['blocks'] <= 65536
    import torch
    big = torch.empty((1, 64, 350, 350, 128), dtype=torch.float16, device='meta')
    other = torch.empty((1, 256, 350, 350, 16), dtype=torch.float16, device='meta')
    small = torch.empty((1, 64, 16, 16, 16), dtype=torch.float16, device='meta')
    knob = ApplyBNReLU.configurators['num_warps']
    assert callable(knob) and knob(big) == stream_table.stream_shape('ApplyBNReLU', 64, big.numel() * 2)['num_warps']
    assert AddStatsBackward.configurators['blocks'](add_grad=big) == \
        stream_table.stream_shape('AddStatsBackward', 64, big.numel() * 2)['blocks']
    saved = {op: {k: dict(v) for k, v in e.items()} for op, e in table.items()}
    try:
        stream_table.set_stream_shape('ApplyBNReLU', blocks=7, num_warps=4, segment=1, key=64)
        stream_table.set_stream_shape('ApplyBNReLU', blocks=9, num_warps=8, segment=4, key='default')
        stream_table.set_stream_shape('ApplyBNReLU', blocks=3, num_warps=4, segment=1, key='small')
        conf = ApplyBNReLU.configurators
        assert (conf['blocks'](big), conf['num_warps'](big), conf['segment'](big)) == (7, 4, 1)
        assert (conf['blocks'](other), conf['num_warps'](other), conf['segment'](other)) == (9, 8, 4)
        assert (conf['blocks'](small), conf['num_warps'](small), conf['segment'](small)) == (3, 4, 1)
        assert ApplyBNReLU.can_be_configured(x=big)
    finally:
        stream_table._table.clear()
        stream_table._table.update(saved)
    assert stream_table.stream_shape('NoSuchOp') == {'blocks': 0, 'num_warps': 0, 'segment': 0}
    assert stream_table.stream_knob('NoSuchOp', 'blocks')(big) == 0


def test_stream_table_round_trips_through_its_file(tmp_path):
    from kerops_amd.settings import stream_table

    before = {op: {k: dict(v) for k, v in e.items()} for op, e in stream_table.load().items()}
    path = str(tmp_path / 'shapes.json')
    try:
        stream_table.set_stream_shape('Stats', blocks=123, num_warps=16, segment=8, key=32)
        stream_table.save(path, note='test')
        assert stream_table.load(path)['Stats']['32'] == {'blocks': 123, 'num_warps': 16, 'segment': 8}
        # the one-shape-per-op form is read as the op's default
        with open(path, 'w') as f:
            f.write('{"shapes": {"Stats": {"blocks": 5, "num_warps": 4, "segment": 1}}}')
        assert stream_table.load(path) == {'Stats': {'default': {'blocks': 5, 'num_warps': 4, 'segment': 1}}}
    finally:
        assert stream_table.load() == before
