"""Comparison helpers that define the reference's pass criteria (kerops/utils.py:6-102).

`allclose_two_stage(input, other, ...)`: a fraction `percentile_strict` of the elements
must satisfy the strict tolerance |input - other| < atol_strict + rtol_strict*|other| and
all remaining ones the narrow tolerance; `other` is the reference side of the relative
term.  `weight_grad_similarity`: cosine similarity close to 1 and norms close.
"""
import torch


def _reporter(debug_info):
    if debug_info is None:
        return lambda msg: None
    if isinstance(debug_info, str):
        if debug_info != 'print':
            raise ValueError(f'Unknown debug_info mode - {debug_info}')
        return print
    return debug_info


def _same_kind(a, b):
    assert a.shape == b.shape
    assert a.dtype == b.dtype
    assert a.device == b.device


@torch.no_grad()
def allclose_two_stage(
    input,
    other,
    rtol_strict=1e-4,
    atol_strict=1e-4,
    percentile_strict=0.99,
    rtol_narrow=1e-3,
    atol_narrow=1e-3,
    debug_info=None,
    precision=None,
):
    say = _reporter(debug_info)
    _same_kind(input, other)
    precision = input.dtype if precision is None else precision

    a = input.reshape(-1).to(precision)
    b = other.reshape(-1).to(precision)
    err = (a - b).abs()
    ref = b.abs()

    strict_ok = err < atol_strict + rtol_strict * ref
    size = a.numel()
    num_true = int(strict_ok.sum().item())
    ratio = num_true / size
    say(f'strict stage - {size=}, {num_true=}, {ratio=} (percentile_strict={percentile_strict})')

    if num_true == size:
        say('every element passed the strict tolerance')
        return True
    if not ratio > percentile_strict:
        say('strict threshold has not been passed')
        return False

    rest = ~strict_ok
    narrow_ok = err[rest] < atol_narrow + rtol_narrow * ref[rest]
    passed = bool(narrow_ok.all().item())
    say('narrow threshold has been passed' if passed else 'narrow threshold has not been passed')
    return passed


def weight_grad_similarity(input, other, rtol_cos=1e-4, atol_cos=1e-4, rtol_len=1e-3, atol_len=1e-3, debug_info=None):
    say = _reporter(debug_info)
    _same_kind(input, other)

    a = input.reshape(-1)
    b = other.reshape(-1)
    cos = torch.nn.functional.cosine_similarity(a, b, dim=0)
    if not torch.allclose(torch.ones_like(cos), cos, rtol=rtol_cos, atol=atol_cos):
        say(f'direction test failed - {cos}')
        return False
    na, nb = torch.norm(a), torch.norm(b)
    if not torch.allclose(na, nb, rtol=rtol_len, atol=atol_len):
        say(f'magnitude test failed - {na=}, {nb=}')
        return False
    say('all stages passed')
    return True
