"""Signature rules of the configuration mechanism (kerops/settings/utils.py:1-34)."""
import inspect


class ConfigurableArg:
    """Annotation that marks a keyword-only parameter as filled by a configurator."""


class CongiguratorError(Exception):
    """Raised by a configurator that cannot serve the given arguments."""


_KW_ONLY = inspect.Parameter.KEYWORD_ONLY
_POSITIONAL = (inspect.Parameter.POSITIONAL_ONLY, inspect.Parameter.POSITIONAL_OR_KEYWORD)


def validate_signature(signature):
    """Configurable parameters must be keyword-only and nothing else may be."""
    for name, param in signature.parameters.items():
        marked = param.annotation is ConfigurableArg
        kw_only = param.kind is _KW_ONLY
        if marked and not kw_only:
            raise RuntimeError(f'ConfigurableArg must be keyword-only - {name}')
        if kw_only and not marked:
            raise RuntimeError(f'non-ConfigurableArg must not be keyword-only - {name}')


def get_config_args(signature):
    return [n for n, p in signature.parameters.items() if p.annotation is ConfigurableArg]


def get_standard_args(signature):
    return [n for n, p in signature.parameters.items() if p.kind in _POSITIONAL]


def configs_match(configurable_args, configurators_names):
    if set(configurable_args) != set(configurators_names):
        raise RuntimeError(f'Configuration mismatch, {configurable_args=}, {configurators_names=}')
