"""`configure` / `confexc` / `ConfiguredFunction` (kerops/settings/wrapper.py:12-107).

Behaviour kept from the reference:
  * `@configure(name=configurator, ...)` wraps a function whose keyword-only
    parameters are annotated `ConfigurableArg`; configurator names must equal those
    parameter names exactly (checked at decoration and in `reconfigure`);
  * on a call, every configurable argument the caller did not pass is produced by
    its configurator: a callable receives the wrapped function's *positional*
    arguments selected by the configurator's own parameter names, any other object
    is used as the value itself; explicitly passed keyword values win;
  * `can_be_configured(**named_args)` dry-runs the callable configurators and
    reports False when one raises `CongiguratorError`;
  * `confexc(*exceptions)` turns the listed exceptions of a configurator into
    `CongiguratorError`.
"""
import functools
import inspect

from .utils import CongiguratorError, configs_match, get_config_args, get_standard_args, validate_signature


class EmptyKwarg:
    """Sentinel for 'the caller did not pass this configurable argument'."""


def _param_names(fn):
    return list(inspect.signature(fn).parameters)


class ConfiguredFunction:
    def __init__(self, origin_function, signature, configurable_args, usual_args, **configurators):
        self.origin_function = origin_function
        self.signature = signature
        self.configurable_args = configurable_args
        self.usual_args = usual_args
        self.configurators = configurators
        # parameter names of each callable configurator, resolved once instead of per call
        self._conf_params = {}
        self._refresh()

    def _refresh(self):
        self._conf_params = {k: _param_names(c) for k, c in self.configurators.items() if callable(c)}
        # positions of those parameters among the wrapped function's positional arguments
        self._conf_index = {k: [self.usual_args.index(p) for p in names if p in self.usual_args]
                            for k, names in self._conf_params.items()}
        self._config_set = frozenset(self.configurable_args)

    def __repr__(self):
        lines = [f'{self.origin_function.__name__}{self.signature}']
        for name, conf in self.configurators.items():
            shown = f"Configurator({', '.join(_param_names(conf))})" if callable(conf) else str(conf)
            lines.append(f'{name}: {shown}')
        return '\n'.join(lines)

    @staticmethod
    def configurator_call(args, configurator, usual_args):
        if not callable(configurator):
            return configurator
        picked = [args[usual_args.index(name)] for name in _param_names(configurator)]
        return configurator(*picked)

    def _resolve(self, name, positional):
        conf = self.configurators[name]
        if not callable(conf):
            return conf
        return conf(*[positional[self.usual_args.index(p)] for p in self._conf_params[name]])

    def __call__(self, *args, **kwargs):
        # common case: every ordinary argument positional, keywords only for configurable ones; the general
        # path below (Signature.bind) costs as much host time as a small kernel takes to run
        if len(args) == len(self.usual_args) and self._config_set.issuperset(kwargs):
            final = {}
            for name in self.configurable_args:
                if name in kwargs:
                    final[name] = kwargs[name]
                else:
                    conf = self.configurators[name]
                    if callable(conf):
                        index = self._conf_index[name]
                        if len(index) != len(self._conf_params[name]):
                            break  # a configurator parameter that is not a positional argument: general path
                        conf = conf(*[args[i] for i in index])
                    final[name] = conf
            else:
                return self.origin_function(*args, **final)
        filled = dict.fromkeys(self.configurable_args, EmptyKwarg)
        filled.update(kwargs)
        bound = self.signature.bind(*args, **filled)
        bound.apply_defaults()
        positional = bound.args
        final = {k: (self._resolve(k, positional) if v is EmptyKwarg else v) for k, v in bound.kwargs.items()}
        return self.origin_function(*positional, **final)

    def can_be_configured(self, **kwargs):
        try:
            for conf in self.configurators.values():
                if callable(conf):
                    conf(**{name: kwargs[name] for name in _param_names(conf)})
        except CongiguratorError:
            return False
        return True

    def reconfigure(self, **new_configurators):
        configs_match(self.configurable_args, new_configurators.keys())
        self.configurators = new_configurators
        self._refresh()


def configure(**configurators):
    def decorate(function):
        signature = inspect.signature(function)
        validate_signature(signature)
        configurable_args = get_config_args(signature)
        usual_args = get_standard_args(signature)
        configs_match(configurable_args, configurators.keys())
        wrapped = ConfiguredFunction(function, signature, configurable_args, usual_args, **configurators)
        return functools.wraps(function)(wrapped)

    return decorate


def confexc(*exceptions):
    def decorate(configurator):
        @functools.wraps(configurator)
        def guarded(*args, **kwargs):
            try:
                return configurator(*args, **kwargs)
            except exceptions as e:
                raise CongiguratorError(str(e))

        return guarded

    return decorate
