"""Warning categories of the DiffLUT API (same names as difflut/utils/warnings.py:26-78,
because user code and tests filter on them)."""
import functools
import warnings


class DiffLUTWarning(UserWarning):
    """Base category for DiffLUT-specific warnings."""


class PerformanceWarning(RuntimeWarning):
    """Something works but is slower than it could be."""


class ConfigurationWarning(UserWarning):
    """A configuration that is valid but probably not intended."""


class DefaultValueWarning(ConfigurationWarning):
    """An optional parameter was left out and its default is used."""


class CUDAWarning(PerformanceWarning):
    """Device-extension availability."""


def warn_default_value(param_name, param_value, stacklevel=2):
    warnings.warn(f"Parameter '{param_name}' was not provided, using default value: {param_value}",
                  category=DefaultValueWarning, stacklevel=stacklevel + 1)


def configure_warnings(action="default", category=None, module_pattern="difflut"):
    if category is None:
        warnings.filterwarnings(action, module=module_pattern)
    else:
        warnings.filterwarnings(action, category=category, module=module_pattern)


def suppress_warnings(func):
    @functools.wraps(func)
    def wrapper(*args, **kwargs):
        with warnings.catch_warnings():
            warnings.filterwarnings("ignore", module="difflut")
            return func(*args, **kwargs)

    return wrapper


def enable_all_warnings():
    configure_warnings("always")


def disable_all_warnings():
    configure_warnings("ignore")


def disable_cuda_warnings():
    configure_warnings("ignore", category=PerformanceWarning)


def enable_strict_mode():
    configure_warnings("error")
