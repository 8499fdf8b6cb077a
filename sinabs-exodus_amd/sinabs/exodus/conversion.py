"""Swap sinabs layers for their EXODUS equivalents and back
(API of reference sinabs/exodus/conversion.py).

The mapping needs the plain sinabs layer classes.  With upstream sinabs installed they are
``sinabs.layers.*``, exactly as in the reference.  Without it, pass any module that offers
classes of the same six names with an ``arg_dict`` property through ``sinabs_layers=``.
"""
from typing import Optional

import torch

from . import layers as el
from ._compat import replace_module

_LAYER_NAMES = ("IAF", "IAFSqueeze", "LIF", "LIFSqueeze", "ExpLeak", "ExpLeakSqueeze")


def _sinabs_layers(sinabs_layers=None):
    if sinabs_layers is not None:
        return sinabs_layers
    try:
        import sinabs.layers as sl
    except ImportError as err:
        raise ImportError(
            "Conversion between sinabs and EXODUS layers needs the `sinabs` package "
            "(or a module with the sinabs layer classes passed as `sinabs_layers=`)."
        ) from err
    return sl


def get_module_map(sinabs_layers=None) -> dict:
    """{sinabs class: EXODUS class} for the six layer types (reference conversion.py:6-13)."""
    sl = _sinabs_layers(sinabs_layers)
    return {getattr(sl, name): getattr(el, name) for name in _LAYER_NAMES}


def __getattr__(name):
    # `conversion.module_map` is a module-level dict in the reference; build it on first use so
    # that importing this module does not require upstream sinabs
    if name == "module_map":
        return get_module_map()
    raise AttributeError(name)


def _convert(model: torch.nn.Module, pairs) -> torch.nn.Module:
    for source_class, target_class in pairs:
        model = replace_module(
            model, source_class,
            mapper_fn=lambda module, replacement=target_class: replacement(**module.arg_dict),
        )
    return model


def exodus_to_sinabs(model: torch.nn.Module, sinabs_layers: Optional[object] = None) -> torch.nn.Module:
    """Replace all EXODUS layers with the sinabs equivalent (e.g. to move to a machine without
    GPU). Constructor arguments are carried over; the original model is not modified."""
    return _convert(model, [(ex, sn) for sn, ex in get_module_map(sinabs_layers).items()])


def sinabs_to_exodus(model: torch.nn.Module, sinabs_layers: Optional[object] = None) -> torch.nn.Module:
    """Replace all sinabs layers with EXODUS equivalents. Constructor arguments are carried over;
    the original model is not modified."""
    return _convert(model, list(get_module_map(sinabs_layers).items()))
