"""Takes the optimizer and initializer descriptions of the reference's Python package as they are.

A `kraken.pytorch.optim.*` or `kraken.pytorch.initializer.*` object answers `type()` (an
OptimType / InitializerType value, common/info.h:46-60) and `conf()` (the string map that travels
to Optim::Create, ps/optim/optim.cc:23-101, and Initializer::Create,
ps/initializer/initializer.cc:22-61). Anything that answers those two calls is handed to the
engine's own conf parsers; an api.Optim / api.Initializer passes through. The reference's classes
themselves stay where they are: this module restates none of them.
"""
from . import api


def _described(x):
    return callable(getattr(x, "type", None)) and callable(getattr(x, "conf", None))


def as_optim(o):
    """An api.Optim from an api.Optim or from a description with type() and conf(); None stays None."""
    if o is None or isinstance(o, api.Optim):
        return o
    if _described(o):
        return api.Optim.create(int(o.type()), dict(o.conf()))
    raise TypeError("an optimizer is an api.Optim or answers type() and conf(), not %r" % (o,))


def as_initializer(i, seed=None):
    """The same for initializers. seed: this engine's extension to the conf map (the reference's
    random initializers cannot be seeded)."""
    if i is None or isinstance(i, api.Initializer):
        return i
    if _described(i):
        conf = dict(i.conf())
        if seed is not None:
            conf["seed"] = str(seed)
        return api.Initializer.create(int(i.type()), conf)
    raise TypeError("an initializer is an api.Initializer or answers type() and conf(), not %r" % (i,))
