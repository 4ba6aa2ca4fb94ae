"""The optimizer and initializer descriptions of the reference's Python package, with its
constructor arguments: `kraken/pytorch/optim.py` (Adagrad, Adam, RMSprop, SGD) and
`kraken/pytorch/initializer.py` (Constant / Uniform / Normal / XavierUniform / XavierNormal).

Each class answers `type()` and `conf()` exactly as the reference's does: the conf is the
string map that travels to Optim::Create (ps/optim/optim.cc) and Initializer::Create
(ps/initializer/initializer.cc:22-61). `build()` hands that map to the engine's own parsers,
so a description goes wherever `api.Optim` / `api.Initializer` go. Needs neither torch nor a GPU.
"""
from . import api


class Optim:
    """pytorch/optim.py:7-13"""

    def type(self):
        raise NotImplementedError

    def conf(self):
        raise NotImplementedError

    def build(self):
        return api.Optim.create(self.type(), self.conf())


def _flag(b):
    return "true" if b else "false"


class Adagrad(Optim):
    """pytorch/optim.py:16-35"""

    def __init__(self, weight_decay=None, eps=1e-10):
        self._weight_decay, self._eps = weight_decay, eps

    def type(self):
        return api.OptimType.kAdagrad

    def conf(self):
        conf = {}
        if self._weight_decay:
            conf["weight_decay"] = str(self._weight_decay)
        conf["eps"] = str(self._eps)
        return conf


class Adam(Optim):
    """pytorch/optim.py:38-71"""

    def __init__(self, weight_decay=None, beta1=0.9, beta2=0.999, eps=1e-08, amsgrad=False):
        self._weight_decay, self._beta1, self._beta2, self._eps, self._amsgrad = (
            weight_decay, beta1, beta2, eps, amsgrad)

    def type(self):
        return api.OptimType.kAdam

    def conf(self):
        conf = {}
        if self._weight_decay:
            conf["weight_decay"] = str(self._weight_decay)
        conf["beta1"] = str(self._beta1)
        conf["beta2"] = str(self._beta2)
        conf["eps"] = str(self._eps)
        conf["amsgrad"] = _flag(self._amsgrad)
        return conf


class RMSprop(Optim):
    """pytorch/optim.py:74-108"""

    def __init__(self, weight_decay=None, momentum=None, alpha=0.99, eps=1e-8, centered=False):
        self._weight_decay, self._momentum, self._alpha, self._eps, self._centered = (
            weight_decay, momentum, alpha, eps, centered)

    def type(self):
        return api.OptimType.kRMSprop

    def conf(self):
        conf = {}
        if self._weight_decay:
            conf["weight_decay"] = str(self._weight_decay)
        if self._momentum:
            conf["momentum"] = str(self._momentum)
        conf["alpha"] = str(self._alpha)
        conf["eps"] = str(self._eps)
        conf["centered"] = _flag(self._centered)
        return conf


class SGD(Optim):
    """pytorch/optim.py:111-141"""

    def __init__(self, momentum=None, dampening=None, weight_decay=None, nesterov=False):
        self._momentum, self._dampening, self._weight_decay, self._nesterov = (
            momentum, dampening, weight_decay, nesterov)

    def type(self):
        return api.OptimType.kSGD

    def conf(self):
        conf = {}
        if self._momentum:
            conf["momentum"] = str(self._momentum)
        if self._dampening:
            conf["dampening"] = str(self._dampening)
        if self._weight_decay:
            conf["weight_decay"] = str(self._weight_decay)
        conf["nesterov"] = _flag(self._nesterov)
        return conf


class Initializer:
    """pytorch/initializer.py:7-13"""

    def type(self):
        raise NotImplementedError

    def conf(self):
        raise NotImplementedError

    def build(self, seed=None):
        conf = dict(self.conf())
        if seed is not None:
            conf["seed"] = str(seed)
        return api.Initializer.create(self.type(), conf)


class ConstantInitializer(Initializer):
    """pytorch/initializer.py:16-26"""

    def __init__(self, value=0.0):
        self._value = value

    def type(self):
        return api.InitializerType.kConstant

    def conf(self):
        return {"value": str(self._value)}


class UniformInitializer(Initializer):
    """pytorch/initializer.py:29-40"""

    def __init__(self, lower=0.0, upper=1.0):
        self._lower, self._upper = lower, upper

    def type(self):
        return api.InitializerType.kUniform

    def conf(self):
        return {"lower": str(self._lower), "upper": str(self._upper)}


class NormalInitializer(Initializer):
    """pytorch/initializer.py:43-54"""

    def __init__(self, mean=0.0, stddev=1.0):
        self._mean, self._stddev = mean, stddev

    def type(self):
        return api.InitializerType.kNormal

    def conf(self):
        return {"mean": str(self._mean), "stddev": str(self._stddev)}


class XavierUniformInitializer(Initializer):
    """pytorch/initializer.py:57-67"""

    def __init__(self, gain=1.0):
        self._gain = gain

    def type(self):
        return api.InitializerType.kXavierUniform

    def conf(self):
        return {"gain": str(self._gain)}


class XavierNormalInitializer(Initializer):
    """pytorch/initializer.py:70-80"""

    def __init__(self, gain=1.0):
        self._gain = gain

    def type(self):
        return api.InitializerType.kXavierNormal

    def conf(self):
        return {"gain": str(self._gain)}


def as_optim(o):
    """An api.Optim from either kind of description (None stays None)."""
    return o.build() if isinstance(o, Optim) else o


def as_initializer(i):
    return i.build() if isinstance(i, Initializer) else i
