"""Descriptions of optimizers and initializers in the reference's Python form reach the engine's
structs. A description is anything that answers type() and conf() the way
kraken/pytorch/optim.py and kraken/pytorch/initializer.py do; the conf maps below are the ones
those files produce (optim.py:26-35, 56-71, 93-108, 126-141; initializer.py:16-80), spelled out
by hand. Runs without a GPU."""
import pytest

from kraken_amd import api, configs


class Described:
    def __init__(self, type_, conf):
        self._type, self._conf = type_, conf

    def type(self):
        return self._type

    def conf(self):
        return self._conf


def test_optim_descriptions_reach_the_engine_structs():
    # Adam(weight_decay=0.125, beta1=0.5, beta2=0.75, eps=0.25, amsgrad=True).conf()
    o = configs.as_optim(Described(1, {"weight_decay": "0.125", "beta1": "0.5", "beta2": "0.75", "eps": "0.25",
                                       "amsgrad": "true"})).raw
    assert (o.type, o.has_weight_decay, o.weight_decay, o.beta1, o.beta2, o.eps, o.amsgrad) == (
        1, 1, 0.125, 0.5, 0.75, 0.25, 1)
    # SGD(momentum=0.5, dampening=0.25, nesterov=True).conf(): unset options are left out
    o = configs.as_optim(Described(3, {"momentum": "0.5", "dampening": "0.25", "nesterov": "true"})).raw
    assert (o.type, o.has_momentum, o.momentum, o.has_dampening, o.dampening, o.nesterov, o.has_weight_decay) == (
        3, 1, 0.5, 1, 0.25, 1, 0)
    # RMSprop(momentum=0.5, alpha=0.75, centered=True).conf()
    o = configs.as_optim(Described(2, {"momentum": "0.5", "alpha": "0.75", "eps": "1e-08", "centered": "true"})).raw
    assert (o.type, o.has_momentum, o.momentum, o.alpha, o.centered) == (2, 1, 0.5, 0.75, 1)
    # Adagrad(eps=0.5).conf(); and the defaults of Adagrad().conf() == {"eps": "1e-10"}
    o = configs.as_optim(Described(0, {"eps": "0.5"})).raw
    assert (o.type, o.eps, o.has_weight_decay) == (0, 0.5, 0)
    assert configs.as_optim(Described(0, {"eps": "1e-10"})).raw.eps == pytest.approx(1e-10)


def test_initializer_descriptions_reach_the_engine_structs():
    i = configs.as_initializer(Described(1, {"lower": "-0.5", "upper": "0.25"}), seed=7).raw
    assert (i.type, i.a, i.b, i.seed) == (1, -0.5, 0.25, 7)
    i = configs.as_initializer(Described(2, {"mean": "0.5", "stddev": "2.0"})).raw
    assert (i.type, i.a, i.b) == (2, 0.5, 2.0)
    assert configs.as_initializer(Described(0, {"value": "0.5"})).raw.a == 0.5
    assert configs.as_initializer(Described(4, {"gain": "1.5"})).raw.a == 1.5


def test_engine_objects_pass_through_and_others_are_refused():
    assert configs.as_optim(None) is None and configs.as_initializer(None) is None
    same = api.Optim.create(api.OptimType.kSGD)
    assert configs.as_optim(same) is same
    init = api.Initializer.create(api.InitializerType.kConstant, {"value": "1"})
    assert configs.as_initializer(init) is init
    with pytest.raises(TypeError):
        configs.as_optim("adam")
    with pytest.raises(TypeError):
        configs.as_initializer(3)
