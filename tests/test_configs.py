"""The reference's Python descriptions of optimizers and initializers (kraken/pytorch/optim.py,
initializer.py): the conf maps they produce, spelled out here by hand from those files, and the
structs the engine's conf parsers make of them. Runs without a GPU."""
import pytest

from kraken_amd import api, configs


def test_optim_confs_as_the_reference_writes_them():
    # pytorch/optim.py:26-35: weight_decay only when set, eps always
    assert configs.Adagrad().conf() == {"eps": "1e-10"}
    assert configs.Adagrad(weight_decay=0.01, eps=1e-6).conf() == {"weight_decay": "0.01", "eps": "1e-06"}
    # :56-71
    assert configs.Adam().conf() == {"beta1": "0.9", "beta2": "0.999", "eps": "1e-08", "amsgrad": "false"}
    assert configs.Adam(weight_decay=0.1, amsgrad=True).conf()["amsgrad"] == "true"
    # :93-108
    assert configs.RMSprop().conf() == {"alpha": "0.99", "eps": "1e-08", "centered": "false"}
    assert configs.RMSprop(momentum=0.9, centered=True).conf() == {
        "momentum": "0.9", "alpha": "0.99", "eps": "1e-08", "centered": "true"}
    # :126-141
    assert configs.SGD().conf() == {"nesterov": "false"}
    assert configs.SGD(momentum=0.9, dampening=0.1, weight_decay=0.01, nesterov=True).conf() == {
        "momentum": "0.9", "dampening": "0.1", "weight_decay": "0.01", "nesterov": "true"}
    assert [c().type() for c in (configs.Adagrad, configs.Adam, configs.RMSprop, configs.SGD)] == [0, 1, 2, 3]


def test_initializer_confs_as_the_reference_writes_them():
    assert configs.ConstantInitializer(0.5).conf() == {"value": "0.5"}
    assert configs.UniformInitializer(-1.0, 2.0).conf() == {"lower": "-1.0", "upper": "2.0"}
    assert configs.NormalInitializer().conf() == {"mean": "0.0", "stddev": "1.0"}
    assert configs.XavierUniformInitializer(2.0).conf() == {"gain": "2.0"}
    assert configs.XavierNormalInitializer().conf() == {"gain": "1.0"}
    assert [c().type() for c in (configs.ConstantInitializer, configs.UniformInitializer,
                                 configs.NormalInitializer, configs.XavierUniformInitializer,
                                 configs.XavierNormalInitializer)] == [0, 1, 2, 3, 4]


def test_build_reaches_the_engine_structs():
    o = configs.Adam(weight_decay=0.125, beta1=0.5, beta2=0.75, eps=0.25, amsgrad=True).build().raw
    assert (o.type, o.has_weight_decay, o.weight_decay, o.beta1, o.beta2, o.eps, o.amsgrad) == (
        1, 1, 0.125, 0.5, 0.75, 0.25, 1)
    o = configs.SGD(momentum=0.5, dampening=0.25, nesterov=True).build().raw
    assert (o.type, o.has_momentum, o.momentum, o.has_dampening, o.dampening, o.nesterov, o.has_weight_decay) == (
        3, 1, 0.5, 1, 0.25, 1, 0)
    o = configs.RMSprop(momentum=0.5, alpha=0.75, centered=True).build().raw
    assert (o.type, o.has_momentum, o.momentum, o.alpha, o.centered) == (2, 1, 0.5, 0.75, 1)
    o = configs.Adagrad(eps=0.5).build().raw
    assert (o.type, o.eps, o.has_weight_decay) == (0, 0.5, 0)
    i = configs.UniformInitializer(-0.5, 0.25).build(seed=7).raw
    assert (i.type, i.a, i.b, i.seed) == (1, -0.5, 0.25, 7)
    i = configs.NormalInitializer(0.5, 2.0).build().raw
    assert (i.type, i.a, i.b) == (2, 0.5, 2.0)
    assert configs.XavierNormalInitializer(1.5).build().raw.a == 1.5
    assert configs.as_optim(None) is None and configs.as_initializer(None) is None
    same = api.Optim.create(api.OptimType.kSGD)
    assert configs.as_optim(same) is same
    with pytest.raises(NotImplementedError):
        configs.Optim().type()
