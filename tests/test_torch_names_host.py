"""The reference's Python-side names without a GPU: what is exported, how install() puts the
names on a module, and the argument checks that need no engine."""
import types

import pytest


def test_names_and_install():
    from cswap_amd import torch_names as names

    mod = types.SimpleNamespace()
    names.install(mod)
    # the five calls of the reference's model and training files (CIFAR10/cifar10.py:86,106; models/vgg.py:23-45)
    for n in ("cswapinit_", "cswapinit", "cswapsetratio", "cswappre", "cswappost"):
        assert callable(getattr(mod, n)) and getattr(mod, n) is getattr(names, n)
    names.uninstall(mod)
    assert not hasattr(mod, "cswappre")
    # the reference's policy codes (Execution.h:70,86,107)
    assert (names.KEEP, names.RAW, names.ZVC, names.ZFP) == (0, 2, 3, 6)


def test_calls_before_cswapinit__say_so():
    import torch

    from cswap_amd import torch_names as names

    names.cswapclose()
    with pytest.raises(RuntimeError, match="cswapinit_"):
        names.cswapsetratio(128)
    with pytest.raises(RuntimeError, match="cswapinit_"):
        names.cswapinit()
    with pytest.raises(ValueError):
        names.cswappre(torch.zeros(4), 5)
    names.cswappost(torch.zeros(4), None, 0)      # a post without its pre changes nothing
    assert names.stats() == {}
