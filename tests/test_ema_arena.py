"""Host-side rules of the EMA output arenas (no GPU needed): an arena counts as
free only when nothing, in Python or in C++, can still reach its tensors."""
import torch

from tspipe_amd import _lib
from tspipe_amd import ema as ema_mod


def _arena():
    return ema_mod._Arena([torch.zeros(8, 4), torch.zeros(16), torch.zeros(2, 2, 3)])


def test_python_references_keep_an_arena_busy():
    arena = _arena()
    assert arena.is_free()
    held = arena.views[1]
    assert not arena.is_free()
    del held
    assert arena.is_free()
    alias = arena.views[0].view(-1)  # a further alias of the storage, no reference to the view object
    assert not arena.is_free()
    del alias
    assert arena.is_free()


def test_a_cpp_holder_alone_keeps_an_arena_busy():
    # what autograd does when it saves a tensor for backward: the TensorImpl
    # gains an owner, the Python refcount and the storage's use count do not change
    host = _lib.host_helper()
    arena = _arena()
    if host is not None:
        host.hold(arena.views[2])
        try:
            assert not arena.is_free()
        finally:
            host.drop()
        assert arena.is_free()
    # the same through autograd itself
    leaf = arena.views[0]
    leaf.requires_grad_()
    loss = (leaf * leaf).sum()  # the multiplication saves `leaf` for its backward
    del leaf
    assert not arena.is_free()
    del loss
    arena.views[0].requires_grad_(False)
    assert arena.is_free()


def test_python_fallback_check_sees_the_cpp_holder(monkeypatch):
    arena = _arena()
    monkeypatch.setattr(_lib, "host_helper", lambda: None)
    assert arena.is_free()
    leaf = arena.views[1]
    leaf.requires_grad_()
    loss = (leaf * leaf).sum()
    del leaf
    assert not arena.is_free()
    del loss
