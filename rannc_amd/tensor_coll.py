"""Collective helpers under the names ``pyrannc/tensor_coll.py:4-17`` gives them.  Each is one call into the
extension's entry points of ``src/main.cpp:78-136`` (``allreduce_tensor(tensor, sum)``, ``bcast_tensor``,
``all_gather``); with one rank they leave their argument as it is."""
from . import _pyrannc


def _allreduce(t, take_sum: bool):
    _pyrannc.allreduce_tensor(t, take_sum)      # in place; the extension returns nothing


def _allreduce_sum(t):
    """``t`` becomes its sum over all ranks."""
    _allreduce(t, True)


def _allreduce_min(t):
    """``t`` becomes its minimum over all ranks."""
    _allreduce(t, False)


def bcast(t, root):
    """The tensor rank ``root`` holds, on every rank."""
    return _pyrannc.bcast_tensor(t, root)


def all_gather(ten, buf):
    """``buf`` receives every rank's ``ten`` in rank order."""
    _pyrannc.all_gather(ten, buf)
