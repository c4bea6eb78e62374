"""Registers the fake (meta) implementations of the ``DrissTorch`` operators.

The operator library declares this module as the home of its fake implementations, as the
reference does (src/register_ops.cpp:14, ``impl_abstract_pystub("driss_torch.abstract_impls")``),
and torch checks that the registrations really come from it.  The shape functions themselves
live in ``driss_torch_amd/abstract_impls.py``.
"""
from torch.library import register_fake

from driss_torch_amd.abstract_impls import FAKE_IMPLS

for _op, _fn in FAKE_IMPLS.items():
    register_fake(_op)(_fn)
