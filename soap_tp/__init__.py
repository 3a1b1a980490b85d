"""Import-name alias: ``import soap_tp`` resolves to the MI355X implementation, so code written
against the reference package runs unchanged.  Every module path the reference's tests and
scripts import (``soap_tp.soap``, ``soap_tp.ops``, ``soap_tp.ops.factorizations``,
``.preconditioners``, ``.optimizer``, ``._utils``, ``soap_tp.slate_bindings``,
``soap_tp.elpa_bindings``) is registered as the very module object of ``soap_tp_amd``, so a
function imported through either name is the same object."""
import sys

import soap_tp_amd
from soap_tp_amd import ops, soap, soap_step
from soap_tp_amd.ops import _common, _utils, factorizations, optimizer, preconditioners

from . import elpa_bindings, slate_bindings

for _name, _module in (
    ("soap", soap),
    ("ops", ops),
    ("ops._common", _common),
    ("ops._utils", _utils),
    ("ops.factorizations", factorizations),
    ("ops.optimizer", optimizer),
    ("ops.preconditioners", preconditioners),
):
    sys.modules[f"{__name__}.{_name}"] = _module

__all__ = ["ops", "soap_step", "elpa_bindings", "slate_bindings"]
