"""Import-name alias: ``import soap_tp`` resolves to the MI355X implementation, so code written
against the reference package (``from soap_tp import soap_step``; ``soap_tp.ops``) runs
unchanged."""
import sys

import soap_tp_amd
from soap_tp_amd import ops, soap_step

sys.modules.setdefault("soap_tp.ops", ops)

__all__ = ["ops", "soap_step"]
