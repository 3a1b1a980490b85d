"""MI355X-native single-GPU implementation of soap-tp's SOAP step.

``soap_step`` and the ``ops`` entry points keep the reference's names and signatures
(src/soap_tp/__init__.py); the work is done by hand-written gfx950 kernels in
``libsoap_mi355.so`` (built by ``python -m soap_tp_amd.build``).
"""
from . import ops
from .soap import soap_step
from .optim import SOAP
from .state_io import load_state, pack_state, save_state, unpack_state, validate_state

__all__ = ["ops", "soap_step", "SOAP", "save_state", "load_state", "pack_state", "unpack_state", "validate_state"]
