"""Optional stage dumps in the reference's ``SOAP_PROFILE`` format.

With ``SOAP_PROFILE=1`` (optionally ``SOAP_PROFILE_STEPS=a,b``) every intermediate of a step
is printed as one ``SOAP_PROFILE {json}`` line with the keys ``impl``, ``step``, ``stage``,
``shape``, ``dtype``, ``values`` and the stage names the reference emits
(src/soap_tp/soap.py:26-120 and the stage list of scripts/compare_soap_profiles.py:35-55), so
its profile comparer can read a run of this package unchanged.  Dumps copy tensors to the host
and therefore synchronise; they are off unless requested.
"""
from __future__ import annotations

import json
import os

from torch import Tensor


def enabled(step: int) -> bool:
    if os.environ.get("SOAP_PROFILE", "").lower() not in {"1", "true", "yes"}:
        return False
    requested = os.environ.get("SOAP_PROFILE_STEPS")
    if not requested:
        return True
    wanted = {int(token) for token in (part.strip() for part in requested.split(",")) if token}
    return step in wanted


def dump(stage: str, step: int, tensor: Tensor, logical_shape=None) -> None:
    if not enabled(step):
        return
    data = tensor.detach()
    if logical_shape is not None:
        data = data[: logical_shape[0], : logical_shape[1]]
    record = {
        "impl": "tp",
        "step": step,
        "stage": stage,
        "shape": list(data.shape),
        "dtype": str(data.dtype).removeprefix("torch."),
        "values": data.cpu().reshape(-1).tolist(),
    }
    print("SOAP_PROFILE " + json.dumps(record, separators=(",", ":")), flush=True)
