"""``torch.optim.Optimizer`` around ``soap_step``: the caller side of the reference's entry point.

The reference leaves learning rate, weight decay and the parameter update to the integrating
optimizer (README.md:43-60: ``local_parameter.add_(update_shard, alpha=-learning_rate)``).  This
class is that integration for one GPU, with the hyper-parameter names, defaults, first-step
behaviour and decoupled weight decay of the original SOAP optimizer the reference vendors as its
ground truth (tests/reference/soap.py:46-143, :145-345):

* matrices (2-D parameters) go through ``soap_step`` with a per-parameter state dictionary;
* vectors and scalars are not preconditioned (``precondition_1d=False`` in the original): they get
  the same bias-corrected Adam formula through the library's Adam kernel;
* the very first ``step()`` only initialises state and leaves every parameter unchanged
  (tests/reference/soap.py:203-204);
* ``p -= lr * update`` and then ``p -= lr * weight_decay * p`` (:296-304).

Independent parameters are issued round-robin on a small pool of side streams (default priority)
forked from and joined back into the current stream, so the launch-bound steps of small matrices
overlap each other and the tails of large ones.  The step that initialises states (two eigensolves
per matrix, tens of thousands of launches each) issues them from one host thread per side stream.
"""
from __future__ import annotations

import threading
from typing import Any, Dict, Iterable, List, Optional, Tuple

import torch
from torch import Tensor

from .ops import adam_update
from .soap import soap_step
from .state_io import pack_state, unpack_state

__all__ = ["SOAP"]


class SOAP(torch.optim.Optimizer):
    """SOAP for parameters that live on one MI355X.

    Arguments mirror tests/reference/soap.py:46-143 where they exist there.  ``shampoo_beta < 0``
    means "use ``betas[1]``"; ``precondition_frequency`` is ``soap_step``'s
    ``basis_refresh_interval``; ``basis_implementation`` selects the initial eigensolver
    (``"elpa"``: fp64, ``"eigh"``: fp32) as in src/soap_tp/soap.py:136.  Parameters with more
    than two dimensions are rejected unless ``flatten_nd`` is set, in which case they are
    preconditioned as ``(shape[0], prod(shape[1:]))`` matrices.  ``streams`` is the number of side
    streams used for independent parameters (0: everything on the current stream).
    """

    def __init__(
        self,
        params: Iterable,
        lr: float = 3e-3,
        betas: Tuple[float, float] = (0.95, 0.95),
        shampoo_beta: float = -1.0,
        eps: float = 1e-8,
        weight_decay: float = 0.01,
        precondition_frequency: int = 10,
        basis_implementation: str = "elpa",
        block_size: int = 128,
        flatten_nd: bool = False,
        streams: int = 2,
    ):
        if lr < 0.0:
            raise ValueError(f"lr must be non-negative, got {lr}.")
        if not (0.0 <= betas[0] < 1.0 and 0.0 <= betas[1] < 1.0):
            raise ValueError(f"betas must be in [0, 1), got {betas}.")
        if shampoo_beta >= 1.0:
            raise ValueError(f"shampoo_beta must be below 1, got {shampoo_beta}.")
        if eps <= 0.0:
            raise ValueError(f"eps must be positive, got {eps}.")
        if weight_decay < 0.0:
            raise ValueError(f"weight_decay must be non-negative, got {weight_decay}.")
        if precondition_frequency <= 0:
            raise ValueError("precondition_frequency must be positive.")
        if basis_implementation not in {"elpa", "eigh"}:
            raise ValueError(f"basis_implementation must be 'elpa' or 'eigh', got {basis_implementation!r}.")
        if streams < 0 or streams > 8:
            raise ValueError(f"streams must be in 0..8, got {streams}.")
        defaults = dict(lr=lr, betas=tuple(betas), shampoo_beta=shampoo_beta, eps=eps, weight_decay=weight_decay,
                        precondition_frequency=precondition_frequency, basis_implementation=basis_implementation,
                        block_size=block_size, flatten_nd=flatten_nd)
        super().__init__(params, defaults)
        self._stream_count = streams
        self._streams: Dict[torch.device, List[torch.cuda.Stream]] = {}

    # ---- one parameter -----------------------------------------------------------------------

    @staticmethod
    def _matrix_view(tensor: Tensor, flatten_nd: bool) -> Optional[Tensor]:
        if tensor.ndim == 2 and tensor.size(0) > 1 and tensor.size(1) > 1:
            return tensor
        if tensor.ndim > 2:
            if not flatten_nd:
                raise ValueError(
                    f"parameter of shape {tuple(tensor.shape)} has more than two dimensions; pass flatten_nd=True "
                    "to precondition it as a (shape[0], prod(shape[1:])) matrix."
                )
            return tensor.reshape(tensor.size(0), -1)
        return None

    def _step_parameter(self, p: Tensor, group: Dict[str, Any]) -> None:
        grad = p.grad
        if grad.is_sparse:
            raise RuntimeError("SOAP does not support sparse gradients.")
        if not p.is_cuda:
            raise ValueError("SOAP parameters must live on the GPU: this build has no CPU path.")
        state = self.state[p]
        beta1, beta2 = group["betas"]
        lr = group["lr"]
        matrix_grad = self._matrix_view(grad, group["flatten_nd"])
        if matrix_grad is not None:
            soap_state = state.setdefault("soap", {})
            rows, columns = matrix_grad.shape
            update = soap_step(
                matrix_grad, soap_state, global_shape=(rows, columns), shard_dim=1,
                block_size=group["block_size"], process_grid_shape=(1, 1),
                preconditioner_beta=group["shampoo_beta"] if group["shampoo_beta"] >= 0 else beta2,
                beta1=beta1, beta2=beta2, eps=group["eps"],
                basis_refresh_interval=group["precondition_frequency"],
                basis_implementation=group["basis_implementation"],
            )
            first = int(soap_state["step"]) == 0
            update = update.view(p.shape) if update.shape != p.shape else update
        else:
            # not preconditioned: Adam on the parameter viewed as one column
            first = "step" not in state
            if first:
                state["step"] = 0
                state["exp_avg"] = torch.zeros(p.numel(), 1, dtype=torch.float32, device=p.device)
                state["exp_avg_sq"] = torch.zeros(p.numel(), 1, dtype=torch.float32, device=p.device)
                update = None
            else:
                state["step"] += 1
                step = state["step"]
                for name in ("exp_avg", "exp_avg_sq"):  # a checkpoint load may have cast them
                    if state[name].dtype != torch.float32:
                        state[name] = state[name].to(torch.float32)
                column = grad.detach().to(torch.float32).reshape(-1, 1)
                bias_correction2 = 1.0 - beta2 ** step
                update = adam_update(column, state["exp_avg"], state["exp_avg_sq"], step, beta1, beta2,
                                     group["eps"] / bias_correction2 ** 0.5).view(p.shape)
        if first:
            return  # the first gradient only initialises state (tests/reference/soap.py:203-204)
        p.add_(update.to(p.dtype), alpha=-lr)
        if group["weight_decay"] > 0.0:
            p.add_(p, alpha=-lr * group["weight_decay"])

    # ---- all parameters ----------------------------------------------------------------------

    def _side_streams(self, device: torch.device) -> List[torch.cuda.Stream]:
        if device not in self._streams:
            self._streams[device] = [torch.cuda.Stream(device=device) for _ in range(self._stream_count)]
        return self._streams[device]

    def _uninitialised(self, p: Tensor) -> bool:
        """A parameter that soap_step preconditions and whose state has not been initialised yet."""
        preconditioned = p.ndim > 2 or (p.ndim == 2 and p.size(0) > 1 and p.size(1) > 1)
        return preconditioned and not self.state[p].get("soap")

    def _step_on_threads(self, device, streams, items) -> None:
        """The initialising step: an eigensolve is tens of thousands of launches and the host does not run
        that far ahead of the device, so parameters issued one after the other by one thread do not
        overlap on the device however many streams they are spread over.  One host thread per side
        stream takes every len(streams)-th parameter (the library calls release the interpreter lock)."""
        failures = []

        def worker(slot: int) -> None:
            try:
                with torch.cuda.device(device), torch.cuda.stream(streams[slot]), torch.no_grad():
                    for p, group in items[slot::len(streams)]:
                        self._step_parameter(p, group)
            except BaseException as error:  # re-raised by the calling thread
                failures.append(error)

        threads = [threading.Thread(target=worker, args=(slot,), name=f"soap-init-{slot}") for slot in range(len(streams))]
        for thread in threads:
            thread.start()
        for thread in threads:
            thread.join()
        if failures:
            raise failures[0]

    @torch.no_grad()
    def step(self, closure=None):
        loss = None
        if closure is not None:
            with torch.enable_grad():
                loss = closure()
        work = [(p, group) for group in self.param_groups for p in group["params"] if p.grad is not None]
        if self._stream_count == 0 or len(work) < 2:
            for p, group in work:
                self._step_parameter(p, group)
            return loss
        by_device: Dict[torch.device, List[Tuple[Tensor, Dict[str, Any]]]] = {}
        for p, group in work:
            by_device.setdefault(p.device, []).append((p, group))
        for device, items in by_device.items():
            if not device.type == "cuda":
                raise ValueError("SOAP parameters must live on the GPU: this build has no CPU path.")
            main = torch.cuda.current_stream(device)
            streams = self._side_streams(device)
            for stream in streams:
                stream.wait_stream(main)
            # largest first, so the long steps start early and the small ones fill in
            order = sorted(range(len(items)), key=lambda i: -items[i][0].numel())
            if any(self._uninitialised(items[index][0]) for index in order):
                self._step_on_threads(device, streams, [items[index] for index in order])
            else:
                for slot, index in enumerate(order):
                    p, group = items[index]
                    with torch.cuda.stream(streams[slot % len(streams)]):
                        self._step_parameter(p, group)
            for stream in streams:
                main.wait_stream(stream)
        return loss

    # ---- checkpoints -------------------------------------------------------------------------

    def state_dict(self):
        """As ``torch.optim.Optimizer.state_dict``, with each parameter's eight strided SOAP buffers
        packed into plain contiguous tensors plus their layout (see ``soap_tp_amd.state_io``)."""
        base = super().state_dict()
        packed = {}
        for key, value in base["state"].items():
            entry = dict(value)
            if "soap" in entry:
                entry["soap"] = pack_state(entry["soap"])
            packed[key] = entry
        return {"state": packed, "param_groups": base["param_groups"]}

    def load_state_dict(self, state_dict):
        # torch casts floating-point state tensors to the parameter's dtype; the SOAP buffers are
        # fp32 by contract, so they are taken out before and put back after the base class runs.
        held = {}
        stripped = {}
        for key, value in state_dict["state"].items():
            entry = dict(value)
            if "soap" in entry:
                held[key] = entry.pop("soap")
            stripped[key] = entry
        super().load_state_dict({"state": stripped, "param_groups": state_dict["param_groups"]})
        if not held:
            return
        index_to_param = {}
        index = 0
        for group in self.param_groups:
            for p in group["params"]:
                index_to_param[index] = p
                index += 1
        saved_ids = [i for group in state_dict["param_groups"] for i in group["params"]]
        for position, saved_id in enumerate(saved_ids):
            if saved_id in held:
                p = index_to_param[position]
                self.state[p]["soap"] = unpack_state(held[saved_id], device=p.device)
