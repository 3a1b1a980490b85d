"""Writes tests/golden/soap_trajectory.npz.

Runs the ORIGINAL full-matrix SOAP optimizer that the reference vendors as its numerical
ground truth (tests/reference/soap.py of the reference checkout) on the configuration of the
reference's end-to-end test (tests/unit/test_soap.py:33-54,417-438: seed 42, 10 iterations,
refresh every 2, preconditioner beta 0.75, betas (0.8, 0.9), eps 1e-6, lr 1, no weight decay,
N(0, 2) gradients from ``torch.Generator(seed + 1)``) and stores, per shape, the gradients fed
in and the updates (parameter deltas) that came out.  It exists to pin the step SEQUENCING of
the CPU oracle, which no closed form covers.

Run it only where the reference checkout is present (never on the GPU box):
    python tests/golden/make_soap_trajectory.py /root/reference
"""
import runpy
import sys
from pathlib import Path

import numpy as np
import torch

SEED = 42
ITERATIONS = 10
SHAPES = ((8, 8), (20, 20), (12, 12), (12, 20), (20, 12))
CONFIG = dict(preconditioner_beta=0.75, beta1=0.8, beta2=0.9, eps=1e-6, basis_refresh_interval=2)


def main(reference_root: str) -> None:
    optimizer_class = runpy.run_path(str(Path(reference_root) / "tests" / "reference" / "soap.py"))["SOAP"]
    arrays = {}
    for rows, columns in SHAPES:
        parameter_generator = torch.Generator().manual_seed(SEED)
        gradient_generator = torch.Generator().manual_seed(SEED + 1)
        parameter = torch.nn.Parameter(
            torch.normal(mean=0, std=1, size=(rows, columns), generator=parameter_generator, dtype=torch.float32)
        )
        optimizer = optimizer_class(
            [parameter], lr=1.0, betas=(CONFIG["beta1"], CONFIG["beta2"]),
            shampoo_beta=CONFIG["preconditioner_beta"], eps=CONFIG["eps"], weight_decay=0.0,
            precondition_frequency=CONFIG["basis_refresh_interval"], max_precond_dim=max(rows, columns),
            merge_dims=False, precondition_1d=False, normalize_grads=False, correct_bias=True,
        )
        gradients, updates = [], []
        for _ in range(ITERATIONS):
            gradient = torch.normal(mean=0, std=2, size=(rows, columns), generator=gradient_generator,
                                    dtype=torch.float32)
            before = parameter.detach().clone()
            parameter.grad = gradient.clone()
            optimizer.step()
            parameter.grad = None
            gradients.append(gradient.numpy().copy())
            updates.append((before - parameter.detach()).numpy().copy())
        arrays[f"gradients_{rows}x{columns}"] = np.stack(gradients)
        arrays[f"updates_{rows}x{columns}"] = np.stack(updates)
    out = Path(__file__).resolve().parent / "soap_trajectory.npz"
    np.savez_compressed(out, **arrays)
    print(f"wrote {out} ({out.stat().st_size} bytes)")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
