"""Stage-by-stage diff of two ``SOAP_PROFILE`` logs.

    python -m soap_tp_amd.compare_profiles REFERENCE.log CANDIDATE.log [--tolerance 1e-4] [--steps 1,2]

Both logs hold lines ``SOAP_PROFILE {"impl":..,"step":..,"stage":..,"shape":[..],"values":[..]}``
as written by the reference (src/soap_tp/soap.py:26-120, tests/reference/soap.py:27-44) and by
``soap_tp_amd._profile``; any other text is skipped.  The tool answers the question the
reference's scripts/compare_soap_profiles.py answers — at which stage of which step do two
implementations part — with the same treatment of the one legitimate ambiguity: eigenvector
columns are defined up to sign, so the candidate's basis columns are aligned to the reference's
and the same signs are applied to everything expressed in eigenbasis coordinates (projected
gradient, momentum, coordinate update) before the relative L2 error is taken.  Variance is a
square and parameter-space tensors do not depend on the signs, so they are compared as they are.

Exit status 0 if every common stage is within the tolerance, 1 otherwise, 2 for unusable input.
"""
from __future__ import annotations

import argparse
import json
import sys
from typing import Dict, Iterable, List, Optional, Tuple

import torch

MARKER = "SOAP_PROFILE "

STAGES = (
    "gradient", "left_preconditioner", "right_preconditioner", "left_basis", "right_basis",
    "momentum_before_adam", "variance_before_adam", "gradient_2d", "projected_gradient",
    "momentum_after_adam", "variance_after_adam", "denominator", "coordinate_update", "backrotated_update",
    "returned_update", "left_preconditioner_after_step", "right_preconditioner_after_step",
    "left_basis_after_step", "right_basis_after_step", "momentum_after_step", "variance_after_step",
    "parameter_after_step",
)
RANK = {name: i for i, name in enumerate(STAGES)}

# stages in the coordinates of the bases the step started with / ended with
IN_CURRENT_BASES = {"momentum_before_adam", "projected_gradient", "momentum_after_adam", "coordinate_update"}
IN_NEXT_BASES = {"momentum_after_step"}
BASIS_STAGES = {"left_basis", "right_basis", "left_basis_after_step", "right_basis_after_step"}

Key = Tuple[int, str]


def read_log(lines: Iterable[str], origin: str) -> Dict[Key, torch.Tensor]:
    """``{(step, stage): float64 tensor}``; a stage dumped twice in a step keeps the last dump."""
    found: Dict[Key, torch.Tensor] = {}
    for number, line in enumerate(lines, 1):
        at = line.find(MARKER)
        if at < 0:
            continue
        try:
            record = json.loads(line[at + len(MARKER):])
            body = record.get("tensor", record)
            shape = [int(extent) for extent in body["shape"]]
            tensor = torch.tensor(body["values"], dtype=torch.float64).reshape(shape)
            found[(int(record["step"]), str(record["stage"]))] = tensor
        except (ValueError, KeyError, TypeError, RuntimeError) as error:
            raise ValueError(f"{origin}:{number}: unusable SOAP_PROFILE line ({error})") from error
    return found


def column_signs(reference: torch.Tensor, candidate: torch.Tensor) -> Tuple[torch.Tensor, float]:
    """+-1 per column such that ``candidate * signs`` points along ``reference``; also the smallest
    |cosine| met (a value far below 1 means the columns differ by more than a sign)."""
    dots = (reference * candidate).sum(0)
    norms = reference.norm(dim=0) * candidate.norm(dim=0)
    cosines = torch.where(norms > 0, dots / norms.clamp_min(1e-300), torch.ones_like(dots))
    signs = torch.where(dots < 0, -torch.ones_like(dots), torch.ones_like(dots))
    return signs, float(cosines.abs().min()) if cosines.numel() else 1.0


def relative_l2(reference: torch.Tensor, candidate: torch.Tensor) -> float:
    scale = float(reference.norm())
    difference = float((reference - candidate).norm())
    return difference / scale if scale > 0 else difference


def compare(reference: Dict[Key, torch.Tensor], candidate: Dict[Key, torch.Tensor],
            steps: Optional[List[int]] = None) -> List[dict]:
    rows = []
    common_steps = sorted({step for step, _ in reference} & {step for step, _ in candidate})
    for step in common_steps:
        if steps is not None and step not in steps:
            continue
        signs = {}
        for stage in BASIS_STAGES:
            if (step, stage) in reference and (step, stage) in candidate \
                    and reference[(step, stage)].shape == candidate[(step, stage)].shape:
                signs[stage] = column_signs(reference[(step, stage)], candidate[(step, stage)])
        stage_names = sorted({stage for s, stage in reference if s == step} & {stage for s, stage in candidate if s == step},
                             key=lambda name: (RANK.get(name, len(RANK)), name))
        for stage in stage_names:
            ref, cand = reference[(step, stage)], candidate[(step, stage)]
            row = {"step": step, "stage": stage, "shape": list(ref.shape), "flipped": 0, "min_cosine": None}
            if ref.shape != cand.shape:
                row.update(error=float("inf"), max_abs=float("inf"), note=f"shape {list(cand.shape)} differs")
                rows.append(row)
                continue
            if stage in BASIS_STAGES and stage in signs:
                column, cosine = signs[stage]
                cand = cand * column
                row.update(flipped=int((column < 0).sum()), min_cosine=cosine)
            elif stage in IN_CURRENT_BASES or stage in IN_NEXT_BASES:
                suffix = "_after_step" if stage in IN_NEXT_BASES else ""
                left, right = signs.get("left_basis" + suffix), signs.get("right_basis" + suffix)
                if left is None and suffix:  # bases unchanged by the step were not dumped again
                    left, right = signs.get("left_basis"), signs.get("right_basis")
                if left is not None and right is not None and ref.ndim == 2 \
                        and ref.shape == (left[0].numel(), right[0].numel()):
                    cand = cand * left[0][:, None] * right[0][None, :]
            row.update(error=relative_l2(ref, cand), max_abs=float((ref - cand).abs().max()) if ref.numel() else 0.0)
            rows.append(row)
    return rows


def render(rows: List[dict], tolerance: float) -> str:
    lines = [f"{'step':>4}  {'stage':<34} {'shape':<14} {'rel L2':>10} {'max abs':>10}  notes"]
    for row in rows:
        notes = []
        if row.get("note"):
            notes.append(row["note"])
        if row["flipped"]:
            notes.append(f"{row['flipped']} columns sign-flipped")
        if row["min_cosine"] is not None and row["min_cosine"] < 0.99:
            notes.append(f"min |cos| {row['min_cosine']:.3f}: more than a sign differs")
        if not row["error"] <= tolerance:
            notes.append("ABOVE TOLERANCE")
        lines.append(f"{row['step']:>4}  {row['stage']:<34} {str(row['shape']):<14} {row['error']:>10.3e} "
                     f"{row['max_abs']:>10.3e}  {'; '.join(notes)}")
    return "\n".join(lines)


def first_divergence(rows: List[dict], tolerance: float) -> Optional[dict]:
    for row in rows:
        if not row["error"] <= tolerance:
            return row
    return None


def main(argv: Optional[List[str]] = None) -> int:
    parser = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    parser.add_argument("reference_log")
    parser.add_argument("candidate_log")
    parser.add_argument("--tolerance", type=float, default=1e-4, help="relative L2 bound per stage (default 1e-4)")
    parser.add_argument("--steps", default=None, help="comma-separated steps to compare (default: all common steps)")
    args = parser.parse_args(argv)
    try:
        with open(args.reference_log) as handle:
            reference = read_log(handle, args.reference_log)
        with open(args.candidate_log) as handle:
            candidate = read_log(handle, args.candidate_log)
    except (OSError, ValueError) as error:
        print(error, file=sys.stderr)
        return 2
    if not reference or not candidate:
        print("no SOAP_PROFILE lines found in one of the logs", file=sys.stderr)
        return 2
    steps = [int(token) for token in args.steps.split(",")] if args.steps else None
    rows = compare(reference, candidate, steps)
    if not rows:
        print("the logs have no step and stage in common", file=sys.stderr)
        return 2
    print(render(rows, args.tolerance))
    only_reference = sorted(set(reference) - set(candidate))
    only_candidate = sorted(set(candidate) - set(reference))
    if only_reference:
        print(f"only in {args.reference_log}: {len(only_reference)} stage dumps, e.g. {only_reference[:3]}")
    if only_candidate:
        print(f"only in {args.candidate_log}: {len(only_candidate)} stage dumps, e.g. {only_candidate[:3]}")
    worst = first_divergence(rows, args.tolerance)
    if worst is None:
        print(f"all {len(rows)} common stages within {args.tolerance:g}")
        return 0
    print(f"first stage above {args.tolerance:g}: step {worst['step']} {worst['stage']} (rel L2 {worst['error']:.3e})")
    return 1


if __name__ == "__main__":
    sys.exit(main())
