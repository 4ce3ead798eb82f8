"""Tensor comparison metrics used by the accuracy tooling (counterpart of the reference's
``get_deff``, my_utils/ops_util.py:86-189: same arguments that matter, same return shape)."""
from typing import Dict, Optional, Tuple

import torch

from . import Logger

ABS_STEPS = (1e-5, 1e-4, 1e-3, 1e-2, 1e-1)
REL_STEPS = (0.01, 0.05, 0.1, 0.2, 0.3, 0.5)


def get_deff(x: torch.Tensor, y: torch.Tensor, verbose: bool = True, strict_threshold: float = 1e-3,
             loose_abs_threshold: float = 1e-4, loose_rel_threshold: float = 0.3, relative_error: bool = True,
             cosine_similarity: bool = True, sample_region: Optional[tuple] = None) -> Tuple[torch.Tensor, float, float, Dict]:
    """Returns ``(mean |x-y|, fraction with |x-y| <= strict_threshold, fraction "loosely equal", metrics)``.
    Loosely equal: |x-y| < loose_abs_threshold, or y within ``loose_rel_threshold`` (relative) of x on x's side of 0."""
    if x.shape != y.shape:
        raise ValueError(f"Shape mismatch: x {tuple(x.shape)}, y {tuple(y.shape)}")
    if sample_region is not None:
        x, y = x[sample_region], y[sample_region]
    xf, yf = x.float(), y.float()
    err = (xf - yf).abs()
    n = err.numel()
    strict = float((err <= strict_threshold).sum()) / n
    lo = torch.minimum(xf * (1 - loose_rel_threshold), xf * (1 + loose_rel_threshold))
    hi = torch.maximum(xf * (1 - loose_rel_threshold), xf * (1 + loose_rel_threshold))
    loose = float(((err < loose_abs_threshold) | ((yf >= lo) & (yf <= hi))).sum()) / n
    rel = err / (xf.abs() + 1e-8)
    metrics: Dict = {
        "abs_error_ratios": {f"<= {t}": float((err <= t).sum()) / n for t in ABS_STEPS},
        "rel_error_ratios": {f"<= {int(t * 100)}%": float((rel <= t).sum()) / n for t in REL_STEPS},
        "max_abs_error": float(err.max()),
    }
    if relative_error:
        metrics["mean_relative_error"] = float(rel.mean())
    if cosine_similarity:
        metrics["cosine_similarity"] = float(torch.nn.functional.cosine_similarity(xf.reshape(-1), yf.reshape(-1), dim=0))
    mean_err = err.mean()
    if verbose:
        Logger.log(f"mean abs error {float(mean_err):.3e}, strict {strict * 100:.2f}%, loose {loose * 100:.2f}%, {metrics}")
    return mean_err, strict, loose, metrics
