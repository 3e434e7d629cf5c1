"""Scalar helpers of the step prologue (Python doubles, as in the reference)."""

from __future__ import annotations


def debias(beta: float, step: int) -> float:
    """Adam-style debias term ``1 - beta**step``  (optimi/utils.py:26-28)."""
    return 1 - beta**step


def debias_beta(beta: float, step: int) -> float:
    """Beta with the debias correction folded in, ``(beta**t - beta) / (beta**t - 1)``,
    equal to ``beta * (1 - beta**(t-1)) / (1 - beta**t)``  (optimi/utils.py:31-36)."""
    bt = beta**step
    return (bt - beta) / (bt - 1)
