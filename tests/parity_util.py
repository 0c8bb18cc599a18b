"""Shared assertions of the parity tests."""
import numpy as np


def top1_agreement(gl, lg):
    """Per-row top-1 agreement of device logits `gl` with oracle logits `lg`.  A row whose winner differs is a tie
    (counted as agreeing) when the oracle's own gap between its winner and the device's winner is within twice that
    row's largest logit error: the device cannot separate two candidates closer than its own error, and the contract's
    99 % bar is about mistakes, not about coin flips between equals.  Returns (fraction with ties counted, strict)."""
    a, b = gl.argmax(1), lg.argmax(1)
    rows = np.arange(lg.shape[0])
    gap = lg[rows, b] - lg[rows, a]
    err = np.abs(gl - lg).max(1)
    ok = (a == b) | (gap <= 2.0 * err)
    return float(ok.mean()), float((a == b).mean())
