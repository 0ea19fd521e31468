"""The parity bars of the model-level tests, in one place.

f32: rel 1e-4 per element, measured against max(|ref|, rms of the row): a logit near zero is a sum that
cancels, and its error scales with the terms of the sum, not with the result.
bf16 mode (against the f32 oracle fed the parameters the device stores): rel 2e-2 of the row's largest
value for every element, and rel 2e-2 of the row's norm for the row as a whole.  Rounding every matmul
operand to 8 bits of mantissa is noise at the scale of the row, not of each element.
"""
import numpy as np

RTOL_F32 = 1e-4
RTOL_BF16 = 2e-2


def rows(a):
    a = np.asarray(a)
    return a.reshape(-1, a.shape[-1]).astype(np.float64)


def rel_err_f32(ref, got):
    r, g = rows(ref), rows(got)
    floor = np.sqrt(np.mean(r * r, axis=1, keepdims=True))
    return float(np.max(np.abs(r - g) / np.maximum(np.maximum(np.abs(r), floor), 1e-30)))


def rel_err_bf16(ref, got):
    """(worst element error over the row maximum, worst row-norm error), over all rows"""
    r, g = rows(ref), rows(got)
    d = np.abs(r - g)
    mx = np.maximum(np.abs(r).max(axis=1), 1e-30)
    nr = np.maximum(np.linalg.norm(r, axis=1), 1e-30)
    return float(np.max(d.max(axis=1) / mx)), float(np.max(np.linalg.norm(d, axis=1) / nr))


def assert_f32(ref, got, what=""):
    e = rel_err_f32(ref, got)
    assert e <= RTOL_F32, f"{what}: f32 rel err {e:.3e} above {RTOL_F32}"


def assert_bf16(ref, got, what=""):
    em, en = rel_err_bf16(ref, got)
    assert em <= RTOL_BF16 and en <= RTOL_BF16, f"{what}: bf16 rel err {em:.3e} (max), {en:.3e} (norm) above {RTOL_BF16}"


def per_row_bf16(ref, got):
    """Per row: max(element error over the row maximum, row-norm error)."""
    r, g = rows(ref), rows(got)
    d = np.abs(r - g)
    return np.maximum(d.max(axis=1) / np.maximum(np.abs(r).max(axis=1), 1e-30),
                      np.linalg.norm(d, axis=1) / np.maximum(np.linalg.norm(r, axis=1), 1e-30))


def assert_logits(ref, got, mode, what=""):
    (assert_bf16 if mode == "bf16" else assert_f32)(ref, got, what)


def top2_margin(logits):
    """top-1 minus top-2 over the rms of the row, per row"""
    r = rows(logits)
    s = np.sort(r, axis=1)
    return (s[:, -1] - s[:, -2]) / np.maximum(np.sqrt(np.mean(r * r, axis=1)), 1e-30)


def top2_gap_over_max(logits):
    """top-1 minus top-2 over the largest magnitude of the row, per row"""
    r = rows(logits)
    s = np.sort(r, axis=1)
    return (s[:, -1] - s[:, -2]) / np.maximum(np.abs(r).max(axis=1), 1e-30)
