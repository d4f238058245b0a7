"""Parity metrics used by every comparison against the oracle."""
import numpy as np


def rel_l2(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def cosine(a, b):
    a = np.asarray(a, np.float64).ravel()
    b = np.asarray(b, np.float64).ravel()
    return float(a.dot(b) / max(np.linalg.norm(a) * np.linalg.norm(b), 1e-30))


def psnr(a, ref):
    """PSNR in dB with peak = range of the reference tensor."""
    a = np.asarray(a, np.float64).ravel()
    ref = np.asarray(ref, np.float64).ravel()
    mse = float(np.mean((a - ref) ** 2))
    peak = float(ref.max() - ref.min())
    if mse == 0:
        return float("inf")
    return 10.0 * np.log10(peak * peak / mse)
