"""Independent numpy statements of the V:N:M layout used to cross-check the
oracle and the library (derived from the index expressions of
src/format/format_sr_nm.cpp:368-374, :385-404, :509-536 of the reference)."""
import glob
import os

import numpy as np

GOLDEN_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def rel_err(got, exact):
    """max |got - exact| / max(|exact|, rms(exact) / 16): a true relative error wherever an entry is not far below the
    typical magnitude of the result (there the error of an fp32-accumulated sum is absolute by nature), so the 1e-2
    bound means the same on outputs of magnitude 0.3 as on outputs of magnitude 30."""
    got = np.asarray(got, dtype=np.float64)
    exact = np.asarray(exact, dtype=np.float64)
    floor = max(float(np.sqrt(np.mean(exact * exact))) / 16.0, 2.0 ** -14)
    return float((np.abs(got - exact) / np.maximum(np.abs(exact), floor)).max())


def fp16_steps(got, exact):
    """max |got - exact| in units of the fp16 spacing at max(|exact|, rms(exact) / 16) (0.5 = correctly rounded wherever
    the entry is not far below the result's typical magnitude)."""
    got = np.asarray(got, dtype=np.float64)
    exact = np.asarray(exact, dtype=np.float64)
    floor = max(float(np.sqrt(np.mean(exact * exact))) / 16.0, 2.0 ** -14)
    spacing = np.spacing(np.maximum(np.abs(exact), floor).astype(np.float16)).astype(np.float64)
    return float((np.abs(got - exact) / spacing).max())


def golden_cases():
    return sorted(glob.glob(os.path.join(GOLDEN_DIR, "vnm_*.npz")))


def ksp_of(cols, n, m):
    groups = -(-cols // m)
    return -(-(groups * n) // 16) * 16


def slot_maps(rows, ksp):
    """value index of slot 0 and (metadata word, bit shift) for every (row, group)."""
    ngroups = ksp // 2
    r = np.arange(rows)[:, None]
    g = np.arange(ngroups)[None, :]
    R16, q, p, s = r // 16, (r % 16) // 4, (r % 4) // 2, r % 2
    t, u = g // 4, g % 4
    vi = R16 * 16 * ksp + t * 128 + q * 32 + u * 8 + p * 4 + s * 2
    wi = (r // 32) * (ksp // 8) * 16 + t * 16 + ((r % 32) // 16) * 8 + q * 2 + p
    sh = s * 16 + u * 4 + 0 * g
    return vi, wi, sh


def numpy_decode(values, meta, columns, rows, cols, n, m, v):
    ksp = ksp_of(cols, n, m)
    ngroups = ksp // 2
    vi, wi, sh = slot_maps(rows, ksp)
    columns = np.asarray(columns, dtype=np.int64).reshape(rows // v, ngroups, 4)
    dense = np.zeros((rows, cols), values.dtype)
    nib = (np.asarray(meta, dtype=np.uint32)[wi] >> sh.astype(np.uint32)) & 0xF
    for j in range(2):
        pos = ((nib >> (2 * j)) & 3).astype(np.int64)
        cl = np.take_along_axis(columns[np.arange(rows) // v], pos[..., None], axis=-1)[..., 0]
        dcol = np.arange(ngroups)[None, :] * m + cl
        ok = dcol < cols
        rr = np.broadcast_to(np.arange(rows)[:, None], dcol.shape)
        dense[rr[ok], dcol[ok]] = values[(vi + j)[ok]]
    return dense


def random_conforming(rows, cols, n, m, v, seed, integer=False, dtype=np.float32):
    """Random matrix obeying V:N:M exactly (every kept entry non-zero) + its pattern."""
    rng = np.random.default_rng(seed)
    ksp = ksp_of(cols, n, m)
    ngroups = ksp // 2
    full = cols // m
    columns = np.zeros((rows // v, ngroups, 4), np.uint32)
    for b in range(rows // v):
        for g in range(full):
            columns[b, g] = np.sort(rng.choice(m, 4, replace=False))
        if cols % m:
            columns[b, full] = np.arange(4)
    dense = np.zeros((rows, cols), dtype)
    mask = np.zeros((rows, cols), np.int32)
    for r in range(rows):
        for g in range(-(-cols // m)):
            cand = [int(g * m + c) for c in columns[r // v, g] if g * m + c < cols]
            keep = rng.choice(len(cand), min(2, len(cand)), replace=False)
            for k in keep:
                val = rng.integers(1, 5) * rng.choice([-1, 1]) if integer else rng.standard_normal() + 3.0
                dense[r, cand[k]] = val
                mask[r, cand[k]] = 1
    return dense, mask, columns.reshape(-1)
