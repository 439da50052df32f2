"""Seeded synthetic workloads: clustered voxel clouds, features and weights.

Shapes follow the benchmark configurations: Gaussian clusters (sigma in voxels)
plus uniform noise on an integer (z, y, x) grid, de-duplicated.  Points that
fall outside the grid are rejected (not clipped).
"""
from typing import Sequence

import numpy as np


def clustered_voxels(rng: np.random.Generator, n_target: int, grid: Sequence[int], n_clusters: int,
                     sigma: float = 15.0, noise_frac: float = 0.10, batch: int = 0) -> np.ndarray:
    """[N, 4] int32 (batch, z, y, x) unique coordinates, N close to n_target,
    sorted by linear coordinate."""
    grid = np.asarray(grid, dtype=np.int64)
    n_noise = int(round(n_target * noise_frac))
    n_clu = n_target - n_noise
    centers = rng.uniform(0, grid, size=(n_clusters, 3))
    pts = []
    have = 0
    # oversample: rejection at the grid border and de-duplication both lose points
    # (clusters too small for the count asked for saturate: stop when two rounds in a row add
    # less than a hundredth of what is missing, and return what there is)
    stalled = 0
    while have < n_clu and stalled < 2:
        want = int((n_clu - have) * 1.5) + 1024
        cid = rng.integers(0, n_clusters, size=want)
        p = np.rint(centers[cid] + rng.normal(0.0, sigma, size=(want, 3))).astype(np.int64)
        ok = np.all((p >= 0) & (p < grid), axis=1)
        pts = [np.unique(np.concatenate(pts + [p[ok]]), axis=0)]
        stalled = stalled + 1 if pts[0].shape[0] - have < (n_clu - have) // 100 + 1 else 0
        have = pts[0].shape[0]
    clu = np.unique(np.concatenate(pts), axis=0)
    if clu.shape[0] > n_clu:
        clu = clu[np.sort(rng.choice(clu.shape[0], n_clu, replace=False))]
    noise = np.stack([rng.integers(0, g, size=n_noise) for g in grid], axis=1)
    allp = np.unique(np.concatenate([clu, noise]), axis=0)
    out = np.zeros((allp.shape[0], 4), dtype=np.int32)
    out[:, 0] = batch
    out[:, 1:] = allp
    return out


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even float32 -> bfloat16 bit patterns (uint16)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    out = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16).astype(np.uint16)
    out[np.isnan(x)] = 0x7FFF
    return out


def bf16_bits_to_f32(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
