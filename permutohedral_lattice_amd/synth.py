"""Seeded synthetic inputs of the shapes the filter is benchmarked and tested on (numpy, host).

All images are channels-last float32, as the LatticeFilter op takes them
(reference: src/LatticeFilterKernel.cpp:111-124).
"""
import numpy as np


def blob_image(height, width, seed, channels=3, n_blobs=12, noise=0.05):
    """Sum of Gaussian colour blobs (sigma 20-80 px) plus uniform noise, clipped to [0, 1]."""
    rng = np.random.default_rng(seed)
    yy, xx = np.meshgrid(np.arange(height, dtype=np.float32), np.arange(width, dtype=np.float32),
                         indexing="ij")
    img = np.zeros((height, width, channels), np.float32)
    for _ in range(n_blobs):
        cy, cx = rng.uniform(0, height), rng.uniform(0, width)
        sigma = rng.uniform(20.0, 80.0)
        colour = rng.uniform(0.0, 1.0, channels).astype(np.float32)
        g = np.exp(-((yy - cy) ** 2 + (xx - cx) ** 2) / (2.0 * sigma * sigma)).astype(np.float32)
        img += g[..., None] * colour
    img += rng.uniform(-noise, noise, img.shape).astype(np.float32)
    return np.clip(img, 0.0, 1.0).astype(np.float32)


def uniform_image(shape, seed):
    return np.random.default_rng(seed).uniform(0.0, 1.0, shape).astype(np.float32)


def normal_image(shape, seed):
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)


def ellipsoid_volume(depth, height, width, seed, n_ellipsoids=8, noise_sigma=0.05):
    """Piecewise-constant ellipsoids (later ones overwrite earlier ones) plus Gaussian noise."""
    rng = np.random.default_rng(seed)
    zz, yy, xx = np.meshgrid(np.arange(depth, dtype=np.float32),
                             np.arange(height, dtype=np.float32),
                             np.arange(width, dtype=np.float32), indexing="ij")
    vol = np.zeros((depth, height, width), np.float32)
    scale = min(depth, height, width) / 128.0
    for _ in range(n_ellipsoids):
        c = rng.uniform(0, 1, 3) * np.array([depth, height, width])
        ax = np.array([rng.uniform(10, 50), rng.uniform(20, 100), rng.uniform(20, 100)]) * scale
        inside = (((zz - c[0]) / ax[0]) ** 2 + ((yy - c[1]) / ax[1]) ** 2
                  + ((xx - c[2]) / ax[2]) ** 2) <= 1.0
        vol[inside] = rng.uniform(0, 1)
    vol += rng.normal(0.0, noise_sigma, vol.shape).astype(np.float32)
    return vol.astype(np.float32)[..., None]


def softmax_logits(shape, seed):
    """softmax over the last axis of N(0,1) logits."""
    z = normal_image(shape, seed).astype(np.float64)
    z -= z.max(axis=-1, keepdims=True)
    e = np.exp(z)
    return (e / e.sum(axis=-1, keepdims=True)).astype(np.float32)


def bilateral_positions(guide, theta_alpha, theta_beta):
    """Feature rows (coords / theta_alpha, guide / theta_beta) for one channels-last item;
    same formula as the reference's feature builder (src/PermutohedralLatticeCPU.h:452-474),
    here with numpy float32 division (IEEE, so identical results)."""
    guide = np.asarray(guide, np.float32)
    sdims = guide.shape[:-1]
    grids = np.meshgrid(*[np.arange(s, dtype=np.float32) for s in sdims], indexing="ij")
    cols = [(g / np.float32(theta_alpha)).reshape(-1) for g in grids]
    flat = guide.reshape(-1, guide.shape[-1])
    cols += [flat[:, c] / np.float32(theta_beta) for c in range(flat.shape[1])]
    return np.stack(cols, axis=1).astype(np.float32)


def spatial_positions(sdims, theta_gamma):
    grids = np.meshgrid(*[np.arange(s, dtype=np.float32) for s in sdims], indexing="ij")
    cols = [(g / np.float32(theta_gamma)).reshape(-1) for g in grids]
    return np.stack(cols, axis=1).astype(np.float32)
