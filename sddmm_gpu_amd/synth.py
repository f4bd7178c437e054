"""Seeded synthetic inputs of the five benchmark shapes.

Every generator returns a dict with
  n_rows, n_cols, nnz      python ints
  row_ptr   int32 [n_rows+1]
  row_ind   int32 [nnz]        (row, col)-sorted, duplicates removed
  col_ind   int32 [nnz]
  val       fp32  [nnz]
  W         fp32  [n_rows, K]  row-major
  H         fp32  [n_cols, K]
  K, seed, name
as torch tensors on the requested device.  torch is used only as an array
library with a seedable generator that runs on the host or on the GPU; the
same code makes the small inputs of the CPU tests and the full-size inputs of
the GPU runs.  `scale` shrinks the matrix dimensions (and with them nnz) while
keeping the distributions, so parity tests can run a CPU check in seconds.
"""
from __future__ import annotations

import math
import torch


def _gen(seed: int, device) -> torch.Generator:
    g = torch.Generator(device=device)
    g.manual_seed(int(seed))
    return g


def _finish(name, n_rows, n_cols, keys, val_fn, K, wh_fn, seed, device, g):
    """keys: int64 row*n_cols+col, unsorted, possibly with duplicates."""
    keys = torch.unique(keys)  # sorted, duplicates removed -> (row, col) order
    row = torch.div(keys, n_cols, rounding_mode="floor")
    col = keys - row * n_cols
    nnz = int(keys.numel())
    if nnz >= 2**31:
        raise ValueError("nnz does not fit int32 offsets")
    counts = torch.bincount(row, minlength=n_rows)
    row_ptr = torch.zeros(n_rows + 1, dtype=torch.int64, device=device)
    row_ptr[1:] = torch.cumsum(counts, 0)
    out = dict(name=name, n_rows=int(n_rows), n_cols=int(n_cols), nnz=nnz, K=int(K), seed=int(seed),
               row_ptr=row_ptr.to(torch.int32), row_ind=row.to(torch.int32), col_ind=col.to(torch.int32))
    del keys, row, col
    out["val"] = val_fn(nnz, g)
    out["W"] = wh_fn((n_rows, K), g)
    out["H"] = wh_fn((n_cols, K), g)
    return out


def _uniform_pm1(device):
    return lambda shape, g: (torch.rand(shape, generator=g, device=device, dtype=torch.float32) * 2.0 - 1.0)


def _normal(sigma, device):
    return lambda shape, g: (torch.randn(shape, generator=g, device=device, dtype=torch.float32) * sigma)


def _uniform_01_open_left(device):
    # (0, 1]: 1 - U with U in [0, 1)
    return lambda n, g: (1.0 - torch.rand(n, generator=g, device=device, dtype=torch.float32))


def _draws_for_unique(weights: torch.Tensor, targets: torch.Tensor) -> torch.Tensor:
    """Number of iid draws from `weights` whose expected number of DISTINCT
    outcomes equals each target (E[unique](m) = sum_c 1-exp(-m w_c), inverted
    on a geometric grid by interpolation)."""
    n = weights.numel()
    w = weights.double()
    w = w / w.sum()
    grid = torch.unique(torch.cat([
        torch.arange(0, 64, dtype=torch.float64, device=w.device),
        torch.logspace(0, math.log10(60.0 / float(w.min())), 400, dtype=torch.float64, device=w.device)]))
    uniq = (1.0 - torch.exp(-grid[:, None] * w[None, :])).sum(1)  # increasing in m
    t = targets.double().clamp(max=float(n) * 0.999)
    idx = torch.searchsorted(uniq, t).clamp(1, grid.numel() - 1)
    u0, u1, g0, g1 = uniq[idx - 1], uniq[idx], grid[idx - 1], grid[idx]
    m = g0 + (g1 - g0) * (t - u0) / (u1 - u0).clamp(min=1e-30)
    return torch.ceil(m).long().clamp(min=1)


def _rows_by_popularity(n_rows, n_cols, deg, weights, g, device, chunk_draws=1 << 26):
    """For each row r draw columns iid from `weights` so that about deg[r]
    distinct columns result; returns int64 keys row*n_cols+col (with dups)."""
    cdf = torch.cumsum(weights.double(), 0)
    cdf = (cdf / cdf[-1]).float()
    m = _draws_for_unique(weights, deg)
    ends = torch.cumsum(m, 0)
    keys = []
    r0 = 0
    while r0 < n_rows:
        base = int(ends[r0 - 1]) if r0 > 0 else 0
        r1 = int(torch.searchsorted(ends, torch.tensor([base + chunk_draws], device=device)).item())
        r1 = max(r1, r0 + 1)
        r1 = min(r1, n_rows)
        total = int(ends[r1 - 1]) - base
        rows = torch.repeat_interleave(torch.arange(r0, r1, device=device), m[r0:r1], output_size=total)
        u = torch.rand(total, generator=g, device=device, dtype=torch.float32)
        cols = torch.searchsorted(cdf, u).clamp(max=n_cols - 1)
        keys.append(torch.unique(rows * n_cols + cols))
        del rows, u, cols
        r0 = r1
    return torch.cat(keys)


def uniform_random(n_rows=4096, n_cols=4096, density=0.01, K=32, seed=1, device="cpu"):
    """Config 1: nonzeros placed uniformly at random, values U(0,1], W/H U[-1,1]."""
    g = _gen(seed, device)
    m = int(round(n_rows * n_cols * density))
    keys = torch.randint(0, n_rows * n_cols, (m,), generator=g, device=device, dtype=torch.int64)
    return _finish("uniform", n_rows, n_cols, keys, _uniform_01_open_left(device), K, _uniform_pm1(device), seed, device, g)


def bag_of_words(n_rows=1500, n_cols=12419, mean_row=497.5, K=256, seed=2, device="cpu", zipf_s=1.1, shuffle_cols=True):
    """Config 2: Zipf(1.1) word frequencies, lognormal document lengths,
    geometric(p=0.4) counts stored as fp32, W/H N(0, 0.1)."""
    g = _gen(seed, device)
    sigma = 0.8
    mu = math.log(mean_row) - sigma * sigma / 2
    deg = torch.exp(torch.randn(n_rows, generator=g, device=device) * sigma + mu).clamp(1, n_cols * 0.9)
    w = torch.arange(1, n_cols + 1, device=device, dtype=torch.float64) ** (-zipf_s)
    if shuffle_cols:
        w = w[torch.randperm(n_cols, generator=g, device=device)]
    keys = _rows_by_popularity(n_rows, n_cols, deg, w, g, device)

    def counts(n, g):
        u = 1.0 - torch.rand(n, generator=g, device=device, dtype=torch.float32)  # (0,1]
        return torch.floor(torch.log(u) / math.log(1.0 - 0.4)) + 1.0

    return _finish("bag_of_words", n_rows, n_cols, keys, counts, K, _normal(0.1, device), seed, device, g)


def recommender(n_rows=480189, n_cols=17770, K=128, seed=3, device="cpu", zipf_s=0.9, beta=1.42,
                max_deg=17000, shuffle_cols=True):
    """Config 3: user degrees from a truncated power law x^-beta on
    [1, max_deg] (mean about 209 at full size), item popularity Zipf(0.9),
    integer ratings 1..5 as fp32, W/H N(0, 0.05)."""
    g = _gen(seed, device)
    M = float(min(max_deg, int(n_cols * 0.95)))
    u = torch.rand(n_rows, generator=g, device=device, dtype=torch.float64)
    e = 1.0 - beta
    deg = (1.0 - u * (1.0 - M ** e)) ** (1.0 / e)
    deg = deg.clamp(1.0, M)
    w = torch.arange(1, n_cols + 1, device=device, dtype=torch.float64) ** (-zipf_s)
    if shuffle_cols:
        w = w[torch.randperm(n_cols, generator=g, device=device)]
    keys = _rows_by_popularity(n_rows, n_cols, deg, w, g, device)
    ratings = lambda n, g: torch.randint(1, 6, (n,), generator=g, device=device).float()
    return _finish("recommender", n_rows, n_cols, keys, ratings, K, _normal(0.05, device), seed, device, g)


def rmat(scale=22, n_edges=200_000_000, K=64, seed=4, device="cpu", a=0.57, b=0.19, c=0.19, d=0.05,
         chunk=1 << 25):
    """Config 4: R-MAT graph of 2^scale vertices, duplicates removed, values
    1.0, W/H U[-1,1]."""
    g = _gen(seed, device)
    n = 1 << scale
    keys = []
    done = 0
    while done < n_edges:
        m = min(chunk, n_edges - done)
        row = torch.zeros(m, dtype=torch.int64, device=device)
        col = torch.zeros(m, dtype=torch.int64, device=device)
        for _ in range(scale):
            u = torch.rand(m, generator=g, device=device, dtype=torch.float32)
            rbit = (u >= a + b).long()                       # quadrants c, d -> lower half
            cbit = (((u >= a) & (u < a + b)) | (u >= a + b + c)).long()  # quadrants b, d -> right half
            row = row * 2 + rbit
            col = col * 2 + cbit
        keys.append(torch.unique(row * n + col))
        del row, col
        done += m
    keys = torch.cat(keys)
    ones = lambda k, g: torch.ones(k, dtype=torch.float32, device=device)
    return _finish("rmat", n, n, keys, ones, K, _uniform_pm1(device), seed, device, g)


def banded(n=1 << 20, per_row=64, half_band=2048, K=512, seed=5, device="cpu"):
    """Config 5: per_row columns per row drawn uniformly inside +-half_band of
    the diagonal (clipped at the edges, duplicates removed), values U(0,1],
    W/H N(0, 0.02)."""
    g = _gen(seed, device)
    rows = torch.arange(n, device=device, dtype=torch.int64).repeat_interleave(per_row)
    off = torch.randint(-half_band, half_band + 1, (n * per_row,), generator=g, device=device, dtype=torch.int64)
    cols = (rows + off).clamp(0, n - 1)
    keys = rows * n + cols
    del rows, off, cols
    return _finish("banded", n, n, keys, _uniform_01_open_left(device), K, _normal(0.02, device), seed, device, g)


def make(config: int, scale: float = 1.0, device="cpu", K=None, seed=None):
    """Config 1..5 of the benchmark list; scale<1 shrinks the dimensions."""
    kw = {}
    if K is not None:
        kw["K"] = K
    if seed is not None:
        kw["seed"] = seed
    s = float(scale)
    if config == 1:
        n = max(8, int(4096 * s))
        return uniform_random(n, n, device=device, **kw)
    if config == 2:
        return bag_of_words(max(4, int(1500 * s)), max(16, int(12419 * s)), mean_row=max(2.0, 497.5 * s),
                            device=device, **kw)
    if config == 3:
        return recommender(max(4, int(480189 * s)), max(32, int(17770 * math.sqrt(s))),
                           max_deg=max(4, int(17000 * math.sqrt(s))), device=device, **kw)
    if config == 4:
        sc = max(4, 22 + int(round(math.log2(s)))) if s < 1 else 22
        return rmat(sc, max(16, int(200_000_000 * s)), device=device, **kw)
    if config == 5:
        n = max(64, int((1 << 20) * s))
        return banded(n, per_row=64 if n >= 4096 else 8, half_band=min(2048, n // 2), device=device, **kw)
    raise ValueError("config must be 1..5")
