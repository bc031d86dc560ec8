"""Seeded synthetic workloads C1..C5 used by the benchmark and the parity tests.

Every tensor comes from a `torch.Generator(device='cpu')` seeded with
`1000*config + stream` (stream 1 = structure matrix / centres, 2 = data latents,
assignments or rows, 3 = queries drawn separately, 4 = directions, 5 = additive
noise), so the same arrays can be regenerated on any machine.  Data and queries
of one config are one draw of N+nq rows (first N = data) unless noted.
"""
import torch


def _gen(config, stream):
    g = torch.Generator(device="cpu")
    g.manual_seed(1000 * config + stream)
    return g


# (N, nq, dim, num_comp, num_simp, k) of the full-size configurations
SHAPES = {
    1: dict(n=3000, nq=500, dim=100, m=2, l=10, k=10),
    2: dict(n=1_000_000, nq=10_000, dim=128, m=2, l=10, k=10),
    3: dict(n=10_000_000, nq=10_000, dim=96, m=3, l=8, k=100),
    4: dict(n=1_000_000, nq=5_000, dim=960, m=2, l=12, k=10),
    5: dict(n=1_000_000, nq=10_000, dim=64, m=2, l=15, k=50),
}


def c1(n=3000, nq=500):
    """(100x50 N(0,1)) . (50x(n+nq) U[0,1)), transposed; dim 100."""
    a = torch.randn(100, 50, generator=_gen(1, 1))
    z = torch.rand(50, n + nq, generator=_gen(1, 2))
    x = (a @ z).T.contiguous()
    return x[:n].contiguous(), x[n:].contiguous()


def c2(n=1_000_000, nq=10_000, centres=1000, dim=128):
    """Gaussian mixture: centres U[0,255], sigma 20, clipped at 0, rounded."""
    c = torch.rand(centres, dim, generator=_gen(2, 1)) * 255.0
    a = torch.randint(0, centres, (n + nq,), generator=_gen(2, 2))
    g = _gen(2, 5)
    x = torch.empty(n + nq, dim)
    step = 1 << 18
    for s in range(0, n + nq, step):
        e = min(n + nq, s + step)
        noise = torch.randn(e - s, dim, generator=g)
        x[s:e] = torch.round(torch.clamp(c[a[s:e]] + 20.0 * noise, min=0.0))
    return x[:n].contiguous(), x[n:].contiguous()


def c3(n=10_000_000, nq=10_000, dim=96):
    """N(0,1) rows scaled to unit L2 norm."""
    g = _gen(3, 2)
    x = torch.empty(n + nq, dim)
    step = 1 << 20
    for s in range(0, n + nq, step):
        e = min(n + nq, s + step)
        r = torch.randn(e - s, dim, generator=g)
        x[s:e] = r / r.norm(dim=1, keepdim=True)
    return x[:n].contiguous(), x[n:].contiguous()


def c4(n=1_000_000, nq=5_000, dim=960, latent=32, sigma=0.1):
    """32-dim manifold in 960 dims plus N(0, 0.01) noise (variance 0.01)."""
    a = torch.randn(dim, latent, generator=_gen(4, 1))
    gz, gn = _gen(4, 2), _gen(4, 5)
    x = torch.empty(n + nq, dim)
    step = 1 << 16
    for s in range(0, n + nq, step):
        e = min(n + nq, s + step)
        z = torch.rand(latent, e - s, generator=gz) * 2.0 - 1.0
        x[s:e] = (a @ z).T + sigma * torch.randn(e - s, dim, generator=gn)
    return x[:n].contiguous(), x[n:].contiguous()


def c5_batch(batch, n=1_000_000, dim=64):
    """One of the 20 incremental N(0,1) batches."""
    g = torch.Generator(device="cpu")
    g.manual_seed(5002 + batch)
    return torch.randn(n, dim, generator=g)


def c5_queries(nq=10_000, dim=64):
    return torch.randn(nq, dim, generator=_gen(5, 3))


def directions(config, num_indices, dim):
    """Unnormalised N(0,1) direction draws for a config (stream 4)."""
    return torch.randn(num_indices, dim, generator=_gen(config, 4))


def exact_knn(X, Q, k, query_chunk=256, point_chunk=1 << 20):
    """Exact k nearest neighbours (ids, ascending by distance) of the rows of Q among the
    rows of X, on the device the tensors live on: recall ground truth.  A fast
    ||x||^2 - 2 q.x pass over blocks of points picks a pool of candidates per block
    (the matrix product's rounding and very long top-k rows are both kept out of the
    answer that way), whose distances are then recomputed in float64 for the final cut."""
    n = X.shape[0]
    pool = min(n, max(2 * k, k + 64))
    xn = (X * X).sum(1)
    out = []
    for q0 in range(0, Q.shape[0], query_chunk):
        q = Q[q0:q0 + query_chunk]
        cands = []
        for p0 in range(0, n, point_chunk):
            xb = X[p0:p0 + point_chunk]
            d2 = xn[None, p0:p0 + point_chunk] - 2.0 * (q @ xb.T)
            cands.append(d2.topk(min(pool, xb.shape[0]), dim=1, largest=False).indices + p0)
        cand = torch.cat(cands, 1)
        best = None
        for c0 in range(0, cand.shape[1], 4096):       # bounded memory for the float64 pass
            cc = cand[:, c0:c0 + 4096]
            d = (X[cc].double() - q[:, None, :].double()).norm(dim=2)
            if best is not None:
                d = torch.cat([best[0], d], 1)
                cc = torch.cat([best[1], cc], 1)
            top = d.topk(min(k, d.shape[1]), dim=1, largest=False)
            best = (top.values, torch.gather(cc, 1, top.indices))
        out.append(best[1])
    return torch.cat(out)


def recall_at_k(ids, truth):
    """Fraction of the true neighbours (rows of `truth`) found in the same rows of `ids`."""
    hit = (ids.long()[:, :, None] == truth.long()[:, None, :]).any(2).float().sum().item()
    return hit / truth.numel()
