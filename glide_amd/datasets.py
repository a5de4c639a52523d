"""Seeded synthetic datasets with the shapes of the benchmark configurations, and the fbin file format.

File formats follow the reference's load.cuh:8-128: fbin = u32 num, u32 dim, then num*dim values row-major.
"""
import numpy as np


def gmm_clipped(num, dim=128, components=64, mean_hi=160.0, sigma=25.0, seed=1234, mixture_seed=99):
    """Gaussian mixture with means uniform in [0, mean_hi], clipped to [0, 255] and rounded to integers.

    The mixture (means) depends only on `mixture_seed`, so base vectors and queries drawn with different
    `seed`s come from the same distribution.
    """
    means = np.random.default_rng(mixture_seed).uniform(0.0, mean_hi, size=(components, dim)).astype(np.float32)
    rng = np.random.default_rng(seed)
    out = np.empty((num, dim), dtype=np.float32)
    step = 1 << 18
    for s in range(0, num, step):
        e = min(num, s + step)
        comp = rng.integers(0, components, size=e - s)
        x = means[comp] + rng.standard_normal((e - s, dim), dtype=np.float32) * np.float32(sigma)
        out[s:e] = np.rint(np.clip(x, 0.0, 255.0))
    return out


def gmm_normalized(num, dim=96, components=256, sigma=0.3, seed=1234, mixture_seed=98):
    """Gaussian mixture with N(0,1) means, each row L2-normalised (cosine configuration)."""
    means = np.random.default_rng(mixture_seed).standard_normal((components, dim)).astype(np.float32)
    rng = np.random.default_rng(seed)
    comp = rng.integers(0, components, size=num)
    x = means[comp] + rng.standard_normal((num, dim), dtype=np.float32) * np.float32(sigma)
    x /= np.linalg.norm(x, axis=1, keepdims=True).astype(np.float32)
    return x.astype(np.float32)


def beta_scaled(num, dim=960, components=128, seed=1234, mixture_seed=97):
    """Beta(0.5, 2) per dimension, modulated by a per-cluster dimension-wise scale vector; values in [0, 1]."""
    scales = np.random.default_rng(mixture_seed).uniform(0.05, 1.0, size=(components, dim)).astype(np.float32)
    rng = np.random.default_rng(seed)
    out = np.empty((num, dim), dtype=np.float32)
    step = 1 << 16
    for s in range(0, num, step):
        e = min(num, s + step)
        comp = rng.integers(0, components, size=e - s)
        out[s:e] = rng.beta(0.5, 2.0, size=(e - s, dim)).astype(np.float32) * scales[comp]
    return out


def lowdim_integer(num, dim=128, latent=12, spread=20.0, noise=3.0, seed=1234, mixture_seed=0):
    """A `latent`-dimensional Gaussian cloud mapped linearly into `dim` dimensions, centred on 128, plus a little noise,
    clipped to [0, 255] and rounded: integer-valued data of low intrinsic dimension, on which graph search navigates
    well.  The linear map depends only on `mixture_seed`."""
    a = np.random.default_rng(mixture_seed).standard_normal((latent, dim)).astype(np.float32)
    r = np.random.default_rng(seed)
    out = np.empty((num, dim), dtype=np.float32)
    for s in range(0, num, 1 << 18):
        e = min(num, s + (1 << 18))
        z = r.standard_normal((e - s, latent)).astype(np.float32)
        out[s:e] = np.rint(np.clip(z @ a * spread + 128 + r.standard_normal((e - s, dim)).astype(np.float32) * noise, 0, 255))
    return out


def write_fbin(path, matrix):
    matrix = np.ascontiguousarray(matrix)
    with open(path, "wb") as f:
        np.array(matrix.shape, dtype=np.uint32).tofile(f)
        matrix.tofile(f)


def read_fbin(path, dtype=np.float32):
    with open(path, "rb") as f:
        num, dim = np.fromfile(f, dtype=np.uint32, count=2)
        return np.fromfile(f, dtype=dtype, count=int(num) * int(dim)).reshape(int(num), int(dim))


def write_vector(path, vec):
    vec = np.ascontiguousarray(vec, dtype=np.uint32)
    with open(path, "wb") as f:
        np.array([vec.size], dtype=np.uint32).tofile(f)
        vec.tofile(f)


def read_vector(path):
    with open(path, "rb") as f:
        n = int(np.fromfile(f, dtype=np.uint32, count=1)[0])
        return np.fromfile(f, dtype=np.uint32, count=n)


def write_segment(path, starts, lengths):
    starts = np.ascontiguousarray(starts, dtype=np.uint32)
    lengths = np.ascontiguousarray(lengths, dtype=np.uint32)
    with open(path, "wb") as f:
        np.array([starts.size], dtype=np.uint32).tofile(f)
        starts.tofile(f)
        lengths.tofile(f)


def read_segment(path):
    with open(path, "rb") as f:
        n = int(np.fromfile(f, dtype=np.uint32, count=1)[0])
        starts = np.fromfile(f, dtype=np.uint32, count=n)
        lengths = np.fromfile(f, dtype=np.uint32, count=n)
    return starts, lengths


def recall(result_ids, truth_ids, k):
    """Mean fraction of the true top-k found among the returned top-k (small_search.cu:14-36)."""
    hit = 0
    for r, t in zip(result_ids[:, :k], truth_ids[:, :k]):
        hit += len(set(r.tolist()) & set(t.tolist()))
    return hit / float(result_ids.shape[0] * k)


def reachable_recall_bound(graph, centroids, start_points, queries, gt, metric=0):
    """Upper bound on recall@k of ANY beam width on a finished index, from the reference's entry rule alone: a search enters
    through the single start point of the query's nearest centroid (search_kernel.cuh:270-271; one random start point per
    partition, glide_impl.cuh:43-75) and only ever scores neighbours of nodes it has scored, so a true neighbour outside the
    set reachable from that start point over directed graph edges cannot be returned.  Returns (bound, fraction of the
    points reachable from the average start point).  Host-side breadth-first search over the N x D id table."""
    from scipy.sparse import csr_matrix
    from scipy.sparse.csgraph import breadth_first_order
    n, deg = graph.shape
    valid = graph != 0xFFFFFFFF
    indptr = np.concatenate([[0], np.cumsum(valid.sum(1))]).astype(np.int64)
    adj = csr_matrix((np.ones(int(indptr[-1]), np.int8), graph[valid].astype(np.int64), indptr), shape=(n, n))
    q64, c64 = queries.astype(np.float64), centroids.astype(np.float64)
    nearest = ((q64 * q64).sum(1)[:, None] - 2.0 * q64 @ c64.T + (c64 * c64).sum(1)[None]).argmin(1)
    hits, sizes = np.zeros(queries.shape[0]), []
    for c in np.unique(nearest):
        sp = int(start_points[c])
        order = breadth_first_order(adj, sp, directed=True, return_predecessors=False)
        reach = np.zeros(n, bool)
        reach[order] = True
        reach[sp] = bool((graph[order] == sp).any())   # the start point itself is only scored if an edge leads back to it
        sizes.append(reach.mean())
        mine = np.nonzero(nearest == c)[0]
        hits[mine] = reach[gt[mine].astype(np.int64)].mean(1)
    return float(hits.mean()), float(np.mean(sizes)), hits
