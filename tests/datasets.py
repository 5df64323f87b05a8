"""Test and benchmark support: synthetic datasets, a plain k-means trainer, exact ground truth.

Not part of the search path.  The library takes a *trained model* (coarse centres, rotation,
PQ codebooks) through ``build_precomputed``; this module produces such models with ordinary
Lloyd iterations so that tests and the benchmark have realistic index contents.  The trainer does
not try to reproduce cuVS's balanced hierarchical k-means: the contract with the search path is
the layout and meaning of the model tensors, not how they were fitted.

Everything here runs on whatever device the input tensor lives on (CPU in unit tests, the GPU in
the benchmark).
"""
import math

import numpy as np
import torch


def dim_ext_of(dim):
    return ((dim + 1 + 7) // 8) * 8


# --------------------------------------------------------------------------------------------
# synthetic datasets of the benchmark configurations
# --------------------------------------------------------------------------------------------

def gaussian_mixture(n, dim, n_components, sigma, seed, device="cpu", center_scale=1.0,
                     normalize_centers=False, normalize_rows=False, dim_decay=None,
                     chunk=1 << 20, dtype=torch.float32):
    """Rows = centre[c] + N(0, sigma^2), c uniform.  Optional per-dimension decay (anisotropy)."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    centers = torch.randn(n_components, dim, generator=g, device=device) * center_scale
    scale = None
    if dim_decay is not None:
        scale = torch.pow(torch.tensor(dim_decay, device=device),
                          torch.arange(dim, device=device, dtype=torch.float32))
        centers = centers * scale
    if normalize_centers:
        centers = torch.nn.functional.normalize(centers, dim=1)
    out = torch.empty(n, dim, dtype=dtype, device=device)
    for s in range(0, n, chunk):
        m = min(chunk, n - s)
        comp = torch.randint(0, n_components, (m,), generator=g, device=device)
        noise = torch.randn(m, dim, generator=g, device=device) * sigma
        if scale is not None:
            noise = noise * scale
        rows = centers[comp] + noise
        if normalize_rows:
            rows = torch.nn.functional.normalize(rows, dim=1)
        out[s:s + m] = rows.to(dtype)
    return out


def sift_like_u8(n, dim, n_components, seed, device="cpu", chunk=1 << 20):
    """uint8 rows: clamp(round(|N(mu_c, sigma^2 = 25)|), 0, 255), cluster means mu_c ~ U[0, 128]."""
    g = torch.Generator(device=device)
    g.manual_seed(seed)
    means = torch.rand(n_components, dim, generator=g, device=device) * 128.0
    out = torch.empty(n, dim, dtype=torch.uint8, device=device)
    for s in range(0, n, chunk):
        m = min(chunk, n - s)
        comp = torch.randint(0, n_components, (m,), generator=g, device=device)
        rows = means[comp] + torch.randn(m, dim, generator=g, device=device) * 5.0
        out[s:s + m] = rows.abs().round().clamp(0, 255).to(torch.uint8)
    return out


def to_float(x):
    """utils::mapping<float> of cuVS: uint8 / 256, int8 / 128, others widened."""
    if x.dtype == torch.uint8:
        return x.to(torch.float32) * (1.0 / 256.0)
    if x.dtype == torch.int8:
        return x.to(torch.float32) * (1.0 / 128.0)
    return x.to(torch.float32)


# --------------------------------------------------------------------------------------------
# k-means
# --------------------------------------------------------------------------------------------

def assign_nearest(x, centers, chunk=1 << 16, half=False):
    """argmin_c ||x - c||^2 by chunks of rows; `half` uses fp16 GEMMs (for very large inputs)."""
    n = x.shape[0]
    labels = torch.empty(n, dtype=torch.int64, device=x.device)
    cn = (centers.float() ** 2).sum(1)
    ct = centers.t().contiguous()
    if half:
        ct = ct.half()
    for s in range(0, n, chunk):
        xs = to_float(x[s:s + chunk])
        if half:
            d = cn[None, :] - 2.0 * (xs.half() @ ct).float()
        else:
            d = cn[None, :] - 2.0 * (xs @ ct)
        labels[s:s + chunk] = d.argmin(1)
    return labels


def kmeans(x, k, iters, seed, half=False):
    """Plain Lloyd iterations with random initialisation; empty clusters are re-seeded."""
    n, d = x.shape
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    perm = torch.randperm(n, generator=g)[:k].to(x.device)
    centers = to_float(x[perm]).clone()
    if n < k:  # fewer points than clusters: pad with jittered copies
        extra = centers[torch.randint(0, n, (k - n,), generator=g).to(x.device)]
        centers = torch.cat([centers, extra + 1e-3 * torch.randn(k - n, d, generator=g).to(x.device)])
    xf = None
    for _ in range(iters):
        labels = assign_nearest(x, centers, half=half)
        sums = torch.zeros(k, d, dtype=torch.float32, device=x.device)
        counts = torch.zeros(k, dtype=torch.float32, device=x.device)
        for s in range(0, n, 1 << 20):
            xs = to_float(x[s:s + (1 << 20)])
            ls = labels[s:s + (1 << 20)]
            sums.index_add_(0, ls, xs)
            counts.index_add_(0, ls, torch.ones_like(ls, dtype=torch.float32))
        empty = counts == 0
        centers = torch.where(empty[:, None], centers, sums / counts.clamp(min=1)[:, None])
        n_empty = int(empty.sum().item())
        if n_empty > 0:
            repl = torch.randint(0, n, (n_empty,), generator=g).to(x.device)
            centers[empty] = to_float(x[repl])
    del xf
    return centers


def batched_kmeans(x, k, iters, seed):
    """Independent k-means problems in one batch.  x: [M, n, p] -> centres [M, k, p]."""
    M, n, p = x.shape
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    if n >= k:
        idx = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(M)]).to(x.device)
    else:
        idx = torch.randint(0, n, (M, k), generator=g).to(x.device)
    centers = torch.gather(x, 1, idx[:, :, None].expand(-1, -1, p)).clone()
    if n < k:
        centers = centers + 1e-3 * torch.randn(M, k, p, generator=g).to(x.device)
    for _ in range(iters):
        cn = (centers ** 2).sum(2)                      # [M, k]
        d = cn[:, None, :] - 2.0 * torch.bmm(x, centers.transpose(1, 2))
        labels = d.argmin(2)                            # [M, n]
        sums = torch.zeros(M, k, p, dtype=torch.float32, device=x.device)
        sums.scatter_add_(1, labels[:, :, None].expand(-1, -1, p), x)
        counts = torch.zeros(M, k, dtype=torch.float32, device=x.device)
        counts.scatter_add_(1, labels, torch.ones(M, n, dtype=torch.float32, device=x.device))
        empty = counts == 0
        centers = torch.where(empty[:, :, None], centers, sums / counts.clamp(min=1)[:, :, None])
    return centers


# --------------------------------------------------------------------------------------------
# model training
# --------------------------------------------------------------------------------------------

def make_rotation(dim, rot_dim, force_random, seed, device):
    """Identity when dim == rot_dim and not forced, else a random matrix with orthonormal columns
    (role of make_rotation_matrix, cuVS ivf_pq_build_common.cu:235-261)."""
    if dim == rot_dim and not force_random:
        return torch.eye(rot_dim, dim, dtype=torch.float32, device=device)
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    a = torch.randn(rot_dim, rot_dim, generator=g, dtype=torch.float64)
    q, _ = torch.linalg.qr(a)
    return q[:, :dim].to(torch.float32).contiguous().to(device)


def train_model(x, n_lists, pq_dim, pq_bits, metric="sqeuclidean", codebook_kind="subspace",
                kmeans_iters=10, pq_iters=10, seed=137, force_random_rotation=False,
                max_pq_train=1 << 16, half_assign=False):
    """Fit coarse centres and PQ codebooks on the rows of `x` (any supported element type).

    Returns a dict of float32 tensors on x's device with the shapes cuvsIvfPqBuildPrecomputed
    takes: centers [n_lists, dim_ext] (column dim = squared norm), centers_rot [n_lists, rot_dim],
    rotation_matrix [rot_dim, dim], pq_centers [pq_dim | n_lists, pq_len, 1 << pq_bits].
    """
    dev = x.device
    n, dim = x.shape
    pq_len = (dim + pq_dim - 1) // pq_dim
    rot_dim = pq_len * pq_dim
    book = 1 << pq_bits
    xs = x
    if metric == "cosine":
        xs = torch.nn.functional.normalize(to_float(x), dim=1)
    centers = kmeans(xs, n_lists, kmeans_iters, seed, half=half_assign)
    if metric == "cosine":
        centers = torch.nn.functional.normalize(centers, dim=1)
    rotation = make_rotation(dim, rot_dim, force_random_rotation, seed + 7, dev)
    padded = torch.zeros(n_lists, dim_ext_of(dim), dtype=torch.float32, device=dev)
    padded[:, :dim] = centers
    padded[:, dim] = (centers ** 2).sum(1)
    centers_rot = (centers @ rotation.t()).contiguous()

    # residuals of a training subsample in the rotated space
    g = torch.Generator(device="cpu")
    g.manual_seed(seed + 1)
    m = min(n, max_pq_train)
    sel = torch.randperm(n, generator=g)[:m].to(dev)
    xt = to_float(xs[sel])
    labels = assign_nearest(xt, centers, half=half_assign)
    res = ((xt - centers[labels]) @ rotation.t()).reshape(m, pq_dim, pq_len)
    if codebook_kind == "subspace":
        cb = batched_kmeans(res.permute(1, 0, 2).contiguous(), book, pq_iters, seed + 2)
        pq_centers = cb.transpose(1, 2).contiguous()          # [pq_dim, pq_len, book]
    else:
        pq_centers = torch.empty(n_lists, pq_len, book, dtype=torch.float32, device=dev)
        pool = res.reshape(-1, pq_len)
        for l in range(n_lists):
            pts = res[labels == l].reshape(-1, pq_len)
            if pts.shape[0] < book:  # too few residuals in this list: top up from the global pool
                extra = pool[torch.randint(0, pool.shape[0], (book * 4,), generator=g).to(dev)]
                pts = torch.cat([pts, extra])
            cb = batched_kmeans(pts[None], book, pq_iters, seed + 3 + l)[0]
            pq_centers[l] = cb.t()
    return {"centers": padded.contiguous(), "centers_rot": centers_rot,
            "rotation_matrix": rotation.contiguous(), "pq_centers": pq_centers.contiguous()}


# --------------------------------------------------------------------------------------------
# exact ground truth and recall
# --------------------------------------------------------------------------------------------

def exact_knn(dataset, queries, k, metric="sqeuclidean", row_chunk=1 << 18, half=False):
    """Exact top-k ids by brute force on the original vectors (fp32, or fp16 GEMMs for speed on
    integer-valued data where fp16 products are exact enough to rank)."""
    dev = queries.device
    qf = to_float(queries)
    if metric == "cosine":
        qf = torch.nn.functional.normalize(qf, dim=1)
    nq = qf.shape[0]
    # a chunk's score matrix (and the copies topk makes of it) stays within 4 GiB
    row_chunk = max(4096, min(row_chunk, (1 << 30) // max(nq, 1)))
    best_d = torch.full((nq, k), float("inf"), device=dev)
    best_i = torch.full((nq, k), -1, dtype=torch.int64, device=dev)
    for s in range(0, dataset.shape[0], row_chunk):
        xs = to_float(dataset[s:s + row_chunk])
        if metric == "cosine":
            xs = torch.nn.functional.normalize(xs, dim=1)
        if half:
            ip = (qf.half() @ xs.half().t()).float()
        else:
            ip = qf @ xs.t()
        if metric in ("sqeuclidean", "euclidean"):
            d = (xs ** 2).sum(1)[None, :] - 2.0 * ip
        else:
            d = -ip
        kk = min(k, d.shape[1])
        dd, ii = torch.topk(d, kk, dim=1, largest=False)
        cat_d = torch.cat([best_d, dd], 1)
        cat_i = torch.cat([best_i, ii + s], 1)
        sel = torch.topk(cat_d, k, dim=1, largest=False)[1]
        best_d = torch.gather(cat_d, 1, sel)
        best_i = torch.gather(cat_i, 1, sel)
    return best_i


def recall(found, truth):
    """sum_q |found_q ∩ truth_q| / (Q * k)  (cuVS bench: benchmark.hpp:355-419)."""
    found = np.asarray(found)
    truth = np.asarray(truth)
    hits = 0
    for f, t in zip(found, truth):
        hits += len(set(f.tolist()) & set(t.tolist()))
    return hits / float(truth.shape[0] * truth.shape[1])
