"""Helpers for the GPU parity tests: build an index through the C ABI, read it back for the oracle."""
import numpy as np
import torch

import helpers as H
from cuvs_amd import ivf_pq


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def build_gpu_index(model, data, pq_dim, pq_bits, metric="sqeuclidean", codebook_kind="subspace",
                    ids=None, labels=None, batches=1):
    params = ivf_pq.IndexParams(n_lists=model["centers"].shape[0], metric=metric, pq_bits=pq_bits,
                                pq_dim=pq_dim, codebook_kind=codebook_kind)
    dev = {k: to_dev(v) for k, v in model.items()}
    index = ivf_pq.build_precomputed(params, data.shape[1], dev["pq_centers"], dev["centers"],
                                     dev["centers_rot"], dev["rotation_matrix"])
    n = data.shape[0]
    bounds = np.linspace(0, n, batches + 1).astype(int)
    for b in range(batches):
        s, e = bounds[b], bounds[b + 1]
        if e == s:
            continue
        ivf_pq.extend(index, to_dev(data[s:e]), to_dev(ids[s:e]) if ids is not None else None,
                      labels=to_dev(labels[s:e].astype(np.int32)) if labels is not None else None)
    return index


def unpack_bits(flat, pq_dim, pq_bits):
    """bit-contiguous rows -> one code per byte"""
    n = flat.shape[0]
    out = np.zeros((n, pq_dim), dtype=np.uint8)
    wide = flat.astype(np.uint32)
    wide = np.concatenate([wide, np.zeros((n, 2), dtype=np.uint32)], axis=1)
    for j in range(pq_dim):
        bit = j * pq_bits
        pair = wide[:, bit // 8] | (wide[:, bit // 8 + 1] << 8)
        out[:, j] = (pair >> (bit % 8)) & ((1 << pq_bits) - 1)
    return out


def read_back(orc, index, model, dim, pq_dim, pq_bits, metric="sqeuclidean", codebook_kind="subspace"):
    """Oracle index holding exactly what the GPU index holds (sizes, ids, codes, in list order)."""
    sizes = index.list_sizes.cpu().numpy().astype(np.uint32)
    datas, inds, all_codes = [], [], []
    for l in range(len(sizes)):
        if sizes[l] == 0:
            datas.append(np.zeros(0, dtype=np.uint8))
            inds.append(np.zeros(0, dtype=np.int64))
            all_codes.append(np.zeros((0, pq_dim), dtype=np.uint8))
            continue
        flat = index.list_data(l).cpu().numpy()
        codes = unpack_bits(flat, pq_dim, pq_bits)
        # the device-side bit-contiguous unpacking agrees with the oracle's on the same bytes
        packed = orc.pack_list(codes, pq_bits)
        assert np.array_equal(orc.unpack_list_contiguous(packed, int(sizes[l]), pq_dim, pq_bits), flat)
        datas.append(packed)
        inds.append(index.list_indices(l).cpu().numpy())
        all_codes.append(codes)
    ix = H.oracle_index(orc, model, dim, pq_dim, pq_bits, metric, codebook_kind)
    ix.set_lists(sizes, datas, inds)
    return ix, all_codes


def read_back_bulk(orc, index, host_model, dim, pq_dim, pq_bits, metric="sqeuclidean", codebook_kind="subspace"):
    """read_back for large indexes: no per-list cross-checks, 8-bit codes taken as they come out of
    the unpack entry point (one byte per code already)."""
    sizes = index.list_sizes.cpu().numpy().astype(np.uint32)
    datas, inds = [], []
    for l in range(len(sizes)):
        if sizes[l] == 0:
            datas.append(np.zeros(0, dtype=np.uint8))
            inds.append(np.zeros(0, dtype=np.int64))
            continue
        flat = index.list_data(l, n_rows=int(sizes[l])).cpu().numpy()
        codes = flat if pq_bits == 8 else unpack_bits(flat, pq_dim, pq_bits)
        datas.append(orc.pack_list(codes, pq_bits))
        inds.append(index.list_indices(l).cpu().numpy())
    ix = H.oracle_index(orc, host_model, dim, pq_dim, pq_bits, metric, codebook_kind)
    ix.set_lists(sizes, datas, inds)
    return ix
