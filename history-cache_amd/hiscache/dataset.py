"""ProcessedDataset: the on-disk layout the reference reads, ``<path>/processed/*``.

Files and element types (raw little-endian arrays, no headers):
``num_nodes.txt`` (decimal text; /root/reference/hiscache/history_cache.py:17-20),
``sorted_indices.dat`` (int64 node ids, hottest last; history_cache.py:124-134),
``node_features.dat`` ([num_nodes, feature_dim] float32, float16 for mag240m;
history_cache.py:141-149), ``csr_ptr_undirected.dat`` / ``csr_idx_undirected.dat`` (int64 CSR;
/root/reference/test/test_cache.py:19-25,43-49), ``split/time/train_idx.dat`` (int64;
test/test_cache.py:54-56) and, beside it, ``valid_idx.dat`` / ``test_idx.dat`` for the trainer's evaluation.  ``node_labels.dat`` (int64) is this package's name for the labels,
which the reference takes from its external loader.
"""
import os
from os import path

import numpy as np
import torch

from .feature_store import PinnedFeatureStore
from .sampler import NeighborSampler

_FILES = {
    "ptr": ("csr_ptr_undirected.dat", np.int64),
    "idx": ("csr_idx_undirected.dat", np.int64),
    "hot": ("sorted_indices.dat", np.int64),
    "labels": ("node_labels.dat", np.int64),
    "train": (path.join("split", "time", "train_idx.dat"), np.int64),
    "valid": (path.join("split", "time", "valid_idx.dat"), np.int64),
    "test": (path.join("split", "time", "test_idx.dat"), np.int64),
}


class ProcessedDataset:

    def __init__(self, root, feature_dim, feature_dtype=np.float32):
        self.dir = path.join(str(root), "processed")
        self.feature_dim = int(feature_dim)
        self.feature_dtype = np.dtype(feature_dtype)
        with open(path.join(self.dir, "num_nodes.txt")) as f:
            self.num_nodes = int(f.readline())

    def _array(self, key, mmap=False):
        name, dtype = _FILES[key]
        p = path.join(self.dir, name)
        if not path.exists(p):
            raise FileNotFoundError(p)
        return np.memmap(p, dtype=dtype, mode="r") if mmap else np.fromfile(p, dtype=dtype)

    def has(self, key):
        return path.exists(path.join(self.dir, _FILES[key][0]))

    def graph(self):
        """(indptr, indices) as NumPy int64; indptr must have num_nodes + 1 entries."""
        indptr, indices = self._array("ptr"), self._array("idx")
        if indptr.shape[0] != self.num_nodes + 1 or int(indptr[-1]) != indices.shape[0]:
            raise ValueError("CSR files do not match num_nodes.txt")
        return indptr, indices

    def hot_ids(self):
        return self._array("hot")

    def labels(self):
        return self._array("labels")

    def train_idx(self):
        return self._array("train")

    def split_idx(self, split):
        """Node ids of a split: "train", "valid" or "test" (``split/time/<split>_idx.dat``)."""
        if split not in ("train", "valid", "test"):
            raise KeyError(split)
        return self._array(split)

    def feature_store(self, device="cuda:0", out_dtype=None, chunk_rows=1 << 20, in_device_memory=False,
                      hot_rows=0, prefetch_cus=0):
        """Pinned, GPU-mapped copy of ``node_features.dat``, read from disk in chunks (the file is
        never held twice in memory).  ``in_device_memory``: the matrix goes to the GPU's own memory
        instead (288 GB hold the papers100M matrix, 57 GB, beside its history table), and the store's
        gathers read it there.  ``hot_rows``: for a matrix that stays in host memory, copies of that many
        rows, the last (hottest) entries of ``sorted_indices.dat``, are kept in device memory and served from
        there (the reference's feature cache, history_cache.py:124-142).  ``prefetch_cus``: see
        ``PinnedFeatureStore`` (the stream of the read-ahead is kept to that many compute units)."""
        p = path.join(self.dir, "node_features.dat")
        want = self.num_nodes * self.feature_dim * self.feature_dtype.itemsize
        if os.path.getsize(p) != want:
            raise ValueError(f"{p}: {os.path.getsize(p)} bytes, expected {want}")
        src = np.memmap(p, dtype=self.feature_dtype, mode="r", shape=(self.num_nodes, self.feature_dim))
        tdtype = {np.dtype(np.float32): torch.float32, np.dtype(np.float16): torch.float16}[self.feature_dtype]
        if in_device_memory:
            buf = torch.empty((self.num_nodes, self.feature_dim), dtype=tdtype, device=device)
            for lo in range(0, self.num_nodes, chunk_rows):
                hi = min(self.num_nodes, lo + chunk_rows)
                buf[lo:hi].copy_(torch.from_numpy(np.array(src[lo:hi])))       # a writable copy of the chunk
        else:
            buf = torch.empty((self.num_nodes, self.feature_dim), dtype=tdtype, pin_memory=True)
            dst = buf.numpy()
            for lo in range(0, self.num_nodes, chunk_rows):
                hi = min(self.num_nodes, lo + chunk_rows)
                dst[lo:hi] = src[lo:hi]
        del src
        store = PinnedFeatureStore(buf, device=device, out_dtype=out_dtype or torch.float32, prefetch_cus=prefetch_cus)
        if hot_rows and not in_device_memory:
            order = self.hot_ids()
            store.set_hot_rows(torch.from_numpy(np.array(order[max(0, len(order) - int(hot_rows)):])))
        return store

    def sampler(self, fanout, device="cuda:0", seed=0, emit_view=False, view_edges=False, replay_slots=0):
        """``emit_view``: every batch carries the transposed view of its CSR (``batch.view``), so that the
        layers' backward builds none; ``view_edges`` adds the edge slots the relational layer reads;
        ``replay_slots``: see ``NeighborSampler`` (one HIP-graph launch per batch; a batch's arrays are
        overwritten that many batches later)."""
        indptr, indices = self.graph()
        labels = self.labels() if self.has("labels") else None
        return NeighborSampler(indptr, indices, fanout, labels=labels, seed=seed, device=device,
                               emit_view=emit_view, view_edges=view_edges, replay_slots=replay_slots)


def write_processed(root, indptr, indices, features, hot_ids=None, labels=None, train_idx=None, valid_idx=None,
                    test_idx=None):
    """Write a dataset in the layout above (for tests and for converting in-memory graphs)."""
    d = path.join(str(root), "processed")
    os.makedirs(path.join(d, "split", "time"), exist_ok=True)
    n = len(indptr) - 1
    with open(path.join(d, "num_nodes.txt"), "w") as f:
        f.write(f"{n}\n")
    np.ascontiguousarray(indptr, dtype=np.int64).tofile(path.join(d, _FILES["ptr"][0]))
    np.ascontiguousarray(indices, dtype=np.int64).tofile(path.join(d, _FILES["idx"][0]))
    feats = np.ascontiguousarray(features)
    if feats.shape[0] != n:
        raise ValueError("features must have one row per node")
    feats.tofile(path.join(d, "node_features.dat"))
    for key, arr in (("hot", hot_ids), ("labels", labels), ("train", train_idx), ("valid", valid_idx),
                     ("test", test_idx)):
        if arr is not None:
            np.ascontiguousarray(arr, dtype=np.int64).tofile(path.join(d, _FILES[key][0]))
    return d
