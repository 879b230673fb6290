"""HisCache for MI355X: the package a user of the reference's ``hiscache`` imports.

Exports follow /root/reference/hiscache/__init__.py:1-6 for the single-GPU hot path, plus
``HistoryCache`` (which the reference README imports from the package but its ``__init__`` omits).
``HistoryTrainer`` is the single-GPU loop around the path; the multi-GPU trainer and the communication helpers are not
part of this package.
"""
from hiscache_backend import count_history_reconstruct, get_graph_structure_score, record_history

from .dataset import ProcessedDataset, write_processed
from .feature_store import PinnedFeatureStore
from .history_cache import HistoryCache
from .history_model import (HistoryRGCN, HistorySAGE, MyRGCNConvHistory2, MySageConvHistory, get_model,
                            prefer_low_latency_gemm, typed_csr)
from .history_table import HistoryTable
from .history_trainer import HistoryTrainer
from . import hotness
from .recorded import RecordedIteration
from .ring_cache import RingHistoryCache
from .sampler import NeighborSampler
from .util import Config, backward_on_this_thread, make_config, quantile_threshold

__all__ = [
    "HistoryCache", "HistoryTable", "HistoryTrainer", "hotness", "RingHistoryCache", "RecordedIteration", "HistorySAGE", "HistoryRGCN", "MySageConvHistory", "MyRGCNConvHistory2", "typed_csr", "get_model", "prefer_low_latency_gemm",
    "PinnedFeatureStore", "NeighborSampler", "ProcessedDataset", "write_processed", "Config", "make_config", "quantile_threshold", "backward_on_this_thread",
    "count_history_reconstruct", "get_graph_structure_score", "record_history",
]
