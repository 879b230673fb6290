"""HistoryTrainer: the loop around the path -- sample, ``lookup_and_load``, forward, loss, backward, optimizer,
``update_history`` -- with the method names and attributes of the reference's trainer
(/root/reference/hiscache/history_trainer.py:15-255: ``cxg_train_epoch`` :176-193, ``cxg_eval_epoch`` :195-227,
``train`` :229-255, ``cxg_just_load`` :144-174, ``batch_to_file`` :134-141).

The reference takes its loader, its UVM store, optimizer, scheduler, loss and evaluator from two external packages
(``cxgnndl.get_loader`` / ``cxgnndl.UVM``, ``cxgnncomp.get_optimizer`` ...).  Here they come from the dataset
directory the configuration names (``ProcessedDataset``: graph, features, splits, hotness order), the device
sampler (one batch ahead on its side stream, every batch with the transposed view of its CSR) and torch (Adam,
NLL on the log-softmax the models return, accuracy).  What the hardware adds is opt-in: the feature matrix in
device memory or its hottest rows there, and the iteration recorded per padded batch shape and replayed
(``RecordedIteration``).
"""
import time

import numpy as np
import torch

from .dataset import ProcessedDataset
from .history_cache import HistoryCache
from .history_model import HistoryRGCN, get_model
from .recorded import RecordedIteration
from .ring_cache import RingHistoryCache
from .util import backward_on_this_thread, log


def _option(config, dotted, default):
    node = config
    for key in dotted.split("."):
        if not hasattr(node, "get") or node.get(key) is None:
            return default
        node = node[key]
    return node


class HistoryTrainer:

    def __init__(self, config, dataset=None, fanout=None, batch_size=None, lr=None, num_epochs=None, eval_begin=None,
                 features_in_device_memory=False, hot_rows=0, cache_bytes=None, ring_rows=0, recorded=False,
                 read_ahead=False, replay_slots=4, seed=0, model_factory=None):
        """``config``: the tree ``make_config`` builds (``dl.dataset.path`` names the dataset directory).  The
        loader's settings are arguments, with the configuration's own keys as defaults where it has them
        (``dl.sampler.train.batch_size`` / ``num_neighbors``, ``train.optimizer.lr``, ``train.train.num_epochs`` /
        ``eval_begin``).  ``cache_bytes``: size of the cache's buffer (default: what the configuration's
        ``history.limit`` and the free device memory give, as in the reference).  ``ring_rows`` > 0: the embeddings live in a
        ``RingHistoryCache`` of that many fp16 rows instead (entries age out after ``history.staleness_thres``
        iterations; no feature cache inside it: use ``hot_rows``).  ``recorded``: train through
        ``RecordedIteration`` (batches of ``batch_size`` seeds; the last, shorter batch of an epoch takes the
        ordinary path).  ``read_ahead``: the feature rows of the next batch are read over the host link beside
        the current iteration (on a stream kept to 16 compute units; the epoch then runs on a stream of its
        own), for a matrix that is not wholly in device memory.  ``replay_slots``: the sampler's launches for a
        batch are recorded once per slot and replayed (see ``NeighborSampler``; the trainer never holds more than
        three batches, so four slots are safe; 0 switches it off).  ``model_factory(config, table)``: builds
        the model instead of ``get_model`` (a relational model with its own node-type ranges, say)."""
        self.config = config
        self.device = torch.device(config.dl.device)
        self.feat_mode = config.dl.loading.feat_mode
        self.recorded = bool(recorded)
        if self.recorded and (config.history.method != "grad" or "history" not in self.feat_mode):
            raise ValueError("recorded iterations need the embedding cache with admission by gradient "
                             "(history.method = 'grad', a history_* feat_mode)")
        self.num_layers = int(config.train.model.num_layers)
        self.batch_size = int(batch_size or _option(config, "dl.sampler.train.batch_size", 1000))
        fanout = fanout or _option(config, "dl.sampler.train.num_neighbors", None)
        if fanout is None or len(fanout) != self.num_layers:
            raise ValueError("fanout: one neighbour count per layer")
        self.num_epochs = int(num_epochs if num_epochs is not None else _option(config, "train.train.num_epochs", 1))
        self.eval_begin = int(eval_begin if eval_begin is not None else _option(config, "train.train.eval_begin", 0))
        self.dataset = dataset or ProcessedDataset(config.dl.dataset.path, config.dl.dataset.feature_dim)
        ds = self.dataset
        # the feature store (cxgnndl.UVM's role): pinned host memory read zero-copy, the hottest rows or the whole
        # matrix in device memory on request
        self.read_ahead = bool(read_ahead) and not features_in_device_memory
        # (a matrix stored in fp16 -- the reference loads mag240M's that way, history_cache.py:148-149 -- stays fp16
        # on its way into the first layer: half the bytes over the link)
        self.uvm = ds.feature_store(device=self.device, in_device_memory=features_in_device_memory,
                                    hot_rows=hot_rows, prefetch_cus=16 if self.read_ahead else 0,
                                    out_dtype=torch.float16 if ds.feature_dtype == np.float16 else None)
        self._compute = None
        if ring_rows:
            self.table = RingHistoryCache(self.uvm, ds.num_nodes, config.dl.dataset.feature_dim,
                                          config.train.model.hidden_dim, capacity=int(ring_rows),
                                          num_layers=self.num_layers, table_dtype=torch.float16,
                                          rate=float(config.history.rate), method=config.history.method,
                                          age_limit=int(config.history.staleness_thres), device=self.device)
        else:
            self.table = HistoryCache(uvm=self.uvm, config=config, mode=self.feat_mode, buffer_bytes=cache_bytes)
        self.model = (model_factory or get_model)(config, self.table).to(self.device)
        self.optimizer = torch.optim.Adam(self.model.parameters(),
                                          lr=float(lr or _option(config, "train.optimizer.lr", 1e-3)), fused=True,
                                          capturable=self.recorded)
        self.scheduler = None
        self.loss_fn = torch.nn.functional.nll_loss
        # every batch comes with the transposed view of its CSR; the relational layer also reads the view's edge slots
        if 0 < replay_slots < (3 if self.read_ahead else 2):
            raise ValueError("replay_slots: at least as many as batches are alive at once (2, with the read-ahead 3)")
        self.sampler = ds.sampler(list(fanout), device=self.device, seed=seed, emit_view=True,
                                  view_edges=isinstance(self.model, HistoryRGCN), replay_slots=replay_slots)
        if self.read_ahead:
            # the stream the epoch runs on beside the read-ahead: of a few, the one that the reads slow down least,
            # and on another hardware queue than the sampler's
            pick = getattr(self.uvm, "quiet_stream", None)
            self._compute = (pick(apart_from=[self.sampler.stream()]) if pick is not None
                             else torch.cuda.Stream(device=self.device))                     # default priority
        self.splits = {"train": torch.from_numpy(np.array(ds.train_idx())).to(self.device)}
        for split, key in (("val", "valid"), ("test", "test")):
            if ds.has(key):
                self.splits[split] = torch.from_numpy(np.array(ds.split_idx(key))).to(self.device)
        self._generator = torch.Generator(device=self.device).manual_seed(seed)
        self._step = RecordedIteration(self.model, self.table, self.optimizer, self.num_layers,
                                       loss_fn=self.loss_fn) if self.recorded else None
        self.glb_iter = 0
        self.prof = bool(_option(config, "dl.performance.prof", False))     # train() then runs the profiled epoch
        self.times = None
        self.val_metrics = []
        self.test_metrics = []
        self.best_metric = 0
        self.metric = None
        self.epoch_seconds = []

    def state_dict(self):
        """Model, optimizer, cache contents and the counters, for a checkpoint (the reference's trainer saves
        none): ``torch.save(trainer.state_dict(), path)``."""
        return {"model": self.model.state_dict(), "optimizer": self.optimizer.state_dict(),
                "table": self.table.state_dict(), "glb_iter": self.glb_iter, "best_metric": self.best_metric,
                "val_metrics": list(self.val_metrics), "test_metrics": list(self.test_metrics),
                "generator": self._generator.get_state(), "sampler_batches": self.sampler.batches}

    def load_state_dict(self, state):
        """Resume from ``state_dict``'s result in a trainer built the same way (recordings are made again on
        demand; the sampler continues its sequence of batch keys)."""
        self.model.load_state_dict(state["model"])
        self.optimizer.load_state_dict(state["optimizer"])
        self.table.load_state_dict(state["table"])
        self.glb_iter = int(state["glb_iter"])
        self.best_metric = state["best_metric"]
        self.val_metrics, self.test_metrics = list(state["val_metrics"]), list(state["test_metrics"])
        self._generator.set_state(state["generator"].cpu())
        self.sampler.batches = int(state["sampler_batches"])
        if self._step is not None:
            self._step.clear()

    def close(self):
        """Give the read-ahead stream back (it is made again on demand)."""
        close = getattr(self.uvm, "close", None)
        if close is not None:
            close()

    # ------------------------------------------------------------------ batches
    def _batches(self, ids, shuffle, read_ahead=False):
        """Batches of ``ids``, every one sampled on the sampler's side stream while the one before is in use;
        with ``read_ahead`` a batch is handed out once the next one is drawn and its feature read is under way."""
        if shuffle:
            ids = ids[torch.randperm(ids.numel(), device=self.device, generator=self._generator)]
        chunks = [ids[lo:lo + self.batch_size].contiguous() for lo in range(0, ids.numel(), self.batch_size)]
        if not chunks:
            return
        chunks.append(None)
        pending = self.sampler.sample_async(chunks[0])
        if not read_ahead:
            for nxt in chunks[1:]:
                batch = pending.get()
                pending = self.sampler.sample_async(nxt) if nxt is not None else None
                yield batch
            return
        batch = pending.get()
        pending = self.sampler.sample_async(chunks[1]) if chunks[1] is not None else None
        for k in range(1, len(chunks)):
            nxt = None
            if pending is not None:
                nxt = pending.get()
                pending = self.sampler.sample_async(chunks[k + 1]) if chunks[k + 1] is not None else None
                if self._step is not None:
                    self._step.prefetch(nxt)        # straight into the array the batch's recording reads
                else:
                    self.table.prefetch(nxt, speculative=True, num_layer=self.num_layers)
            yield batch
            batch = nxt

    @staticmethod
    def evaluator(y_pred, y_true):
        """Accuracy of the arg-max class (the evaluator of the node-classification datasets)."""
        return (y_pred.argmax(dim=-1) == y_true).float().mean()

    # ------------------------------------------------------------------ epochs
    def cxg_train_epoch(self):
        if self._compute is None:
            return self._train_epoch()
        # the read-ahead runs beside the iteration only when the iteration is on a stream of its own
        self._compute.wait_stream(torch.cuda.current_stream(self.device))
        with torch.cuda.stream(self._compute):
            self._train_epoch()
        torch.cuda.current_stream(self.device).wait_stream(self._compute)

    def _train_epoch(self):
        self.model.train()
        tepoch = time.time()
        num_layers = len(self.model.convs)
        for batch in self._batches(self.splits["train"], shuffle=True, read_ahead=self.read_ahead):
            if self._step is not None:
                self._step(batch, self.glb_iter)
            else:
                self.optimizer.zero_grad(set_to_none=True)
                self.table.lookup_and_load(batch, num_layers)
                out = self.model(batch)
                loss = self.loss_fn(out, batch.y)
                backward_on_this_thread(loss)
                self.optimizer.step()
                self.table.update_history(batch, self.glb_iter)
            if self.scheduler is not None:
                self.scheduler.step()
            self.glb_iter += 1
        torch.cuda.synchronize(self.device)
        self.epoch_seconds.append(time.time() - tepoch)
        log.info(f"epoch time: {self.epoch_seconds[-1]}")

    def cxg_train_epoch_prof(self):
        """The ordinary epoch with the time of every phase summed over the epoch, as the reference's profiled
        epoch reports it (/root/reference/hiscache/history_trainer.py:77-132: load, forward, loss, backward, step,
        update, sample).  The phases are bracketed by events on the stream instead of host synchronisations, so the
        loop runs as it does unprofiled; ``sample`` is the time the host waited for the sampler.  The sums (seconds)
        are kept in ``self.times`` and logged."""
        self.model.train()
        tepoch = time.time()
        num_layers = len(self.model.convs)
        names = ("load", "forward", "loss", "backward", "step", "update")
        marks = []                                           # per iteration: 7 events around the 6 phases
        cur = torch.cuda.current_stream(self.device)
        waited = 0.0

        def mark(row):
            ev = torch.cuda.Event(enable_timing=True)
            ev.record(cur)
            row.append(ev)

        batches = self._batches(self.splits["train"], shuffle=True)
        while True:
            t0 = time.time()
            batch = next(batches, None)                      # (waits for the sampler's read-back)
            waited += time.time() - t0
            if batch is None:
                break
            row = []
            self.optimizer.zero_grad(set_to_none=True)
            mark(row)
            self.table.lookup_and_load(batch, num_layers)
            mark(row)
            out = self.model(batch)
            mark(row)
            loss = self.loss_fn(out, batch.y)
            mark(row)
            backward_on_this_thread(loss)
            mark(row)
            self.optimizer.step()
            if self.scheduler is not None:
                self.scheduler.step()
            mark(row)
            self.table.update_history(batch, self.glb_iter)
            mark(row)
            marks.append(row)
            self.glb_iter += 1
        torch.cuda.synchronize(self.device)
        self.epoch_seconds.append(time.time() - tepoch)
        self.times = {name: 1e-3 * sum(row[i].elapsed_time(row[i + 1]) for row in marks)
                      for i, name in enumerate(names)}
        self.times["sample"] = waited
        log.info(f"epoch time: {self.epoch_seconds[-1]}")
        log.info(", ".join(f"{k}-time: {v}" for k, v in self.times.items())
                 + f" total-time: {sum(self.times.values())}")

    @torch.no_grad()
    def cxg_just_load(self, num_epochs=3, rate=0.9, staleness=200, score_fn=None):
        """The hit rate of historical embeddings without a model (/root/reference/hiscache/history_trainer.py:144-174):
        over ``num_epochs`` epochs of sampled batches, the share of every batch's layer-1 nodes that a store
        admitting the uncached nodes under the ``rate`` quantile of random scores, and holding an admission for
        ``staleness`` batches, would already hold.  Returns one (hit rate, nodes held) per batch and advances
        ``glb_iter`` as the reference does (which prints them and then leaves the process)."""
        is_cached = torch.zeros(self.table.total_num_node, dtype=torch.int32, device=self.device)
        admitted, out = [], []
        for _ in range(int(num_epochs)):
            for batch in self._batches(self.splits["train"], shuffle=True):
                nodes = batch.sub_to_full[: int(batch.num_node_in_layer[1])]
                held = is_cached[nodes] > 0
                out.append((float(held.sum()) / max(nodes.numel(), 1), int((is_cached > 0).sum())))
                log.info(f"history hitrate {out[-1][0]} {out[-1][1]}")
                rand = score_fn(nodes.numel()) if score_fn is not None else torch.randn(
                    nodes.numel(), device=self.device, generator=self._generator)
                check_in = nodes[(rand < torch.quantile(rand, rate)) & ~held]
                admitted.append(check_in)
                if len(admitted) > staleness:
                    is_cached[admitted.pop(0)] -= 1
                is_cached[check_in] += 1
                self.glb_iter += 1
        return out

    @staticmethod
    def batch_to_file(batch, filename):
        """The batch's CSR and layer sizes as a ``torch.save`` file (history_trainer.py:134-141, without leaving
        the process)."""
        torch.save({"ptr": batch.ptr.cpu(), "idx": batch.idx.cpu(),
                    "num_node_in_layer": torch.as_tensor(batch.num_node_in_layer).cpu()}, filename)

    def cxg_eval_epoch(self, split="val"):
        self.model.eval()
        y_preds, y_trues, losses = [], [], []
        tepoch = time.time()
        num_layers = len(self.model.convs)
        for batch in self._batches(self.splits[split], shuffle=False):
            self.table.lookup_and_load(batch, num_layers, feature_cache_only=True)
            out = self.model(batch)
            losses.append(self.loss_fn(out, batch.y).detach())
            y_preds.append(out.detach())
            y_trues.append(batch.y.detach().clone())
        torch.cuda.synchronize(self.device)
        if not y_preds:
            log.info(f"{split}: no nodes")
            return
        self.metric = self.evaluator(torch.cat(y_preds, dim=0), torch.cat(y_trues, dim=0)).item()
        log.info(f"epoch time: {time.time() - tepoch}")
        log.info(f"{split}-metric: {self.metric}")
        if split == "val":
            self.best_metric = max(self.best_metric, self.metric)
            log.info(f"best-metric: {self.best_metric}")
            self.val_metrics.append(self.metric)
        else:
            self.test_metrics.append(self.metric)

    def train(self):
        for epoch in range(self.num_epochs):
            log.info(f"Epoch {epoch}/{self.num_epochs}")
            if self.prof:
                self.cxg_train_epoch_prof()
            else:
                self.cxg_train_epoch()
            if epoch >= self.eval_begin:
                if "val" in self.splits:
                    self.cxg_eval_epoch(split="val")
                if "test" in self.splits and "mag" not in str(self.config.dl.dataset.name).lower():
                    self.cxg_eval_epoch(split="test")
        if len(self.val_metrics) > 0:
            val, test = np.array(self.val_metrics), np.array(self.test_metrics)
            log.info(f"best-val-metrics: {val.max()} at epoch {val.argmax()}")
            if len(test) == len(val):
                log.info(f"best-test-metrics: {test.max()} valided test-metric {test[val.argmax()]}")
