"""Train a model through the history cache from a YAML configuration.

The role of /root/reference/example/main.py:13-29 (hydra reads the loader package's configuration, then
``HistoryTrainer(config).train()``), without hydra: ``config.yaml`` beside this file holds the keys that are read,
and ``a.b.c=value`` arguments override them the way hydra's command line does.

    python main.py                                     # config.yaml as it is
    python main.py --synthetic 200000                  # write a random dataset of that many nodes first
    python main.py history.rate=0.8 trainer.recorded=true dl.dataset.path=/data/arxiv
"""
import argparse
import logging
import os
import sys

import numpy as np
import yaml

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

import hiscache  # noqa: E402

log = logging.getLogger("hiscache.example")


def load_config(path, overrides=()):
    """The configuration tree of ``path`` with the ``dotted.key=value`` overrides applied (values in YAML
    spelling: ``true``, ``0.5``, ``[15,10]``).  A key that the file does not hold is added."""
    with open(path) as f:
        tree = yaml.safe_load(f) or {}
    for item in overrides:
        key, eq, value = item.partition("=")
        if not eq or not key:
            raise ValueError(f"override '{item}': expected dotted.key=value")
        node = tree
        parts = key.split(".")
        for part in parts[:-1]:
            nxt = node.setdefault(part, {})
            if not isinstance(nxt, dict):
                raise ValueError(f"override '{item}': '{part}' is not a group")
            node = nxt
        node[parts[-1]] = yaml.safe_load(value)
    return hiscache.Config(tree)


def plain(node):
    """The tree as plain dicts (for printing)."""
    return {k: plain(v) for k, v in node.items()} if isinstance(node, dict) else node


def trainer_options(config):
    """The ``trainer`` group as ``HistoryTrainer`` arguments."""
    t = config.get("trainer") or {}
    mb = float(t.get("cache_megabytes", 0) or 0)
    return dict(recorded=bool(t.get("recorded", False)), read_ahead=bool(t.get("read_ahead", False)),
                features_in_device_memory=bool(t.get("features_in_device_memory", False)),
                hot_rows=int(t.get("hot_rows", 0) or 0), ring_rows=int(t.get("ring_rows", 0) or 0),
                cache_bytes=int(mb * 2 ** 20) if mb > 0 else None, seed=int(t.get("seed", 0) or 0))


def write_synthetic(config, num_nodes, degree=12, seed=0):
    """A random graph with features whose leading columns decide the label, hottest nodes by degree, written to
    ``dl.dataset.path`` in the processed layout."""
    rng = np.random.default_rng(seed)
    n, f, c = int(num_nodes), int(config.dl.dataset.feature_dim), int(config.dl.dataset.num_classes)
    if c > f:
        raise ValueError("the synthetic labels need num_classes <= feature_dim")
    indptr = np.arange(0, (n + 1) * degree, degree, dtype=np.int64)
    # (a skewed choice of neighbours, so that a hotness order means something)
    indices = np.minimum((rng.random(n * degree) ** 2 * n).astype(np.int64), n - 1)
    feats = rng.standard_normal((n, f)).astype(np.float32)
    labels = feats[:, :c].argmax(1).astype(np.int64)
    order = hiscache.hotness.hotness_order(np.bincount(indices, minlength=n))
    perm = rng.permutation(n)
    a, b = n * 6 // 10, n * 8 // 10
    return hiscache.write_processed(config.dl.dataset.path, indptr, indices, feats, hot_ids=order.numpy(),
                                    labels=labels, train_idx=perm[:a], valid_idx=perm[a:b], test_idx=perm[b:])


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--config", default=os.path.join(os.path.dirname(os.path.abspath(__file__)), "config.yaml"))
    ap.add_argument("--synthetic", type=int, default=0, metavar="NODES",
                    help="write a random dataset of this many nodes to dl.dataset.path before training")
    ap.add_argument("overrides", nargs="*", help="dotted.key=value")
    args = ap.parse_args(argv)
    logging.basicConfig(level=logging.INFO, format="%(message)s")
    config = load_config(args.config, args.overrides)
    log.info(yaml.safe_dump(plain(config), sort_keys=False))
    if int(config.dl.num_device) > 1:
        # (/root/reference/example/main.py:24-26 hands this case to its multi-device trainer)
        raise SystemExit("dl.num_device > 1: this build runs one process on one device")
    if args.synthetic:
        log.info("dataset written to %s", write_synthetic(config, args.synthetic))
    trainer = hiscache.HistoryTrainer(config, **trainer_options(config))
    try:
        trainer.train()
    finally:
        trainer.close()
    log.info("validation metric per evaluated epoch %s, test metric %s, best validation metric %.4f",
             [round(m, 4) for m in trainer.val_metrics], [round(m, 4) for m in trainer.test_metrics],
             trainer.best_metric)
    return trainer


if __name__ == "__main__":
    main()
