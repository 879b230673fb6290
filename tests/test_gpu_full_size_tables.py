"""The ring cache at the table sizes of the papers100M- and mag240M-shaped configurations: 111 059 956
and 244 160 499 nodes with one 256-wide fp16 row per node (57 and 125 GB of table, byte offsets beyond
2^32 and, for the larger one, beyond 2^36; node ids and slots up to the last one).  Batches have the
configurations' shape (1000 seeds, fanout [15, 10, 5] and [25, 15], ids uniform over all nodes).  The ring's
write position starts 700 slots before the end of the table, so that the first admission runs over the
end and goes on at slot 0, where it evicts entries that were put there beforehand; the first batch comes
back at the end and finds the rows that were admitted then.

The CPU statement runs on arrays of the same size: its three maps are ordinary arrays (2 GB each at the
larger size), its table is a sparse file of the table's size mapped into memory, of which only the rows
that the batches touch are ever written.  Lookups, masks, admitted rows, the three maps in full, the write
position and every table row of a live slot that the statement wrote or read are compared exactly; the
number of non-zero table rows on the device is compared with the statement's count, so that nothing was
written anywhere else."""
import os
import tempfile

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

SIZES = {
    "papers100M": dict(nodes=111_059_956, fanout=[15, 10, 5], layers=3, degree_scale=2.6),
    "mag240M": dict(nodes=244_160_499, fanout=[25, 15], layers=2, degree_scale=1.25),
}
H, FIN, POOL = 256, 32, 1 << 20


def folded_store(feats, device):
    """A feature store over a pool of rows that stands for a matrix of one row per node (which no host here
    holds): ids are folded into the pool.  Test plumbing; the rows that come back are compared below."""
    from hiscache import PinnedFeatureStore

    class Folded(PinnedFeatureStore):
        def masked_get(self, ids, mask):
            return super().masked_get(ids % POOL, mask)

    return Folded(feats, device=device)


def nonzero_rows(table, chunk=1 << 22):
    n = 0
    for lo in range(0, table.shape[0], chunk):
        n += int((table[lo:lo + chunk].view(torch.int16) != 0).any(dim=1).sum().item())
    return n


@pytest.mark.parametrize("name", list(SIZES))
def test_ring_cache_at_the_full_table_size(orc, name):
    from hiscache import RingHistoryCache
    from hiscache.synthetic import direct_power_law_batch, make_batch
    from oracle import host_model
    cfg = SIZES[name]
    N, fanout, L = cfg["nodes"], cfg["fanout"], cfg["layers"]
    need = N * (H * 2 + 3 * 8) + (8 << 30)
    free, _ = torch.cuda.mem_get_info()
    if free < need:
        pytest.skip("needs %.0f GB of device memory, %.0f GB are free" % (need / 1e9, free / 1e9))
    rng = np.random.default_rng(111)
    gen = torch.Generator(device=DEV).manual_seed(111)
    feats = torch.from_numpy(rng.standard_normal((POOL, FIN), dtype=np.float32))
    cache = RingHistoryCache(folded_store(feats, DEV), N, FIN, H, capacity=N, num_layers=L,
                             table_dtype=torch.float16, rate=0.5, age_limit=1 << 30, device=DEV)
    assert cache.table.numel() * 2 > 1 << 35

    # --- initial state, made on the device: 35% of the nodes cached; 200 000 of them sit in slots 0.. (the
    # ones the wrapped ring will evict), the others in the slots up to 700 before the end
    ids = torch.nonzero(torch.rand(N, device=DEV, generator=gen) < 0.35).view(-1)
    ids = ids[torch.randperm(ids.numel(), device=DEV, generator=gen)]
    n_low = 200_000
    n_high = ids.numel() - n_low
    start = N - 700 - n_high
    cache.preload(ids[:n_low])
    cache._header.fill_(start)
    cache.preload(ids[n_low:])
    assert cache.header == N - 700
    cache.table[:n_low].normal_(0.0, 0.5, generator=gen)
    cache.table[start:N - 700].normal_(0.0, 0.5, generator=gen)
    del ids

    with tempfile.TemporaryDirectory() as tmp:
        path = os.path.join(tmp, "table.bin")
        ref_table = np.lib.format.open_memmap(path, mode="w+", dtype=np.uint16, shape=(N, H))
        ref = dict(table=ref_table, f2s=cache.full2slot.cpu().numpy(), s2f=cache.slot2full.cpu().numpy(),
                   checkin=cache.checkin.cpu().numpy(), header=np.array([N - 700], np.int64))
        written = set()                     # slots whose rows the statement holds

        def seed_rows(slots):
            """Copies the initial rows of ``slots`` from the device into the statement's table."""
            slots = np.unique(slots[slots >= 0])
            new = np.array([s for s in slots.tolist() if s not in written], np.int64)
            if new.size:
                rows = cache.table[torch.from_numpy(new).to(DEV)].view(torch.int16).cpu().numpy()
                ref_table[new] = rows.view(np.uint16)
                written.update(new.tolist())

        class Rows:
            """The statement's table read as fp32, a few rows at a time."""
            shape = (N, H)

            def __getitem__(self, slots):
                return ref_table[slots].view(np.float16).astype(np.float32)

        class Labels:
            """Labels of the whole id space folded into a small table."""
            base = rng.integers(0, 16, size=1 << 20)

            def __getitem__(self, ids):
                return self.base[np.asarray(ids) % self.base.size]

        samples = [direct_power_law_batch(N, 1000, fanout, 2.0, 500 + k, degree_scale=cfg["degree_scale"])
                   for k in range(3)]
        # two of the seeds of the second batch are the last node and node 0
        samples[1]["sub_to_full"][:2] = (N - 1, 0)
        assert len(np.unique(samples[1]["sub_to_full"])) == len(samples[1]["sub_to_full"])
        order = [0, 1, 2, 0]
        admitted_total, wrapped, evicted, hits_of_admitted = 0, False, 0, 0
        first_admitted = None
        for it, k in enumerate(order, start=1):
            b = samples[k]
            batch = make_batch(b, Labels(), DEV)
            n1, n_all = int(b["num_node_in_layer"][1]), len(b["sub_to_full"])
            nodes = b["sub_to_full"][:n1]
            assert nodes.max() > N - N // 50            # ids reach the end of the maps
            seed_rows(ref["f2s"][nodes])
            cache.lookup_and_load(batch, L)
            slot, rows = host_model.ring_lookup(ref["f2s"], ref["checkin"], nodes, it, 1 << 30, Rows())
            np.testing.assert_array_equal(cache.sub2embed.cpu().numpy(), slot)
            np.testing.assert_array_equal(cache.cached_embedding.cpu().numpy(), rows)
            used = orc.count_history_reconstruct(b["ptr"], b["idx"], slot, n_all, 1000, L)
            np.testing.assert_array_equal(cache.used_masks[0].cpu().numpy(), used[0])
            x_ref = feats.numpy()[b["sub_to_full"] % POOL] * used[0][:, None]
            np.testing.assert_array_equal(batch.x.cpu().numpy(), x_ref)
            hit = slot != -1
            if it < len(order):
                assert 0.25 < hit.mean() < 0.45
            else:
                hits_of_admitted = int((hit & first_admitted).sum())

            emb = rng.standard_normal((n1, H), dtype=np.float32)
            grad = (rng.standard_normal((n1, H)) * np.exp(rng.normal(-3, 1.5, size=(n1, 1)))).astype(np.float32)
            pe = torch.from_numpy(emb).to(DEV).requires_grad_(True)
            pe.grad = torch.from_numpy(grad).to(DEV)
            cache.produced_embedding = pe
            before = int(ref["header"][0])
            cache.update_history(batch, it)
            score = orc.row_scores(grad)
            thres = float(host_model.quantile_threshold(score, 0.5))
            s2f_before = ref["s2f"].copy()
            rmask, _, slot_of = orc.grad_check(grad, emb, slot, None, None, nodes, thres, 0, orc.NORM_L2, orc.CMP_LT,
                                               ref_table, orc.DT_F16, ref["f2s"], ref["s2f"], ref["checkin"],
                                               ref["header"], it)
            np.testing.assert_array_equal(cache.last_record_mask.cpu().numpy(), rmask)
            assert 0 < rmask.sum() < n1 and not (rmask & hit).any()
            new_slots = slot_of[rmask]
            written.update(new_slots.tolist())
            admitted_total += int(rmask.sum())
            if it == 1:
                first_admitted = rmask.copy()
                wrapped = int(ref["header"][0]) < before
                assert new_slots.max() == N - 1 and new_slots.min() == 0
            evicted += int((s2f_before[new_slots] != -1).sum())
            assert cache.header == int(ref["header"][0])
            np.testing.assert_array_equal(cache.full2slot.cpu().numpy(), ref["f2s"])
            np.testing.assert_array_equal(cache.slot2full.cpu().numpy(), ref["s2f"])
            np.testing.assert_array_equal(cache.checkin.cpu().numpy(), ref["checkin"])
            held = np.fromiter(written, np.int64, len(written))
            held.sort()
            got = cache.table[torch.from_numpy(held).to(DEV)].view(torch.int16).cpu().numpy().view(np.uint16)
            np.testing.assert_array_equal(got, ref_table[held])
        assert wrapped and evicted > 0
        assert hits_of_admitted > 0          # rows stored across the end of the ring were served again
        # nothing was written outside the preloaded windows and the admitted slots (a normal row of 256
        # values is never all zero; the slots of evicted entries were non-zero before)
        fresh = admitted_total - evicted
        assert fresh == 700
        assert nonzero_rows(cache.table) == n_low + n_high + fresh
        got = cache.stats()
        assert got["rows_admitted"] == admitted_total and got["lookups"] == len(order)
        del ref_table
    del cache
    torch.cuda.empty_cache()


def test_row_gathers_from_a_feature_matrix_of_the_full_size():
    """The papers100M feature matrix at its real size in device memory (111 M x 128 fp32, 57 GB): rows whose contents
    are a function of their number, read through ``hc_gather_rows`` (several rows per wave) and through the hot tier
    (a 111 M-entry slot map, 50 M device copies whose slots run against the row order), the last row included --
    byte offsets beyond 2^35."""
    import hiscache_backend as be
    N, F = 111_000_000, 128
    need = N * F * 4 + 50_000_000 * F * 4 + N * 4 + (6 << 30)
    free, _ = torch.cuda.mem_get_info()
    if free < need:
        pytest.skip("needs %.0f GB of device memory, %.0f GB are free" % (need / 1e9, free / 1e9))
    col = torch.arange(F, device=DEV, dtype=torch.float32) / 256.0

    def rows_of(ids):                                  # what row ``ids[i]`` of the matrix holds
        return (ids % 99_991).to(torch.float32)[:, None] + (ids // 99_991 % 7).to(torch.float32)[:, None] * 0.5 + col

    matrix = torch.empty((N, F), dtype=torch.float32, device=DEV)
    step = 4_000_000
    for lo in range(0, N, step):
        hi = min(N, lo + step)
        matrix[lo:hi] = rows_of(torch.arange(lo, hi, device=DEV))
    gen = torch.Generator(device=DEV).manual_seed(7)
    ids = torch.randint(0, N, (150_000,), device=DEV, generator=gen)
    ids[0], ids[1], ids[2] = N - 1, 0, -1                                   # (-1 addresses the last row)
    mask = torch.rand(150_000, device=DEV, generator=gen) < 0.9
    want = rows_of(torch.where(ids < 0, ids + N, ids)) * mask[:, None]
    assert torch.equal(be.gather_rows(matrix, ids, mask=mask), want)
    # the hot tier: nodes [61 M, 111 M) have copies, in reverse order
    n_hot = 50_000_000
    slot = torch.full((N,), -1, dtype=torch.int32, device=DEV)
    slot[N - n_hot:] = torch.arange(n_hot - 1, -1, -1, dtype=torch.int32, device=DEV)
    hot = torch.empty((n_hot, F), dtype=torch.float32, device=DEV)
    for lo in range(0, n_hot, step):
        hi = min(n_hot, lo + step)
        hot[lo:hi] = rows_of(N - 1 - torch.arange(lo, hi, device=DEV))
    out = torch.full((150_000, F), -1.0, device=DEV)
    _, cold = be.gather_rows_hot(hot, slot, ids, mask=mask, out=out)
    wrapped = torch.where(ids < 0, ids + N, ids)
    is_hot = wrapped >= N - n_hot
    assert torch.equal(cold.bool(), mask & ~is_hot)
    done = ~(mask & ~is_hot)
    assert torch.equal(out[done], want[done]) and bool((out[~done] == -1.0).all())
    be.gather_rows_flagged(matrix, ids, cold, out)                           # (the other tier, here device memory too)
    assert torch.equal(out, want)
    assert int(is_hot[mask].sum()) > 50_000 and int(cold.sum()) > 50_000
