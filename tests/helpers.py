"""Shared generators for the tests (small seeded CSR blocks and cache states)."""
import numpy as np


def random_csr(rng, n_rows, n_src, max_deg, zero_frac=0.2, hub=None):
    """CSR with degrees in [0, max_deg]; a fraction of rows is empty; optional hub row degree."""
    deg = rng.integers(1, max_deg + 1, size=n_rows)
    deg[rng.random(n_rows) < zero_frac] = 0
    if hub is not None and n_rows > 0:
        deg[rng.integers(0, n_rows)] = hub
    ptr = np.zeros(n_rows + 1, np.int64)
    np.cumsum(deg, out=ptr[1:])
    idx = rng.integers(0, n_src, size=int(ptr[-1]), dtype=np.int64)
    return ptr, idx


def random_hmap(rng, n, frac):
    h = np.full(n, -1, np.int64)
    hit = rng.random(n) < frac
    h[hit] = rng.integers(0, 1000, size=int(hit.sum()))
    return h


def layered_batch(rng, n_full, n_seed, fanout, avg_deg=8):
    """A small layered-CSR mini-batch (see hiscache.synthetic.sample_layered_batch)."""
    from hiscache.synthetic import sample_layered_batch, uniform_graph
    indptr, indices = uniform_graph(n_full, avg_deg, int(rng.integers(1 << 30)))
    seeds = rng.choice(n_full, size=n_seed, replace=False)
    return sample_layered_batch(indptr, indices, seeds, fanout, rng)


def power_law_graph(rng, num_nodes, degree_scale, alpha=2.0, max_degree=2000, popular=True):
    """CSR of a directed graph with Zipf(alpha) out-degrees (scaled, capped) and neighbour ids skewed
    towards popular nodes (a cubed uniform scattered by a multiplicative hash), multi-edges possible:
    the shape of a citation graph, small enough to hold on the host."""
    raw = np.minimum(rng.zipf(alpha, size=num_nodes), 1 << 20).astype(np.float64)
    deg = np.minimum(np.floor(raw * degree_scale), max_degree).astype(np.int64)
    indptr = np.zeros(num_nodes + 1, np.int64)
    np.cumsum(deg, out=indptr[1:])
    E = int(indptr[-1])
    if popular:
        u = rng.random(E)
        indices = ((u * u * u * num_nodes).astype(np.int64) * 2654435761) % num_nodes
    else:
        indices = rng.integers(0, num_nodes, size=E, dtype=np.int64)
    return indptr, indices.astype(np.int64)


# ---- inputs that can be rebuilt bit for bit from a seed (fixtures then hold seeds and outputs only) --------
_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x):
    """The splitmix64 finaliser on uint64 arrays (wrap-around arithmetic, no floating point)."""
    with np.errstate(over="ignore"):
        z = (x + np.uint64(0x9E3779B97F4A7C15)) & _M64
        z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
        z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
        return z ^ (z >> np.uint64(31))


def exact_rows(seed, n, width, octaves=13):
    """[n, width] float32 built from integer hashes and exactly representable operations only (no library
    random stream, no transcendental function), so that any NumPy on any machine rebuilds the same bits:
    entry = (sum of four 16-bit fields of a hash - 131070) / 65536, a bell-shaped value in (-2, 2), times a
    per-row scale 2^-k * (1 + m/256) with k < octaves, which spreads the row norms over several octaves the
    way gradient rows are spread."""
    cell = np.arange(n * width, dtype=np.uint64).reshape(n, width)
    with np.errstate(over="ignore"):
        h = _splitmix64(cell * np.uint64(2) + np.uint64(seed) * np.uint64(0x100000001B3))
        hr = _splitmix64(np.arange(n, dtype=np.uint64) * np.uint64(2) + np.uint64(1)
                         + np.uint64(seed) * np.uint64(0x100000001B3))
    f = [((h >> np.uint64(16 * q)) & np.uint64(0xFFFF)).astype(np.int64) for q in range(4)]
    value = (f[0] + f[1] + f[2] + f[3] - 131070).astype(np.float64) / 65536.0
    k = (hr % np.uint64(octaves)).astype(np.int64)
    m = ((hr >> np.uint64(8)) & np.uint64(0xFF)).astype(np.float64)
    scale = np.ldexp(1.0 + m / 256.0, -k)
    return (value * scale[:, None]).astype(np.float32)


def exact_sum_rows(seed, n, width, octaves=9):
    """[n, width] float32 whose row sums (of the values, of their magnitudes) are exact in fp32 in ANY order
    of summation: entry = q * 2^-(10 + k) with an integer |q| <= 4096 from a hash and a per-row k < octaves,
    so a row's partial sums are integers below 2^24 in units of 2^-(10 + k).  Scores built from such rows do
    not depend on how a library folds a row."""
    cell = np.arange(n * width, dtype=np.uint64).reshape(n, width)
    with np.errstate(over="ignore"):
        h = _splitmix64(cell * np.uint64(2) + np.uint64(seed) * np.uint64(0x100000001B3))
        hr = _splitmix64(np.arange(n, dtype=np.uint64) * np.uint64(2) + np.uint64(1)
                         + np.uint64(seed) * np.uint64(0x100000001B3))
    q = (h & np.uint64(0x1FFF)).astype(np.int64) - 4096
    k = (hr % np.uint64(octaves)).astype(np.int64)
    return np.ldexp(q.astype(np.float64), -(10 + k)[:, None]).astype(np.float32)


def affine_ids(n_full, count, a, b):
    """`count` distinct node ids (a * i + b) mod n_full; a must be coprime with n_full."""
    assert np.gcd(a, n_full) == 1 and count <= n_full
    return ((np.arange(count, dtype=np.int64) * a + b) % n_full).astype(np.int64)
