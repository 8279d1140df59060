"""Seeded synthetic workloads for the sparse pull / push path.

Everything is a pure function of integers so that the same table snapshot can
be materialised on the GPU in bulk (torch int64 arithmetic, wrapping like
uint64) and on the host for just the keys a batch touches (numpy uint64).

    sign          = splitmix64(zipf_id),  zipf_id in [1, vocab]
    resident set  = { splitmix64(i) : 1 <= i <= resident }
    snapshot row  = w[c] ~ U(-0.01, 0.01) from hash(seed, sign, c); fresh state
"""
import numpy as np

MASK64 = (1 << 64) - 1


def splitmix64(x):
    """splitmix64 finaliser on a numpy uint64 array (wraps mod 2^64)."""
    x = np.asarray(x, dtype=np.uint64).copy()
    with np.errstate(over="ignore"):
        x += np.uint64(0x9E3779B97F4A7C15)
        x = (x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        x = (x ^ (x >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        x = x ^ (x >> np.uint64(31))
    return x


def _i64(c):
    """Python int (uint64 value) -> the int64 with the same bits."""
    c &= MASK64
    return c - (1 << 64) if c >= (1 << 63) else c


def splitmix64_torch(x):
    """Same function on a torch int64 tensor holding uint64 bit patterns."""

    def lsr(v, k):
        return (v >> k) & ((1 << (64 - k)) - 1)

    x = x + _i64(0x9E3779B97F4A7C15)
    x = (x ^ lsr(x, 30)) * _i64(0xBF58476D1CE4E5B9)
    x = (x ^ lsr(x, 27)) * _i64(0x94D049BB133111EB)
    return x ^ lsr(x, 31)


def snapshot_rows(signs, dim, seed=0, scale=0.01):
    """float32 [n, dim] weights of the snapshot for numpy uint64 signs."""
    signs = np.asarray(signs, dtype=np.uint64)
    cols = splitmix64(np.uint64(seed * 4096) + np.arange(dim, dtype=np.uint64))
    h = splitmix64(signs[:, None] ^ cols[None, :])
    u24 = (h >> np.uint64(40)).astype(np.float32)
    return (u24 * np.float32(2.0 ** -23) - np.float32(1.0)) * np.float32(scale)


def snapshot_rows_torch(signs, dim, seed=0, scale=0.01):
    """Same values for a torch int64 tensor of signs (on any device)."""
    import torch

    cols_np = splitmix64(np.uint64(seed * 4096) + np.arange(dim, dtype=np.uint64)).view(np.int64)
    cols = torch.from_numpy(cols_np.copy()).to(signs.device)
    h = splitmix64_torch(signs[:, None] ^ cols[None, :])
    u24 = ((h >> 40) & ((1 << 24) - 1)).to(torch.float32)
    return (u24 * (2.0 ** -23) - 1.0) * scale


def zipf_ids(rng, n, s, vocab):
    """Bounded Zipf(s) ids in [1, vocab] by inverting the continuous CDF."""
    u = rng.random(n)
    a = 1.0 - s
    x = (1.0 + u * (float(vocab) ** a - 1.0)) ** (1.0 / a)
    ids = np.floor(x).astype(np.int64)
    return np.clip(ids, 1, vocab).astype(np.uint64)


# The five workload shapes (batch rows x slots, id-list lengths, vocabulary,
# resident keys, embedding dim, optimizer, gradient sigma).
CONFIGS = {
    "cfg1": dict(batch=1024, slots=8, lens="one", zipf_s=1.1, vocab=10 ** 6, resident=10 ** 6, dim=8,
                 opt="AdaGrad", hyper=dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8), grad_sigma=0.01,
                 fresh=0.0),
    "cfg2": dict(batch=4096, slots=26, lens="one", zipf_s=1.05, vocab=10 ** 8, resident=5 * 10 ** 7, dim=16,
                 opt="Adam", hyper=dict(learning_rate=1e-3, beta1=0.9, beta2=0.999, epsilon=1e-8), grad_sigma=1e-3,
                 fresh=0.0),
    "cfg3": dict(batch=16384, slots=100, lens="poisson3", zipf_s=1.1, vocab=10 ** 9, resident=5 * 10 ** 8, dim=16,
                 opt="AdaGrad", hyper=dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8), grad_sigma=1e-3,
                 fresh=0.0),
    "cfg4": dict(batch=8192, slots=40, lens="one", zipf_s=1.1, vocab=10 ** 8, resident=10 ** 8, dim=64,
                 opt="AdaGrad", hyper=dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8), grad_sigma=1e-2,
                 fresh=0.2),
    "cfg5": dict(batch=32768, slots=64, lens="one", zipf_s=1.2, vocab=15 * 10 ** 8, resident=15 * 10 ** 8, dim=16,
                 opt="AdaGrad", hyper=dict(learning_rate=0.01, initial_g2sum=0.1, epsilon=1e-8), grad_sigma=1e-3,
                 fresh=0.0, dense_total=2 * 10 ** 8),
}


def make_batch(cfg, batch_index=0, scale=1.0):
    """Per-slot int64 sign arrays of one batch of workload `cfg` (a dict of
    CONFIGS).  `scale` < 1 shrinks the number of batch rows (for CPU-sized
    samples of the same distribution)."""
    rng = np.random.default_rng(batch_index)
    rows = max(1, int(cfg["batch"] * scale))
    out = []
    for _ in range(cfg["slots"]):
        if cfg["lens"] == "poisson3":
            lens = np.clip(rng.poisson(3.0, rows), 1, 20)
            n = int(lens.sum())
        else:
            n = rows
        ids = zipf_ids(rng, n, cfg["zipf_s"], cfg["vocab"])
        signs = splitmix64(ids)
        if cfg["fresh"] > 0:
            fresh = rng.random(n) < cfg["fresh"]
            signs = np.where(fresh, rng.integers(0, 1 << 64, n, dtype=np.uint64), signs)
        out.append(signs.view(np.int64))
    return out


CLICK_RATE = 0.2  # share of lookups whose feature label is 1 (the label of their example)


def make_labels(values, batch_index=0, rate=CLICK_RATE):
    """Per-slot int64 feature labels (0 / 1) for the lookups of one batch."""
    rng = np.random.default_rng(2_000_003 + batch_index)
    return [(rng.random(len(v)) < rate).astype(np.int64) for v in values]


def make_grads(counts, dim, sigma, seed=0):
    """Per-slot float32 [U_s, dim] gradients ~ N(0, sigma)."""
    rng = np.random.default_rng(1_000_003 + seed)
    return [(rng.standard_normal((int(u), dim)) * sigma).astype(np.float32) for u in counts]


def populate_table(tn, handle, resident, dim, chunk=1 << 23):
    """Loads the resident set splitmix64(1..resident) with its snapshot rows into a sparse
    table on the GPU, in chunks (signs and rows are generated on the device)."""
    import torch

    for lo in range(1, resident + 1, chunk):
        hi = min(resident + 1, lo + chunk)
        ids = torch.arange(lo, hi, dtype=torch.int64, device="cuda")
        signs = splitmix64_torch(ids)
        w = snapshot_rows_torch(signs, dim)
        tn.ops.table_load_rows(handle, signs, w)
        del ids, signs, w
    torch.cuda.synchronize()
