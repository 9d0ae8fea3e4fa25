"""Seeded synthetic inputs for the five benchmark configurations.

numpy `default_rng` streams, so any machine regenerates identical bytes.  Each
generator returns a dict with float32 `coords` (or `x`), int32 `row_splits`,
`K` and a `name`; `scale` shrinks the point count (same distribution, same
number of blobs / events) for parity tests that have to finish in seconds.
"""
import numpy as np


def cfg1_uniform_small(scale=1.0):
    """N=10 000, D=3, uniform in [0,1), row_splits [0, 6000, 10000], K=16."""
    n = int(round(10000 * scale))
    rng = np.random.default_rng(1001)
    coords = rng.random((n, 3)).astype(np.float32)
    rs = np.array([0, int(round(6000 * scale)), n], dtype=np.int32)
    return dict(name="cfg1_uniform_10k_d3_k16", coords=coords, row_splits=rs, K=16)


def cfg2_blobs_4events(scale=1.0):
    """N=200 000, D=4, 4 events of 50 000: 200 Gaussian blobs (sigma 0.02) + 10 % noise, K=40."""
    per = int(round(50000 * scale))
    rng = np.random.default_rng(1002)
    parts = []
    for _ in range(4):
        centres = rng.random((200, 4))
        n_noise = per // 10
        n_blob = per - n_noise
        which = rng.integers(0, 200, size=n_blob)
        blob = centres[which] + rng.normal(0.0, 0.02, size=(n_blob, 4))
        noise = rng.random((n_noise, 4))
        ev = np.concatenate([blob, noise], axis=0)
        ev = ev[rng.permutation(per)]
        parts.append(ev)
    coords = np.concatenate(parts, axis=0).astype(np.float32)
    rs = (np.arange(5) * per).astype(np.int32)
    return dict(name="cfg2_blobs_200k_d4_k40", coords=coords, row_splits=rs, K=40)


def cfg3_gravnet(scale=1.0):
    """GravNetOp input: N=300 000 x 64 N(0,1), 2 events; S=4, P=32, k=40, out 64."""
    per = int(round(150000 * scale))
    rng = np.random.default_rng(1003)
    x = rng.standard_normal((2 * per, 64)).astype(np.float32)
    rs = np.array([0, per, 2 * per], dtype=np.int32)
    g = np.random.default_rng(2003).standard_normal((2 * per, 64)).astype(np.float32)
    return dict(name="cfg3_gravnet_300k_c64_s4_p32_k40", x=x, row_splits=rs, K=40,
                in_channels=64, out_channels=64, space_dimensions=4, propagate_dimensions=32,
                out_grad=g, weight_seed=1003)


def cfg4_zipf_blobs(scale=1.0):
    """N=1 000 000, D=3, one event: 500 blobs (sigma 0.01, Zipf(1.2) sizes) + 20 % noise, K=64."""
    n = int(round(1000000 * scale))
    rng = np.random.default_rng(1004)
    centres = rng.random((500, 3))
    p = np.arange(1, 501, dtype=np.float64) ** -1.2
    p /= p.sum()
    n_noise = n // 5
    n_blob = n - n_noise
    which = rng.choice(500, size=n_blob, p=p)
    blob = centres[which] + rng.normal(0.0, 0.01, size=(n_blob, 3))
    noise = rng.random((n_noise, 3))
    coords = np.concatenate([blob, noise], axis=0)
    coords = coords[rng.permutation(n)].astype(np.float32)
    rs = np.array([0, n], dtype=np.int32)
    gd = np.random.default_rng(2004).standard_normal((n, 64)).astype(np.float32)
    return dict(name="cfg4_zipf_blobs_1m_d3_k64", coords=coords, row_splits=rs, K=64, grad_distsq=gd)


def cfg5_many_events_d8(scale=1.0):
    """N=500 000, D=8, uniform in [-1,1), 64 events with lognormal(8.5, 0.6) sizes, K=100."""
    n = int(round(500000 * scale))
    rng = np.random.default_rng(1005)
    sizes = rng.lognormal(8.5, 0.6, size=64)
    sizes = np.floor(sizes / sizes.sum() * n).astype(np.int64)
    sizes[np.argmax(sizes)] += n - sizes.sum()
    rs = np.concatenate([[0], np.cumsum(sizes)]).astype(np.int32)
    coords = (rng.random((n, 8)) * 2.0 - 1.0).astype(np.float32)
    return dict(name="cfg5_events64_500k_d8_k100", coords=coords, row_splits=rs, K=100)


CONFIGS = {
    "cfg1": cfg1_uniform_small,
    "cfg2": cfg2_blobs_4events,
    "cfg3": cfg3_gravnet,
    "cfg4": cfg4_zipf_blobs,
    "cfg5": cfg5_many_events_d8,
}


def oc_workload(scale=1.0):
    """Truth indices for the object-condensation helper: 4 events of 50 000 vertices, 500 objects per event with
    sizes ~ rank^-1 (a few large showers, many small ones), 10 % noise vertices (-1), shuffled inside the event;
    object ids restart at 0 in every event.  Returns (int64 truth indices [200 000], int64 row_splits [5])."""
    rng = np.random.default_rng(1006)
    per_event = int(round(50000 * scale))
    n_obj = 500
    p = 1.0 / np.arange(1, n_obj + 1)
    p /= p.sum()
    parts = []
    for _ in range(4):
        t = rng.choice(n_obj, size=per_event, p=p)
        t[rng.random(per_event) < 0.1] = -1
        parts.append(t)
    a = np.concatenate(parts).astype(np.int64)
    rs = (np.arange(5) * per_event).astype(np.int64)
    return a, rs
