"""LibSVM text I/O and the seeded synthetic workloads the benchmarks and parity tests run on.

Feature values are always float32-exact: the reference parses "%d:%f" into a float
(src/thundersvm/dataset.cpp:76-79), so every loader and generator here rounds to float32 and then
widens to float64.  Feature indices are 1-based as in LibSVM files.
"""
import numpy as np


class CsrData:
    """Rows in CSR form: ptr int64[n+1], col int32[nnz] (1-based feature ids), val float64[nnz], y float64[n]."""

    def __init__(self, ptr, col, val, y=None):
        self.ptr = np.ascontiguousarray(ptr, dtype=np.int64)
        self.col = np.ascontiguousarray(col, dtype=np.int32)
        self.val = np.ascontiguousarray(val, dtype=np.float64)
        self.y = None if y is None else np.ascontiguousarray(y, dtype=np.float64)

    @property
    def n(self):
        return len(self.ptr) - 1

    @property
    def nnz(self):
        return int(self.ptr[-1])

    @property
    def n_features(self):
        return int(self.col.max()) if len(self.col) else 0

    def rows(self, idx):
        idx = np.asarray(idx, dtype=np.int64)
        lens = self.ptr[idx + 1] - self.ptr[idx]
        ptr = np.zeros(len(idx) + 1, dtype=np.int64)
        np.cumsum(lens, out=ptr[1:])
        take = np.repeat(self.ptr[idx] - ptr[:-1], lens) + np.arange(ptr[-1])
        return CsrData(ptr, self.col[take], self.val[take], None if self.y is None else self.y[idx])

    def to_dense(self, n_cols=None):
        """Dense float64 [n, n_cols] with column c holding feature id c (column 0 stays zero for 1-based data)."""
        n_cols = n_cols or self.n_features + 1
        out = np.zeros((self.n, n_cols))
        r = np.repeat(np.arange(self.n), np.diff(self.ptr))
        keep = self.col < n_cols
        out[r[keep], self.col[keep]] = self.val[keep]
        return out


def from_dense(x, y=None, keep_zeros=False):
    """Dense [n, d] -> CsrData with 1-based feature ids, dropping zeros unless keep_zeros."""
    x = np.asarray(x, dtype=np.float32).astype(np.float64)
    n, d = x.shape
    if keep_zeros:
        ptr = np.arange(n + 1, dtype=np.int64) * d
        col = np.tile(np.arange(1, d + 1, dtype=np.int32), n)
        return CsrData(ptr, col, x.reshape(-1), y)
    mask = x != 0
    ptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(mask.sum(axis=1), out=ptr[1:])
    col = (np.nonzero(mask)[1] + 1).astype(np.int32)
    return CsrData(ptr, col, x[mask], y)


def load_libsvm(path):
    """Parse a LibSVM text file (label idx:val ...).  Values are rounded to float32 like the reference loader."""
    ys, ptr, col, val = [], [0], [], []
    with open(path) as fh:
        for line in fh:
            parts = line.split()
            if not parts:
                continue
            ys.append(float(parts[0]))
            for tup in parts[1:]:
                i, v = tup.split(":")
                col.append(int(i))
                val.append(float(v))
            ptr.append(len(col))
    val32 = np.asarray(val, dtype=np.float64).astype(np.float32)
    return CsrData(ptr, col, val32.astype(np.float64), ys)


def save_libsvm(path, data, rows_per_write=100000):
    """LibSVM text with nine significant digits (float32-exact values survive the round trip)."""
    n = data.n
    ptr = data.ptr.tolist()
    y = data.y.tolist() if data.y is not None else [0.0] * n
    with open(path, "w") as fh:
        for r0 in range(0, n, rows_per_write):
            r1 = min(n, r0 + rows_per_write)
            e0, e1 = ptr[r0], ptr[r1]
            toks = ["%d:%.9g" % cv for cv in zip(data.col[e0:e1].tolist(), data.val[e0:e1].tolist())]
            fh.write("".join("%.9g %s\n" % (y[i], " ".join(toks[ptr[i] - e0:ptr[i + 1] - e0])) for i in range(r0, r1)))


# ----------------------------------------------------------------------------------------------
# The five benchmark workloads.  seed = 20240 + workload number.  `scale` shrinks the row count
# for parity tests; scale=1 is the full benchmark shape.
# ----------------------------------------------------------------------------------------------
def _rng(cfg):
    return np.random.Generator(np.random.PCG64(20240 + cfg))


def workload_c1(scale=1.0):
    """4000x32 dense, two Gaussian blobs at +-0.5, 80/20 split.  CLI: -s 0 -t 2 -g 0.5 -c 100 -e 0.001."""
    rng = _rng(1)
    n = max(int(4000 * scale), 64)
    y = np.where(np.arange(n) % 2 == 0, 1.0, -1.0)
    x = rng.standard_normal((n, 32)) + 0.5 * y[:, None]
    perm = rng.permutation(n)
    x, y = x[perm], y[perm]
    ntr = int(n * 0.8)
    return dict(train=from_dense(x[:ntr], y[:ntr]), test=from_dense(x[ntr:], y[ntr:]),
                params=dict(svm_type=0, kernel_type=2, gamma=0.5, C=100.0, epsilon=0.001), name="C1")


def workload_c2(scale=1.0):
    """100000x784 pixel-like (k/255, ~80% zeros), hyperplane+quadratic labels, 5% flips; 10000 held out."""
    rng = _rng(2)
    n = max(int(100000 * scale), 256)
    nte = max(int(10000 * scale), 64)
    d = 784
    w = rng.standard_normal(d)
    u = rng.standard_normal(d)

    def gen(m):
        k = rng.integers(0, 256, size=(m, d)).astype(np.float32)
        zero = rng.random((m, d)) < 0.8
        k[zero] = 0
        return (k / np.float32(255)).astype(np.float32)

    x = gen(n)
    xt = gen(nte)
    score = x.astype(np.float64) @ w + (x.astype(np.float64) ** 2) @ u
    med = np.median(score)
    y = np.where(score > med, 1.0, -1.0)
    flip = rng.random(n) < 0.05
    y[flip] = -y[flip]
    st = xt.astype(np.float64) @ w + (xt.astype(np.float64) ** 2) @ u
    yt = np.where(st > med, 1.0, -1.0)
    return dict(train=from_dense(x, y), test=from_dense(xt, yt),
                params=dict(svm_type=0, kernel_type=2, gamma=0.125, C=10.0), name="C2")


def workload_c3(scale=1.0, kernel="rbf"):
    """72000x20958 CSR, ~50 nnz/row, Zipf(1.1) columns, lognormal values, L2-normalised rows."""
    rng = _rng(3)
    n = max(int(72000 * scale), 256)
    d = 20958
    ranks = np.arange(1, d + 1, dtype=np.float64)
    pz = ranks ** -1.1
    pz /= pz.sum()
    nnz_row = np.maximum(rng.poisson(50, size=n), 1)
    wcols = rng.choice(d, size=400, replace=False, p=pz)
    w = np.zeros(d + 1)
    w[wcols + 1] = rng.standard_normal(400)
    # every row's draws at once: each row draws until it holds nnz_row distinct columns (more draws than needed are
    # made up front and the first nnz_row distinct ones kept, in draw order), columns ascending per row
    n_draw = 2 * nnz_row + 16
    row_of = np.repeat(np.arange(n, dtype=np.int64), n_draw)
    drawn = rng.choice(d, size=int(n_draw.sum()), replace=True, p=pz).astype(np.int64) + 1
    _, first = np.unique(row_of * (d + 2) + drawn, return_index=True)   # first occurrence of every (row, column)
    first.sort()
    r = row_of[first]
    start = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(np.bincount(r, minlength=n), out=start[1:])
    keep = first[np.arange(len(first)) - start[r] < nnz_row[r]]
    key = np.sort(row_of[keep] * (d + 2) + drawn[keep])
    row_of, col = key // (d + 2), (key % (d + 2)).astype(np.int32)
    ptr = np.zeros(n + 1, dtype=np.int64)
    np.cumsum(np.bincount(row_of, minlength=n), out=ptr[1:])
    v = rng.lognormal(0.0, 1.0, size=len(col))
    norm = np.sqrt(np.add.reduceat(v * v, ptr[:-1]))
    val = (v / norm[row_of]).astype(np.float32).astype(np.float64)
    score = np.add.reduceat(val * w[col], ptr[:-1])
    y = np.where(score > np.median(score), 1.0, -1.0)
    flip = rng.random(n) < 0.03
    y[flip] = -y[flip]
    params = dict(svm_type=0, kernel_type=0, C=1.0) if kernel == "linear" else dict(svm_type=0, kernel_type=2, gamma=1.0, C=1.0)
    return dict(train=CsrData(ptr, col, val, y), test=None, params=params, name="C3-" + kernel)


def workload_c4(scale=1.0, n_test=0):
    """500000x54: 10 standardised Gaussian-mixture features + 4-way and 40-way one-hots, 7 skewed classes."""
    rng = _rng(4)
    n = max(int(500000 * scale), 700)
    pri = np.array([0.36, 0.49, 0.06, 0.005, 0.016, 0.03, 0.035])
    pri = pri / pri.sum()
    means = rng.standard_normal((7, 10)) * 1.5
    scales = 0.5 + rng.random((7, 10))
    p4 = rng.dirichlet(np.ones(4) * 0.7, size=7)
    p40 = rng.dirichlet(np.ones(40) * 0.3, size=7)

    def gen(m):
        cls = rng.choice(7, size=m, p=pri)
        cont = means[cls] + scales[cls] * rng.standard_normal((m, 10))
        c4 = (rng.random(m)[:, None] > np.cumsum(p4[cls], axis=1)).sum(axis=1).clip(0, 3)
        c40 = (rng.random(m)[:, None] > np.cumsum(p40[cls], axis=1)).sum(axis=1).clip(0, 39)
        return cls, cont, c4, c40

    cls, cont, c4, c40 = gen(n)
    mu, sd = cont.mean(axis=0), cont.std(axis=0)

    def assemble(cls, cont, c4, c40):
        m = len(cls)
        x = np.zeros((m, 54), dtype=np.float32)
        x[:, :10] = ((cont - mu) / sd).astype(np.float32)
        x[np.arange(m), 10 + c4] = 1
        x[np.arange(m), 14 + c40] = 1
        return from_dense(x, (cls + 1).astype(np.float64))

    out = dict(train=assemble(cls, cont, c4, c40), test=None,
               params=dict(svm_type=0, kernel_type=2, gamma=1.0, C=3.0), name="C4")
    if n_test:
        out["test"] = assemble(*gen(n_test))
    return out


def workload_c5(scale=1.0):
    """400000x90 standard normal, y = sin(w1.x) + 0.5 (w2.x)^2 + N(0, 0.1^2); 200000 predict rows."""
    rng = _rng(5)
    n = max(int(400000 * scale), 256)
    nte = max(int(200000 * scale), 128)
    d = 90
    w1 = rng.standard_normal(d)
    w1 /= np.linalg.norm(w1)
    w2 = rng.standard_normal(d)
    w2 /= np.linalg.norm(w2)

    def gen(m):
        x = rng.standard_normal((m, d)).astype(np.float32)
        xd = x.astype(np.float64)
        y = np.sin(xd @ w1) + 0.5 * (xd @ w2) ** 2 + 0.1 * rng.standard_normal(m)
        return from_dense(x, y.astype(np.float32).astype(np.float64), keep_zeros=True)

    return dict(train=gen(n), test=gen(nte),
                params=dict(svm_type=3, kernel_type=2, gamma=0.05, C=10.0, p=0.1), name="C5")
