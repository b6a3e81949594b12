"""CPU-only check of the accumulation plans the sketch kernels run on (binned plans for long
rows first, row-list plans at the end).

The two GPU passes are replayed here in numpy, reading only the plan's tables: pass A permutes
each chunk's records into its image, pass B collects a bin's segments and adds every bucket's
terms in the order the plan lists them.  If the tables are right this reproduces the oracle's
update bit for bit (same terms, same ascending-column order)."""
import numpy as np
import pytest

A, B = 994443, 609478


def build_plan(n, d, w, chunk=0, tbin=0):
    from conef_amd import _lib
    lib = _lib.load()
    nb = lib.conef_plan_bytes(n, d, w, chunk, tbin)
    assert nb > 0
    buf = np.zeros(nb, np.uint8)
    assert lib.conef_plan_build_host(buf.ctypes.data, nb, n, d, w, A, B, chunk, tbin) == 0
    i32, i64 = buf[:128].view(np.int32), buf[:128].view(np.int64)
    h = {"C": int(i32[9]), "nchunks": int(i32[10]), "T": int(i32[11]), "nbins": int(i32[12]),
         "maxrec": int(i32[13])}
    h["pos"] = buf[int(i64[7]):int(i64[7]) + 2 * d].view(np.uint16)
    h["seg"] = buf[int(i64[8]):int(i64[8]) + 4 * h["nbins"] * (h["nchunks"] + 1)].view(np.uint32).reshape(
        h["nbins"], h["nchunks"] + 1)
    h["csr"] = buf[int(i64[9]):int(i64[9]) + 4 * (w + 1)].view(np.uint32)
    h["ent"] = buf[int(i64[10]):int(i64[10]) + 2 * d].view(np.uint16)
    assert int(i64[13]) >= 4 * n * d
    h["pk"] = buf[int(i64[11]):int(i64[11]) + 4 * d].view(np.uint32)
    return h


def replay(h, vec, cs, beta, oracle):
    n, d = vec.shape
    w = cs.shape[1]
    C, T = h["C"], h["T"]
    staging = np.full(n * d, np.nan, np.float32)
    for c in range(h["nchunks"]):                                   # pass A
        c0, c1 = c * C, min(d, (c + 1) * C)
        img = np.full((c1 - c0, n), np.nan, np.float32)
        p = h["pos"][c0:c1].astype(np.int64)
        assert sorted(p.tolist()) == list(range(c1 - c0))           # a permutation of the chunk
        img[p, :] = vec[:, c0:c1].T
        staging[c0 * n:c1 * n] = img.reshape(-1)
    out = cs.copy()
    omb = 1.0 - float(np.float32(beta))
    for bn in range(h["nbins"]):                                    # pass B
        seg = h["seg"][bn]
        total = int(seg[-1] >> 16)
        assert total <= h["maxrec"]
        img = np.empty((total, n), np.float32)
        for c in range(h["nchunks"]):
            start, off = int(seg[c] & 0xffff), int(seg[c] >> 16)
            ln = int(seg[c + 1] >> 16) - off
            src = (c * C + start) * n
            img[off:off + ln] = staging[src:src + ln * n].reshape(ln, n)
        for j in range(bn * T, min(w, (bn + 1) * T)):
            for e in range(int(h["csr"][j]), int(h["csr"][j + 1])):
                en = int(h["ent"][e])
                sign = 1.0 if en >> 15 else -1.0
                for r in range(n):
                    v = float(img[en & 0x7fff, r])
                    term = np.float32(sign * v - omb * float(cs[r, j]))
                    out[r, j] = np.float32(out[r, j] + term)
    assert not np.isnan(out).any()
    return out


@pytest.mark.parametrize("n,d,w,chunk,tbin", [(5, 9000, 900, 1024, 64), (1, 5000, 5000, 2048, 128),
                                              (8, 3001, 77, 1024, 64), (3, 30011, 4000, 0, 0),
                                              (11, 9000, 900, 1024, 64), (9, 30011, 4000, 0, 0)])
def test_plan_replay_matches_oracle_bit_for_bit(oracle, n, d, w, chunk, tbin):
    rng = np.random.RandomState(d)
    h = build_plan(n, d, w, chunk, tbin)
    vec = rng.randn(n, d).astype(np.float32)
    cs0 = rng.randn(n, w).astype(np.float32)
    got = replay(h, vec, cs0, 0.9, oracle)
    want = cs0.copy()
    oracle.cs_update(vec, want, 0.9)
    np.testing.assert_array_equal(got, want)


def test_plan_tables_are_consistent(oracle):
    n, d, w = 5, 50_000, 5_000
    h = build_plan(n, d, w)
    bucket, sign = oracle.hash_table(d, w)
    assert h["csr"][0] == 0 and h["csr"][-1] == d
    np.testing.assert_array_equal(np.diff(h["csr"].astype(np.int64)), np.bincount(bucket, minlength=w))
    bins = bucket // h["T"]
    np.testing.assert_array_equal(h["seg"][:, -1] >> 16, np.bincount(bins, minlength=h["nbins"]))
    assert h["maxrec"] == np.bincount(bins, minlength=h["nbins"]).max()
    np.testing.assert_array_equal(h["pk"] & 0x7fffffff, bucket.astype(np.uint32))
    np.testing.assert_array_equal(h["pk"] >> 31, (sign > 0).astype(np.uint32))
    # entries of a bucket carry that bucket's signs, in ascending column order
    order = np.lexsort((np.arange(d), bucket))
    np.testing.assert_array_equal(h["ent"] >> 15, (sign[order] > 0).astype(np.uint16))


def build_rowlist(n, d, w):
    from conef_amd import _lib
    lib = _lib.load()
    nb = lib.conef_plan_bytes(n, d, w, 0, 0)
    assert nb > 0
    buf = np.zeros(nb, np.uint8)
    assert lib.conef_plan_build_host(buf.ctypes.data, nb, n, d, w, A, B, 0, 0) == 0
    assert lib.conef_plan_kind(buf.ctypes.data) == 1
    assert lib.conef_plan_workspace_bytes(buf.ctypes.data) == 0
    i64 = buf[:136].view(np.int64)
    csr = buf[int(i64[9]):int(i64[9]) + 4 * (w + 1)].view(np.uint32)
    ent = buf[int(i64[10]):int(i64[10]) + 2 * d].view(np.uint16)
    pk = buf[int(i64[11]):int(i64[11]) + 4 * d].view(np.uint32)
    order = buf[int(i64[16]):int(i64[16]) + 2 * w].view(np.uint16)
    # the walk's bucket order: every bucket once, longest list first, equal lengths by index
    lengths = np.diff(csr.astype(np.int64))
    np.testing.assert_array_equal(order.astype(np.int64), np.argsort(-lengths, kind="stable"))
    return csr, ent, pk


@pytest.mark.parametrize("n,d,w", [(3, 17, 5), (40, 5760, 1152), (7, 24576, 100), (100, 650, 65), (2, 100, 300)])
def test_rowlist_plan_replay_matches_oracle_bit_for_bit(oracle, n, d, w):
    """Walking the per-bucket column lists the way the kernel does reproduces the oracle's update."""
    csr, ent, pk = build_rowlist(n, d, w)
    bucket, sign = oracle.hash_table(d, w)
    np.testing.assert_array_equal(pk & 0x7fffffff, bucket.astype(np.uint32))
    np.testing.assert_array_equal(pk >> 31, (sign > 0).astype(np.uint32))
    assert csr[0] == 0 and csr[-1] == d
    rng = np.random.RandomState(d)
    vec = rng.randn(n, d).astype(np.float32)
    cs0 = rng.randn(n, w).astype(np.float32)
    omb = 1.0 - float(np.float32(0.9))
    got = cs0.copy()
    for j in range(w):
        cols = ent[csr[j]:csr[j + 1]].astype(np.int64)
        assert (np.diff(cols & 0x7fff) > 0).all()                       # ascending columns
        for en in cols:
            s = 1.0 if en >> 15 else -1.0
            term = (s * vec[:, en & 0x7fff].astype(np.float64) - omb * cs0[:, j].astype(np.float64)).astype(np.float32)
            got[:, j] = got[:, j] + term
    want = cs0.copy()
    oracle.cs_update(vec, want, 0.9)
    np.testing.assert_array_equal(got, want)


def build_panels(n, d, w):
    from conef_amd import _lib
    lib = _lib.load()
    nb = lib.conef_plan_bytes(n, d, w, 0, 0)
    assert nb > 0
    buf = np.zeros(nb, np.uint8)
    assert lib.conef_plan_build_host(buf.ctypes.data, nb, n, d, w, A, B, 0, 0) == 0
    assert lib.conef_plan_kind(buf.ctypes.data) == 2
    assert lib.conef_plan_workspace_bytes(buf.ctypes.data) == 0
    i32, i64 = buf[:128].view(np.int32), buf[:136].view(np.int64)
    pc = int(i32[9])
    assert pc % 8 == 0 and int(i32[10]) == (d + pc - 1) // pc
    epos = buf[int(i64[10]):int(i64[10]) + 2 * d].view(np.uint16)
    entg = buf[int(i64[7]):int(i64[7]) + 4 * d].view(np.uint32)
    colb = buf[int(i64[9]):int(i64[9]) + 2 * d].view(np.uint16)
    pk = buf[int(i64[11]):int(i64[11]) + 4 * d].view(np.uint32)
    return pc, epos, entg, colb, pk


@pytest.mark.parametrize("n,d,w", [(600, 25_088, 2508), (257, 30_001, 12_000), (1030, 40_000, 400)])
def test_panel_plan_replay_matches_oracle_bit_for_bit(oracle, n, d, w):
    """The kernel's two steps, panel after panel, from the plan's tables alone: every column's term
    is parked at the entry the plan names for it, then the first entry of a bucket's group adds the
    group's terms in the order they sit in."""
    pc, epos, entg, colb, pk = build_panels(n, d, w)
    assert pc <= 4096
    bucket, sign = oracle.hash_table(d, w)
    np.testing.assert_array_equal(pk & 0x7fffffff, bucket.astype(np.uint32))
    np.testing.assert_array_equal(pk >> 31, (sign > 0).astype(np.uint32))
    np.testing.assert_array_equal(colb, bucket.astype(np.uint16))
    np.testing.assert_array_equal(epos >> 15, (sign > 0).astype(np.uint16))
    rows = 3                                                    # the tables are the same for every row
    rng = np.random.RandomState(d)
    vec = rng.randn(rows, d).astype(np.float32)
    cs0 = rng.randn(rows, w).astype(np.float32)
    omb = 1.0 - float(np.float32(0.9))
    got = cs0.copy()
    for c0 in range(0, d, pc):
        cols = min(pc, d - c0)
        e = (epos[c0:c0 + cols] & 0x7fff).astype(np.int64)
        assert sorted(e.tolist()) == list(range(cols))                         # a permutation of the panel
        e_b = (entg[c0:c0 + cols] & 0xffff).astype(np.int64)
        np.testing.assert_array_equal(e_b[e], colb[c0:c0 + cols])              # every entry names its column's bucket
        assert (np.diff(e_b) >= 0).all()                                      # grouped by bucket ...
        lens = (entg[c0:c0 + cols] >> 16).astype(np.int64)                    # ... the first of a group carries its length
        first = np.concatenate([[True], np.diff(e_b) != 0])
        assert (lens[~first] == 0).all()
        np.testing.assert_array_equal(lens[first], np.diff(np.concatenate([np.flatnonzero(first), [cols]])))
        col_of = np.empty(cols, np.int64)
        col_of[e] = np.arange(cols)
        assert (np.diff(col_of)[np.diff(e_b) == 0] > 0).all()                 # ... ascending columns inside a group
        # park
        s = np.where(epos[c0:c0 + cols] >> 15, 1.0, -1.0)
        terms = np.empty((cols, rows), np.float32)
        v = vec[:, c0:c0 + cols].astype(np.float64)
        decay = omb * cs0[:, colb[c0:c0 + cols].astype(np.int64)].astype(np.float64)
        terms[e, :] = (s[None, :] * v - decay).astype(np.float32).T
        # walk
        for k in np.flatnonzero(lens):
            for kk in range(k, k + lens[k]):
                got[:, e_b[k]] = got[:, e_b[k]] + terms[kk, :]
    want = cs0.copy()
    oracle.cs_update(vec, want, 0.9)
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize("n,d,w,kind", [(5, 1_300_000, 130_000, 0), (640, 5760, 1152, 1), (33278, 650, 65, 1),
                                        (7, 24_576, 1228, 1), (8, 20_000, 1000, 1), (8, 20_000, 18_000, 0),
                                        (8, 30_000, 27_000, 0), (1, 1, 1, 1), (3, 8191, 8191, 1), (20_000, 66, 6, 1),
                                        (5, 24_577, 100, 0), (33, 1023, 2046, 1),
                                        # rows too long for whole row lists: tall matrices take the panels, matrices
                                        # with few rows (or a sketch too wide for LDS) the binned passes in row groups
                                        (4096, 25_088, 2508, 2), (4096, 25_088, 12_544, 2), (16, 50_000, 5000, 0),
                                        (9, 100_000, 10_000, 0), (64, 200_000, 20_000, 0), (9, 1_300_000, 130_000, 0),
                                        (2000, 30_000, 30_000, 0), (1024, 24_577, 2457, 2)])
def test_which_kind_of_plan_a_shape_gets(n, d, w, kind):
    from conef_amd import _lib
    lib = _lib.load()
    nb = lib.conef_plan_bytes(n, d, w, 0, 0)
    assert nb > 0
    buf = np.zeros(nb, np.uint8)
    assert lib.conef_plan_build_host(buf.ctypes.data, nb, n, d, w, A, B, 0, 0) == 0
    assert lib.conef_plan_kind(buf.ctypes.data) == kind


def test_plan_argument_checks():
    from conef_amd import _lib
    lib = _lib.load()
    assert lib.conef_plan_bytes(9, 100_000, 100, 0, 0) > 0        # long rows and more than 8 of them: binned, in row groups
    assert lib.conef_plan_bytes(9, 1000, 100, 0, 0) > 0           # short rows: row lists, any number of rows
    assert lib.conef_plan_bytes(9, 1000, 100, 1024, 64) > 0       # a binned plan was asked for
    assert lib.conef_plan_bytes(8 * 65536, 100_000, 100, 1024, 64) == 0   # more row groups than a grid dimension holds
    assert lib.conef_plan_bytes(0, 1000, 100, 0, 0) == -1
    buf = np.zeros(64, np.uint8)
    assert lib.conef_plan_build_host(buf.ctypes.data, 64, 5, 1000, 100, A, B, 0, 0) == -1   # buffer too small
    assert lib.conef_plan_workspace_bytes(buf.ctypes.data) == -1                            # not a plan
