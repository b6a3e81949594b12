"""PowerSGD rounds at ranks above 32.

The reference's hooks take any ``matrix_approximation_rank`` (communication/powerSGD_hook.py:146-160);
the kernels of this package keep the rank dimension in registers or in one 32-wide matrix-core tile.
A wider factor is therefore cut into column chunks of at most 32, each a contiguous [rows, width]
matrix of its own, and the round (powerSGD_hook.py:473-564) is put together from the batch entry
points on those chunks:

  * the products are independent per chunk: P_c = X Q_c, Q_c = X^T P_c;
  * the Gram-Schmidt of the reference (powerSGD_hook.py:21-43: normalise a column, take its component
    out of every later column) runs chunk by chunk: chunk b is orthogonalised by the kernels, then
    every later chunk loses its components along chunk b, A_c <- A_c - Q_b (Q_b^T A_c).  Taking the
    components along the (orthogonal) columns of Q_b out one after the other, as the reference does,
    or all at once differs by the rounding of the dot products only;
  * M = P Q^T is the sum of the chunks' products: the first chunk's launch leaves its product in the
    matrix and the residual X - M_0 in a scratch buffer, the next takes that residual as its input,
    and the products are added up in chunk order.

Nothing here is tuned: a bucket's round is some forty launches where rank 32 takes ten.  It exists so
that a rank the reference accepts is not refused.
"""
import ctypes

import torch

from . import _lib

CHUNK = 32


def chunk_widths(rank):
    """Column chunks of a rank-``rank`` factor: the remainder first, then whole chunks of 32, so that
    a later chunk is never narrower than an earlier one (the projection of chunk c against chunk b
    is a product whose long side is chunk c's)."""
    return ([rank % CHUNK] if rank % CHUNK else []) + [CHUNK] * (rank // CHUNK)


def _items(entries):
    """A PsgdItem table from (x, err, p, q, n, m, r) tuples of device pointers and sizes."""
    arr = (_lib.PsgdItem * max(len(entries), 1))()
    for it, (x, err, p, q, n, m, r) in zip(arr, entries):
        it.x, it.err, it.p, it.q, it.n, it.m, it.r, it.w = x, err, p, q, n, m, r, 1
    return arr


class _Factor:
    """The column chunks of the [rows, rank] factors of a bucket's matrices, two buffers a chunk:
    a projection reads one and writes the other, so chunk c, projected c times by the time its own
    turn comes, ends up in buffer c % 2."""

    def __init__(self, shapes, device):
        # shapes: (rows, rank) per matrix
        self.shapes = shapes
        self.widths = [chunk_widths(r) for _, r in shapes]
        self.offsets = [[sum(w[:c]) for c in range(len(w))] for w in self.widths]
        self.buf = [[(torch.empty(rows, wd, device=device), torch.empty(rows, wd, device=device)) for wd in w]
                    for (rows, _), w in zip(shapes, self.widths)]
        self.coef = [torch.empty(CHUNK * CHUNK, device=device) for _ in shapes]
        self.most = max(len(w) for w in self.widths)
        self.gs = []          # per block b: (ptrs, rows, ranks, count) of conef_gram_schmidt_batch_f32
        self.proj = []        # per block b: [(item table, count)] of the later chunks' projections, one per later chunk index
        for b in range(self.most):
            members = [k for k, w in enumerate(self.widths) if len(w) > b]
            mats = [self.buf[k][b][b % 2] for k in members]
            self.gs.append(((ctypes.c_void_p * len(mats))(*[t.data_ptr() for t in mats]),
                            (ctypes.c_int64 * len(mats))(*[t.shape[0] for t in mats]),
                            (ctypes.c_int32 * len(mats))(*[t.shape[1] for t in mats]), len(mats)))
            # later chunks lose their components along chunk b: one launch pair per later chunk index (the
            # matrices of a bucket each keep one coefficient buffer, so a pair holds one chunk per matrix)
            groups = []
            for c in range(b + 1, self.most):
                entries = []
                for k in members:
                    if len(self.widths[k]) <= c:
                        continue
                    qb = self.buf[k][b][b % 2]
                    src, dst = self.buf[k][c][b % 2], self.buf[k][c][(b + 1) % 2]
                    # C = A_c^T Q_b ([w_c, w_b], into coef), then A_c - Q_b C^T into the other buffer
                    entries.append((src.data_ptr(), dst.data_ptr(), qb.data_ptr(), self.coef[k].data_ptr(),
                                    src.shape[0], src.shape[1], qb.shape[1]))
                if entries:
                    groups.append((_items(entries), len(entries)))
            self.proj.append(groups)

    def start(self, k, c):
        """Where chunk c of matrix k is written before the orthogonalisation."""
        return self.buf[k][c][0]

    def final(self, k, c):
        """Where it is afterwards."""
        return self.buf[k][c][c % 2]

    def split(self, factors):
        for k, f in enumerate(factors):
            for c, (o, wd) in enumerate(zip(self.offsets[k], self.widths[k])):
                self.start(k, c).copy_(f[:, o:o + wd])

    def merge(self, factors, where):
        for k, f in enumerate(factors):
            for c, (o, wd) in enumerate(zip(self.offsets[k], self.widths[k])):
                f[:, o:o + wd].copy_(where(k, c))

    def orthogonalize(self, lib, eps, ws_ptr, ws_len, stream):
        """The reference's Gram-Schmidt over all columns, chunk by chunk."""
        for b in range(self.most):
            ptrs, rows, ranks, count = self.gs[b]
            _lib.check(lib.conef_gram_schmidt_batch_f32(ptrs, rows, ranks, count, eps, ws_ptr, ws_len, stream),
                       "conef_gram_schmidt_batch_f32")
            for table, cnt in self.proj[b]:
                _lib.check(lib.conef_psgd_mtp_batch_f32(table, cnt, ws_ptr, ws_len, stream), "conef_psgd_mtp_batch_f32")
                _lib.check(lib.conef_psgd_pqt_batch_f32(table, cnt, 1, 0.0, 0, 0, stream), "conef_psgd_pqt_batch_f32")


class WideRound:
    """The launches of one bucket's round at a rank above 32, built once per bucket layout."""

    def __init__(self, work, ps, qs, device):
        lib = _lib.load()
        self.work = work
        self.p = _Factor([(n, r) for _, n, m, r in work], device)
        self.q = _Factor([(m, r) for _, n, m, r in work], device)
        count = len(work)
        mq, mtp = [], []
        for k, (matrix, n, m, r) in enumerate(work):
            for c in range(len(self.p.widths[k])):
                wd = self.p.widths[k][c]
                # P_c = X Q_c with the orthogonalised Q_c; Q_c = X^T P_c with the orthogonalised P_c
                mq.append((matrix.data_ptr(), None, self.p.start(k, c).data_ptr(), self.q.final(k, c).data_ptr(), n, m, wd))
                mtp.append((matrix.data_ptr(), None, self.p.final(k, c).data_ptr(), self.q.start(k, c).data_ptr(), n, m, wd))
        self.mq, self.mtp, self.n_products = _items(mq), _items(mtp), len(mq)
        # M = sum of the chunks' products, the residual handed from chunk to chunk
        total = sum(n * m for _, n, m, _ in work)
        self.res = [torch.empty(max(total, 1), device=device), torch.empty(max(total, 1), device=device)]
        self.own_dest = torch.empty(max(total, 1), device=device)
        self.chain = []           # per chunk index: (items, count, [(k, offset of matrix k in the scratch buffers)])
        offs, off = [], 0
        for _, n, m, _ in work:
            offs.append(off)
            off += n * m
        self.offs = offs
        for c in range(self.p.most):
            members = [k for k in range(count) if len(self.p.widths[k]) > c]
            entries = []
            for k in members:
                matrix, n, m, r = work[k]
                x = matrix.data_ptr() if c == 0 else self.res[(c - 1) % 2].data_ptr() + 4 * offs[k]
                err = self.res[c % 2].data_ptr() + 4 * offs[k]          # the last chunk's goes to the destination, per step
                entries.append((x, err, self.p.final(k, c).data_ptr(), self.q.start(k, c).data_ptr(), n, m, self.p.widths[k][c]))
            self.chain.append((_items(entries), len(entries), members))
        need = [lib.conef_psgd_batch_workspace_bytes(self.mq, self.n_products),
                lib.conef_psgd_batch_workspace_bytes(self.mtp, self.n_products)]
        for f in (self.p, self.q):
            for groups in f.proj:
                for table, cnt in groups:
                    need.append(lib.conef_psgd_batch_workspace_bytes(table, cnt))
        if min(need) < 0:
            raise ValueError("a matrix of this bucket does not fit the PowerSGD kernels")
        self.ws_need = max(max(need), 256)

    def run(self, lib, ps, qs, dest, eps, ws_ptr, ws_len, stream):
        """ps, qs: the state's [n, r] / [m, r] views; dest[k]: device pointer the residual of matrix k
        goes to (None: nobody wants it).  On entry every matrix holds X (its error already added) and
        qs the factors the round starts from; on exit the matrices hold P Q^T and ps, qs the round's
        factors, as powerSGD_hook.py:473-564 leaves them."""
        work = self.work
        self.q.split(qs)
        self.q.orthogonalize(lib, eps, ws_ptr, ws_len, stream)
        _lib.check(lib.conef_psgd_mq_batch_f32(self.mq, self.n_products, 0, 0.0, 0, 0, ws_ptr, ws_len, stream),
                   "conef_psgd_mq_batch_f32")
        self.p.orthogonalize(lib, eps, ws_ptr, ws_len, stream)
        self.p.merge(ps, self.p.final)
        _lib.check(lib.conef_psgd_mtp_batch_f32(self.mtp, self.n_products, ws_ptr, ws_len, stream), "conef_psgd_mtp_batch_f32")
        self.q.merge(qs, self.q.start)
        for c, (table, cnt, members) in enumerate(self.chain):
            for i, k in enumerate(members):
                if c == len(self.p.widths[k]) - 1:                 # the matrix's last chunk leaves the round's residual
                    table[i].err = dest[k] if dest[k] is not None else self.own_dest.data_ptr() + 4 * self.offs[k]
            _lib.check(lib.conef_psgd_pqt_batch_f32(table, cnt, 1, 0.0, 0, 0, stream), "conef_psgd_pqt_batch_f32")
            if c > 0:
                # this chunk's product sits where its input was: add it to the matrix (x += e; e = 0)
                for k in members:
                    matrix, n, m, _ = work[k]
                    rc = lib.conef_ef_passthrough_f32(matrix.data_ptr(), self.res[(c - 1) % 2].data_ptr() + 4 * self.offs[k],
                                                      n * m, stream)
                    _lib.check(rc, "conef_ef_passthrough_f32")
