"""CPU oracle for the ConEF compress + error-feedback path (numpy front end).

TEST INFRASTRUCTURE ONLY.  This module wraps ``libconef_oracle.so`` (built from
``conef_oracle.c`` next to it) and restates, on numpy arrays, the per-bucket
logic of the reference hooks at world size 1 (every all-reduce is the identity
followed by a division by 1).  Only tests, the smoke check and the CPU-baseline
leg of the benchmark may import it; the shipped package never does.

Reference lines restated here (paths relative to the reference checkout):
  communication/compressors/CountSketch.py:102-182        -> DenseCS
  communication/compressors/CountSketchHash3.py:152-238   -> DenseCSHash3
  communication/compressors/halfCountSketch.py:110-197    -> HalfDenseCS
  communication/RandomBlock_hook.py:138-295               -> RandomBlockOracle
  communication/UnbiasedRandomBlock_hook.py:98-219        -> UnbiasedRandomBlockOracle
  communication/powerSGD_hook.py:280-580                  -> PowerSGDOracle
  communication/hPowerSGD_hook.py:90-97,274-570           -> HPowerSGDOracle, topk_sparsify
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libconef_oracle.so")

HASH_A = 994443   # CountSketch.py:112
HASH_B = 609478   # CountSketch.py:113

_lib_handle = None


def build():
    """Compile the C restatement (gcc, a second or two)."""
    subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libconef_oracle.so"])


def _lib():
    global _lib_handle
    if _lib_handle is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        f32p = ctypes.POINTER(ctypes.c_float)
        i32p = ctypes.POINTER(ctypes.c_int32)
        i64, i32, f32 = ctypes.c_int64, ctypes.c_int32, ctypes.c_float
        L.conef_oracle_mix.restype = i32
        L.conef_oracle_mix.argtypes = [i32, i32, i32]
        L.conef_oracle_hash.restype = i32
        L.conef_oracle_hash.argtypes = [i32, i32, i32, i32]
        L.conef_oracle_median3.restype = f32
        L.conef_oracle_median3.argtypes = [f32, f32, f32]
        L.conef_oracle_hash_table.restype = None
        L.conef_oracle_hash_table.argtypes = [i32p, i32p, i64, i32, i32, i32, i32, i32]
        L.conef_oracle_cs_query.restype = None
        L.conef_oracle_cs_query.argtypes = [f32p, f32p, i64, i64, i32, f32, i32, i32]
        L.conef_oracle_cs_update.restype = None
        L.conef_oracle_cs_update.argtypes = [f32p, f32p, i64, i64, i32, f32, i32, i32]
        L.conef_oracle_cs3_query.restype = None
        L.conef_oracle_cs3_query.argtypes = [f32p, f32p, f32p, f32p, i64, i64, i32, f32]
        L.conef_oracle_cs3_update.restype = None
        L.conef_oracle_cs3_update.argtypes = [f32p, f32p, f32p, f32p, i64, i64, i32, f32]
        L.conef_oracle_gram_schmidt.restype = None
        L.conef_oracle_gram_schmidt.argtypes = [f32p, i64, i64, i64, f32]
        for name in ("conef_oracle_mq", "conef_oracle_mtp"):
            getattr(L, name).restype = None
            getattr(L, name).argtypes = [f32p, f32p, f32p, i64, i64, i64]
        L.conef_oracle_pqt.restype = None
        L.conef_oracle_pqt.argtypes = [f32p, f32p, f32p, i64, i64, i64]
        L.conef_oracle_randblock_conef_step.restype = None
        L.conef_oracle_randblock_conef_step.argtypes = [f32p, f32p, f32p, i64, i64, i32, i64, i64,
                                                        f32, f32, i32, i32]
        _lib_handle = L
    return _lib_handle


def _f32(a):
    assert isinstance(a, np.ndarray) and a.dtype == np.float32 and a.flags["C_CONTIGUOUS"], \
        "oracle wants C-contiguous float32 numpy arrays"
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def _i32(a):
    assert a.dtype == np.int32 and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_int32))


# ------------------------------------------------------------------ scalars --

def mix(value, a=HASH_A, b=HASH_B):
    """Pre-modulo hash value (always >= 0)."""
    return int(_lib().conef_oracle_mix(value, a, b))


def hash_bucket(value, w, a=HASH_A, b=HASH_B):
    return int(_lib().conef_oracle_hash(value, w, a, b))


def median3(a, b, c):
    return float(_lib().conef_oracle_median3(a, b, c))


def hash_table(d, w, a=HASH_A, b=HASH_B, sa=None, sb=None):
    """(bucket[d], sign[d]) as int32 arrays; sign is +1/-1."""
    sa = a + 2 if sa is None else sa
    sb = b + 3 if sb is None else sb
    bucket = np.empty(d, dtype=np.int32)
    sign = np.empty(d, dtype=np.int32)
    _lib().conef_oracle_hash_table(_i32(bucket), _i32(sign), d, w, a, b, sa, sb)
    return bucket, sign


def sketch_width(d, sketch_size):
    """CountSketch.py:107"""
    return max(int(d * sketch_size), 1)


# ----------------------------------------------------------- raw operations --

def cs_query(x, cs, alpha, a=HASH_A, b=HASH_B):
    n, d = x.shape
    assert cs.shape[0] == n
    _lib().conef_oracle_cs_query(_f32(x), _f32(cs), n, d, cs.shape[1], np.float32(alpha), a, b)


def cs_update(vec, cs, beta, a=HASH_A, b=HASH_B):
    n, d = vec.shape
    assert cs.shape[0] == n
    _lib().conef_oracle_cs_update(_f32(vec), _f32(cs), n, d, cs.shape[1], np.float32(beta), a, b)


def cs3_query(x, cs0, cs1, cs2, alpha):
    n, d = x.shape
    _lib().conef_oracle_cs3_query(_f32(x), _f32(cs0), _f32(cs1), _f32(cs2), n, d, cs0.shape[1],
                                  np.float32(alpha))


def cs3_update(vec, cs0, cs1, cs2, beta):
    n, d = vec.shape
    _lib().conef_oracle_cs3_update(_f32(vec), _f32(cs0), _f32(cs1), _f32(cs2), n, d, cs0.shape[1],
                                   np.float32(beta))


def gram_schmidt(a, eps=0.0):
    """In place on a C-contiguous [rows, cols] float32 array."""
    rows, cols = a.shape
    _lib().conef_oracle_gram_schmidt(_f32(a), rows, cols, cols, np.float32(eps))


def mq(mat, q):
    n, m = mat.shape
    r = q.shape[1]
    p = np.empty((n, r), dtype=np.float32)
    _lib().conef_oracle_mq(_f32(mat), _f32(q), _f32(p), n, m, r)
    return p


def mtp(mat, p):
    n, m = mat.shape
    r = p.shape[1]
    q = np.empty((m, r), dtype=np.float32)
    _lib().conef_oracle_mtp(_f32(mat), _f32(p), _f32(q), n, m, r)
    return q


def pqt(p, q):
    n, r = p.shape
    m = q.shape[0]
    mat = np.empty((n, m), dtype=np.float32)
    _lib().conef_oracle_pqt(_f32(p), _f32(q), _f32(mat), n, m, r)
    return mat


def randblock_conef_step(x, cs, payload, start, block, alpha, beta, a=HASH_A, b=HASH_B):
    """All-C fused restatement of one RandomBlock+ConEF step (used for CPU timing)."""
    n, m = x.shape
    _lib().conef_oracle_randblock_conef_step(_f32(x), _f32(cs), _f32(payload), n, m, cs.shape[1],
                                             start, block, np.float32(alpha), np.float32(beta), a, b)


def randblock_conef_step_threaded(x, cs, payload, start, block, alpha, beta, threads, a=HASH_A, b=HASH_B):
    """The same step with the rows of the sketch (they are independent: every row reads and writes
    only its own cells) spread over ``threads`` host threads; the foreign calls release the GIL.
    Same arithmetic per row, so bit-identical to ``randblock_conef_step``.  Used for CPU timing."""
    from concurrent.futures import ThreadPoolExecutor
    n, m = x.shape
    numel = n * m
    end = min(start + block, numel)
    rest = block - (end - start)
    flat = x.reshape(-1)

    def per_row(fn):
        with ThreadPoolExecutor(max_workers=max(1, min(threads, n))) as pool:
            list(pool.map(fn, range(n)))

    per_row(lambda r: cs_query(x[r:r + 1], cs[r:r + 1], alpha, a, b))
    payload[:end - start] = flat[start:end]
    cp = x.copy()
    cpf = cp.reshape(-1)
    cpf[start:end] = 0
    if rest > 0:
        payload[end - start:] = flat[:rest]
        cpf[:rest] = 0
    per_row(lambda r: cs_update(cp[r:r + 1], cs[r:r + 1], beta, a, b))
    flat[:] = 0
    flat[start:end] = payload[:end - start]
    if rest > 0:
        flat[:rest] = payload[end - start:]


def block_bounds(numel, ratio, start):
    """RandomBlock_hook.py:216-223 -> (block, end, rest)."""
    block = max(1, int(ratio * numel))
    end = min(start + block, numel)
    rest = block - (end - start)
    return block, end, rest


def topk_sparsify(err, topk_ratio):
    """hPowerSGD_hook.py:90-97: keep the k = max(1, int(0.5*ratio*numel)) entries of largest
    magnitude, zero the rest, in place.  The reference calls topk(sorted=False) and so leaves
    ties open; here ties on the threshold magnitude keep the lowest flat indices."""
    flat = err.reshape(-1)
    k = max(1, int(0.5 * topk_ratio * flat.size))
    order = np.argsort(-np.abs(flat), kind="stable")[:k]
    vals = flat[order].copy()
    flat[:] = 0
    flat[order] = vals
    return k


def should_compress(n, m, rank, min_rate):
    """powerSGD_hook.py:46-70"""
    return (n + m) * rank * min_rate < n * m


# ------------------------------------------------------- compressor classes --

class DenseCS:
    """CountSketch.py:102-182 on numpy."""

    def __init__(self, N, D, sketch_size):
        self.N, self.D = N, D
        self.range = sketch_width(D, sketch_size)
        self.cs = np.zeros((N, self.range), dtype=np.float32)
        self.a, self.b = HASH_A, HASH_B

    def update(self, vec, beta):
        cs_update(vec.reshape(self.N, self.D), self.cs, beta, self.a, self.b)

    def query(self, x, alpha):
        cs_query(x.reshape(self.N, self.D), self.cs, alpha, self.a, self.b)

    def clean(self, alpha):
        self.cs *= np.float32(alpha)


class HalfDenseCS(DenseCS):
    """halfCountSketch.py:110-197: fp16 storage, fp32 arithmetic, whole-sketch casts around
    every call (:152,168,176,194)."""

    def __init__(self, N, D, sketch_size):
        super().__init__(N, D, sketch_size)
        self.cs = self.cs.astype(np.float16)

    def update(self, vec, beta):
        cs32 = self.cs.astype(np.float32)
        cs_update(vec.reshape(self.N, self.D), cs32, beta, self.a, self.b)
        self.cs = cs32.astype(np.float16)

    def query(self, x, alpha):
        cs32 = self.cs.astype(np.float32)
        cs_query(x.reshape(self.N, self.D), cs32, alpha, self.a, self.b)
        self.cs = cs32.astype(np.float16)

    def clean(self, alpha):
        # halfCountSketch.py:196-197: mul_ on the fp16 tensor (computed in fp32, rounded to fp16)
        self.cs = (self.cs.astype(np.float32) * np.float32(alpha)).astype(np.float16)


class DenseCSHash3:
    """CountSketchHash3.py:152-238 on numpy."""

    def __init__(self, N, D, sketch_size):
        self.N, self.D = N, D
        self.range = sketch_width(D, sketch_size)
        self.cs0 = np.zeros((N, self.range), dtype=np.float32)
        self.cs1 = np.zeros((N, self.range), dtype=np.float32)
        self.cs2 = np.zeros((N, self.range), dtype=np.float32)

    def update(self, vec, beta):
        cs3_update(vec.reshape(self.N, self.D), self.cs0, self.cs1, self.cs2, beta)

    def query(self, x, alpha):
        cs3_query(x.reshape(self.N, self.D), self.cs0, self.cs1, self.cs2, alpha)

    def clean(self, alpha):
        for c in (self.cs0, self.cs1, self.cs2):
            c *= np.float32(alpha)


# ------------------------------------------------------------ hook oracles --
# A "bucket" is a flat float32 numpy buffer plus the list of parameter shapes laid out in it,
# exactly what GradBucket.buffer()/gradients() give the reference hooks.

def split_bucket(flat, shapes):
    """Per-parameter views into the flat buffer (GradBucket.gradients())."""
    out, off = [], 0
    for shp in shapes:
        cnt = int(np.prod(shp)) if len(shp) else 1
        out.append(flat[off:off + cnt].reshape(shp))
        off += cnt
    assert off == flat.size
    return out


class RandomBlockOracle:
    """RandomBlock_hook.py:16-135 (state) and :138-295 (hook body) at world size 1."""

    def __init__(self, compression_ratio=0.1, use_error_compression=False, beta=0.9, sketch_size=0.5,
                 use_error_feedback=True, random_seed=42):
        self.compression_ratio = compression_ratio
        self.use_error_compression = use_error_compression
        self.use_error_feedback = use_error_feedback
        self.beta, self.sketch_size = beta, sketch_size
        self.rng = np.random.RandomState(random_seed)   # :92
        self.error_dict = {}
        self.compressed_tensor_memory = {}
        self.last_starts = []

    def step(self, bucket_index, flat, shapes):
        """Runs one compressed step in place on ``flat``; returns the payload."""
        if bucket_index not in self.error_dict:
            self.error_dict[bucket_index] = []
        errs = self.error_dict[bucket_index]
        mats = []
        for t in split_bucket(flat, shapes):                      # :170-193
            if t.ndim <= 1:
                continue
            mat = t.reshape(t.shape[0], -1)
            cnt = len(mats)
            if not self.use_error_compression:
                if len(errs) <= cnt:
                    errs.append(np.zeros_like(mat))
                mat += errs[cnt]                                    # :182
                errs[cnt] = mat.copy()                              # :184
            else:
                if len(errs) <= cnt:
                    errs.append(DenseCS(mat.shape[0], mat.shape[1], self.sketch_size))
                errs[cnt].query(mat, 1 - self.beta)                 # :190
            mats.append(mat)
        blocks = [max(1, int(self.compression_ratio * m.size)) for m in mats]
        if bucket_index not in self.compressed_tensor_memory:       # :205-209
            self.compressed_tensor_memory[bucket_index] = np.empty(sum(blocks), dtype=np.float32)
        payload = self.compressed_tensor_memory[bucket_index]
        idx, sel = 0, []
        self.last_starts = []
        for mat, err, block in zip(mats, errs, blocks):             # :215-245
            flatm = mat.reshape(-1)
            start = int(self.rng.choice(flatm.size))                # :218
            self.last_starts.append(start)
            end = min(start + block, flatm.size)
            rest = block - (end - start)
            payload[idx:idx + end - start] = flatm[start:end]
            if rest > 0:
                payload[idx + end - start:idx + block] = flatm[:rest]
            if not self.use_error_compression:
                ef = err.reshape(-1)
                ef[start:end] = 0                                    # :228
                if rest > 0:
                    ef[:rest] = 0                                    # :240
            else:
                cp = mat.copy()                                      # :231
                cpf = cp.reshape(-1)
                cpf[start:end] = 0
                if rest > 0:
                    cpf[:rest] = 0
                err.update(cp, self.beta)                            # :234 / :243 (exactly once)
            sel.append((start, end, rest, block, idx))
            idx += block
        for mat, (start, end, rest, block, idx) in zip(mats, sel):   # :271-281
            flatm = mat.reshape(-1)
            flatm[:] = 0
            flatm[start:end] = payload[idx:idx + end - start]
            if rest > 0:
                flatm[:rest] = payload[idx + end - start:idx + block]
        return payload


class UnbiasedRandomBlockOracle:
    """UnbiasedRandomBlock_hook.py:12-95 (state) and :98-219 (hook body) at world size 1."""

    def __init__(self, compression_ratio=0.1, random_seed=42):
        self.compression_ratio = compression_ratio
        self.rng = np.random.RandomState(random_seed)   # :74
        self.compressed_tensor_memory = {}
        self.last_starts = []

    def step(self, bucket_index, flat, shapes):
        tens = [t for t in split_bucket(flat, shapes) if t.ndim > 1]
        blocks = [max(1, int(self.compression_ratio * t.size)) for t in tens]
        if bucket_index not in self.compressed_tensor_memory:
            self.compressed_tensor_memory[bucket_index] = np.empty(sum(blocks), dtype=np.float32)
        payload = self.compressed_tensor_memory[bucket_index]
        idx = 0
        self.last_starts = []
        for t, block in zip(tens, blocks):
            f = t.reshape(-1)
            prob = np.float32(block / f.size)                        # :155, fp32 tensor / python float
            start = int(self.rng.choice(f.size))                     # :157
            self.last_starts.append(start)
            end = min(start + block, f.size)
            rest = block - (end - start)
            payload[idx:idx + end - start] = f[start:end] / prob     # :161-162
            if rest > 0:
                payload[idx + end - start:idx + block] = f[:rest] / prob
            f[:] = 0                                                  # :200
            f[start:end] = payload[idx:idx + end - start]
            if rest > 0:
                f[:rest] = payload[idx + end - start:idx + block]
            idx += block
        return payload


class PowerSGDOracle:
    """powerSGD_hook.py:89-277 (state) and :280-580 (hook body) at world size 1.
    ``error_mode``: None (no EF), 'ef' (dense error over the whole bucket), 'conef' (count sketch
    per compressed matrix), 'conef_v2' (C2CS_hook_v2, :791-1092: the sketch is DenseCS(m, n) over
    the [m,n] re-view of the matrix's memory, :918-920,1074-1076), 'topk'
    (hPowerSGD_hook.py:393-400,549-554: dense per-matrix error, sparsified by magnitude after
    each step)."""

    def __init__(self, matrix_approximation_rank=1, min_compression_rate=2, error_mode="ef", beta=0.9,
                 sketch_size=0.5, topk_ratio=0.4, warm_start=True, orthogonalization_epsilon=0,
                 random_seed=0):
        self.rank = matrix_approximation_rank
        self.min_rate = min_compression_rate
        self.error_mode = error_mode
        self.beta, self.sketch_size, self.topk_ratio = beta, sketch_size, topk_ratio
        self.warm_start = warm_start
        self.eps = orthogonalization_epsilon
        self.rng = np.random.RandomState(random_seed)   # :218
        self.error_dict, self.p_memory_dict, self.q_memory_dict = {}, {}, {}
        self.last_seed = None

    def step(self, bucket_index, flat, shapes):
        import torch  # only for the seeded CPU randn that initialises Q (:485-493)

        cp_flat = None
        if self.error_mode == "ef":                                   # :359-375
            if bucket_index in self.error_dict:
                flat += self.error_dict[bucket_index]
            else:
                self.error_dict[bucket_index] = np.zeros_like(flat)
            cp_flat = flat.copy()
        elif self.error_mode in ("conef", "conef_v2", "topk"):
            self.error_dict.setdefault(bucket_index, {})
        mats, copies, ranks = [], [], []
        for t in split_bucket(flat, shapes):                          # :394-418
            mat = t.reshape(t.shape[0], -1)
            n, m = mat.shape
            r = min(n, m, self.rank)
            if not should_compress(n, m, r, self.min_rate):
                continue
            cnt = len(mats)
            errs = self.error_dict.get(bucket_index)
            if self.error_mode == "conef":
                if cnt not in errs:
                    errs[cnt] = DenseCS(n, m, self.sketch_size)
                errs[cnt].query(mat, 1 - self.beta)                   # :409
                copies.append(mat.copy())                             # :410
            elif self.error_mode == "conef_v2":
                if cnt not in errs:
                    errs[cnt] = DenseCS(m, n, self.sketch_size)       # :918
                errs[cnt].query(mat.reshape(m, n), 1 - self.beta)     # :920 (a view of the same memory)
                copies.append(mat.copy())
            elif self.error_mode == "topk":
                if cnt not in errs:
                    errs[cnt] = np.zeros_like(mat)
                mat += errs[cnt]                                      # hPowerSGD_hook.py:399
                copies.append(mat.copy())
            mats.append(mat)
            ranks.append(r)
        need_randomize = (not self.warm_start) or bucket_index not in self.p_memory_dict   # :434-436
        if need_randomize:
            self.p_memory_dict[bucket_index] = [np.empty((m.shape[0], r), dtype=np.float32)
                                                for m, r in zip(mats, ranks)]
            self.q_memory_dict[bucket_index] = [np.empty((m.shape[1], r), dtype=np.float32)
                                                for m, r in zip(mats, ranks)]
        ps, qs = self.p_memory_dict[bucket_index], self.q_memory_dict[bucket_index]
        if not need_randomize:
            for q in qs:
                gram_schmidt(q, self.eps)                             # :475-477
        else:
            with torch.random.fork_rng(devices=[]):                   # :479-494
                self.last_seed = int(self.rng.randint(1_000_000_000))
                torch.manual_seed(self.last_seed)
                for q in qs:
                    q[...] = torch.randn(*q.shape, device="cpu", dtype=torch.float32).numpy()
                    gram_schmidt(q, self.eps)
        for i, (mat, q) in enumerate(zip(mats, qs)):
            ps[i][...] = mq(np.ascontiguousarray(mat), q)             # :498
        for p in ps:
            gram_schmidt(p, self.eps)                                 # :527-528
        for i, (mat, p) in enumerate(zip(mats, ps)):
            qs[i][...] = mtp(np.ascontiguousarray(mat), p)            # :532
        for mat, p, q in zip(mats, ps, qs):
            mat[...] = pqt(p, q)                                      # :551
        if self.error_mode == "ef":
            self.error_dict[bucket_index] = cp_flat - flat            # :558
        elif self.error_mode == "conef":
            for cnt, (mat, cp) in enumerate(zip(mats, copies)):
                cp -= mat                                             # :563
                self.error_dict[bucket_index][cnt].update(cp, self.beta)   # :564
        elif self.error_mode == "conef_v2":
            for cnt, (mat, cp) in enumerate(zip(mats, copies)):
                n, m = mat.shape
                cp -= mat                                             # :1075
                self.error_dict[bucket_index][cnt].update(cp.reshape(m, n), self.beta)   # :1076
        elif self.error_mode == "topk":
            for cnt, (mat, cp) in enumerate(zip(mats, copies)):
                err = cp - mat                                        # hPowerSGD_hook.py:553
                topk_sparsify(err, self.topk_ratio)                   # :554
                self.error_dict[bucket_index][cnt] = err
        if not self.warm_start:
            self.p_memory_dict.clear()
            self.q_memory_dict.clear()


class BatchedPowerSGDOracle:
    """batched_powerSGD_hook (powerSGD_hook.py:583-787) at world size 1: the flat bucket, padded
    with zeros to a square of side ceil(sqrt(length)) (:657-663), is one matrix; dense error over
    the padded length (:669-687); P, Q are [side, rank]; Q is orthogonalised on every call (:733)."""

    def __init__(self, matrix_approximation_rank=1, use_error_feedback=True, warm_start=True,
                 orthogonalization_epsilon=0, random_seed=0):
        self.rank = matrix_approximation_rank
        self.use_error_feedback, self.warm_start = use_error_feedback, warm_start
        self.eps = orthogonalization_epsilon
        self.rng = np.random.RandomState(random_seed)
        self.error_dict, self.p_memory_dict, self.q_memory_dict = {}, {}, {}

    def step(self, bucket_index, flat, shapes=None):
        import math

        import torch

        total = flat.shape[0]
        side = math.ceil(math.sqrt(total))
        while side * side < total:          # guard against sqrt rounding on large lengths
            side += 1
        padded = np.zeros(side * side, dtype=np.float32)
        padded[:total] = flat
        cp = None
        if self.use_error_feedback:
            if bucket_index in self.error_dict:
                padded += self.error_dict[bucket_index]
            else:
                self.error_dict[bucket_index] = np.zeros_like(padded)
            cp = padded.copy()
        mat = padded.reshape(side, side)
        if not self.warm_start or bucket_index not in self.p_memory_dict:
            self.p_memory_dict[bucket_index] = np.empty((side, self.rank), dtype=np.float32)
            with torch.random.fork_rng(devices=[]):
                torch.manual_seed(int(self.rng.randint(1_000_000_000)))
                self.q_memory_dict[bucket_index] = torch.randn(side, self.rank, device="cpu",
                                                               dtype=torch.float32).numpy().copy()
        p, q = self.p_memory_dict[bucket_index], self.q_memory_dict[bucket_index]
        gram_schmidt(q, self.eps)
        p[...] = mq(mat, q)
        gram_schmidt(p, self.eps)
        q[...] = mtp(mat, p)
        mat[...] = pqt(p, q)
        if self.use_error_feedback:
            self.error_dict[bucket_index] = cp - padded
        if not self.warm_start:
            self.p_memory_dict.clear()
            self.q_memory_dict.clear()
        flat[...] = padded[:total]
