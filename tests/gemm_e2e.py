"""The Gemm layer of the end-to-end configuration (N=8192, 5 limbs of 40 bits, y = W x with W 16x64) as a
CKKS evaluation: 15 hoisted rotations of the input, 16 plaintext products accumulated, two rotate-and-add
steps to fold the 64 partial sums into 16, one rescale.  The same sequence runs on the CPU oracle and, through
the C-ABI, on the GPU; inputs (keys, ciphertext, encoded weights) come from ckks_host.

Packing: x sits in slots 0..63 and repeats with period 64.  With u_d[k] = W[k mod 16][(k+d) mod 64],
z = sum_{d<16} u_d * rot(x, d) holds in slot k the partial sum of row k mod 16 over columns k+d, d<16, and
y_i = z_i + z_{i+16} + z_{i+32} + z_{i+48}.  (The compiler's Gemm programs have the same shape:
per-diagonal rotate, encode, multiply-accumulate, then log-step rotate-and-add:
fhe-cmplr/rtlib/ant/example/eg_fhertlib_gemm.inc.)
"""
import numpy as np

ROWS, COLS = 16, 64
CFG = (8192, 5, 40, 40, 3)
ROTS = list(range(1, ROWS)) + [32, 16]


def make_problem(seed):
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1.0, 1.0, COLS).astype(np.float32)
    w = rng.normal(0.0, 0.1, (ROWS, COLS)).astype(np.float32)
    return x, w


def diagonals(w):
    k = np.arange(COLS)
    return [w[k % ROWS, (k + d) % COLS].astype(np.float64) for d in range(ROWS)]


def prepare(host, x, w):
    """Keys, the encrypted input and the encoded diagonals (all host arrays)."""
    o = host.o
    L, scale = o.L, 2.0 ** CFG[3]
    keys = {r: host.rotation_key(o.find_automorphism_index(r)) for r in ROTS}
    orders = {r: o.automorphism_order(o.find_automorphism_index(r), True) for r in ROTS}
    ct = host.encrypt(host.encode(x.astype(np.float64), scale, L), host.public_key(), L)
    pts = [host.encode(u, scale, L) for u in diagonals(w)]
    return dict(keys=keys, orders=orders, ct=ct, pts=pts, scale=scale)


def evaluate(ev, prob, level):
    """ev: an evaluator (OracleEval / GpuEval).  Returns the result ciphertext at level-1 as host arrays."""
    c0, c1 = ev.put(prob["ct"][0]), ev.put(prob["ct"][1])
    pts = [ev.put(p) for p in prob["pts"]]
    rots = list(range(1, ROWS))
    rotated = [(c0, c1)] + ev.rotations(c0, c1, [prob["keys"][r] for r in rots], [prob["orders"][r] for r in rots], level)
    acc0, acc1 = ev.zeros(level), ev.zeros(level)
    for (r0, r1), pt in zip(rotated, pts):
        ev.mul_plain_acc(acc0, acc1, r0, r1, pt, level)
    for r in (32, 16):
        (s0, s1), = ev.rotations(acc0, acc1, [prob["keys"][r]], [prob["orders"][r]], level)
        acc0, acc1 = ev.add(acc0, s0, level), ev.add(acc1, s1, level)
    r0, r1 = ev.rescale(acc0, acc1, level)
    return ev.get(r0), ev.get(r1)


class OracleEval:
    def __init__(self, o):
        self.o, self.n = o, o.N

    def put(self, a):
        return np.array(a, dtype=np.int64)

    def get(self, a):
        return a

    def zeros(self, level):
        return np.zeros(level * self.n, np.int64)

    def rotations(self, c0, c1, keys, orders, level):
        digits = self.o.precomp(c1, level, True)
        return [self.o.fast_rotate(c0, digits, k, od, level) for k, od in zip(keys, orders)]

    def mul_plain_acc(self, acc0, acc1, r0, r1, pt, level):
        acc0[:] = self.o.poly("add", acc0, self.o.poly("mul", r0, pt, level), level)
        acc1[:] = self.o.poly("add", acc1, self.o.poly("mul", r1, pt, level), level)

    def add(self, a, b, level):
        return self.o.poly("add", a, b, level)

    def rescale(self, c0, c1, level):
        return self.o.rescale(c0, level, True), self.o.rescale(c1, level, True)


class GpuEval:
    """Every step is one call through the C-ABI; data stays in HBM between steps."""

    def __init__(self, g):
        self.g, self.n = g, g.N
        self._keys = {}

    def put(self, a):
        return self.g.upload(a)

    def get(self, a):
        return a.get()

    def zeros(self, level):
        return self.g.alloc(level * self.n)

    def _dev(self, arr):
        k = id(arr)
        if k not in self._keys:
            self._keys[k] = (arr, self.g.upload(arr))
        return self._keys[k][1]

    def rotations(self, c0, c1, keys, orders, level):
        m, n = len(keys), level * self.n
        s0, s1 = self.g.alloc(m * n), self.g.alloc(m * n)
        self.g.rotate_batch(s0, s1, c0, c1, [self._dev(k) for k in keys], [self._dev(od) for od in orders], level)
        return [(s0.view(i * n, n), s1.view(i * n, n)) for i in range(m)]

    def mul_plain_acc(self, acc0, acc1, r0, r1, pt, level):
        tmp = self.g.alloc(level * self.n)
        for acc, r in ((acc0, r0), (acc1, r1)):
            self.g.poly("mul", tmp, r, pt, level)
            self.g.poly("add", acc, acc, tmp, level)
        tmp.free()

    def add(self, a, b, level):
        self.g.poly("add", a, a, b, level)
        return a

    def rescale(self, c0, c1, level):
        r0, r1 = self.g.alloc((level - 1) * self.n), self.g.alloc((level - 1) * self.n)
        self.g.rescale_ciph(r0, r1, c0, c1, level)
        return r0, r1


def decode_result(host, r0, r1, level_out, scale_out):
    slots = host.decrypt_decode(r0, r1, level_out, scale_out)
    return np.real(slots[:ROWS])
