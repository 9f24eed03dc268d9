"""CPU oracle for the QMoE sub-1-bit codec: Python side.

TEST INFRASTRUCTURE ONLY.  Imported by ``tests/``, by ``__graft_entry__.smoke()``
and by ``bench.py``'s cpu_baseline leg, as the checker or the timed CPU figure;
never by the shipped package.

Two things live here:

* ``COracle`` - ctypes access to ``oracle/_build/libsub1_oracle.so`` (the C
  restatement in ``sub1_oracle.c``; build it with ``make -C oracle``).
* A second, independent restatement in Python/numpy of the same reference
  semantics, written with different algorithms so that agreement between the
  two is evidence rather than repetition:

  - ``enumerate_dictionary``   closed form of sub1.py:49-57 (bounded DFS + sort,
                               no heap)
  - ``pack_dec`` / ``flat_trie``  sub1.py:60-72 / sub1.py:74-97
  - ``greedy_row``             test.py:86-100 (dict-of-dict trie walk)
  - ``expand_codes``           test.py:103-115 (works on the entry strings, not
                               on the packed dec words)

Reference line numbers are into the reference checkout (sub1.py, test.py,
sub1_cuda_kernel.cu).
"""
import ctypes
import os
import subprocess

import numpy as np

COUNT = 2 ** 16      # sub1.py:30
ZEROS = .885         # sub1.py:31
MAX_PAIRS = 14       # sub1.py:54
TRIE_ROOT = COUNT    # sub1.py:89

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, '_build', 'libsub1_oracle.so')


def build_c_oracle():
    """Compile oracle/sub1_oracle.c (gcc only, a second or two)."""
    subprocess.check_call(['make', '-C', _HERE, '-s'])
    return _LIB_PATH


# --------------------------------------------------------------------- bf16 --

def f32_to_bf16_bits(a):
    """float32 array -> uint16 bf16 bit patterns, round-to-nearest-even."""
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7fff + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


# ----------------------------------------------- independent Python oracle --

def pair_probabilities(zeros=ZEROS):
    """The nine pair probabilities, index r = 3a+b, value (1.0*p[a])*p[b] in
    IEEE double (the association sub1.py:37-43 produces)."""
    p = [zeros, (1 - zeros) / 2, (1 - zeros) / 2]
    return [(1. * p[a]) * p[b] for a in range(3) for b in range(3)]


def enumerate_dictionary(count=COUNT, max_pairs=MAX_PAIRS, zeros=ZEROS):
    """Dictionary entries as tuples of pair symbols, in index order.

    sub1.py:49-57 pops a min-heap keyed (negated probability, pair list) and
    pushes the nine extensions of every popped string shorter than max_pairs.
    An extension's key is strictly larger than its parent's, so the pop order
    is the sorted order of ALL strings of 1..max_pairs pairs under
    (key, list-lexicographic), where a string's key is the left-to-right double
    product (((-1*q[s0])*q[s1])*...).  This function takes that closed form
    literally: enumerate every string whose key is below a cut, sort, truncate.
    """
    q = pair_probabilities(zeros)
    cut = -1e-5
    while True:
        found = []
        stack = [(-1., ())]
        while stack:
            key, seq = stack.pop()
            if len(seq) == max_pairs:
                continue
            for s in range(9):
                k = key * q[s]
                if k <= cut:            # keys only grow along a string
                    child = (k, seq + (s,))
                    found.append(child)
                    stack.append(child)
        if len(found) >= count:
            break
        total = sum(9 ** n for n in range(1, max_pairs + 1))
        if len(found) == total:
            raise ValueError('fewer than %d strings exist' % count)
        cut /= 4
    found.sort()
    # everything below the cut was enumerated, so the first `count` are exact
    return [seq for _, seq in found[:count]]


def pack_dec(entries):
    """uint32 words of the decode table (returned as int32), sub1.py:60-72."""
    dec = np.zeros(2 * len(entries), dtype=np.uint32)
    for i, seq in enumerate(entries):
        for half in range(2):
            word = 0
            for j, r in enumerate(seq[7 * half:7 * half + 7]):
                word |= ((r % 3) | ((r // 3) << 2)) << (4 * j)
            dec[2 * i + half] = (word << 4) | len(seq)
    return dec.astype(np.int32)


def dict_trie(entries):
    """Nested-dict trie {symbol: subtrie, -1: entry index}, sub1.py:74-84."""
    root = {}
    for i, seq in enumerate(entries):
        node = root
        for s in seq:
            node = node.setdefault(s, {})
        node[-1] = i
    return root


def flat_trie(entries):
    """int32 [count+1, 9] child table with the root in the last row,
    sub1.py:86-97."""
    n = len(entries)
    index = {seq: i for i, seq in enumerate(entries)}
    arr = np.full((n + 1, 9), -1, dtype=np.int32)
    for seq, i in index.items():
        parent = index[seq[:-1]] if len(seq) > 1 else n
        arr[parent, seq[-1]] = i
    return arr


def row_to_pairs(trits):
    """Pair symbols of one row: 3*w[i+1] + w[i]; an odd tail keeps w[i] only
    (sub1_cuda_kernel.cu:223-228)."""
    t = [int(v) for v in trits]
    if len(t) % 2:
        t.append(0)
    return [3 * t[i + 1] + t[i] for i in range(0, len(t), 2)]


def greedy_row(pairs, root):
    """Greedy longest-match parse of one row over the nested-dict trie,
    test.py:86-100."""
    out = []
    node = root
    for s in pairs:
        if s not in node:
            out.append(node[-1])
            node = root
        node = node[s]
    if -1 in node:
        out.append(node[-1])
    return out


def expand_codes(codes, entries, width):
    """Symbols of one row from its codes, via the entry strings
    (test.py:103-115: low digit first, digits past the width dropped)."""
    out = []
    for c in codes:
        for r in entries[int(c)]:
            out.append(r % 3)
            out.append(r // 3)
    if len(out) not in (width, width + 1):
        raise ValueError('codes cover %d weights, row has %d' % (len(out), width))
    return out[:width]


# ------------------------------------------------------------- C oracle ----

class COracle:
    """ctypes front end of sub1_oracle.c.  Arrays are numpy, bf16 values are
    uint16 bit patterns."""

    def __init__(self, path=_LIB_PATH):
        if not os.path.exists(path):
            build_c_oracle()
        self.lib = ctypes.CDLL(path)
        L = self.lib
        vp = ctypes.c_void_p
        L.sub1o_build_tables.argtypes = [vp, vp]
        L.sub1o_build_tables.restype = ctypes.c_int
        L.sub1o_dictionary_entries.argtypes = [vp, vp]
        L.sub1o_dictionary_entries.restype = ctypes.c_int
        L.sub1o_encode.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, vp,
                                   ctypes.c_int64, vp]
        L.sub1o_encode.restype = ctypes.c_int64
        L.sub1o_decode.argtypes = [vp, vp, vp, ctypes.c_int, ctypes.c_int, vp]
        L.sub1o_decode.restype = ctypes.c_int
        L.sub1o_dequant.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, vp]
        L.sub1o_dequant.restype = None
        for name in ('sub1o_matvec_lanes', 'sub1o_matvec_seq', 'sub1o_matvec_wave'):
            f = getattr(L, name)
            f.argtypes = [vp] * 6 + [ctypes.c_int, ctypes.c_int]
            f.restype = None
        L.sub1o_matvec_gap.argtypes = [vp] * 6 + [ctypes.c_int, ctypes.c_int]
        L.sub1o_matvec_gap.restype = ctypes.c_int
        L.sub1o_gap_entries.argtypes = [vp, vp, ctypes.c_int, ctypes.c_int, vp, ctypes.c_int]
        L.sub1o_gap_entries.restype = ctypes.c_int
        L.sub1o_matvec_f64.argtypes = [vp] * 5 + [ctypes.c_int, ctypes.c_int]
        L.sub1o_matvec_f64.restype = None
        L.sub1o_expert_ffn.argtypes = [vp] * 10 + [ctypes.c_int] * 3
        L.sub1o_expert_ffn.restype = None
        self._tables = None

    @staticmethod
    def _p(a):
        return a.ctypes.data_as(ctypes.c_void_p)

    def tables(self):
        """(dec int32[131072], trie int32[65537, 9]), cached."""
        if self._tables is None:
            dec = np.zeros(2 * COUNT, dtype=np.int32)
            trie = np.zeros((COUNT + 1, 9), dtype=np.int32)
            rc = self.lib.sub1o_build_tables(self._p(dec), self._p(trie))
            if rc:
                raise RuntimeError('sub1o_build_tables failed: %d' % rc)
            self._tables = (dec, trie)
        return self._tables

    def entries(self):
        """(list of pair-symbol tuples, float64 keys) in index order."""
        raw = np.zeros((COUNT, 15), dtype=np.uint8)
        keys = np.zeros(COUNT, dtype=np.float64)
        rc = self.lib.sub1o_dictionary_entries(self._p(raw), self._p(keys))
        if rc:
            raise RuntimeError('sub1o_dictionary_entries failed: %d' % rc)
        return [tuple(int(v) for v in row[1:1 + row[0]]) for row in raw], keys

    def encode(self, w_tern, trie=None):
        """int32 [H, W] symbols -> (codes uint16 [C], row_off int32 [H+1])."""
        trie = self.tables()[1] if trie is None else trie
        w_tern = np.ascontiguousarray(w_tern, dtype=np.int32)
        h, w = w_tern.shape
        cap = h * ((w + 1) // 2)          # one code per pair at worst
        codes = np.zeros(max(cap, 1), dtype=np.uint16)
        row_off = np.zeros(h + 1, dtype=np.int32)
        n = self.lib.sub1o_encode(self._p(trie), self._p(w_tern), h, w,
                                  self._p(codes), cap, self._p(row_off))
        if n < 0:
            raise RuntimeError('sub1o_encode overflow')
        return codes[:n].copy(), row_off

    def decode(self, codes, row_off, width, dec=None):
        """-> uint8 [H, W] symbols."""
        dec = self.tables()[0] if dec is None else dec
        codes = np.ascontiguousarray(codes, dtype=np.uint16)
        row_off = np.ascontiguousarray(row_off, dtype=np.int32)
        h = row_off.shape[0] - 1
        tern = np.zeros((h, width), dtype=np.uint8)
        rc = self.lib.sub1o_decode(self._p(dec), self._p(codes), self._p(row_off),
                                   h, width, self._p(tern))
        if rc:
            raise ValueError('row %d does not cover its width' % (rc - 1))
        return tern

    def dequant(self, tern, ter_minmax):
        tern = np.ascontiguousarray(tern, dtype=np.uint8)
        mm = np.ascontiguousarray(ter_minmax, dtype=np.uint16)
        h, w = tern.shape
        out = np.zeros((h, w), dtype=np.uint16)
        self.lib.sub1o_dequant(self._p(tern), self._p(mm), h, w, self._p(out))
        return out

    def _matvec(self, fn, codes, row_off, ter_minmax, x, y, dec):
        dec = self.tables()[0] if dec is None else dec
        codes = np.ascontiguousarray(codes, dtype=np.uint16)
        row_off = np.ascontiguousarray(row_off, dtype=np.int32)
        mm = np.ascontiguousarray(ter_minmax, dtype=np.uint16)
        x = np.ascontiguousarray(x, dtype=np.uint16)
        h = row_off.shape[0] - 1
        y = np.zeros(h, dtype=np.uint16) if y is None else \
            np.array(y, dtype=np.uint16, copy=True)
        fn(self._p(dec), self._p(codes), self._p(row_off), self._p(mm),
           self._p(x), self._p(y), h, x.shape[0])
        return y

    def matvec_lanes(self, codes, row_off, ter_minmax, x, y=None, dec=None):
        """Reference kernel arithmetic; returns y (+= onto the given y)."""
        return self._matvec(self.lib.sub1o_matvec_lanes, codes, row_off,
                            ter_minmax, x, y, dec)

    def matvec_seq(self, codes, row_off, ter_minmax, x, y=None, dec=None):
        """Per-symbol stream-order arithmetic; returns y."""
        return self._matvec(self.lib.sub1o_matvec_seq, codes, row_off,
                            ter_minmax, x, y, dec)

    def matvec_wave(self, codes, row_off, ter_minmax, x, y=None, dec=None):
        """Wavefront-per-row order (codeword i in lane i mod 64, butterfly over
        the 64 lane sums); returns y."""
        return self._matvec(self.lib.sub1o_matvec_wave, codes, row_off,
                            ter_minmax, x, y, dec)

    def matvec_gap(self, codes, row_off, ter_minmax, x, y=None, dec=None):
        """Prepared-stream order (groups of 72 gap entries, one fused
        multiply-add per entry); returns y."""
        return self._matvec(self.lib.sub1o_matvec_gap, codes, row_off,
                            ter_minmax, x, y, dec)

    def gap_entries(self, row_codes, width, dec=None):
        """uint8 steps of one row's prepared stream."""
        dec = self.tables()[0] if dec is None else dec
        row_codes = np.ascontiguousarray(row_codes, dtype=np.uint16)
        cap = width + width // 40 + 8
        out = np.zeros(cap, dtype=np.uint8)
        n = self.lib.sub1o_gap_entries(self._p(dec), self._p(row_codes), row_codes.shape[0],
                                       width, self._p(out), cap)
        if n < 0 or n > cap:
            raise ValueError('the codes do not cover the width')
        return out[:n].copy()

    def matvec_f64(self, tern, ter_minmax, x):
        """-> (y float64 [H], sum |w*x| float64 [H]) on the decoded matrix."""
        tern = np.ascontiguousarray(tern, dtype=np.uint8)
        mm = np.ascontiguousarray(ter_minmax, dtype=np.uint16)
        x = np.ascontiguousarray(x, dtype=np.uint16)
        h, w = tern.shape
        y = np.zeros(h, dtype=np.float64)
        ya = np.zeros(h, dtype=np.float64)
        self.lib.sub1o_matvec_f64(self._p(tern), self._p(mm), self._p(x),
                                  self._p(y), self._p(ya), h, w)
        return y, ya

    def expert_ffn(self, wi, wo, x, order=0, dec=None):
        """wo(relu(wi(x))) for one token.  wi/wo = (codes, row_off, ter_minmax).
        order: 0 lane order, 1 per-symbol stream order, 2 prepared-stream
        order, 3 wavefront-per-row order.
        Returns (y uint16 [d_model], h uint16 [d_ff])."""
        dec = self.tables()[0] if dec is None else dec
        a = [np.ascontiguousarray(wi[0], dtype=np.uint16),
             np.ascontiguousarray(wi[1], dtype=np.int32),
             np.ascontiguousarray(wi[2], dtype=np.uint16),
             np.ascontiguousarray(wo[0], dtype=np.uint16),
             np.ascontiguousarray(wo[1], dtype=np.int32),
             np.ascontiguousarray(wo[2], dtype=np.uint16)]
        x = np.ascontiguousarray(x, dtype=np.uint16)
        d_model = x.shape[0]
        d_ff = a[1].shape[0] - 1
        y = np.zeros(d_model, dtype=np.uint16)
        h = np.zeros(d_ff, dtype=np.uint16)
        self.lib.sub1o_expert_ffn(self._p(dec), *[self._p(v) for v in a],
                                  self._p(x), self._p(y), self._p(h),
                                  d_model, d_ff, order)
        return y, h


# ------------------------------------------------- synthetic workloads -----

def synthetic_ternary(height, width, p_zero, seed):
    """Seeded iid symbols {0,1,2} with P(0)=p_zero, P(1)=P(2)=(1-p_zero)/2,
    per-row scale s ~ U(0.01, 0.05) stored as ter_minmax = (bf16(-s), bf16(+s)).
    Returns (w_tern int32 [H,W], ter_minmax uint16 [2H])."""
    rng = np.random.default_rng(seed)
    u = rng.random((height, width))
    t = np.zeros((height, width), dtype=np.int32)
    t[u >= p_zero] = 1
    t[u >= p_zero + (1 - p_zero) / 2] = 2
    s = rng.uniform(0.01, 0.05, size=height).astype(np.float32)
    mm = np.empty(2 * height, dtype=np.uint16)
    mm[0::2] = f32_to_bf16_bits(-s)
    mm[1::2] = f32_to_bf16_bits(s)
    return t, mm


def synthetic_activation(width, seed):
    """x ~ N(0,1) rounded to bf16 (uint16 bit patterns)."""
    rng = np.random.default_rng(seed)
    return f32_to_bf16_bits(rng.standard_normal(width).astype(np.float32))
