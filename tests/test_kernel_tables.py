"""The renumbered code space and its decode table (sub1_build_kernel_tables),
checked on the CPU against the dictionary itself: decoding every kernel code
through the table, the way the kernels do, must give back exactly the entry
the code stands for."""
import numpy as np

from qmoe_amd import _lib


def build():
    lib = _lib.load()
    recode = np.zeros(65536, dtype=np.uint16)
    table = np.zeros(16384, dtype=np.uint32)
    nb = np.zeros(1, dtype=np.int32)
    words = np.zeros(1, dtype=np.int32)
    assert lib.sub1_build_kernel_tables(recode.ctypes.data, table.ctypes.data,
                                        nb.ctypes.data, words.ctypes.data) == 0
    return recode, table, int(nb[0]), int(words[0])


def decode_kernel_code(c, table, nb):
    """(pair count, [(position, symbol)] in slot order) as the kernels see code c."""
    idx = c if c < nb else nb + ((c - nb) >> 3)
    word = int(table[idx])
    slots = []
    empty_seen = False
    for j, shift in enumerate((0, 8, 24)):                    # bytes 0, 1, 3 hold the slots
        f = ((word >> shift) & 0xfe) | ((c >> j) & 1)         # low bit comes from the code
        if f in (4, 5) and j < 2 or f in (0x82, 0x83) and j == 2:
            empty_seen = True
            continue                                          # a zero dword: empty slot
        assert not empty_seen                                 # non-zeros fill the slots from slot 0
        m, rem = divmod(f, 6)
        assert rem < 4 and f < 128
        slots.append((2 * m + rem // 2, 1 + (rem & 1)))
    advance = (word >> 16) & 0xff
    assert advance % 6 == 0
    return advance // 6, slots


def test_sizes_and_bijection():
    recode, table, nb, words = build()
    assert nb == 8224 and words == 8224 + 7164            # 61.5 KB of table
    assert words <= 16384 and nb % 8 == 0
    assert np.array_equal(np.sort(recode), np.arange(65536, dtype=np.uint16))
    # the index the kernels compute: min(c, (c >> 3) + nb - nb/8)
    c = np.arange(65536)
    direct = np.where(c < nb, c, nb + ((c - nb) >> 3))
    assert np.array_equal(np.minimum(c, (c >> 3) + nb - nb // 8), direct)
    assert direct.max() == words - 1


def test_every_code_decodes_to_its_entry(entries):
    recode, table, nb, _ = build()
    for e, seq in enumerate(entries):
        want = []
        for j, r in enumerate(seq):
            if r % 3:
                want.append((2 * j, r % 3))
            if r // 3:
                want.append((2 * j + 1, r // 3))
        npairs, slots = decode_kernel_code(int(recode[e]), table, nb)
        assert npairs == len(seq)
        assert sorted(slots) == want
        # non-zeros that feed the same sum keep their column order
        for sym in (1, 2):
            cols = [p for p, s in slots if s == sym]
            assert cols == sorted(cols)


def test_size_query_only():
    lib = _lib.load()
    nb = np.zeros(1, dtype=np.int32)
    assert lib.sub1_build_kernel_tables(None, None, nb.ctypes.data, None) == 0
    assert nb[0] == 8224
