"""Pins the oracle's dictionary (oracle/sub1_oracle.c sub1o_build_tables and
oracle/sub1_oracle.py enumerate_dictionary) WITHOUT trusting either:

  * golden: SHA-256 and samples of the tables the reference's own setup()
    produced (tests/golden/dictionary_golden.json, made by
    tests/golden/make_dictionary_golden.py);
  * known answers derived by hand from reference sub1.py:31-72
    (p0=.885, p1=p2=.0575: pair probabilities .783225, .0508875, .00330625);
  * brute force on a tiny dictionary (all 819 strings of <= 3 pairs sorted);
  * structural invariants of the construction;
  * two implementations with different algorithms (C heap, Python DFS+sort).
"""
import hashlib
import itertools
import json
import os

import numpy as np

from oracle import sub1_oracle as so

GOLDEN = os.path.join(os.path.dirname(__file__), 'golden', 'dictionary_golden.json')


def test_tables_match_reference_golden(oracle):
    with open(GOLDEN) as f:
        g = json.load(f)
    dec, trie = oracle.tables()
    assert hashlib.sha256(dec.tobytes()).hexdigest() == g['dec_sha256']
    assert hashlib.sha256(trie.tobytes()).hexdigest() == g['trie_sha256']
    for i, words in g['dec_samples'].items():
        assert [int(dec[2 * int(i)]), int(dec[2 * int(i) + 1])] == words
    for r, row in g['trie_samples'].items():
        assert [int(v) for v in trie[int(r)]] == row


def test_python_restatement_matches_c(oracle, entries):
    ent = so.enumerate_dictionary()
    assert ent == entries
    dec, trie = oracle.tables()
    assert np.array_equal(so.pack_dec(ent), dec)
    assert np.array_equal(so.flat_trie(ent), trie)


def test_hand_derived_known_answers(oracle, entries):
    z = lambda n: (0,) * n
    # zero runs of 1..12 pairs outrank every string with a non-zero
    assert entries[:12] == [z(n) for n in range(1, 13)]
    # .0508875 > .783225**13 = .0417: the four single-non-zero pairs come next,
    # in symbol order because their keys tie
    assert entries[12:16] == [(1,), (2,), (3,), (6,)]
    assert entries[16] == z(13)
    assert entries[17:25] == [(0, 1), (0, 2), (0, 3), (0, 6), (1, 0), (2, 0), (3, 0), (6, 0)]
    assert entries[25] == z(14)
    dec, trie = oracle.tables()
    assert dec[0] == 1 and dec[1] == 1                 # one zero pair, length 1
    assert dec[24] == (1 << 4) | 1 and dec[25] == 1    # pair symbol 1: even weight = 1
    assert dec[26] == (2 << 4) | 1                     # symbol 2: even weight = 2
    assert dec[28] == (1 << 6) | 1                     # symbol 3: odd weight = 1
    assert dec[30] == (2 << 6) | 1                     # symbol 6: odd weight = 2
    assert dec[50] == 14 and dec[51] == 14             # fourteen zero pairs
    root = trie[so.TRIE_ROOT]
    assert list(root[[0, 1, 2, 3, 6]]) == [0, 12, 13, 14, 15]
    assert all(root >= 0)                              # every single pair is an entry


def test_brute_force_tiny_dictionary():
    q = so.pair_probabilities()
    strings = []
    for n in (1, 2, 3):
        for seq in itertools.product(range(9), repeat=n):
            key = -1.
            for s in seq:
                key = key * q[s]
            strings.append((key, seq))
    strings.sort()
    for count in (9, 64, 300, 819):
        assert so.enumerate_dictionary(count=count, max_pairs=3) == \
            [seq for _, seq in strings[:count]]


def test_structural_invariants(oracle, entries):
    dec, trie = oracle.tables()
    keys = oracle.entries()[1]
    assert len(set(entries)) == so.COUNT
    index = {seq: i for i, seq in enumerate(entries)}
    assert np.all(np.diff(keys) >= 0)                  # probability never increases
    for i, seq in enumerate(entries):
        assert 1 <= len(seq) <= so.MAX_PAIRS
        if len(seq) > 1:
            assert index[seq[:-1]] < i                 # prefix closed, parent first
    lens = np.array([len(s) for s in entries])
    assert np.array_equal(dec[0::2] & 15, lens) and np.array_equal(dec[1::2] & 15, lens)
    # digits beyond the entry's length are zero
    u = dec.view(np.uint32).reshape(-1, 2).astype(np.uint64)
    digits = (u[:, 0] >> 4) | ((u[:, 1] >> 4) << 28)
    assert not np.any(digits >> (4 * lens).astype(np.uint64))
    # no digit equals 3
    assert not np.any(digits & (digits >> np.uint64(1)) & np.uint64(0x55555555555555))
    # at most three non-zero weights per entry: what the one-word slot form relies on
    nz = np.array([sum((r % 3 != 0) + (r // 3 != 0) for r in s) for s in entries])
    assert nz.max() == 3
    # the trie holds each entry exactly once
    vals = trie[trie >= 0]
    assert np.array_equal(np.sort(vals), np.arange(so.COUNT))
