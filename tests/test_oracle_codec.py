"""Pins the oracle's encoder and decoder (sub1o_encode / sub1o_decode /
sub1o_dequant) by means that do not repeat their code:

  * known answers for all-zero rows (a zero run of 14 pairs is entry 25, of 6
    pairs entry 5, of 10 pairs entry 9 - see the dictionary known answers);
  * encode -> decode round trips where the DECODE side is the independent
    Python expansion of the entry strings (never the packed dec words);
  * the greedy parse restated as "longest dictionary string that prefixes the
    rest of the row", evaluated with a Python set;
  * greedy maximality of every emitted code;
  * a second encoder (nested-dict trie walk, reference test.py:86-100
    semantics) that must agree code for code;
  * edge cases: odd widths (reference sub1_cuda_kernel.cu:226 drops the
    missing high digit), width 1 and 2, rows that end exactly on an entry.
"""
import numpy as np
import pytest

from oracle import sub1_oracle as so


def rows_of(codes, row_off):
    return [codes[row_off[r]:row_off[r + 1]] for r in range(len(row_off) - 1)]


@pytest.mark.parametrize('width,full,tail_entry', [(768, 27, 5), (3072, 109, 9), (28, 1, None)])
def test_all_zero_rows_known_answer(oracle, width, full, tail_entry):
    t = np.zeros((3, width), dtype=np.int32)
    codes, row_off = oracle.encode(t)
    per_row = full + (tail_entry is not None)
    assert list(row_off) == [0, per_row, 2 * per_row, 3 * per_row]
    for row in rows_of(codes, row_off):
        assert list(row[:full]) == [25] * full
        if tail_entry is not None:
            assert row[full] == tail_entry


@pytest.mark.parametrize('height,width,p0', [(64, 768, 0.9), (32, 3072, 0.9), (16, 2080, 0.88),
                                             (40, 767, 0.9), (8, 1, 0.5), (8, 2, 0.5),
                                             (8, 29, 0.3), (8, 56, 0.0)])
def test_round_trip_against_independent_expansion(oracle, entries, height, width, p0):
    t, _ = so.synthetic_ternary(height, width, p0, seed=width)
    codes, row_off = oracle.encode(t)
    assert row_off[0] == 0 and row_off[-1] == len(codes)
    for r, row in enumerate(rows_of(codes, row_off)):
        assert so.expand_codes(row, entries, width) == list(t[r])
    # the C decoder says the same
    assert np.array_equal(oracle.decode(codes, row_off, width), t)


def test_greedy_is_longest_prefix_match(oracle, entries):
    known = set(entries)
    t, _ = so.synthetic_ternary(24, 600, 0.885, seed=7)
    codes, row_off = oracle.encode(t)
    for r, row in enumerate(rows_of(codes, row_off)):
        pairs = tuple(so.row_to_pairs(t[r]))
        pos = 0
        for c in row:
            n = 1
            while pos + n < len(pairs) and n < so.MAX_PAIRS and pairs[pos:pos + n + 1] in known:
                n += 1
            assert entries[c] == pairs[pos:pos + n]
            pos += n
        assert pos == len(pairs)


def test_emitted_codes_cannot_be_extended(oracle, entries):
    _, trie = oracle.tables()
    t, _ = so.synthetic_ternary(16, 1024, 0.9, seed=3)
    codes, row_off = oracle.encode(t)
    for r, row in enumerate(rows_of(codes, row_off)):
        pairs = so.row_to_pairs(t[r])
        pos = 0
        for c in row[:-1]:
            pos += len(entries[c])
            assert trie[c, pairs[pos]] == -1
        assert pos + len(entries[row[-1]]) == len(pairs)


def test_second_encoder_agrees(oracle, entries):
    root = so.dict_trie(entries)
    for width, p0 in [(768, 0.9), (333, 0.7), (2080, 0.885)]:
        t, _ = so.synthetic_ternary(12, width, p0, seed=width + 1)
        codes, row_off = oracle.encode(t)
        for r, row in enumerate(rows_of(codes, row_off)):
            assert so.greedy_row(so.row_to_pairs(t[r]), root) == list(row)


def test_row_ending_exactly_on_a_leaf(oracle, entries):
    # 14 zero pairs then a non-zero pair: [0]^14 is emitted when pair 15 cannot
    # extend it, and the single pair is flushed at the row end
    t = np.zeros((1, 30), dtype=np.int32)
    t[0, 28] = 2
    codes, row_off = oracle.encode(t)
    assert list(codes) == [25, 13] and list(row_off) == [0, 2]
    t[0, 28], t[0, 29] = 0, 1                       # pair symbol 3
    assert list(oracle.encode(t)[0]) == [25, 14]


def test_decode_rejects_wrong_coverage(oracle):
    with pytest.raises(ValueError):
        oracle.decode(np.array([25], dtype=np.uint16), np.array([0, 1], dtype=np.int32), 30)


def test_dequant_values(oracle):
    t, mm = so.synthetic_ternary(8, 64, 0.5, seed=11)
    w = oracle.dequant(t.astype(np.uint8), mm)
    lut = np.stack([np.zeros(8, np.uint16), mm[0::2], mm[1::2]], axis=1)
    assert np.array_equal(w, np.take_along_axis(lut, t.astype(np.int64), axis=1))
    # scales are U(0.01, 0.05), min = -max
    f = so.bf16_bits_to_f32(mm)
    assert np.all(f[0::2] == -f[1::2]) and np.all((f[1::2] > 0.0099) & (f[1::2] < 0.0501))
