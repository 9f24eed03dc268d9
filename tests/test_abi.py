"""CPU-side checks of the shipped library: it loads, exports every function
include/sub1_hip.h declares, builds the same dictionary as the oracle (and so
as the reference, see test_oracle_dictionary.py), and rejects bad arguments
before touching a GPU."""
import ctypes
import os
import re

import numpy as np
import pytest

from qmoe_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, 'include', 'sub1_hip.h')).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return re.findall(r'\b(sub1_[a-z0-9_]+)\s*\(', text)


def test_every_declared_symbol_is_exported_and_bound():
    names = set(declared_functions())
    assert {'sub1_matvec', 'sub1_pack_count', 'sub1_pack_emit', 'sub1_decode',
            'sub1_moe_grouped', 'sub1_build_tables'} <= names
    lib = _lib.load()
    for name in names:
        assert hasattr(lib, name), name
        assert name in _lib.PROTOTYPES, name
    assert set(_lib.PROTOTYPES) == names
    assert lib.sub1_abi_version() == 4


def test_header_constants_match_binding():
    text = open(os.path.join(ROOT, 'include', 'sub1_hip.h')).read()
    assert int(re.search(r'#define SUB1_MAX_WIDTH (\d+)', text).group(1)) == _lib.MAX_WIDTH
    assert int(re.search(r'#define SUB1_DICT_ENTRIES (\d+)', text).group(1)) == _lib.DICT_ENTRIES


def test_library_dictionary_equals_oracle(oracle):
    lib = _lib.load()
    dec = np.zeros(_lib.DEC_WORDS, dtype=np.int32)
    trie = np.zeros(_lib.TRIE_ROWS * 9, dtype=np.int32)
    assert lib.sub1_build_tables(dec.ctypes.data, trie.ctypes.data) == 0
    odec, otrie = oracle.tables()
    assert np.array_equal(dec, odec)
    assert np.array_equal(trie.reshape(-1, 9), otrie)
    # either output may be omitted
    assert lib.sub1_build_tables(None, None) == 0


def test_bad_arguments_are_refused_on_the_host():
    lib = _lib.load()
    one = ctypes.c_void_p(256)          # aligned, never dereferenced: checks come first
    odd = ctypes.c_void_p(257)
    assert lib.sub1_matvec(None, one, one, one, one, one, 8, 8, None) == -1
    assert b'NULL' in lib.sub1_last_error()
    assert lib.sub1_matvec(one, one, one, one, one, one, 8, 0, None) == -2
    assert lib.sub1_matvec(one, one, one, one, one, one, 0, 8, None) == -2
    assert lib.sub1_matvec(one, odd, one, one, one, one, 8, 8, None) == -3
    assert lib.sub1_pack_count(None, one, one, 8, 8, None) == -1
    assert lib.sub1_pack_count(one, one, one, 0, 8, None) == -2
    assert lib.sub1_pack_emit(one, one, None, 8, 8, None) == -1
    assert lib.sub1_decode(one, one, None, one, one, one, one, 8, 8, None) == -1
    assert lib.sub1_decode(one, one, one, None, None, one, None, 8, 8, None) == -1
    st = _lib.MoeStack()
    assert lib.sub1_moe_grouped(ctypes.byref(st), one, one, one, 4, one, 1 << 20, None) == -1
    # the grouped launch on the packed layout stages a row of activations in LDS
    wide = _lib.MoeStack(256, 256, 256, 256, 256, 256, 256, 256, 1, _lib.MAX_WIDTH + 1, 8)
    assert lib.sub1_moe_grouped(ctypes.byref(wide), one, one, one, 4, one, 1 << 30, None) == -2
    with pytest.raises(_lib.Sub1Error) as err:
        _lib.check(lib.sub1_matvec(one, one, one, one, one, one, 8, 0, None))
    assert err.value.status == -2 and 'width' in str(err.value)


def test_workspace_size():
    """The workspace holds a fixed head (control words and the tagged copy of h
    for launches of a token or two), a 64-byte word per token and h; its size
    is a multiple of 256, grows with the batch, and h of 64 tokens of a
    Switch-c-2048 layer fits what the static array of the entry point that
    does not allocate keeps for it."""
    lib = _lib.load()
    head = lib.sub1_moe_workspace_bytes(0, 3072)
    assert head == lib.sub1_moe_workspace_bytes(0, 8) and head % 256 == 0
    assert head >= 64 * 4 + 2 * 12288 * 8
    last = head
    for tokens in (1, 2, 3, 64, 65, 1000):
        need = lib.sub1_moe_workspace_bytes(tokens, 6144)
        assert need % 256 == 0 and need > last
        assert head + tokens * (64 + 6144 * 2) <= need < head + tokens * (64 + 6144 * 2) + 256
        last = need
    # the static array: control words for STATIC_MAX_TOKENS, h in the rest
    h_room = _lib.STATIC_SCRATCH_BYTES - lib.sub1_moe_workspace_bytes(_lib.STATIC_MAX_TOKENS, 0)
    assert 64 * 6144 * 2 <= h_room < 128 * 6144 * 2
    assert lib.sub1_moe_workspace_bytes(-1, 8) == 0


def test_python_surface_imports_without_a_gpu():
    from qmoe_amd import sub1, sub1_hip
    assert sub1.dec.shape == (_lib.DEC_WORDS,) and sub1.trie.shape == (_lib.TRIE_ROWS, 9)
    lin = sub1.Sub1Linear(16, 5)
    assert set(dict(lin.named_buffers())) == {'w_comp', 'row_off', 'ter_minmax', 'weight'}
    assert lin.w_comp.dtype.__str__() == 'torch.int16' and lin.row_off.shape == (17,)
    assert lin.ter_minmax.shape == (32,) and lin.weight.numel() == 0
    assert callable(sub1_hip.sub1matvec) and callable(sub1_hip.sub1pack)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it exits with a message that
    says so, before touching any GPU."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    res = subprocess.run([sys.executable, os.path.join(root, 'bench.py'), '--gpus', '2'],
                         capture_output=True, text=True, timeout=120)
    assert res.returncode != 0
    assert 'one GPU' in res.stderr
