"""Writes tests/golden/dictionary_golden.json from the reference's own
dictionary builder.

Run once, in the authoring container only (it needs the reference checkout):

    python tests/golden/make_dictionary_golden.py [/root/reference]

Why the reference is executed at all: the complete index order of the 65536
dictionary entries depends on IEEE-double products and Python tuple/list
tie-breaking deep in the table; closed forms, invariants and two independent
restatements pin it only up to "all restatements read the source the same
way".  The reference's `sub1` module cannot be imported (it imports the
unbuilt CUDA extension and indexes an empty GPU list at import), so only the
body of its `setup()` function is compiled, from the syntax tree, and called;
nothing else of the module runs.

The fixture holds data only: SHA-256 of the two tables' bytes and a few
hundred sampled words, so a mismatch can be localised.
"""
import ast
import hashlib
import heapq
import json
import os
import sys

import numpy as np
import torch


def reference_setup(ref_root):
    path = os.path.join(ref_root, 'sub1.py')
    with open(path) as f:
        tree = ast.parse(f.read(), filename=path)
    funcs = [n for n in tree.body if isinstance(n, ast.FunctionDef) and n.name == 'setup']
    if len(funcs) != 1:
        raise RuntimeError('expected exactly one setup() in %s' % path)
    module = ast.Module(body=funcs, type_ignores=[])
    scope = {'heapq': heapq, 'np': np, 'torch': torch}
    exec(compile(module, path, 'exec'), scope)
    dec, trie = scope['setup']()
    return dec.numpy(), trie.numpy()


def main():
    ref_root = sys.argv[1] if len(sys.argv) > 1 else '/root/reference'
    dec, trie = reference_setup(ref_root)
    assert dec.dtype == np.int32 and dec.shape == (131072,)
    assert trie.dtype == np.int32 and trie.shape == (65537, 9)
    entry_ids = sorted(set(list(range(0, 65536, 257)) + list(range(40)) + [65535]))
    trie_rows = sorted(set(list(range(0, 65537, 1021)) + [65536]))
    golden = {
        'source': 'reference sub1.py setup(), executed from its syntax tree',
        'dec_sha256': hashlib.sha256(dec.tobytes()).hexdigest(),
        'trie_sha256': hashlib.sha256(trie.tobytes()).hexdigest(),
        'dec_samples': {str(i): [int(dec[2 * i]), int(dec[2 * i + 1])] for i in entry_ids},
        'trie_samples': {str(r): [int(v) for v in trie[r]] for r in trie_rows},
    }
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), 'dictionary_golden.json')
    with open(out, 'w') as f:
        json.dump(golden, f, indent=1, sort_keys=True)
    print('wrote', out, golden['dec_sha256'], golden['trie_sha256'])


if __name__ == '__main__':
    main()
