"""ctypes binding of libsub1_hip.so (the C ABI declared in include/sub1_hip.h)."""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, 'libsub1_hip.so')

SUB1_OK = 0
DICT_ENTRIES = 65536
DEC_WORDS = 2 * DICT_ENTRIES
TRIE_ROWS = DICT_ENTRIES + 1
MAX_WIDTH = 12288
PREPARED_MAX_WIDTH = 12288
STATIC_SCRATCH_BYTES = 1 << 20   # SUB1_STATIC_SCRATCH_BYTES
STATIC_MAX_TOKENS = 512           # SUB1_STATIC_MAX_TOKENS

_vp = ctypes.c_void_p
_int = ctypes.c_int
_i64 = ctypes.c_int64


class MoeStack(ctypes.Structure):
    """struct sub1_moe_stack"""
    _fields_ = [('dec', _vp), ('w_comp', _vp), ('wi_code_base', _vp),
                ('wo_code_base', _vp), ('wi_row_off', _vp), ('wo_row_off', _vp),
                ('wi_minmax', _vp), ('wo_minmax', _vp), ('experts', ctypes.c_int32),
                ('d_model', ctypes.c_int32), ('d_ff', ctypes.c_int32)]


class MoeLayers(ctypes.Structure):
    """struct sub1_moe_layers"""
    _fields_ = [('dec', _vp), ('wi_w_comp', _vp), ('wo_w_comp', _vp), ('wi_row_off', _vp),
                ('wo_row_off', _vp), ('wi_minmax', _vp), ('wo_minmax', _vp),
                ('experts', ctypes.c_int32), ('d_model', ctypes.c_int32), ('d_ff', ctypes.c_int32)]


class MoePrepared(ctypes.Structure):
    """struct sub1_moe_prepared"""
    _fields_ = [('meta', _vp), ('codes', _vp), ('meta_bytes', _i64), ('code_bytes', _i64),
                ('total_chunks', _i64), ('experts', ctypes.c_int32),
                ('d_model', ctypes.c_int32), ('d_ff', ctypes.c_int32),
                ('max_chunks', ctypes.c_int32 * 2)]


class MatrixSet(ctypes.Structure):
    """struct sub1_matrix_set"""
    _fields_ = [('dec', _vp), ('w_comp', _vp), ('code_base', _vp), ('row_off', _vp),
                ('ter_minmax', _vp), ('count', ctypes.c_int32), ('height', ctypes.c_int32),
                ('width', ctypes.c_int32)]


class MatrixPrepared(ctypes.Structure):
    """struct sub1_matrix_prepared"""
    _fields_ = [('meta', _vp), ('codes', _vp), ('meta_bytes', _i64), ('code_bytes', _i64),
                ('total_chunks', _i64), ('count', ctypes.c_int32), ('height', ctypes.c_int32),
                ('width', ctypes.c_int32), ('max_chunks', ctypes.c_int32)]


class Tiles(ctypes.Structure):
    """struct sub1_tiles"""
    _fields_ = [('meta', _vp), ('entries', _vp), ('meta_bytes', _i64), ('entry_bytes', _i64),
                ('total_chunks', _i64), ('count', ctypes.c_int32), ('height', ctypes.c_int32),
                ('width', ctypes.c_int32)]


# every symbol include/sub1_hip.h declares, with its prototype
PROTOTYPES = {
    'sub1_last_error': (ctypes.c_char_p, []),
    'sub1_abi_version': (_int, []),
    'sub1_last_kernel': (ctypes.c_char_p, []),
    'sub1_build_tables': (_int, [_vp, _vp]),
    'sub1_matvec': (_int, [_vp] * 6 + [_int, _int, _vp]),
    'sub1_matvec_tokens': (_int, [_vp] * 6 + [_int, _int, _int, _i64, _i64, _vp]),
    'sub1_pack_count': (_int, [_vp, _vp, _vp, _int, _int, _vp]),
    'sub1_pack_emit': (_int, [_vp, _vp, _vp, _int, _int, _vp]),
    'sub1_decode': (_int, [_vp] * 7 + [_int, _int, _vp]),
    'sub1_moe_workspace_bytes': (_i64, [_int, _int]),
    'sub1_moe_grouped': (_int, [ctypes.POINTER(MoeStack), _vp, _vp, _vp, _int, _vp,
                                _i64, _vp]),
    'sub1_moe_prepared_meta_bytes': (_i64, [_int, _int, _int]),
    'sub1_moe_prepare_layout': (_int, [ctypes.POINTER(MoeStack), _vp, _i64,
                                       ctypes.POINTER(MoePrepared), _vp]),
    'sub1_moe_prepare_codes': (_int, [ctypes.POINTER(MoeStack), ctypes.POINTER(MoePrepared),
                                      _vp]),
    'sub1_moe_prepare_layout_from_layers': (_int, [ctypes.POINTER(MoeLayers), _vp, _i64,
                                                   ctypes.POINTER(MoePrepared), _vp]),
    'sub1_moe_prepare_codes_from_layers': (_int, [ctypes.POINTER(MoeLayers),
                                                  ctypes.POINTER(MoePrepared), _vp]),
    'sub1_moe_prepared_entry_counts': (_int, [ctypes.POINTER(MoePrepared),
                                              ctypes.POINTER(_i64), ctypes.POINTER(_i64), _vp]),
    'sub1_moe_grouped_prepared': (_int, [ctypes.POINTER(MoePrepared), _vp, _vp, _vp, _int,
                                         _vp, _i64, _vp]),
    'sub1_moe_grouped_prepared_static': (_int, [ctypes.POINTER(MoePrepared), _vp, _vp, _vp, _int,
                                                _vp]),
    'sub1_moe_prepared_decode': (_int, [ctypes.POINTER(MoePrepared), _int, _int, _vp, _vp]),
    'sub1_matrix_prepared_meta_bytes': (_i64, [_int, _int, _int]),
    'sub1_matrix_prepare_layout': (_int, [ctypes.POINTER(MatrixSet), _vp, _i64,
                                          ctypes.POINTER(MatrixPrepared), _vp]),
    'sub1_matrix_prepare_codes': (_int, [ctypes.POINTER(MatrixSet),
                                         ctypes.POINTER(MatrixPrepared), _vp]),
    'sub1_matvec_prepared': (_int, [ctypes.POINTER(MatrixPrepared), _vp, _vp, _i64, _vp, _i64,
                                    _int, _vp]),
    'sub1_matrix_prepared_decode': (_int, [ctypes.POINTER(MatrixPrepared), _int, _vp, _vp]),
    'sub1_tiles_meta_bytes': (_i64, [_int, _int, _int]),
    'sub1_tiles_layout': (_int, [ctypes.POINTER(MatrixSet), _vp, _i64, ctypes.POINTER(Tiles), _vp]),
    'sub1_tiles_entries': (_int, [ctypes.POINTER(MatrixSet), ctypes.POINTER(Tiles), _vp]),
    'sub1_matvec_tiles': (_int, [ctypes.POINTER(Tiles), _int, _vp, _i64, _vp, _i64, _int, _vp]),
    'sub1_tiles_decode': (_int, [ctypes.POINTER(Tiles), _int, _vp, _vp]),
    'sub1_route_from_mask': (_int, [_vp, _int, _int, _int, _vp, _vp, _vp]),
    'sub1_timing_begin': (_int, [_vp]),
    'sub1_timing_end': (_int, [_vp, ctypes.POINTER(ctypes.c_double)]),
    'sub1_init': (_int, []),
    'sub1_fault_flags': (_int, [ctypes.POINTER(ctypes.c_int32)]),
    'sub1_fault_words_host': (_vp, []),
    'sub1_clear_faults': (_int, []),
    'sub1_fault_epoch': (_i64, []),
    'sub1_static_scratch_reset': (_int, [_vp]),
    'sub1_static_scratch_pointer': (_int, [ctypes.POINTER(ctypes.c_void_p)]),
    'sub1_set_wait_limit_us': (_int, [_i64]),
    'sub1_test_overstate_wait': (_int, [_int]),
    'sub1_test_tiles_kernel': (_int, [_int]),
    'sub1_unregister_dec': (_int, [_vp]),
}

_lib = None


class Sub1Error(RuntimeError):
    def __init__(self, status, message):
        super().__init__('libsub1_hip status %d: %s' % (status, message))
        self.status = status


def load():
    """The loaded library.  There is no fallback: a missing library is an error."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                '%s is missing: build it with `python -m qmoe_amd.build` '
                '(hipcc, gfx950); there is no CPU fallback' % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(status):
    if status != SUB1_OK:
        raise Sub1Error(status, load().sub1_last_error().decode())


class Sub1Fault(RuntimeError):
    """A launch could not finish its work and said so through the library's
    sticky fault flags; outputs since the last check may be wrong."""


_fault_words = None


def check_faults():
    """Raise Sub1Fault if a launch has set a fault flag: a wait between
    workgroups gave up at its time limit (that launch's output is wrong), or a
    `dec` buffer changed under the table cached for its address.  Reads host
    memory, synchronises nothing: it reports what the GPU has got to so far.
    The flags stay up until clear_faults()."""
    global _fault_words
    if _fault_words is None:
        lib = load()
        check(lib.sub1_init())
        _fault_words = (ctypes.c_int32 * 2).from_address(lib.sub1_fault_words_host())
    if _fault_words[0] or _fault_words[1]:
        what = []
        if _fault_words[0]:
            what.append('a wait between workgroups ran into its time limit, so the output of '
                        'that launch is wrong')
        if _fault_words[1]:
            what.append('a dec tensor no longer holds what the table cached for its address '
                        'was derived from (sub1_unregister_dec before freeing one)')
        raise Sub1Fault('libsub1_hip: ' + '; '.join(what) + ' [sticky: clear_faults() resets]')


def clear_faults(stream=None):
    """Reset the fault flags, once the work that raised them has ended.  A wait
    fault may have left control words of its workspace at other values than
    zero: the stacks zero their workspaces again before the next launch (they
    compare fault_epoch(), which this call moves on), and the static scratch
    is zeroed here, on `stream` (the legacy default stream if None)."""
    lib = load()
    before = lib.sub1_fault_epoch()
    check(lib.sub1_clear_faults())
    if lib.sub1_fault_epoch() != before:
        check(lib.sub1_static_scratch_reset(stream))


def fault_epoch():
    """Wait faults cleared so far (see clear_faults)."""
    return load().sub1_fault_epoch()
