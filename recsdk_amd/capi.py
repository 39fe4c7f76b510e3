"""ctypes binding of librecsdk_hip.so (the C ABI declared in include/recsdk_hip.h).

The library is loaded from recsdk_amd/lib/.  It is never built here: run `python -m recsdk_amd.build`
(or __graft_entry__.build()) first.  There is no CPU fallback: every op raises if the library is missing.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int32, c_int64, c_uint32, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "librecsdk_hip.so")

OK = 0
EINVAL = -1
ENULL = -3
ENOMEM = -10
EOVERFLOW = -16
EHIP = -100
ENOTFOUND = -101
ECAPACITY = -102

DT_F32, DT_F16, DT_I32, DT_BF16, DT_I64 = 0, 1, 2, 3, 4
OPT_SGD, OPT_ADAGRAD, OPT_ADAM = 0, 1, 2
POOL_SUM, POOL_MEAN, POOL_NONE = 0, 1, 2
CHANNEL_TRAIN, CHANNEL_EVAL = 0, 1


class RecsdkError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"recsdk error {code}: {message}")
        self.code = code


_lib = None

# name -> (restype, argtypes); every symbol include/recsdk_hip.h declares
class InitializerDesc(ctypes.Structure):
    """recsdk_initializer_desc_t"""
    _fields_ = [("kind", c_int32), ("start", c_uint32), ("len", c_uint32), ("value_or_mean", c_float),
                ("stddev", c_float), ("seed", c_uint32), ("init_k", c_float)]


INIT_CONSTANT, INIT_RANDOM_NORMAL, INIT_TRUNCATED_NORMAL = 0, 1, 2


def initializer_descs(descs):
    """[(kind, start, len, value_or_mean, stddev, seed, init_k), ...] -> ctypes array"""
    arr = (InitializerDesc * max(len(descs), 1))()
    for i, d in enumerate(descs):
        arr[i] = InitializerDesc(int(d[0]), int(d[1]), int(d[2]), float(d[3]), float(d[4]), int(d[5]), float(d[6]))
    return arr


PROTOTYPES = {
    "recsdk_version": (c_int32, []),
    "recsdk_last_error": (c_char_p, []),
    "recsdk_set_small_batch_keys": (c_int32, [c_int64]),
    "recsdk_profile_start": (c_int32, [c_char_p]),
    "recsdk_profile_stop": (c_int32, []),
    "recsdk_profile_get": (c_int32, [c_int32, c_char_p, c_int32, POINTER(c_int64), POINTER(ctypes.c_double)]),
    "recsdk_calib_copy": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p]),
    "recsdk_graph_node_kinds": (c_int32, [c_void_p, POINTER(c_int32), c_int64, POINTER(c_int64)]),
    "recsdk_sorter_create": (c_int32, [c_int64, c_int32, POINTER(c_void_p)]),
    "recsdk_sorter_destroy": (c_int32, [c_void_p]),
    "recsdk_sort_pairs": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int32, c_void_p]),
    "recsdk_lookup_by_addr": (c_int32, [c_void_p, c_int64, c_int32, c_int32, c_void_p, c_void_p]),
    "recsdk_update_by_addr": (c_int32, [c_void_p, c_int64, c_int32, c_int32, c_void_p, c_int32, c_void_p]),
    "recsdk_lazy_adam": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_void_p, c_void_p, c_float,
                                   c_float, c_float, c_float, c_void_p]),
    "recsdk_sgd": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p, c_float, c_float, c_void_p]),
    "recsdk_unique_create": (c_int32, [c_int64, c_int32, POINTER(c_void_p)]),
    "recsdk_unique_destroy": (c_int32, [c_void_p]),
    "recsdk_unique_run": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int64,
                                    c_void_p]),
    "recsdk_unique_results": (c_int32, [c_void_p, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                        POINTER(c_void_p)]),
    "recsdk_unique_fetch": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "recsdk_unique_expand": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "recsdk_unique_total": (c_int32, [c_void_p, c_void_p, POINTER(c_int64)]),
    "recsdk_unique_set_lists": (c_int32, [c_void_p, c_int32]),
    "recsdk_unique_set_counts": (c_int32, [c_void_p, c_int32]),
    "recsdk_unique_set_max_table_keys": (c_int32, [c_void_p, c_int64]),
    "recsdk_unique_run_noalloc": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_int64, c_void_p,
                                            c_void_p, c_void_p, c_void_p, c_void_p]),
    "recsdk_regroup_create": (c_int32, [c_int64, POINTER(c_void_p)]),
    "recsdk_regroup_destroy": (c_int32, [c_void_p]),
    "recsdk_unique_sharded": (c_int32, [c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int64, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(c_int32)]),
    "recsdk_unique_sorted": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "recsdk_tables_create": (c_int32, [c_int32, POINTER(c_int64), POINTER(c_int32), POINTER(c_int64),
                                       POINTER(c_int64), c_int64, POINTER(c_void_p)]),
    "recsdk_tables_destroy": (c_int32, [c_void_p]),
    "recsdk_tables_key2offset": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p]),
    "recsdk_tables_evict": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_void_p]),
    "recsdk_tables_maintain": (c_int32, [c_void_p, c_void_p, POINTER(c_int32)]),
    "recsdk_tables_stats": (c_int32, [c_void_p, c_void_p, POINTER(c_int64), POINTER(c_int64), POINTER(c_int64)]),
    "recsdk_tables_evict_pos": (c_int32, [c_void_p, c_int32, c_void_p, POINTER(c_int64), c_int64,
                                          POINTER(c_int64)]),
    "recsdk_rows_create": (c_int32, [c_int32, c_int32, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                     POINTER(c_int64), POINTER(c_void_p)]),
    "recsdk_rows_destroy": (c_int32, [c_void_p]),
    "recsdk_gather_unique": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "recsdk_sparse_apply": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_float, c_float, c_float,
                                      c_float, c_float, c_void_p]),
    "recsdk_sparse_apply_lr_dev": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p, c_float, c_float,
                                      c_float, c_float, c_void_p]),
    "recsdk_faae_create": (c_int32, [c_int32, POINTER(c_int64), POINTER(c_int32), POINTER(c_int32), POINTER(c_int32),
                                     POINTER(c_int32), c_int64, POINTER(c_void_p)]),
    "recsdk_faae_destroy": (c_int32, [c_void_p]),
    "recsdk_faae_admit": (c_int32, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_int64,
                                    POINTER(c_int64), c_void_p]),
    "recsdk_faae_admit_distinct": (c_int32, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_int64,
                                    POINTER(c_int64), c_void_p]),
    "recsdk_faae_admit_distinct_dev": (c_int32, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_int64,
                                                 c_void_p, c_void_p]),
    "recsdk_faae_evict_dev": (c_int32, [c_void_p, c_int32, c_void_p, c_int64, c_void_p, c_void_p]),
    "recsdk_faae_count_add": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_void_p]),
    "recsdk_faae_count_filter": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_void_p]),
    "recsdk_faae_record_timestamp": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_void_p]),
    "recsdk_faae_evict": (c_int32, [c_void_p, c_int32, c_void_p, c_int64, POINTER(c_int64), c_void_p]),
    "recsdk_faae_stats": (c_int32, [c_void_p, c_void_p, POINTER(c_int64), POINTER(c_int64)]),
    "recsdk_faae_dump": (c_int32, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, POINTER(c_int64),
                                   c_void_p]),
    "recsdk_swap_create": (c_int32, [c_int64, c_int64, c_int64, POINTER(c_void_p)]),
    "recsdk_swap_destroy": (c_int32, [c_void_p]),
    "recsdk_swap_compute": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p]),
    "recsdk_swap_counts": (c_int32, [c_void_p, c_void_p, POINTER(c_int64), POINTER(c_int64), POINTER(c_int64)]),
    "recsdk_swap_remove": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p]),
    "recsdk_swap_export": (c_int32, [c_void_p, c_void_p, c_void_p]),
    "recsdk_om_create": (c_int32, [c_int64, c_int64, POINTER(c_void_p)]),
    "recsdk_om_destroy": (c_int32, [c_void_p]),
    "recsdk_om_compute": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "recsdk_om_counts": (c_int32, [c_void_p, c_void_p, POINTER(c_int64), POINTER(c_int64), POINTER(c_int64),
                                   POINTER(c_int64)]),
    "recsdk_om_remove": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p]),
    "recsdk_om_export": (c_int32, [c_void_p, c_void_p, c_void_p]),
    "recsdk_om_copy_state": (c_int32, [c_void_p, c_void_p, c_void_p]),
    "recsdk_faae_load": (c_int32, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_int64, c_int32, c_int64, c_void_p]),
    "recsdk_tables_export": (c_int32, [c_void_p, c_int32, c_void_p, c_void_p, c_int64, c_void_p, POINTER(c_int64)]),
    "recsdk_tables_load_keys": (c_int32, [c_void_p, c_int32, c_void_p, c_int64, c_void_p]),
    "recsdk_ckpt_write_keys": (c_int32, [c_char_p, c_void_p, c_int64, c_void_p]),
    "recsdk_ckpt_read_keys": (c_int32, [c_char_p, c_int32, c_int32, c_int32, c_void_p, c_void_p, c_int64,
                                        POINTER(c_int64)]),
    "recsdk_ckpt_write_rows": (c_int32, [c_char_p, c_void_p, c_int64, c_int32, c_int64, c_void_p]),
    "recsdk_ckpt_read_rows": (c_int32, [c_char_p, c_void_p, c_int64, c_int32, c_void_p, c_int64, c_void_p]),
    "recsdk_hostrows_swap_out_dev": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p]),
    "recsdk_hostrows_swap_in_dev": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p]),
    "recsdk_hostrows_on_link_start": (c_int32, [c_void_p, c_void_p]),
    "recsdk_hostrows_swap_dev": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                                           c_int64, c_void_p]),
    "recsdk_hostrows_serialize": (c_int32, [c_void_p, c_void_p, c_int64, POINTER(c_int64)]),
    "recsdk_hostrows_deserialize": (c_int32, [c_void_p, c_void_p, c_int64]),
    "recsdk_hostrows_save": (c_int32, [c_void_p, c_char_p, c_int32, c_int32]),
    "recsdk_hostrows_load": (c_int32, [c_void_p, c_char_p, c_int32, c_int32]),
    "recsdk_read_emb_key": (c_int32, [c_void_p, c_int32, c_int64, c_void_p, c_void_p, c_int32, c_int32, c_int64, c_void_p,
                                      c_void_p, c_void_p, POINTER(c_int64), c_void_p]),
    "recsdk_padding_keys_mask": (c_int32, [c_void_p, c_int64, c_void_p, c_int32, c_void_p, c_void_p]),
    "recsdk_hot_create": (c_int32, [c_int32, c_void_p, c_int64, POINTER(c_void_p)]),
    "recsdk_hot_destroy": (c_int32, [c_void_p]),
    "recsdk_hot_split": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_void_p]),
    "recsdk_initializer_create": (c_int32, [c_void_p, c_int32, POINTER(c_void_p)]),
    "recsdk_initializer_destroy": (c_int32, [c_void_p]),
    "recsdk_initializer_generate": (c_int32, [c_void_p, c_void_p, c_int64, c_int32]),
    "recsdk_hostrows_create": (c_int32, [c_int64, c_int32, c_void_p, c_int32, POINTER(c_void_p)]),
    "recsdk_hostrows_destroy": (c_int32, [c_void_p]),
    "recsdk_hostrows_gather": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_int32]),
    "recsdk_hostrows_scatter": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_int32]),
    "recsdk_hostrows_gather_and_remove": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p]),
    "recsdk_hostrows_remove": (c_int32, [c_void_p, c_void_p, c_int64]),
    "recsdk_hostrows_find_rows": (c_int32, [c_void_p, c_void_p, c_int64, c_int32, c_void_p]),
    "recsdk_hostrows_size": (c_int32, [c_void_p, POINTER(c_int64)]),
    "recsdk_hostrows_arena": (c_int32, [c_void_p, POINTER(c_void_p)]),
    "recsdk_hostrows_export": (c_int32, [c_void_p, c_void_p, c_void_p, c_int64, POINTER(c_int64)]),
    "recsdk_hostrows_swap_out": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p]),
    "recsdk_hostrows_swap_in": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_int64, c_void_p]),
    "recsdk_tbe_forward": (c_int32, [c_void_p, c_int32, c_int64, c_void_p, c_void_p, c_int64, c_int32, c_void_p,
                                     c_void_p, c_int32, c_int64, c_int64, c_int32, c_void_p, c_void_p]),
    "recsdk_tbe_create": (c_int32, [c_int32, c_int64, POINTER(c_void_p)]),
    "recsdk_tbe_destroy": (c_int32, [c_void_p]),
    "recsdk_tbe_backward": (c_int32, [c_void_p, c_int32, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_int64,
                                      c_int32, c_void_p, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int32,
                                      c_void_p, c_void_p, c_float, c_float, c_float, c_float, c_int64, c_void_p]),
    "recsdk_tbe_backward_unique": (c_int32, [c_void_p, c_int32, c_void_p, c_void_p, c_int32, c_void_p, c_void_p, c_int64,
                                             c_int32, c_void_p, c_void_p, c_int32, c_int64, c_int64, c_int32, c_void_p,
                                             c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_float, c_float, c_float,
                                             c_float, c_int64, c_void_p]),
}


def lib():
    """Returns the loaded library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RecsdkError(EINVAL, f"{LIB_PATH} is missing: build it with `python -m recsdk_amd.build`")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


def check(code):
    if code != OK:
        msg = lib().recsdk_last_error()
        raise RecsdkError(code, msg.decode() if msg else "")
    return code


def profile_start(prefix=""):
    check(lib().recsdk_profile_start(prefix.encode()))


def profile_stop():
    """Stops timing and returns {kernel name: (launches, total_ms)}."""
    n = lib().recsdk_profile_stop()
    out = {}
    for i in range(n):
        name = ctypes.create_string_buffer(128)
        cnt = c_int64()
        ms = ctypes.c_double()
        check(lib().recsdk_profile_get(i, name, 128, ctypes.byref(cnt), ctypes.byref(ms)))
        out[name.value.decode()] = (cnt.value, ms.value)
    return out
