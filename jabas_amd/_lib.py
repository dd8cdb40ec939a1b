"""ctypes binding of libjabas_sync.so (the C ABI declared in include/jabas_sync.h).

The structures below mirror the header field for field. There is no fallback: when
the shared library is missing, :func:`lib` raises, and every product path that reaches
for a kernel fails with that error instead of computing on the CPU.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# JABAS_SYNC_LIB points at another build of the same library (kernel tuning experiments)
LIB_PATH = os.environ.get("JABAS_SYNC_LIB") or os.path.join(_HERE, "csrc", "libjabas_sync.so")

MAX_K = 16
MAX_GROUPS = 16
STATS_STRIDE = 40
GRAM_MAX_K = 16
GRAM_STRIDE = 256
STATS_GRAM_MAX_K = 8
STATIC_MAX_NUMEL = 1 << 26
STEP_SCALARS_BYTES = 688

F32, BF16 = 0, 1
OPT_NONE, OPT_SGD, OPT_ADAM, OPT_ADAMW, OPT_ADAM_AMSGRAD, OPT_ADAMW_AMSGRAD = 0, 1, 2, 3, 4, 5
STATS_NONE, STATS_FULL, STATS_SIMILARITY, STATS_GRAM = 0, 1, 2, 3

STAT_DOT_AB, STAT_NORM_A, STAT_NORM_B, STAT_NORM_AGG, STAT_NORM_VSW0 = 0, 1, 2, 3, 4


def stat_pair(K, a, b):
    """Slot of sum g_a*g_b (a < b < K) in a row of level STATS_GRAM: JABAS_STAT_PAIR of the header."""
    return STAT_NORM_VSW0 + K + a * (2 * K - a - 1) // 2 + (b - a - 1)

OK = 0
ERR_NULL, ERR_K, ERR_ALIGN, ERR_DTYPE, ERR_OPT, ERR_GROUP = -1, -2, -3, -4, -5, -6
ERR_WORKSPACE, ERR_PLAN, ERR_SIZE, ERR_LAUNCH, ERR_ALIAS, ERR_STATE = -7, -8, -9, -10, -11, -12
RDV_WAITING, RDV_LAUNCHED, RDV_LAUNCHED_ROW0, RDV_LAUNCHED_ROW1, RDV_UNKNOWN = 0, 1, 2, 3, 4


class JabasSpan(C.Structure):
    _fields_ = [
        ("grads", C.c_void_p * MAX_K),
        ("agg_out", C.c_void_p),
        ("param", C.c_void_p),
        ("state1", C.c_void_p),
        ("state2", C.c_void_p),
        ("state3", C.c_void_p),
        ("fanout", C.c_void_p * (MAX_K - 1)),
        ("numel", C.c_uint64),
        ("n_fanout", C.c_uint32),
        ("bound_begin", C.c_uint32),
        ("bound_count", C.c_uint32),
        ("state_block_log2", C.c_uint32),
        ("state_block_pos", C.c_uint32),
        ("reserved", C.c_uint32),
    ]


class JabasBound(C.Structure):
    _fields_ = [("start", C.c_uint64), ("group", C.c_uint32), ("reserved", C.c_uint32)]


class JabasGroup(C.Structure):
    _fields_ = [("lr", C.c_double), ("weight_decay", C.c_double), ("step", C.c_int64)]


class JabasStepArgs(C.Structure):
    _fields_ = [
        ("K", C.c_int32),
        ("grad_dtype", C.c_int32),
        ("weight", C.c_float * MAX_K),
        ("stats", C.c_int32),
        ("half_id", C.c_uint8 * MAX_K),
        ("half_weight", C.c_float * MAX_K),
        ("opt_kind", C.c_int32),
        ("n_groups", C.c_int32),
        ("first_step", C.c_int32),
        ("nesterov", C.c_int32),
        ("momentum", C.c_double),
        ("dampening", C.c_double),
        ("beta1", C.c_double),
        ("beta2", C.c_double),
        ("eps", C.c_double),
        ("groups", JabasGroup * MAX_GROUPS),
        ("grad_scale", C.c_void_p),
        ("scalars_dev", C.c_void_p),
    ]


# name -> (restype, argtypes); one entry per symbol the header declares.
SIGNATURES = {
    "jabas_sync_version": (C.c_char_p, []),
    "jabas_status_string": (C.c_char_p, [C.c_int]),
    "jabas_step_scalars_encode": (C.c_int, [C.POINTER(JabasStepArgs), C.c_void_p, C.c_size_t]),
    "jabas_step_scalars_upload": (C.c_int, [C.POINTER(JabasStepArgs), C.c_void_p, C.c_void_p]),
    "jabas_sync_workspace_bytes": (C.c_size_t, [C.c_uint64, C.c_int32]),
    "jabas_plan_bytes": (C.c_size_t, [C.POINTER(JabasSpan), C.c_uint32, C.c_uint32, C.c_int32]),
    "jabas_plan_encode": (C.c_int, [C.POINTER(JabasSpan), C.c_uint32, C.POINTER(JabasBound), C.c_uint32,
                                    C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_size_t]),
    "jabas_plan_chunks": (C.c_int64, [C.c_void_p, C.c_int32]),
    "jabas_plan_workspace_bytes": (C.c_size_t, [C.c_void_p]),
    "jabas_sync_fused": (C.c_int, [C.c_void_p, C.c_void_p, C.POINTER(JabasStepArgs), C.c_void_p,
                                   C.c_void_p, C.c_size_t, C.c_void_p]),
    "jabas_sync_bucket": (C.c_int, [C.POINTER(JabasSpan), C.c_void_p, C.POINTER(JabasStepArgs), C.c_void_p,
                                    C.c_void_p, C.c_size_t, C.c_void_p]),
    "jabas_sync_bucket_static": (C.c_int, [C.POINTER(JabasSpan), C.c_void_p, C.POINTER(JabasStepArgs), C.c_void_p,
                                           C.c_void_p]),
    "jabas_aggregate": (C.c_int, [C.POINTER(C.c_void_p), C.c_int32, C.c_int32, C.POINTER(C.c_float),
                                  C.c_void_p, C.c_uint64, C.c_void_p]),
    "jabas_stats": (C.c_int, [C.POINTER(C.c_void_p), C.c_int32, C.c_int32, C.POINTER(C.c_float),
                              C.POINTER(C.c_uint8), C.POINTER(C.c_float), C.c_uint64, C.c_void_p,
                              C.c_void_p, C.c_size_t, C.c_void_p]),
    "jabas_gram": (C.c_int, [C.POINTER(C.c_void_p), C.c_int32, C.c_int32, C.c_uint64, C.c_void_p,
                             C.c_void_p, C.c_size_t, C.c_void_p]),
    "jabas_clip_coef": (C.c_int, [C.c_void_p, C.c_uint32, C.c_double, C.c_double, C.c_void_p, C.c_void_p]),
    "jabas_sgd": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_double, C.c_double,
                            C.c_double, C.c_double, C.c_int32, C.c_int32, C.c_void_p]),
    "jabas_adam": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_double,
                             C.c_double, C.c_double, C.c_double, C.c_double, C.c_int64, C.c_int32,
                             C.c_void_p]),
    "jabas_rdv_create": (C.c_int, [C.c_int32, C.POINTER(C.c_void_p)]),
    "jabas_rdv_destroy": (None, [C.c_void_p]),
    "jabas_rdv_set_bucket": (C.c_int, [C.c_void_p, C.c_uint32, C.POINTER(JabasSpan), C.c_void_p, C.c_void_p,
                                       C.c_void_p, C.c_size_t, C.c_int32]),
    "jabas_rdv_drop_bucket": (C.c_int, [C.c_void_p, C.c_uint32]),
    "jabas_rdv_publish": (C.c_int, [C.c_void_p, C.c_int32, C.c_uint32, C.c_int32, C.c_void_p, C.c_void_p,
                                    C.POINTER(JabasStepArgs), C.c_int32]),
    "jabas_rdv_reset": (C.c_int, [C.c_void_p]),
}

_lib = None


class JabasSyncError(RuntimeError):
    """A libjabas_sync.so entry point returned a negative status."""

    def __init__(self, status, where):
        self.status = status
        try:
            text = lib().jabas_status_string(status).decode()
        except Exception:  # pragma: no cover - library vanished between calls
            text = "?"
        super().__init__(f"{where}: status {status} ({text})")


def lib():
    """Load (once) and return the shared library with typed entry points."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C jabas_amd/csrc` (needs hipcc). There is no CPU fallback.")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(status, where):
    if status != OK:
        raise JabasSyncError(status, where)
