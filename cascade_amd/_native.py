"""ctypes bindings of the C ABI declared in include/cascade_hip.h.

There is no CPU fallback: if the HIP library has not been built, loading fails with an error that says so.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
HIP_LIB_PATH = os.path.join(HERE, "libcascade_hip.so")

CSA_MAX_GENERATIONS = 64
CSA_MAX_PART_SZ = 2147483647
CSA_MAX_INDEX = 1 << 40
CSA_OK, CSA_ERR_ARG, CSA_ERR_TOO_LARGE, CSA_ERR_HIP, CSA_ERR_INTERNAL = 0, -1, -2, -3, -4
CSA_FLAG_KERNEL_TIMING = 1
CSA_TUNE_DEFER_MIN, CSA_TUNE_WINDOW_MIN_CHANGED, CSA_TUNE_XCD_CHUNK, CSA_TUNE_PACK_SYMBOLS, CSA_TUNE_EXPECT_PRESORTED = 0, 1, 2, 3, 4

# every symbol include/cascade_hip.h declares
EXPORTS = (
    "csa_bytes_per_suffix", "csa_create", "csa_destroy", "csa_sort_partition_u16_dev", "csa_sort_partition_u16",
    "csa_pack_keys_u16_dev", "csa_radix_sort_pairs_dev", "csa_verify_sa40_dev", "csa_last_error",
    "csa_partition_id_bits", "csa_partition_ids_u16_dev", "csa_scatter_to_rank_order_dev", "csa_output_cut",
    "csa_stage_slab_u16_dev", "csa_count_messages_dev", "csa_message_offsets_dev", "csa_emit_messages_dev",
    "csa_join_messages_dev", "csa_join_messages_sorted_dev", "csa_sort_init_dev", "csa_sort_rerank_dev",
    "csa_set_device_exclusive", "csa_set_tuning", "csa_radix_sort_pairs_static_dev", "csa_radix_sort_pairs_static_status", "csa_enable_profile_ranges",
    "csa_step_bytes_per_suffix", "csa_workspace_bytes", "csa_create_steps", "csa_scratch_high_water", "csa_last_step_result",
    "csa_sort_init_slabs", "csa_sort_rerank_slabs", "csa_scatter_slabs", "csa_sort_partitions_u16",
)


class CsaSlab(C.Structure):
    """csa_slab of include/cascade_hip.h: one pinned host slab of a partition."""
    _fields_ = [
        ("key", C.c_void_p), ("suf", C.c_void_p), ("beta", C.c_void_p), ("msg_target", C.c_void_p), ("msg_rank", C.c_void_p),
        ("off", C.c_uint64), ("size", C.c_uint64), ("inbox_off", C.c_uint32), ("inbox_sz", C.c_uint32),
        ("outbox_off", C.c_uint32), ("outbox_sz", C.c_uint32),
    ]


class CsaStepResult(C.Structure):
    """csa_step_result of include/cascade_hip.h: what a per-generation partition step reports."""
    _fields_ = [("active", C.c_uint64), ("messages", C.c_uint64), ("unserved", C.c_uint64), ("pills", C.c_uint64),
                ("incoherent_pills", C.c_uint64)]


class CsaStats(C.Structure):
    _fields_ = [
        ("n", C.c_uint64),
        ("key_words", C.c_int32),
        ("generations", C.c_int32),
        ("active", C.c_uint64 * CSA_MAX_GENERATIONS),
        ("groups", C.c_uint64 * CSA_MAX_GENERATIONS),
        ("big", C.c_uint64 * CSA_MAX_GENERATIONS),
        ("passes", C.c_int32 * CSA_MAX_GENERATIONS),
        ("rank_update", C.c_int32 * CSA_MAX_GENERATIONS),
        ("small_only", C.c_int32 * CSA_MAX_GENERATIONS),
        ("dense", C.c_int32 * CSA_MAX_GENERATIONS),
        ("ms", C.c_float * CSA_MAX_GENERATIONS),
        ("ms_output", C.c_float),
        ("ms_total", C.c_float),
        ("radix_launches", C.c_uint64),
        ("radix_pairs", C.c_uint64),
        ("radix_ms", C.c_double),
        ("presorted", C.c_uint64 * CSA_MAX_GENERATIONS),
        ("key_symbols", C.c_uint32),
        ("first_sort_generations", C.c_uint32),
    ]


class CascadeError(RuntimeError):
    def __init__(self, status, message):
        super().__init__(f"cascade_hip status {status}: {message}")
        self.status = status


_lib = None


def load():
    """Loads libcascade_hip.so and declares its prototypes. Raises if the library is missing."""
    global _lib
    if _lib is not None:
        return _lib
    path = os.environ.get("CASCADE_HIP_LIB", HIP_LIB_PATH)  # a differently tuned build of the same library
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -m cascade_amd.build` "
            "(there is no CPU fallback for the partition sort)")
    lib = C.CDLL(path)
    vp, u64, u32, i32 = C.c_void_p, C.c_uint64, C.c_uint32, C.c_int
    lib.csa_bytes_per_suffix.restype = u64
    lib.csa_bytes_per_suffix.argtypes = [i32]
    lib.csa_create.restype = i32
    lib.csa_create.argtypes = [u64, i32, C.POINTER(vp)]
    lib.csa_destroy.restype = None
    lib.csa_destroy.argtypes = [vp]
    lib.csa_set_device_exclusive.restype = C.c_int
    lib.csa_set_device_exclusive.argtypes = [vp, C.c_int]
    lib.csa_set_tuning.restype = C.c_int
    lib.csa_set_tuning.argtypes = [vp, C.c_int, C.c_uint32]
    lib.csa_sort_partition_u16_dev.restype = i32
    lib.csa_sort_partition_u16_dev.argtypes = [vp, vp, u64, u64, vp, vp, u32, C.POINTER(CsaStats)]
    lib.csa_sort_partition_u16.restype = i32
    lib.csa_sort_partition_u16.argtypes = [vp, u64, i32, vp, C.POINTER(CsaStats)]
    lib.csa_sort_partitions_u16.restype = i32
    lib.csa_sort_partitions_u16.argtypes = [u32, vp, vp, vp, i32, vp, C.POINTER(CsaStats)]
    lib.csa_pack_keys_u16_dev.restype = i32
    lib.csa_pack_keys_u16_dev.argtypes = [vp, u64, i32, vp, vp]
    lib.csa_radix_sort_pairs_dev.restype = i32
    lib.csa_radix_sort_pairs_dev.argtypes = [vp, vp, vp, u64, i32, i32, vp]
    lib.csa_radix_sort_pairs_static_dev.restype = i32
    lib.csa_radix_sort_pairs_static_dev.argtypes = [vp, vp, u64, i32, i32, vp]
    lib.csa_radix_sort_pairs_static_status.restype = i32
    lib.csa_radix_sort_pairs_static_status.argtypes = [vp]
    lib.csa_verify_sa40_dev.restype = i32
    lib.csa_verify_sa40_dev.argtypes = [vp, vp, u64, u64, vp, vp, C.POINTER(i32)]
    lib.csa_last_error.restype = C.c_char_p
    lib.csa_last_error.argtypes = []
    lib.csa_partition_id_bits.restype = u32
    lib.csa_partition_id_bits.argtypes = [u32]
    lib.csa_partition_ids_u16_dev.restype = i32
    lib.csa_partition_ids_u16_dev.argtypes = [vp, u64, u64, vp, i32, u32, vp, vp, vp, vp]
    lib.csa_scatter_to_rank_order_dev.restype = i32
    lib.csa_scatter_to_rank_order_dev.argtypes = [vp, vp, vp, u64, vp, vp]
    lib.csa_stage_slab_u16_dev.restype = i32
    lib.csa_stage_slab_u16_dev.argtypes = [vp, u64, vp, u64, i32, vp, u32, u64, i32, vp, vp, vp]
    lib.csa_count_messages_dev.restype = i32
    lib.csa_count_messages_dev.argtypes = [vp, vp, vp, u64, u64, i32, u32, vp, vp]
    lib.csa_message_offsets_dev.restype = i32
    lib.csa_message_offsets_dev.argtypes = [vp, u32, vp]
    lib.csa_emit_messages_dev.restype = i32
    lib.csa_emit_messages_dev.argtypes = [vp, vp, vp, u64, u64, i32, vp, u32, vp, vp, vp, vp]
    lib.csa_join_messages_dev.restype = i32
    lib.csa_join_messages_dev.argtypes = [vp, vp, u32, vp, vp, vp, u64, vp]
    lib.csa_join_messages_sorted_dev.restype = i32
    lib.csa_join_messages_sorted_dev.argtypes = [vp, vp, vp, u32, vp, vp, vp, u64, vp]
    lib.csa_sort_init_dev.restype = i32
    lib.csa_sort_init_dev.argtypes = [vp, vp, i32, vp, vp, u64, u32, vp, vp, vp, vp, vp, vp, vp]
    lib.csa_sort_rerank_dev.restype = i32
    lib.csa_sort_rerank_dev.argtypes = [vp, vp, vp, vp, u64, vp, vp, u32, u64, u32, vp, vp, vp, vp, vp, vp, vp]
    lib.csa_enable_profile_ranges.restype = i32
    lib.csa_enable_profile_ranges.argtypes = [i32]
    lib.csa_step_bytes_per_suffix.restype = u64
    lib.csa_step_bytes_per_suffix.argtypes = [i32]
    lib.csa_workspace_bytes.restype = u64
    lib.csa_workspace_bytes.argtypes = [u64]
    lib.csa_create_steps.restype = i32
    lib.csa_create_steps.argtypes = [u64, i32, C.POINTER(vp)]
    lib.csa_scratch_high_water.restype = u64
    lib.csa_scratch_high_water.argtypes = [vp]
    lib.csa_last_step_result.restype = i32
    lib.csa_last_step_result.argtypes = [vp, C.POINTER(CsaStepResult)]
    lib.csa_sort_init_slabs.restype = i32
    lib.csa_sort_init_slabs.argtypes = [vp, C.POINTER(CsaSlab), u32, u64, i32, u32, u64, vp, vp, vp]
    lib.csa_sort_rerank_slabs.restype = i32
    lib.csa_sort_rerank_slabs.argtypes = [vp, C.POINTER(CsaSlab), u32, u64, u64, u64, u32, u64, vp, vp, vp]
    lib.csa_scatter_slabs.restype = i32
    lib.csa_scatter_slabs.argtypes = [vp, C.POINTER(CsaSlab), u32, u64, u64, u64, vp]
    lib.csa_output_cut.restype = None
    lib.csa_output_cut.argtypes = [u64, u64, u64, u64, u64, C.POINTER(u64 * 6)]
    _lib = lib
    return lib


def check(status):
    if status != CSA_OK:
        raise CascadeError(status, load().csa_last_error().decode())
