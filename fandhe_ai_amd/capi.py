"""ctypes declarations of the C ABI in include/fandhe_rocm.h and of the
measurement / test aids in include/fandhe_rocm_bench.h.

Loads ``fandhe_ai_amd/lib/libfandhe_rocm.so`` (built by ``make -C
fandhe_ai_amd/csrc`` / ``__graft_entry__.build()``).  There is no fallback: if
the library is missing, importing this module raises.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libfandhe_rocm.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        "libfandhe_rocm.so is not built (%s); run `make -C fandhe_ai_amd/csrc` or "
        "`python -c 'import __graft_entry__ as g; g.build()'`" % LIB_PATH)

lib = C.CDLL(LIB_PATH)

# status codes (BackendError, crates/tensor-core/src/device.rs:225-371)
OK, INVALID_ARGUMENT, SHAPE_MISMATCH, DEVICE_MISMATCH, ALLOCATION_FAILED, KERNEL_LAUNCH_FAILED, \
    DEVICE_UNAVAILABLE, TRANSFER_FAILED, UNSUPPORTED, CONTEXT_POISONED, CAPTURE_IN_PROGRESS, STORE_POISONED = range(12)

F32, BF16, I8, E4M3, I32, U32 = range(6)
QW_INT8_CHANNEL, QW_E4M3_TENSOR, QW_E4M3_CHANNEL = 0, 1, 2
ACT_NONE, ACT_RELU = 0, 1

ctx_p = C.c_void_p
buf_p = C.c_void_p
qw_p = C.c_void_p
u32p = C.POINTER(C.c_uint32)
i32p = C.POINTER(C.c_int32)
f32p = C.POINTER(C.c_float)
u64 = C.c_uint64


HOST_VIEW_FN = C.CFUNCTYPE(None, C.c_void_p, C.c_void_p, C.c_uint64)


class DeviceInfo(C.Structure):
    _fields_ = [("ordinal", C.c_int32), ("compute_units", C.c_int32), ("clock_khz", C.c_int32),
                ("wavefront_size", C.c_int32), ("total_memory_bytes", C.c_uint64),
                ("arch", C.c_char * 32), ("name", C.c_char * 128)]


class PoolStats(C.Structure):
    _fields_ = [("alloc_count", u64), ("reuse_count", u64), ("cached_bytes", u64),
                ("pending_return_bytes", u64), ("capacity_waste_bytes", u64), ("released_bytes", u64)]


class PagedLayout(C.Structure):
    _fields_ = [("num_blocks", u64), ("block_size", u64), ("embed_dim", u64)]


class PagedArgs(C.Structure):
    _fields_ = [("layout", PagedLayout), ("batch", u64), ("l_new", u64), ("num_heads", u64),
                ("max_blocks_per_seq", u64), ("scale", C.c_float), ("num_kv_heads", u64)]


class BlockTableState(C.Structure):
    _fields_ = [("seq_len", u64), ("has_batch", u64), ("batch", u64), ("used_blocks", u64), ("free_blocks", u64),
                ("next_unused", u64), ("returned", u64)]


class PagedPlan(C.Structure):
    _fields_ = [("out_numel", u64), ("s_max", u64), ("query_rows", u64), ("workspace_elems", u64)]


class RowSampling(C.Structure):
    """fa_row_sampling: one request's strategy and generator state."""
    _fields_ = [("rng_state", C.c_uint64), ("temperature", C.c_float), ("top_k", C.c_uint32),
                ("strategy", C.c_int32), ("reserved", C.c_uint32)]


class GemmPlan(C.Structure):
    """fa_gemm_plan: the kernel a prefill-shape GEMM is launched with."""
    _fields_ = [("big_ntb", C.c_int32), ("waves", C.c_int32), ("splits", C.c_uint32)]


class DecoderConfig(C.Structure):
    _fields_ = [("n_layers", C.c_uint32), ("d_model", C.c_uint32), ("n_heads", C.c_uint32),
                ("n_kv_heads", C.c_uint32), ("head_dim", C.c_uint32), ("d_ffn", C.c_uint32),
                ("vocab", C.c_uint32), ("block_size", C.c_uint32), ("max_blocks_per_seq", C.c_uint32),
                ("num_blocks", C.c_uint32), ("max_batch", C.c_uint32), ("rms_eps", C.c_float),
                ("rope_theta", C.c_double)]


# name -> (restype, argtypes); every symbol the header declares
SIGNATURES = {
    "fa_last_error_message": (C.c_char_p, []),
    "fa_status_name": (C.c_char_p, [C.c_int32]),
    "fa_abi_version": (C.c_uint32, []),
    "fa_device_count": (C.c_int32, [i32p]),
    "fa_context_create": (C.c_int32, [C.c_int32, C.POINTER(ctx_p)]),
    "fa_context_destroy": (C.c_int32, [ctx_p]),
    "fa_context_info": (C.c_int32, [ctx_p, C.POINTER(DeviceInfo)]),
    "fa_alloc_zeroed": (C.c_int32, [ctx_p, C.c_int, u64, C.POINTER(buf_p)]),
    "fa_alloc_uninit": (C.c_int32, [ctx_p, C.c_int, u64, C.POINTER(buf_p)]),
    "fa_upload": (C.c_int32, [ctx_p, C.c_int, C.c_void_p, u64, C.POINTER(buf_p)]),
    "fa_upload_into": (C.c_int32, [ctx_p, C.c_void_p, u64, buf_p, u64]),
    "fa_download": (C.c_int32, [ctx_p, buf_p, u64, C.c_void_p, u64]),
    "fa_context_poisoned": (C.c_int32, [ctx_p, C.POINTER(C.c_int32)]),
    "fa_download_owned": (C.c_int32, [ctx_p, buf_p, C.c_void_p, u64]),
    "fa_with_host_view": (C.c_int32, [ctx_p, buf_p, C.c_void_p, C.c_void_p]),
    "fa_buffer_free": (C.c_int32, [ctx_p, buf_p]),
    "fa_buffer_numel": (u64, [buf_p]),
    "fa_buffer_dtype": (C.c_int, [buf_p]),
    "fa_buffer_device_ptr": (C.c_void_p, [buf_p]),
    "fa_synchronize_device": (C.c_int32, [ctx_p]),
    "fa_context_stream": (C.c_void_p, [ctx_p]),
    "fa_device_memory_pool_stats": (C.c_int32, [ctx_p, C.POINTER(PoolStats)]),
    "fa_release_cached_device_memory": (C.c_int32, [ctx_p]),
    "fa_size_class_for": (C.c_int32, [u64, C.POINTER(u64)]),
    "fa_gemm_device": (C.c_int32, [ctx_p, buf_p, buf_p, u64, u64, u64, buf_p]),
    "fa_linear_forward_device": (C.c_int32, [ctx_p, buf_p, u64, u64, buf_p, u64, u64, buf_p, u64, C.c_int, buf_p]),
    "fa_qweight_from_f32": (C.c_int32, [ctx_p, buf_p, u64, u64, u64, C.c_int, C.POINTER(qw_p)]),
    "fa_qweight_from_codes": (C.c_int32, [ctx_p, C.c_void_p, f32p, u64, u64, C.c_int, C.POINTER(qw_p)]),
    "fa_qweight_export": (C.c_int32, [ctx_p, qw_p, C.c_void_p, f32p]),
    "fa_qweight_free": (C.c_int32, [ctx_p, qw_p]),
    "fa_qweight_k": (u64, [qw_p]),
    "fa_qweight_n": (u64, [qw_p]),
    "fa_quantize_rows_i8": (C.c_int32, [ctx_p, buf_p, u64, u64, buf_p, buf_p]),
    "fa_linear_w8a8": (C.c_int32, [ctx_p, buf_p, u64, qw_p, buf_p, u64, buf_p, buf_p]),
    "fa_linear_w8a16": (C.c_int32, [ctx_p, buf_p, u64, qw_p, buf_p]),
    "fa_quantize_tensor_e4m3": (C.c_int32, [ctx_p, buf_p, u64, buf_p, buf_p]),
    "fa_gemm_e4m3": (C.c_int32, [ctx_p, buf_p, buf_p, u64, qw_p, buf_p]),
    "fa_quantize_rows_e4m3": (C.c_int32, [ctx_p, buf_p, u64, u64, buf_p, buf_p]),
    "fa_linear_e4m3": (C.c_int32, [ctx_p, buf_p, u64, qw_p, buf_p, u64, buf_p]),
    "fa_gemm_e4m3_rows": (C.c_int32, [ctx_p, buf_p, buf_p, u64, qw_p, buf_p, u64, buf_p]),
    "fa_gemm_w8a8": (C.c_int32, [ctx_p, buf_p, buf_p, u64, qw_p, buf_p, buf_p]),
    "fa_rmsnorm": (C.c_int32, [ctx_p, buf_p, buf_p, C.c_float, u64, u64, buf_p]),
    "fa_rope": (C.c_int32, [ctx_p, buf_p, buf_p, u64, u64, u64, C.c_double, buf_p]),
    "fa_silu_mul": (C.c_int32, [ctx_p, buf_p, buf_p, u64, buf_p]),
    "fa_add": (C.c_int32, [ctx_p, buf_p, buf_p, u64, buf_p]),
    "fa_argmax_rows": (C.c_int32, [ctx_p, buf_p, u64, u64, buf_p]),
    "fa_gather_rows": (C.c_int32, [ctx_p, buf_p, u64, u64, buf_p, u64, buf_p]),
    "fa_convert": (C.c_int32, [ctx_p, buf_p, u64, buf_p]),
    "fa_fill_normal": (C.c_int32, [ctx_p, buf_p, u64, u64, u64, C.c_float, C.c_float]),
    "fa_validate_paged_kv_append": (C.c_int32, [u64, u64, u64, u64, u32p, u64, C.POINTER(PagedLayout)]),
    "fa_validate_paged_attention": (C.c_int32, [u64, u64, u64, u32p, u64, u32p, u64, C.POINTER(PagedArgs),
                                                C.POINTER(PagedPlan)]),
    "fa_paged_kv_append": (C.c_int32, [ctx_p, buf_p, buf_p, buf_p, buf_p, u32p, u64, C.POINTER(PagedLayout)]),
    "fa_paged_attention_forward": (C.c_int32, [ctx_p, buf_p, buf_p, buf_p, u32p, u64, u32p, u64,
                                               C.POINTER(PagedArgs), buf_p]),
    "fa_paged_kv_append_device": (C.c_int32, [ctx_p, buf_p, buf_p, buf_p, buf_p, buf_p, u64, C.POINTER(PagedLayout)]),
    "fa_paged_attention_forward_device": (C.c_int32, [ctx_p, buf_p, buf_p, buf_p, buf_p, buf_p,
                                                      C.POINTER(PagedArgs), buf_p]),
    "fa_paged_attention_decode_static": (C.c_int32, [ctx_p, buf_p, buf_p, buf_p, buf_p, buf_p,
                                                     C.POINTER(PagedArgs), buf_p]),
    "fa_paged_attention_decode_static_max_bytes": (u64, []),
    "fa_sample_rows": (C.c_int32, [ctx_p, buf_p, u64, u64, C.c_int32, C.c_float, u64, buf_p, buf_p]),
    "fa_sampling_weights": (C.c_int32, [ctx_p, buf_p, u64, u64, u64, C.c_int32, C.c_float, u64, buf_p, u64, buf_p]),
    "fa_speculative_accept": (C.c_int32, [ctx_p, buf_p, u64, buf_p, u64, i32p, u64, u64, buf_p, buf_p]),
    "fa_rng_seed": (C.c_int32, [ctx_p, buf_p, u64]),
    "fa_decoder_set_sampling": (C.c_int32, [ctx_p, C.c_void_p, C.c_int32, C.c_float, u64, u64]),
    "fa_rng_state_from_seed": (C.c_int32, [u64, C.POINTER(u64)]),
    "fa_sample_rows_per_row": (C.c_int32, [ctx_p, buf_p, u64, u64, buf_p, buf_p]),
    "fa_decoder_set_row_sampling": (C.c_int32, [ctx_p, C.c_void_p, C.POINTER(RowSampling)]),
    "fa_decoder_read_row_sampling": (C.c_int32, [ctx_p, C.c_void_p, C.POINTER(RowSampling)]),
    "fa_decoder_prefill_padded": (C.c_int32, [ctx_p, C.c_void_p, i32p, C.c_uint32, u32p]),
    "fa_decoder_verify": (C.c_int32, [ctx_p, C.c_void_p, i32p, C.c_uint32, i32p, f32p]),
    "fa_decoder_rewind": (C.c_int32, [ctx_p, C.c_void_p, u32p]),
    "fa_decoder_prefill": (C.c_int32, [ctx_p, C.c_void_p, i32p, C.c_uint32]),
    "fa_probe_matrix_rate": (C.c_int32, [ctx_p, C.c_int32, buf_p, C.c_uint32, buf_p, C.POINTER(C.c_double)]),
    "fa_block_table_create": (C.c_int32, [C.POINTER(C.c_void_p)]),
    "fa_block_table_destroy": (C.c_int32, [C.c_void_p]),
    "fa_block_table_clone": (C.c_int32, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "fa_block_table_alloc": (C.c_int32, [C.c_void_p, u64, u32p, i32p]),
    "fa_block_table_return": (C.c_int32, [C.c_void_p, C.c_uint32]),
    "fa_block_table_reset": (C.c_int32, [C.c_void_p]),
    "fa_block_table_state_get": (C.c_int32, [C.c_void_p, u64, C.POINTER(BlockTableState)]),
    "fa_block_table_extend_for_append": (C.c_int32, [C.c_void_p, u64, u64, u64, u64, u32p, u64, C.POINTER(u64)]),
    "fa_block_table_flatten": (C.c_int32, [C.c_void_p, u64, u32p, u64, C.POINTER(u64)]),
    "fa_block_table_rewind_to": (C.c_int32, [C.c_void_p, u64, u64]),
    "fa_paged_cache_check_config": (C.c_int32, [u64, u64, u64, C.c_int32]),
    "fa_paged_cache_create": (C.c_int32, [ctx_p, u64, u64, u64, C.c_int32, C.POINTER(C.c_void_p)]),
    "fa_paged_cache_destroy": (C.c_int32, [ctx_p, C.c_void_p]),
    "fa_paged_cache_state_get": (C.c_int32, [C.c_void_p, C.POINTER(BlockTableState), i32p]),
    "fa_paged_cache_pools": (C.c_int32, [C.c_void_p, C.POINTER(buf_p), C.POINTER(buf_p)]),
    "fa_paged_cache_block_tables": (C.c_int32, [C.c_void_p, u64, u32p, u64, C.POINTER(u64)]),
    "fa_paged_cache_append": (C.c_int32, [ctx_p, C.c_void_p, buf_p, buf_p, u64, u64]),
    "fa_paged_cache_attention": (C.c_int32, [ctx_p, C.c_void_p, buf_p, u64, u64, u64, u64, C.c_float, buf_p]),
    "fa_paged_cache_rewind_to": (C.c_int32, [C.c_void_p, u64]),
    "fa_paged_cache_clear": (C.c_int32, [C.c_void_p]),
    "fa_paged_cache_snapshot_table": (C.c_int32, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "fa_paged_cache_restore_table": (C.c_int32, [C.c_void_p, C.c_void_p]),
    "fa_graph_capture_begin": (C.c_int32, [ctx_p]),
    "fa_graph_capture_end": (C.c_int32, [ctx_p, C.POINTER(C.c_void_p)]),
    "fa_graph_launch": (C.c_int32, [ctx_p, C.c_void_p]),
    "fa_graph_destroy": (C.c_int32, [ctx_p, C.c_void_p]),
    "fa_decoder_create": (C.c_int32, [ctx_p, C.POINTER(DecoderConfig), C.POINTER(C.c_void_p)]),
    "fa_decoder_destroy": (C.c_int32, [ctx_p, C.c_void_p]),
    "fa_decoder_set_layer": (C.c_int32, [C.c_void_p, C.c_uint32, buf_p, buf_p, qw_p, qw_p, qw_p, qw_p]),
    "fa_decoder_set_head": (C.c_int32, [C.c_void_p, buf_p, buf_p, qw_p]),
    "fa_decoder_kv_pools": (C.c_int32, [C.c_void_p, C.c_uint32, C.POINTER(buf_p), C.POINTER(buf_p)]),
    "fa_decoder_set_sequences": (C.c_int32, [ctx_p, C.c_void_p, C.c_uint32, u32p, u32p]),
    "fa_decoder_set_tokens": (C.c_int32, [ctx_p, C.c_void_p, i32p]),
    "fa_decoder_step": (C.c_int32, [ctx_p, C.c_void_p, C.c_int32]),
    "fa_decoder_read_tokens": (C.c_int32, [ctx_p, C.c_void_p, i32p]),
    "fa_decoder_read_logits": (C.c_int32, [ctx_p, C.c_void_p, f32p]),
    "fa_decoder_logits_buffer": (C.c_int32, [C.c_void_p, C.POINTER(buf_p)]),
    "fa_decoder_read_seq_lens": (C.c_int32, [ctx_p, C.c_void_p, u32p]),
    "fa_set_tuning": (C.c_int32, [C.c_int32, C.c_int32]),
    "fa_timer_create": (C.c_int32, [ctx_p, C.POINTER(C.c_void_p)]),
    "fa_timer_start": (C.c_int32, [ctx_p, C.c_void_p]),
    "fa_timer_stop": (C.c_int32, [ctx_p, C.c_void_p]),
    "fa_timer_elapsed_ms": (C.c_int32, [ctx_p, C.c_void_p, f32p]),
    "fa_timer_destroy": (C.c_int32, [ctx_p, C.c_void_p]),
    "fa_decoder_debug_step_until": (C.c_int32, [ctx_p, C.c_void_p, C.c_int32]),
    "fa_decoder_debug_buffer": (C.c_int32, [C.c_void_p, C.c_int32, C.POINTER(buf_p)]),
    "fa_probe_stream_read": (C.c_int32, [ctx_p, buf_p, u64, u64, C.c_int32, C.c_int32, buf_p]),
    "fa_gemm_f32_form_query": (C.c_int32, [u64, u64, u64, C.POINTER(C.c_int32)]),
    "fa_gemm_plan_query": (C.c_int32, [ctx_p, u64, qw_p, C.POINTER(GemmPlan)]),
    "fa_graph_owned_blocks": (C.c_int32, [C.c_void_p, C.POINTER(C.c_void_p), u64, C.POINTER(u64)]),
    "fa_topology_query": (C.c_int32, [ctx_p, i32p, i32p]),
    "fa_probe_l2_path": (C.c_int32, [ctx_p, buf_p, u64, u64, buf_p, C.c_uint32, C.c_uint32, C.c_int32, C.c_int32, C.c_int32,
                                     C.c_int32, buf_p]),
}

for _name, (_res, _args) in SIGNATURES.items():
    _fn = getattr(lib, _name)        # AttributeError here = the library lacks a declared symbol
    _fn.restype = _res
    _fn.argtypes = _args


def last_error():
    return lib.fa_last_error_message().decode("utf-8", "replace")
