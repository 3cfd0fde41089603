"""ctypes loader of libsplash_hip.so. Fails loudly when the library is missing."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))


def library_path():
    return os.path.join(_HERE, "lib", "libsplash_hip.so")


class SplashError(RuntimeError):
    """A failed C ABI call; .status is the sp_status code."""

    def __init__(self, status, message):
        super().__init__(f"sp_status {status}: {message}")
        self.status = status
        self.message = message


class InvalidArgument(SplashError, ValueError):
    """SP_INVALID_ARGUMENT / SP_UNKNOWN_KERNEL: the operators' std::invalid_argument."""


def _load():
    path = library_path()
    if not os.path.exists(path):
        raise ImportError(
            f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C splash_amd/csrc`); there is no fallback path")
    return ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)


lib = _load()

SP_OK, SP_INVALID_ARGUMENT, SP_BACKEND_ERROR, SP_UNHEALTHY, SP_BUSY, SP_OUT_OF_MEMORY, SP_UNKNOWN_KERNEL, SP_TIMEOUT = range(8)

lib.sp_last_error.restype = ctypes.c_char_p


def check(status):
    if status == SP_OK:
        return
    message = lib.sp_last_error().decode("utf-8", "replace")
    if status in (SP_INVALID_ARGUMENT, SP_UNKNOWN_KERNEL):
        raise InvalidArgument(status, message)
    raise SplashError(status, message)


c_u32, c_u64, c_p, c_int, c_double, c_size = (ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int,
                                              ctypes.c_double, ctypes.c_size_t)
P = ctypes.POINTER


class DeviceInfo(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 64), ("arch", ctypes.c_char * 32), ("compute_units", c_u32),
                ("wavefront_size", c_u32), ("lds_bytes_per_cu", c_u32), ("l2_bytes", c_u32), ("hbm_bytes", c_u64),
                ("clock_khz", c_u32), ("memory_clock_khz", c_u32), ("memory_bus_bits", c_u32)]


class Dispatch(ctypes.Structure):
    _fields_ = [("kernel", ctypes.c_char_p), ("buffer_count", c_u32), ("buffers", P(c_p)), ("params", c_p),
                ("params_bytes", c_u32), ("grid", c_u32 * 3), ("block", c_u32 * 3), ("indirect", c_p),
                ("indirect_offset", c_u64)]


class MemoryStats(ctypes.Structure):
    _fields_ = [("allocated_bytes", c_u64), ("peak_allocated_bytes", c_u64), ("device_current_allocated_bytes", c_u64),
                ("device_peak_allocated_bytes", c_u64)]


class LinearPlan(ctypes.Structure):
    _fields_ = [("rows", c_u32), ("epilogue", c_u32), ("splits", c_u32), ("whole_groups", c_u32), ("storage_rows", c_u32),
                ("float32", c_u32), ("tile", c_u32), ("reserved", c_u32), ("scratch_input", c_u64), ("scratch_partials", c_u64), ("scratch_counters", c_u64)]


class ChainLink(ctypes.Structure):
    _fields_ = [("projection", c_p), ("gate", c_p), ("plan", LinearPlan), ("input", c_p), ("output", c_p), ("residual", c_p),
                ("norm_weight", c_p), ("next_table", c_p), ("table", c_p), ("partials", c_p), ("counters", c_p),
                ("prepared", ctypes.c_int32), ("reserved", c_u32)]


class AttentionGeometry(ctypes.Structure):
    _fields_ = [("q_heads", c_u32), ("kv_heads", c_u32), ("head_dim", c_u32), ("rotary_pairs", c_u32), ("normalize", c_u32), ("gated", c_u32),
                ("int8_queries", c_u32)]


class AttentionRows(ctypes.Structure):
    _fields_ = [("first_row", c_u32), ("rows", c_u32), ("committed", c_u32), ("table_first", c_u32)]


class RopeSequence(ctypes.Structure):
    _fields_ = [("first_row", c_u32), ("rows", c_u32), ("anchor", c_u32)]


class LaneRows(ctypes.Structure):
    _fields_ = [("first", c_u32), ("rows", c_u32)]


class GdnShape(ctypes.Structure):
    _fields_ = [("key_heads", c_u32), ("value_heads", c_u32), ("convolution_dimension", c_u32), ("packed_width", c_u32),
                ("sigmoid_gate", c_u32)]


class GdnStateStrides(ctypes.Structure):
    _fields_ = [("convolution_layer_bytes", c_u64), ("recurrent_layer_bytes", c_u64), ("convolution_state_bytes", c_u64)]


class GdnLane(ctypes.Structure):
    _fields_ = [("first_row", c_u32), ("rows", c_u32), ("pending_path", c_u32), ("reserved", c_u32), ("pending_tape", c_u64),
                ("step_tape", c_u64), ("current_cell", c_u64), ("next_cell", c_u64)]


class GdnDecodeBuffers(ctypes.Structure):
    _fields_ = [(n, c_p) for n in ("packed", "convolution_weights", "states", "tape", "decay_weights", "time_bias", "mixer_norm",
                                   "hidden")] + [("float_norm", c_u32), ("tree_rows", c_p), ("hidden_table", c_p)]


class GdnPrefillBuffers(ctypes.Structure):
    _fields_ = [(n, c_p) for n in ("packed", "convolution_weights", "states", "decay_weights", "time_bias", "mixer_norm")] + \
               [("float_norm", c_u32), ("reserved", c_u32)] + \
               [(n, c_p) for n in ("queries", "keys", "values", "decay", "beta", "recurrent_rows", "hidden")] + \
               [("current_cell", c_u64), ("next_cell", c_u64)]


class GdnPrefillCapture(ctypes.Structure):
    _fields_ = [("tokens", c_u32), ("reserved", c_u32), ("cell", c_u64)]


class StateCodecShape(ctypes.Structure):
    _fields_ = [("layers", c_u32), ("rows", c_u32), ("columns", c_u32), ("bf16_state", c_u32), ("state_layer_bytes", c_u64),
                ("codes_layer_bytes", c_u64)]


class MoeShape(ctypes.Structure):
    _fields_ = [("hidden", c_u32), ("ffn", c_u32), ("experts", c_u32), ("top_k", c_u32), ("shared_slices", c_u32), ("shared_gate", c_u32),
                ("sigmoid_router", c_u32), ("reserved", c_u32)]


MOE_WORKSPACE_FIELDS = ("selected", "weights", "route_slot", "slot_row", "tile_expert", "tile_rows", "tile_total", "tables", "next_tables",
                        "intermediate", "expert_output")


class MoeWorkspace(ctypes.Structure):
    _fields_ = [(n, c_p) for n in MOE_WORKSPACE_FIELDS]


class SamplingBuffers(ctypes.Structure):
    _fields_ = [(n, c_p) for n in ("logits", "tokens", "partial_values", "partial_indices", "draft_probabilities", "uniforms",
                                   "masses", "ranges", "decisions", "input_tokens", "tree_rows", "token_mask")] + [("mask_words", c_u32)] + [
        (n, c_p) for n in ("candidate_ids", "candidate_probabilities", "candidate_draws", "child_uniforms")]


class DenseDimensions(ctypes.Structure):
    _fields_ = [(n, c_u32) for n in ("hidden", "q_heads", "kv_heads", "head_dim", "ffn", "vocabulary", "layers", "rotary_pairs",
                                     "normalize_heads")] + [("rope_theta", ctypes.c_float)]


class VerifyLane(ctypes.Structure):
    _fields_ = [("rows", c_u32), ("committed", c_u32), ("table_first", c_u32), ("temperature", ctypes.c_float),
                ("remaining", c_u32), ("min_p", ctypes.c_float), ("top_k", c_u32), ("top_p", ctypes.c_float)]


class SamplingPolicy(ctypes.Structure):
    _fields_ = [("temperature", ctypes.c_float), ("min_p", ctypes.c_float), ("top_k", c_u32), ("top_p", ctypes.c_float),
                ("constrained", c_u32), ("excludes_stop_tokens", c_u32)]


class SamplingPenalties(ctypes.Structure):
    _fields_ = [("repetition", ctypes.c_float), ("presence", ctypes.c_float), ("frequency", ctypes.c_float), ("table_row", c_u32)]


class ThinkingCutoff(ctypes.Structure):
    _fields_ = [("active", c_u32), ("row", c_u32), ("count", c_u32), ("end", c_u32 * 16), ("also_ends", c_u32), ("waits_for_mask", c_u32)]


class HybridDimensions(ctypes.Structure):
    _fields_ = [(n, c_u32) for n in ("hidden", "vocabulary", "layers", "attention_interval", "q_heads", "kv_heads", "head_dim",
                                     "rotary_pairs", "normalize_heads", "gated_attention")] + [("rope_theta", ctypes.c_float)] + [
        (n, c_u32) for n in ("gdn_key_heads", "gdn_value_heads", "gdn_packed_width", "experts", "top_k", "expert_ffn", "shared_slices",
                             "shared_gate", "dense_ffn")]


class HybridLane(ctypes.Structure):
    _fields_ = [("block", VerifyLane), ("pending_path", c_u32), ("parity", c_u32)]


class HybridLayer(ctypes.Structure):
    _fields_ = [(n, c_p) for n in ("mixer_input", "mixer_output", "input_norm", "post_norm", "query_norm", "key_norm",
                                   "convolution_weights", "decay_weights", "time_bias", "mixer_norm", "router", "gate_images",
                                   "up_images", "down_images")] + [("expert_format", c_u32), ("expert_down_format", c_u32),
                                                                    ("shared_scalar_gate", c_p), ("ffn_gate", c_p), ("ffn_up", c_p),
                                                                    ("ffn_down", c_p)]


class DFlashLayout(ctypes.Structure):
    _fields_ = [(n, c_u32) for n in ("layers", "hidden", "vocabulary", "intermediate", "target_layers")]


DFLASH_LAYER_FIELDS = ("attention_dynamic", "qkv", "output", "mlp_dynamic", "gate", "up", "down", "input_norm", "attention_convolution",
                       "query_norm", "key_norm", "post_attention_norm", "mlp_convolution")


class DFlashLayer(ctypes.Structure):
    _fields_ = [(n, c_p) for n in DFLASH_LAYER_FIELDS]


def _sig(name, restype, *argtypes):
    fn = getattr(lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


_sig("sp_backend_create", c_int, c_int, c_double, P(c_p))
_sig("sp_backend_destroy", None, c_p)
_sig("sp_backend_stop", None, c_p)
_sig("sp_backend_device_info", c_int, c_p, P(DeviceInfo))
_sig("sp_buffer_alloc", c_int, c_p, c_u64, c_int, ctypes.c_char_p, P(c_p))
_sig("sp_buffer_view", c_int, c_p, c_u64, c_u64, P(c_p))
_sig("sp_buffer_retain", None, c_p)
_sig("sp_buffer_release", None, c_p)
_sig("sp_buffer_size", c_u64, c_p)
_sig("sp_buffer_allocated", c_u64, c_p)
_sig("sp_buffer_storage", c_int, c_p)
_sig("sp_buffer_contents", c_p, c_p)
_sig("sp_buffer_gpu_address", c_u64, c_p)
_sig("sp_buffer_same_view", c_int, c_p, c_p)
_sig("sp_buffer_upload", c_int, c_p, c_u64, c_p, c_u64)
_sig("sp_buffer_download", c_int, c_p, c_u64, c_p, c_u64)
_sig("sp_buffer_fill", c_int, c_p, c_u64, c_int, c_u64)
_sig("sp_kernel_exists", c_int, ctypes.c_char_p)
_sig("sp_kernel_names", c_size, ctypes.c_char_p, c_size)
_sig("sp_submit", c_int, c_p, P(Dispatch), c_u32, c_p, c_p, P(c_p))
_sig("sp_ticket_ready", c_int, c_p)
_sig("sp_ticket_wait", c_int, c_p, P(c_double), P(c_double))
_sig("sp_ticket_release", None, c_p)
_sig("sp_backend_set_dispatch_profiling", None, c_p, c_int)
_sig("sp_ticket_wait_profiled", c_int, c_p, P(c_double), P(c_double), P(c_double), c_u32)
_sig("sp_command_create", c_int, c_p, P(Dispatch), c_u32, P(c_p))
_sig("sp_command_submit", c_int, c_p, c_p, c_p, P(c_p))
_sig("sp_command_release", None, c_p)
_sig("sp_command_in_flight", c_int, c_p)
_sig("sp_backend_healthy", c_int, c_p)
_sig("sp_backend_check_health", c_int, c_p)
_sig("sp_backend_unhealthy_reason", c_size, c_p, ctypes.c_char_p, c_size)
_sig("sp_memory_stats", c_int, c_p, P(MemoryStats))
_sig("sp_restart_peaks", None, c_p)
_sig("sp_backend_stream", c_p, c_p)

_sig("spo_graph_create", c_int, P(c_p))
_sig("spo_graph_destroy", None, c_p)
_sig("spo_graph_size", c_u32, c_p)
_sig("spo_graph_kernel", c_size, c_p, c_u32, ctypes.c_char_p, c_size)
_sig("spo_graph_add", c_int, c_p, ctypes.c_char_p, P(c_p), c_u32, c_p, c_u32, P(c_u32), P(c_u32))
_sig("spo_graph_submit", c_int, c_p, c_p, P(c_p))
_sig("spo_graph_record", c_int, c_p, c_p, P(c_p))
_sig("spo_gguf_image_bytes", c_u64, c_u32, c_u32, c_u32)
_sig("spo_gguf_table_bytes", c_u64, c_u32, c_u32)
_sig("spo_gguf_pack_image", c_int, c_u32, c_p, c_u32, c_u32, c_p)
_sig("spo_gguf_rewrite_format", c_u32, c_u32)
_sig("spo_gguf_rewrite", c_int, c_u32, c_p, ctypes.c_uint64, c_p)
_sig("spo_gguf_unpack_image", c_int, c_u32, c_p, c_u32, c_u32, c_p)
_sig("spo_gguf_add_dequant", c_int, c_p, c_u32, c_p, c_p, c_u32, c_u32)
_sig("spo_projection_create", c_int, c_u32, P(c_u32), P(c_u32), c_u32, P(c_p), c_int, P(c_p))
_sig("spo_projection_destroy", None, c_p)
_sig("spo_projection_weight_bytes", c_u64, c_p)
_sig("spo_linear_create", c_int, c_p, P(c_p))
_sig("spo_linear_create_calibrated", c_int, c_u32, c_u32, c_u32, P(c_p))
_sig("spo_linear_destroy", None, c_p)
_sig("spo_linear_plan_for", c_int, c_p, c_p, c_u32, c_u32, P(LinearPlan))
_sig("spo_linear_plan_with", c_int, c_p, P(LinearPlan))
_sig("spo_linear_add", c_int, c_p, c_p, c_p, c_p, P(LinearPlan), c_p, c_p, c_p, c_p, c_p, c_p, c_int)
_sig("spo_linear_add_residual_norm", c_int, c_p, c_p, c_p, P(LinearPlan), c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_int)
_sig("spo_linear_add_swiglu", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u32, c_p, c_p, c_p, c_p)
_sig("spo_linear_set_chain_spin_limit", c_int, c_p, c_u32)
_sig("spo_linear_add_link", c_int, c_p, c_p, P(ChainLink))
_sig("spo_linear_add_chain", c_int, c_p, c_p, P(ChainLink), c_u32, c_p)
_sig("spo_linear_prefill_table_bytes", c_u64, c_u32, c_u32)
_sig("spo_linear_add_prefill", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_u32)
_sig("spo_linear_scratch_size", c_int, c_p, c_u32, c_u32, c_u32, P(c_u64), P(c_u64), P(c_u64))

_sig("spo_kv_page_bytes", c_u64, c_u32, c_u32)
_sig("spo_kv_key_index", c_u64, c_u32, c_u32, c_u32, c_u32)
_sig("spo_kv_value_index", c_u64, c_u32, c_u32, c_u32, c_u32)
_sig("spo_attention_plan_create", c_int, P(AttentionGeometry), P(AttentionRows), c_u32, P(c_p))
_sig("spo_attention_plan_destroy", None, c_p)
_sig("spo_attention_plan_splits", c_u32, c_p)
_sig("spo_attention_workspace", c_int, c_p, P(c_u64))
_sig("spo_attention_add_projection", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u64)
_sig("spo_attention_fuses_projection", c_int, c_p, c_p, P(LinearPlan))
_sig("spo_attention_add_fused_projection", c_int, c_p, c_p, P(ChainLink), c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u64)
_sig("spo_attention_add_attention", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u64, c_p, c_p, c_p)
_sig("spo_attention_chunk_plan_create", c_int, P(AttentionGeometry), P(AttentionRows), c_u32, P(c_p))
_sig("spo_attention_chunk_plan_destroy", None, c_p)
_sig("spo_attention_chunk_plan_dispatches", c_u32, c_p)
_sig("spo_attention_chunk_workspace", c_int, c_p, P(c_u64))
_sig("spo_attention_add_chunk_projection", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u64)
_sig("spo_attention_add_chunk_attention", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u64, c_p, c_p, c_p)
_sig("spo_attention_add_path_commit", c_int, c_p, c_p, c_p, c_p, c_p, c_u64)

_sig("spo_norm_add_rms", c_int, c_p, c_p, c_p, c_p, c_u32, c_u32)
_sig("spo_norm_add_rms_table", c_int, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32)
_sig("spo_embedding_add", c_int, c_p, c_u32, c_p, c_u32, c_u32, c_p, c_p, c_u32)
_sig("spo_rope_add_tree_tables", c_int, c_p, c_p, c_p, c_p, c_p, c_u32, P(RopeSequence), c_u32)
_sig("spo_float_projection_add", c_int, c_p, c_p, c_p, c_u32, c_u32, c_u32, c_p, c_u32, c_u32, c_u32, c_u32)
_sig("spo_gdn_layout", c_int, P(GdnShape), c_u32, P(GdnStateStrides), P(c_u64), P(c_u64))
_sig("spo_gdn_add_decode", c_int, c_p, P(GdnDecodeBuffers), P(GdnShape), c_u32, P(GdnStateStrides), c_u32, P(GdnLane), c_u32)
_sig("spo_gdn_add_prefill", c_int, c_p, P(GdnPrefillBuffers), P(GdnShape), c_u32, c_u32, P(GdnStateStrides), c_u32, P(GdnPrefillCapture), c_u32)
_sig("spo_gdn_add_fold", c_int, c_p, c_p, c_p, c_p, c_u64, c_u64, c_u64, P(GdnShape), c_u32, c_u32, P(GdnStateStrides))
_sig("spo_state_codec_layer_bytes", c_u64, c_u32, c_u32)
for _name in ("spo_state_codec_add_quantize", "spo_state_codec_add_dequantize", "spo_state_codec_add_copy"):
    _sig(_name, c_int, c_p, c_p, c_p, P(StateCodecShape))
_sig("spo_moe_workspace_sizes", c_int, P(MoeShape), c_u32, P(c_u64))
_sig("spo_moe_add_routing", c_int, c_p, c_p, c_u32, P(MoeWorkspace), P(MoeShape), c_u32, c_p, c_p)
_sig("spo_moe_add_routed", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32, P(MoeWorkspace), P(MoeShape), c_u32)
_sig("spo_moe_add_routed_norm", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32, P(MoeWorkspace), P(MoeShape), c_u32, c_p, c_p)
_sig("spo_row_copy_add", c_int, c_p, c_p, c_u32, c_u32, c_u32, c_p, c_u32, c_u32, c_u32, c_u32, c_u32)
_sig("spo_sampling_workspace", c_int, c_u32, P(c_u64))
_sig("spo_sampling_add_verify", c_int, c_p, P(SamplingBuffers), c_u32, c_u32, P(LaneRows), P(SamplingPolicy), c_u32, P(c_u32))
class DraftTreeLane(ctypes.Structure):
    _fields_ = [("anchor", c_u32), ("depth", c_u32), ("children", c_u32), ("chain", c_u32), ("slope", ctypes.c_float),
                ("intercept", ctypes.c_float * 7), ("temperature", ctypes.c_float), ("noise", c_u32 * 2)]


_sig("spo_draft_add_tree", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, P(DraftTreeLane), c_u32)
_sig("spo_draft_add_verify_children", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32)
_sig("spo_draft_add_verify_rows", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32, c_u32, ctypes.c_float)
_sig("spo_draft_add_verify_row_slots", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32, ctypes.c_float)
_sig("spo_draft_attention_workspace", c_int, c_u32, c_u32, P(c_u64))
_sig("spo_draft_attention_add_convolution", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32, c_u32)
_sig("spo_draft_attention_add_prepare", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32)
_sig("spo_draft_attention_add_decode", c_int, c_p, c_p, c_p, P(c_u64), P(c_u64), c_p, c_p, P(c_u32), c_u32, c_u32)
_sig("spo_draft_attention_add_context_prefill", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_u64, c_u64, c_u32, c_u32, c_u32)
_sig("spo_draft_attention_add_context_commit", c_int, c_p, c_p, c_p, c_p, c_p, c_p, P(c_u64), P(c_u64), c_p, c_p, P(c_u32), c_u32, c_u32,
     c_u32, c_u32)
_sig("spo_draft_context_window_bytes", c_int, c_u32, P(c_u64))
_sig("spo_draft_attention_add_window_store", c_int, c_p, c_p, c_p, c_u32, c_u32, c_u32)
_sig("spo_draft_attention_add_window_commit", c_int, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32, c_u32, c_u32)
_sig("spo_draft_attention_add_window_load", c_int, c_p, c_p, c_p, c_u32, c_u32, c_u32)
_sig("spo_draft_attention_add_mask_rows", c_int, c_p, c_p, c_p, c_u32, c_u32)
_sig("spo_dflash_draft_create", c_int, c_p, P(DFlashLayout), c_u32, c_u32, P(c_p))
_sig("spo_dflash_draft_destroy", None, c_p)
_sig("spo_dflash_draft_set_layer", c_int, c_p, c_u32, P(DFlashLayer))
_sig("spo_dflash_draft_set_model", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p)
_sig("spo_dflash_draft_buffer", c_int, c_p, c_u32, c_u32, P(c_p))
_sig("spo_dflash_draft_encode_decode", c_int, c_p, c_p, P(c_u32), c_u32)
_sig("spo_dflash_draft_encode_context_prefill", c_int, c_p, c_p, c_u32, c_u32, c_u32, c_int)
_sig("spo_dflash_draft_encode_context_commit", c_int, c_p, c_p, c_p, c_p, P(c_u32), c_u32, c_u32, c_u32)
_sig("spo_sampling_add_acceptance", c_int, c_p, c_p, c_p, c_p, c_p, c_p, c_p, P(LaneRows), P(c_u32), c_u32, P(c_u32))
_sig("spo_dense_verify_set_penalties", c_int, c_p, c_u32, ctypes.c_float, ctypes.c_float, ctypes.c_float)
_sig("spo_hybrid_verify_set_penalties", c_int, c_p, c_u32, ctypes.c_float, ctypes.c_float, ctypes.c_float)
_sig("spo_dense_verify_set_admission", c_int, c_p, c_u32, c_u32, c_u32)
_sig("spo_hybrid_verify_set_admission", c_int, c_p, c_u32, c_u32, c_u32)
_sig("spo_dense_verify_set_stop_tokens", c_int, c_p, P(c_u32))
_sig("spo_hybrid_verify_set_stop_tokens", c_int, c_p, P(c_u32))
_sig("spo_dense_verify_set_thinking_cutoff", c_int, c_p, c_u32, P(ThinkingCutoff))
_sig("spo_hybrid_verify_set_thinking_cutoff", c_int, c_p, c_u32, P(ThinkingCutoff))
_sig("spo_sampling_rebuild_penalty_words", c_int, c_p, c_u32, c_p, ctypes.c_uint64, ctypes.c_uint64, c_u32, c_u32)
_sig("spo_sampling_add_penalties", c_int, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32, P(LaneRows), P(SamplingPenalties), c_u32)
_sig("spo_sampling_add_penalty_count", c_int, c_p, c_p, c_p, c_p, c_u32, P(LaneRows), P(SamplingPenalties), c_u32)
_sig("spo_sampling_add_thinking_cutoff", c_int, c_p, c_p, c_p, c_p, c_p, c_u32, c_u32, P(LaneRows), P(ThinkingCutoff), c_u32)
_sig("spo_lookup_index_create", c_int, P(c_p))
_sig("spo_lookup_index_destroy", None, c_p)
_sig("spo_lookup_index_append", c_int, c_p, c_p, ctypes.c_uint64)
_sig("spo_lookup_index_match", c_int, c_p, P(c_u32), P(c_u32))
_sig("spo_lookup_index_proposals", c_u32, c_p, c_u32, c_p)
_sig("spo_lookup_agreement", c_u32, c_u32, c_u32, c_p, c_u32, c_u32)
_sig("spo_sampling_greedy_rows_static", c_int, ctypes.c_void_p, c_u32, c_u32, c_u32, ctypes.c_void_p, ctypes.c_void_p)
_sig("spo_verify_check_results", c_int, P(LaneRows), P(c_u32), c_u32, c_u32, c_u32, P(c_u32), P(c_u32), P(c_u32), P(c_u32))
_sig("spo_projection_rows", c_int, c_p, P(c_u32), P(c_u32), c_u32, P(c_p))
_sig("spo_hybrid_verify_set_capture", c_int, c_p, P(c_u32), c_u32, c_p)
_sig("spo_dense_verify_set_staged_prefill", c_int, c_p, c_int)
_sig("spo_dense_verify_set_capture", c_int, c_p, P(c_u32), c_u32, c_p)
_sig("spo_dense_verify_set_chained", c_int, c_p, c_int)
_sig("spo_dense_verify_chain_status", c_int, c_p, ctypes.POINTER(ctypes.c_uint32))
_sig("spo_dense_verify_set_test_children", c_int, c_p, c_int)
_sig("spo_dense_verify_encode_prefill", c_int, c_p, c_p, c_u32, c_u32, c_u32)
_sig("spo_dense_verify_set_fused_prepare", c_int, c_p, c_int)
_sig("spo_dense_verify_results", c_int, c_p, P(VerifyLane), c_u32, P(c_u32), P(c_u32), P(c_u32), P(c_u32))
_sig("spg_dense_dimensions", c_int, c_p, P(DenseDimensions))
_sig("spo_dense_verify_load_gguf", c_int, c_p, c_p)
_sig("spg_hybrid_dimensions", c_int, c_p, P(HybridDimensions))
_sig("spo_hybrid_verify_load_gguf", c_int, c_p, c_p)
_sig("spo_dense_verify_create", c_int, c_p, P(DenseDimensions), c_u32, c_u32, c_u32, P(c_p))
_sig("spo_dense_verify_create_chunked", c_int, c_p, P(DenseDimensions), c_u32, c_u32, c_u32, c_u32, P(c_p))
_sig("spo_dense_verify_destroy", None, c_p)
_sig("spo_dense_verify_set_layer", c_int, c_p, c_u32, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p, c_p)
_sig("spo_dense_verify_set_head", c_int, c_p, c_u32, c_p, c_p, c_p)
_sig("spo_dense_verify_buffer", c_int, c_p, c_int, c_u32, P(c_p))
_sig("spo_dense_verify_page_bytes", c_u64, c_p)
_sig("spo_dense_verify_step_bytes", c_u64, c_p, P(VerifyLane), c_u32)
_sig("spo_dense_verify_encode", c_int, c_p, c_p, P(VerifyLane), c_u32, c_int)
_sig("spo_dense_verify_encode_part", c_int, c_p, c_p, c_u32, c_u32, P(VerifyLane), c_u32)
_sig("spo_hybrid_verify_create", c_int, c_p, P(HybridDimensions), c_u32, c_u32, c_u32, P(c_p))
_sig("spo_hybrid_verify_create_chunked", c_int, c_p, P(HybridDimensions), c_u32, c_u32, c_u32, c_u32, P(c_p))
_sig("spo_hybrid_verify_encode_prefill", c_int, c_p, c_p, c_u32, c_u32, c_u32, c_u32, c_u32, c_u32, c_u32)
_sig("spo_hybrid_verify_destroy", None, c_p)
_sig("spo_hybrid_verify_set_layer", c_int, c_p, c_u32, P(HybridLayer))
_sig("spo_hybrid_verify_set_head", c_int, c_p, c_u32, c_p, c_p, c_p)
_sig("spo_hybrid_verify_buffer", c_int, c_p, c_u32, c_u32, P(c_p))
_sig("spo_hybrid_verify_layout", c_int, c_p, P(c_u64), P(c_u64), P(c_u64), P(GdnStateStrides))
_sig("spo_hybrid_verify_step_bytes", c_u64, c_p, P(HybridLane), c_u32)
_sig("spo_hybrid_verify_encode", c_int, c_p, c_p, P(HybridLane), c_u32, c_int)
_sig("spo_hybrid_verify_encode_part", c_int, c_p, c_p, c_u32, c_u32, P(HybridLane), c_u32)
_sig("spo_hybrid_verify_results", c_int, c_p, P(HybridLane), c_u32, P(c_u32), P(c_u32), P(c_u32), P(c_u32))


# ---- GGUF files (include/splash_gguf.h) ----
class GgufTensor(ctypes.Structure):
    _fields_ = [("ggml_type", c_u32), ("dimensions", c_u32), ("dims", ctypes.c_uint64 * 4), ("bytes", ctypes.c_uint64),
                ("format", c_u32), ("reserved", c_u32)]


_sig("spg_open", c_int, ctypes.c_char_p, P(c_p))
_sig("spg_open_parts", c_int, P(ctypes.c_char_p), c_u32, P(c_p))
_sig("spg_close", None, c_p)
_sig("spg_metadata_unsigned", c_int, c_p, ctypes.c_char_p, P(ctypes.c_uint64))
_sig("spg_metadata_float", c_int, c_p, ctypes.c_char_p, P(c_double))
_sig("spg_metadata_string", ctypes.c_size_t, c_p, ctypes.c_char_p, ctypes.c_char_p, ctypes.c_size_t)
_sig("spg_tensor_count", ctypes.c_uint64, c_p)
_sig("spg_tensor_name", ctypes.c_size_t, c_p, ctypes.c_uint64, ctypes.c_char_p, ctypes.c_size_t)
_sig("spg_tensor_info", c_int, c_p, ctypes.c_uint64, P(GgufTensor))
_sig("spg_find", ctypes.c_int64, c_p, ctypes.c_char_p)
_sig("spg_tensor_data", c_p, c_p, ctypes.c_uint64)
_sig("spg_load_image", c_int, c_p, c_p, ctypes.c_uint64, c_u32, c_u32, P(c_p), P(c_u32), P(c_u32), P(c_u32))
_sig("spg_load_bf16", c_int, c_p, c_p, ctypes.c_uint64, P(c_p), P(ctypes.c_uint64))
