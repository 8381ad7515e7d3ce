"""anemone_amd -- Python bindings of libanemone_hip.so, the MI355X backend and operator prepare functions of the
routed-expert path. Everything here goes through the library's C ABI (include/anemone_backend.h,
include/anemone_ops.h, include/anemone_records.h); there is no CPU fallback: without the built library, or without
a card, the calls fail."""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(HERE, "libanemone_hip.so")
PROBE_LIBRARY_PATH = os.path.join(HERE, "libanemone_probe.so")

STATUS_OK, STATUS_INVALID_ARGUMENT, STATUS_OUT_OF_MEMORY = 0, 1, 2
STATUS_DEVICE_ERROR, STATUS_TIMED_OUT, STATUS_UNSUPPORTED, STATUS_BUSY = 5, 6, 7, 8
WEIGHT_FORMAT_EXL3, WEIGHT_FORMAT_E2M1_SCALED, WEIGHT_FORMAT_E4M3_SCALED, WEIGHT_FORMAT_E4M3_BLOCK128 = 2, 3, 5, 6
WEIGHT_FORMAT_E2M1_GFX950, WEIGHT_FORMAT_E4M3_GFX950 = 7, 8  # the two _SCALED formats in gfx950's own lane order
WEIGHT_FORMAT_E4M3_BLOCK128_GFX950 = 9  # E4M3_BLOCK128's codes in E4M3_GFX950's lane order, its float32 scales as they are
ARITHMETIC_CLASS_GFX950 = 950
BACKEND_NO_KERNEL = 0xFFFFFFFF
LAUNCH_CHAIN, LAUNCH_SIDE, LAUNCH_RESUME, LAUNCH_JOIN, LAUNCH_SIDE_MORE = 0, 1, 2, 3, 4  # kernel_launch.branch
ROUTER_SORT_ROWS = 384
EXL3_TCP_CHUNK_PAIRS = 160
EXL3_EXPERT_LAUNCHES, EXL3_TC_LAUNCHES = 5, 5
EXL3_TC_STATIC_SCRATCH_BYTES = 16 << 20
EXL3_TC_GATE_UP_SLICES, EXL3_TC_DOWN_SLICES = 4, 4
AFFINITY_SQRT_SOFTPLUS, AFFINITY_SIGMOID = 0, 1
SECOND = 1_000_000_000

u8, u32, u64, f32 = C.c_uint8, C.c_uint32, C.c_uint64, C.c_float


class AnemoneError(RuntimeError):
    def __init__(self, what, status):
        super().__init__("%s: status %d (%s)" % (what, status, status_text(status)))
        self.status = status


class KernelLaunch(C.Structure):
    _fields_ = [("kernel", u32), ("grid", u32 * 3), ("block", u32 * 3), ("dynamic_shared_byte_count", u32),
                ("argument_byte_count", u32), ("branch", u32), ("argument", u8 * 192)]


class CardDescription(C.Structure):
    _fields_ = [("name", C.c_char * 96), ("bus_address", C.c_char * 32), ("arithmetic_class", u32),
                ("link_generation", u32), ("link_lane_count", u32), ("reserved_zero", u32),
                ("memory_total_bytes", u64), ("memory_free_bytes", u64), ("memory_reserved_bytes", u64)]


class Range(C.Structure):
    _fields_ = [("byte_offset", u64), ("byte_count", u64)]


class Shape(C.Structure):
    _fields_ = [("output_size", u32), ("input_size", u32), ("bits_per_weight", u32), ("reserved_must_be_zero", u32)]


class Exl3ReconstructRecord(C.Structure):
    _fields_ = [("matrix_offset", u64), ("output_offset", u64), ("input_size", u32), ("output_size", u32),
                ("bits_per_weight", u32), ("reserved_zero", u32)]


class Exl3ExpertRecord(C.Structure):
    _fields_ = [("jobs_offset", u64), ("input_offset", u64), ("operands_offset", u64), ("products_offset", u64),
                ("hidden_offset", u64), ("output_offset", u64), ("input_size", u32), ("inner_size", u32),
                ("pair_count", u32), ("pairs_per_row", u32), ("job_count", u32), ("bits_per_weight", u32),
                ("activation_limit", f32), ("reserved_zero", u32), ("widths_offset", u64)]


class RowSumArguments(C.Structure):
    _fields_ = [("pair_output_offset", u64), ("row_output_offset", u64), ("width", u32), ("pairs_per_row", u32)]


class Exl3TcpRecord(C.Structure):
    _fields_ = [("picks_offset", u64), ("expert_offsets_offset", u64), ("hidden_offset", u64), ("workspace_offset", u64),
                ("output_offset", u64), ("row_count", u32), ("intermediate", u32), ("bits_x2", u32), ("pass_", u32),
                ("activation_limit", f32), ("rotation", u32), ("half_rows", u32), ("part", u32), ("step_offset", u64),
                ("cone_layer", u32), ("two_blocks", u32), ("widths_offset", u64), ("hidden", u32), ("pairs_per_row", u32),
                ("expert_count", u32), ("reserved_zero", u32)]


class Exl3TcRecord(C.Structure):
    _fields_ = [("jobs_offset", u64), ("hidden_offset", u64), ("workspace_offset", u64), ("output_offset", u64),
                ("row_count", u32), ("job_capacity", u32), ("intermediate", u32), ("bits_x2", u32),
                ("activation_limit", f32), ("pass_", u32), ("rotation", u32), ("shared_sum", u32),
                ("shared_offset", u64), ("widths_offset", u64), ("hidden", u32), ("pairs_per_row", u32), ("expert_count", u32),
                ("reserved_zero", u32)]


class RouterKernels(C.Structure):
    _fields_ = [(name, u32) for name in ("select", "wide_select", "wide_count", "wide_place", "wide_jobs",
                                         "wide_small", "select_draft", "projection", "projection_tiles")]


class RoutedExpertsDescription(C.Structure):
    _fields_ = [(name, Range) for name in ("jobs", "expert_weights", "codes", "exponents", "operands", "hidden",
                                           "hidden_codes", "hidden_exponents", "hidden_operands", "pair_output",
                                           "row_output")] + \
               [("gate_up_shape", Shape), ("down_shape", Shape), ("weight_format", C.c_int), ("job_count", u32),
                ("row_count", u32), ("pairs_per_row", u32), ("gate_up_slice_count", u32), ("down_slice_count", u32),
                ("activation_limit", f32), ("reserved_zero", u32)]


class WideExpertGateUpArguments(C.Structure):
    _fields_ = [("tiles_offset", u64), ("pairs_offset", u64), ("codes_offset", u64), ("exponents_offset", u64), ("operands_offset", u64),
                ("hidden_codes_offset", u64), ("hidden_exponents_offset", u64), ("hidden_operands_offset", u64), ("output_size", u32),
                ("input_size", u32), ("tile_count", u32), ("pairs_per_row", u32), ("activation_limit", f32), ("pair_count", u32)]


class WideExpertDownArguments(C.Structure):
    _fields_ = [("tiles_offset", u64), ("pairs_offset", u64), ("codes_offset", u64), ("exponents_offset", u64), ("operands_offset", u64),
                ("output_offset", u64), ("output_size", u32), ("input_size", u32), ("tile_count", u32), ("pair_count", u32)]


class LinearWideExpertsDescription(C.Structure):
    _fields_ = [("experts", RoutedExpertsDescription), ("tiles", Range), ("pairs", Range), ("tile_count", u32), ("reserved_zero", u32)]


class RouterDescription(C.Structure):
    _fields_ = [("experts", C.POINTER(RoutedExpertsDescription)), ("expert_offsets", C.POINTER(u64)),
                ("expert_widths", C.POINTER(u32)), ("step", Range), ("scores", Range), ("bias", Range),
                ("offsets", Range), ("affinities", Range), ("order", C.c_int), ("expert_count", u32),
                ("pick_count", u32), ("affinity_kind", u32), ("route_scale", f32)]


class RouterWideDescription(C.Structure):
    _fields_ = [("expert_offsets", C.POINTER(u64)), ("expert_widths", C.POINTER(u32)), ("step", Range), ("scores", Range),
                ("bias", Range), ("offsets", Range), ("expert_weights", Range), ("affinities", Range), ("picks", Range),
                ("counts", Range), ("pairs", Range), ("runs", Range), ("tiles", Range), ("jobs", Range),
                ("gate_up_shape", Shape), ("down_shape", Shape), ("weight_format", C.c_int), ("order", C.c_int),
                ("row_count", u32), ("reserved_zero", u32), ("expert_count", u32), ("pick_count", u32),
                ("affinity_kind", u32), ("route_scale", f32)]


class RouterProjectionDescription(C.Structure):
    _fields_ = [("weights", Range), ("rows", Range), ("output", Range), ("row_count", u32), ("hidden", u32),
                ("expert_count", u32), ("reserved_zero", u32)]


class LinearKernels(C.Structure):
    _fields_ = [("activation_quantize", u32), ("expert_gate_up", u32 * 5), ("expert_down", u32 * 5), ("expert_row_sum", u32),
                ("trunk_linear_quantized", u32 * 5), ("trunk_linear_bfloat16", u32 * 5), ("trunk_hidden", u32),
                ("trunk_linear_quantized_wide", u32 * 5), ("trunk_linear_bfloat16_wide", u32 * 5),
                ("trunk_linear_quantized_interleaved", u32), ("expert_gate_up_e4m3", u32 * 5), ("expert_down_e4m3", u32 * 5),
                ("expert_gate_up_b128", u32 * 5), ("expert_down_b128", u32 * 5), ("activation_quantize_128", u32),
                ("expert_gate_up_gfx950", u32 * 5), ("expert_down_gfx950", u32 * 5), ("expert_gate_up_e4m3_gfx950", u32 * 5),
                ("expert_down_e4m3_gfx950", u32 * 5), ("expert_gate_up_b128_gfx950", u32 * 5), ("expert_down_b128_gfx950", u32 * 5)]


class ExpertFusedKernels(C.Structure):
    _fields_ = [("gate_up_quantize", u32 * 5), ("shared_join", u32 * 5), ("join", u32), ("gate_up_quantize_e4m3", u32 * 5), ("post", u32)]


class LinearMatrix(C.Structure):
    _fields_ = [("stored", Range), ("shape", Shape), ("weight_format", C.c_int), ("slice_count", u32), ("wide_form", C.c_int),
                ("reserved_zero", u32)]


class TrunkQuantizedDescription(C.Structure):
    _fields_ = [("matrices", LinearMatrix * 2), ("codes", Range), ("exponents", Range), ("operands", Range), ("outputs", Range * 2),
                ("matrix_count", u32), ("row_count", u32)]


class SharedExpertDescription(C.Structure):
    _fields_ = [("gate", LinearMatrix), ("up", LinearMatrix), ("down", LinearMatrix)] + \
               [(name, Range) for name in ("codes", "exponents", "operands", "gate_output", "up_output", "hidden", "hidden_codes",
                                           "hidden_exponents", "hidden_operands", "output")] + \
               [("row_count", u32), ("activation_limit", f32)]


class ExpertJoinDescription(C.Structure):
    _fields_ = [(name, Range) for name in ("pair_output", "shared_output", "streams", "post", "comb", "row_sums")] + \
               [("pairs_per_row", u32), ("row_count", u32), ("width", u32)]


class ExpertSharedJoinDescription(C.Structure):
    _fields_ = [("down", LinearMatrix), ("codes", Range), ("exponents", Range), ("operands", Range), ("join", ExpertJoinDescription)]


class TrunkLinearQuantizedArguments(C.Structure):
    _fields_ = [("weights_offset", u64 * 2), ("output_offset", u64 * 2), ("codes_offset", u64), ("exponents_offset", u64),
                ("operands_offset", u64), ("output_size", u32 * 2), ("input_size", u32), ("row_count", u32)]


class ExpertJoinArguments(C.Structure):
    _fields_ = [("pair_output_offset", u64), ("shared_output_offset", u64), ("streams_offset", u64), ("post_offset", u64),
                ("comb_offset", u64), ("row_sums_offset", u64), ("pairs_per_row", u32), ("reserved_zero", u32)]


class DenseLinearKernels(C.Structure):
    _fields_ = [("products", u32 * 8), ("wide_products", u32 * 2)]


class DenseLinearDescription(C.Structure):
    _fields_ = [("weights", Range), ("rows", Range), ("output", Range), ("step", Range), ("output_size", u32), ("input_size", u32),
                ("row_count", u32), ("weight_type", u32), ("output_type", u32), ("flags", u32), ("output_scale", f32),
                ("epsilon", f32), ("cone_layer", u32)]


class HyperKernelsRecord(C.Structure):
    _fields_ = [(name, u32) for name in ("mix_finish", "final_collapse", "post", "embed", "draft_inputs", "final_kept")]


class HyperSiteDescription(C.Structure):
    _fields_ = [(name, Range) for name in ("streams", "carried_pre", "mixes", "scale", "base", "norm_weight", "post", "comb", "hidden",
                                           "output", "routed_sums")] + [("row_count", u32), ("reserved_zero", u32)]


class SiteFrontKernels(C.Structure):
    _fields_ = [("fronts", u32 * 8)]


class SiteFrontDescription(C.Structure):
    _fields_ = [(name, Range) for name in ("streams", "carried_pre", "mix_weights", "scale", "base", "norm_weight", "post", "comb", "hidden",
                                           "codes", "exponents", "operands", "scratch")] + \
               [("router", C.POINTER(RouterDescription)), ("router_weights", Range), ("kind", u32), ("row_count", u32), ("reserved_zero", u32)]


class ExpertPause(C.Structure):
    _fields_ = [("jobs_offset", u64), ("slots_offset", u64), ("slot_byte_count", u64), ("expert_byte_count", u64), ("matrix_offsets", u64 * 3),
                ("first_host_expert", u32), ("host_expert_count", u32), ("jobs_per_row", u32), ("slot_count", u32), ("card", u32),
                ("after_segment", u32)]


class ExpertSlots(C.Structure):
    _fields_ = [("fields", C.POINTER(u64)), ("pause_mark", u64), ("slot_count", u32), ("next_slot", u32)]


class ExpertHostCopies(C.Structure):
    _fields_ = [("block", C.POINTER(C.c_ubyte)), ("byte_count", u64), ("table_staging_offset", u64)]


class ExpertPauseUpload(C.Structure):
    _fields_ = [("slot", u32), ("host_expert", u32)]


class LinearWideKernels(C.Structure):
    _fields_ = [("wide_expert_gate_up", u32), ("wide_expert_down", u32), ("wide_expert_gate_up_e4m3", u32), ("wide_expert_down_e4m3", u32),
                ("wide_expert_gate_up_b128", u32), ("wide_expert_down_b128", u32)]


class PackTensor(C.Structure):
    """A tensor record as a pack stores it (include/anemone_descriptor.h: struct pack_tensor, 64 bytes)."""
    _fields_ = [("byte_offset_in_extent", u64), ("byte_count", u64), ("extent_index", u32), ("name_byte_offset", u32), ("name_byte_count", u32),
                ("element_type", u32), ("dimension_count", u32), ("dimensions", u32 * 4), ("weight_format", u32), ("bits_per_weight", u32),
                ("reserved_zero", u32 * 1)]


PACK_TENSOR_DTYPE = np.dtype([("byte_offset_in_extent", "<u8"), ("byte_count", "<u8"), ("extent_index", "<u4"), ("name_byte_offset", "<u4"),
                              ("name_byte_count", "<u4"), ("element_type", "<u4"), ("dimension_count", "<u4"), ("dimensions", "<u4", (4,)),
                              ("weight_format", "<u4"), ("bits_per_weight", "<u4"), ("reserved_zero", "<u4", (1,))])


class Exl3PackView(C.Structure):
    _fields_ = [("header_digest", u64), ("file_byte_count", u64), ("tensors", C.c_void_p), ("name_bytes", C.c_void_p), ("tensor_count", u32),
                ("name_byte_count", u32)]


class Exl3DescriptorMatrix(C.Structure):
    _fields_ = [("kind", C.c_char_p), ("outputs", u32), ("inputs", u32)]


class Exl3EstablishedPack(C.Structure):
    _fields_ = [("name", C.c_char_p), ("header_digest", u64), ("file_byte_count", u64)]


class Exl3DescriptorModel(C.Structure):
    _fields_ = [("model_type", C.c_char_p), ("layers", u32), ("experts_per_layer", u32), ("hidden", u32), ("intermediate", u32),
                ("matrices", Exl3DescriptorMatrix * 3), ("established", C.POINTER(Exl3EstablishedPack)), ("established_count", u32),
                ("routes_per_row", u32), ("cone_first_layer", u32)]


class LinearNativeKernels(C.Structure):
    _fields_ = [("native_expert_gate_up", u32), ("native_expert_down", u32), ("native_expert_gate_up_e4m3", u32), ("native_expert_down_e4m3", u32),
                ("native_expert_gate_up_b128", u32), ("native_expert_down_b128", u32)]


class QuantizeDescription(C.Structure):
    _fields_ = [("values", Range), ("codes", Range), ("exponents", Range), ("operands", Range), ("width", u32),
                ("row_count", u32)]


JOB_DTYPE = np.dtype([("gate_offset", "<u8"), ("up_offset", "<u8"), ("down_offset", "<u8"), ("row_count", "<u4"),
                      ("expert", "<u4"), ("pair_index", "<u4", (8,)), ("route_weight", "<f4", (8,))])

_lib = None
_probe_lib = None


def probe_library():
    """Loads libanemone_probe.so (the copy, instruction-rate and self-check kernels: measurement and tests, not part of the
    drop-in library). Its kernel files add themselves to the backend's kernel table as the library is loaded, after which
    Card.kernel finds them like any other."""
    global _probe_lib
    if _probe_lib is None:
        library()
        if not os.path.exists(PROBE_LIBRARY_PATH):
            raise ImportError("%s is missing: run `python -m anemone_amd.build`" % PROBE_LIBRARY_PATH)
        _probe_lib = C.CDLL(PROBE_LIBRARY_PATH)
    return _probe_lib


def library():
    """The loaded library. Raises if it was not built: there is no other implementation to fall back to."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIBRARY_PATH):
            raise ImportError("%s is missing: run `python -m anemone_amd.build` (hipcc, gfx950)" % LIBRARY_PATH)
        lib = C.CDLL(LIBRARY_PATH)
        vp, launch_p = C.c_void_p, C.POINTER(KernelLaunch)
        lib.status_text.restype = C.c_char_p
        lib.status_text.argtypes = [C.c_int]
        signatures = {
            "backend_hip_card_count": [C.POINTER(u32)],
            "backend_hip_card_describe": [u32, C.POINTER(CardDescription)],
            "backend_hip_card_open": [u32, u64, C.POINTER(vp)],
            "backend_hip_staging_allocate": [u64, C.POINTER(vp)],
            "backend_hip_upload_begin": [vp, u64, vp, u64, C.POINTER(u64)],
            "backend_hip_upload_wait": [vp, u64, u64],
            "backend_hip_download_begin": [vp, u64, vp, u64, C.POINTER(u64)],
            "backend_hip_kernel_prepare": [vp, C.c_char_p, C.c_char_p, u32, C.POINTER(u32)],
            "backend_hip_launch_run": [vp, launch_p, u32],
            "backend_hip_launch_run_timed": [vp, launch_p, u32, C.POINTER(C.c_double)],
            "backend_hip_launch_wait": [vp, u64],
            "backend_hip_graph_capture": [vp, launch_p, u32, C.POINTER(u32)],
            "backend_hip_graph_run": [vp, u32],
            "backend_hip_measure_begin": [vp],
            "backend_hip_measure_end": [vp],
            "backend_hip_measure_elapsed_us": [vp, u64, C.POINTER(C.c_double)],
            "backend_hip_kernel_table_entry": [u32, C.POINTER(C.c_char_p), C.POINTER(C.c_char_p), C.POINTER(u32)],
            "exl3_reconstruct_prepare": [C.POINTER(Exl3ReconstructRecord), u64, u32, launch_p],
            "exl3_experts_prepare": [C.POINTER(Exl3ExpertRecord), u64, vp, vp, u32, launch_p],
            "exl3_experts_fast_prepare": [C.POINTER(Exl3ExpertRecord), u64, vp, vp, u32, launch_p],
            "exl3_experts_relaxed_prepare": [C.POINTER(Exl3ExpertRecord), u64, vp, vp, u32, launch_p],
            "exl3_row_sum_prepare": [C.POINTER(RowSumArguments), u32, u64, vp, vp, launch_p],
            "exl3_tc_prepare": [C.POINTER(Exl3TcRecord), u64, vp, vp, launch_p],
            "exl3_tc_prepare_short": [C.POINTER(Exl3TcRecord), u64, vp, vp, launch_p],
            "exl3_tc_prepare_paired": [C.POINTER(Exl3TcRecord), u64, vp, vp, launch_p],
            "exl3_tcp_prepare": [C.POINTER(Exl3TcpRecord), u64, vp, vp, launch_p, C.POINTER(u32)],
            "router_kernels_prepare": [vp, vp, C.POINTER(RouterKernels)],
            "router_select_prepare": [C.POINTER(RouterDescription), u64, C.POINTER(RouterKernels), launch_p],
            "router_projection_prepare": [C.POINTER(RouterProjectionDescription), u64, C.POINTER(RouterKernels), launch_p],
            "router_wide_prepare": [C.POINTER(RouterWideDescription), u64, C.POINTER(RouterKernels), launch_p],
            "router_wide_small_prepare": [C.POINTER(RouterWideDescription), u64, C.POINTER(RouterKernels), launch_p],
            "linear_kernels_prepare": [vp, vp, u32, C.POINTER(LinearKernels)],
            "linear_quantize_prepare": [C.POINTER(QuantizeDescription), u64, C.POINTER(LinearKernels), launch_p],
            "linear_quantize_128_prepare": [C.POINTER(QuantizeDescription), u64, C.POINTER(LinearKernels), launch_p],
            "linear_wide_experts_block128_prepare": [C.POINTER(LinearWideExpertsDescription), u64, C.POINTER(LinearKernels),
                                                     C.POINTER(LinearWideKernels), launch_p],
            "linear_routed_experts_prepare": [C.POINTER(RoutedExpertsDescription), u64, C.POINTER(LinearKernels), launch_p],
            "linear_default_slice_count": [C.c_int, C.c_int, C.c_int, C.POINTER(Shape), u32, C.POINTER(u32)],
            "linear_wide_kernels_prepare": [vp, vp, u32, C.POINTER(LinearWideKernels)],
            "linear_wide_experts_prepare": [C.POINTER(LinearWideExpertsDescription), u64, C.POINTER(LinearKernels),
                                            C.POINTER(LinearWideKernels), launch_p],
            "linear_native_kernels_prepare": [vp, vp, u32, C.POINTER(LinearNativeKernels)],
            "linear_native_experts_prepare": [C.POINTER(LinearWideExpertsDescription), u64, C.POINTER(LinearKernels),
                                              C.POINTER(LinearNativeKernels), launch_p],
            "weight_format_gfx950_pack": [C.c_int, C.POINTER(Shape), vp, u64, vp, u64],
            "weight_format_gfx950_unpack": [C.c_int, C.POINTER(Shape), vp, u64, vp, u64],
            "expert_fused_kernels_prepare": [vp, vp, u32, C.POINTER(ExpertFusedKernels)],
            "expert_producer_prepare": [C.POINTER(RoutedExpertsDescription), Range, u64, C.POINTER(LinearKernels),
                                        C.POINTER(ExpertFusedKernels), launch_p],
            "linear_trunk_quantized_prepare": [C.POINTER(TrunkQuantizedDescription), u64, C.POINTER(LinearKernels), launch_p],
            "linear_shared_expert_prepare": [C.POINTER(SharedExpertDescription), u64, C.POINTER(LinearKernels), launch_p],
            "expert_join_prepare": [C.POINTER(ExpertJoinDescription), u64, C.POINTER(ExpertFusedKernels), launch_p],
            "dense_linear_kernels_prepare": [vp, vp, C.POINTER(DenseLinearKernels)],
            "dense_linear_prepare": [C.POINTER(DenseLinearDescription), u64, C.POINTER(DenseLinearKernels), launch_p],
            "hyper_kernels_prepare": [vp, vp, C.POINTER(HyperKernelsRecord)],
            "hyper_site_prepare": [C.POINTER(HyperSiteDescription), u64, C.POINTER(HyperKernelsRecord), launch_p],
            "expert_pause_plan": [C.POINTER(ExpertPause), vp, u64, C.POINTER(ExpertSlots), C.POINTER(ExpertPauseUpload), C.POINTER(u32),
                                  C.POINTER(u32)],
            "expert_pause_run": [vp, vp, C.POINTER(ExpertPause), u32, C.POINTER(ExpertSlots), vp, vp, u64, C.POINTER(u32)],
            "site_front_kernels_prepare": [vp, vp, C.POINTER(SiteFrontKernels)],
            "site_front_prepare": [C.POINTER(SiteFrontDescription), u64, C.POINTER(RouterKernels), C.POINTER(SiteFrontKernels), launch_p],
            "site_front_check": [vp, vp, Range, vp, u64, C.POINTER(u32)],
            "expert_host_copies_attach": [vp, C.POINTER(ExpertPause), u32, C.POINTER(u64), u64, vp, u64, u64, u64, C.POINTER(ExpertHostCopies),
                                          C.POINTER(u64)],
            "expert_post_prepare": [C.POINTER(ExpertJoinDescription), u64, u32, launch_p],
            "exl3_descriptor_check": [C.c_char_p, C.POINTER(Exl3PackView), C.POINTER(Exl3DescriptorModel), C.c_char_p, u64, C.c_bool],
            "exl3_descriptor_tc_check": [C.c_char_p, C.POINTER(Exl3DescriptorModel), u32, u32],
            "expert_shared_join_prepare": [C.POINTER(ExpertSharedJoinDescription), u64, C.POINTER(LinearKernels),
                                           C.POINTER(ExpertFusedKernels), launch_p],
        }
        for name, argtypes in signatures.items():
            function = getattr(lib, name)
            function.restype = C.c_int
            function.argtypes = argtypes
        lib.expert_host_copies_detach.restype = None
        lib.expert_host_copies_detach.argtypes = [vp, C.POINTER(ExpertHostCopies)]
        lib.backend_hip_card_close.restype = None
        lib.backend_hip_card_close.argtypes = [vp, u64]
        lib.backend_hip_staging_free.restype = None
        lib.backend_hip_staging_free.argtypes = [vp]
        lib.backend_hip_format_supported.restype = C.c_bool
        lib.backend_hip_format_supported.argtypes = [u32, C.c_int]
        lib.backend_hip_kernel_table_count.restype = u32
        lib.exl3_scratch_byte_count.restype = u64
        lib.exl3_scratch_byte_count.argtypes = [u32, u32]
        lib.anemone_sha256.restype = None
        lib.anemone_sha256.argtypes = [vp, u64, vp]
        lib.exl3_width_name.restype = C.c_char_p
        lib.exl3_width_name.argtypes = [u32]
        _lib = lib
    return _lib


def status_text(status):
    return library().status_text(status).decode()


def check(status, what):
    if status != STATUS_OK:
        raise AnemoneError(what, status)


def gfx950_pack(weight_format, outputs, inputs, stored):
    """A matrix of the reference's E2M1_SCALED / E4M3_SCALED bytes (or of E4M3_BLOCK128's) in gfx950's lane order
    (weight_format names the GFX950 format): the library's load-time re-lay-out, weight_format_gfx950_pack."""
    stored = np.ascontiguousarray(stored, dtype=np.uint8)
    packed = np.empty_like(stored)
    shape = Shape(outputs, inputs, 4 if weight_format == WEIGHT_FORMAT_E2M1_GFX950 else 8, 0)
    check(library().weight_format_gfx950_pack(weight_format, C.byref(shape), stored.ctypes.data, stored.nbytes, packed.ctypes.data, packed.nbytes),
          "weight_format_gfx950_pack")
    return packed


def gfx950_unpack(weight_format, outputs, inputs, packed):
    packed = np.ascontiguousarray(packed, dtype=np.uint8)
    stored = np.empty_like(packed)
    shape = Shape(outputs, inputs, 4 if weight_format == WEIGHT_FORMAT_E2M1_GFX950 else 8, 0)
    check(library().weight_format_gfx950_unpack(weight_format, C.byref(shape), packed.ctypes.data, packed.nbytes, stored.ctypes.data, stored.nbytes),
          "weight_format_gfx950_unpack")
    return stored


def backend_table():
    """Address of `backend_hip_value`, the table a prepare function takes as its backend."""
    return C.addressof(C.c_char.in_dll(library(), "backend_hip_value"))


def card_count():
    count = u32(0)
    check(library().backend_hip_card_count(C.byref(count)), "card_count")
    return count.value


def exl3_tcp_layout(rows, picks, experts, hidden, intermediate):
    """The prefill workspace's parts (byte offsets) as exl3_tcp_layout_of of the library's records lays them."""
    rounded = lambda n: (n + 255) // 256 * 256
    pairs, blocks = rows * picks, (rows + ROUTER_SORT_ROWS - 1) // ROUTER_SORT_ROWS
    layout = {"chunk_capacity": pairs // EXL3_TCP_CHUNK_PAIRS + experts, "counts": 0}
    layout["runs"] = layout["counts"] + rounded(blocks * experts * 4)
    layout["header"] = layout["runs"] + rounded(experts * 8)
    layout["chunks"] = layout["header"] + 256
    layout["sorted"] = layout["chunks"] + rounded(layout["chunk_capacity"] * 16)
    layout["place_of"] = layout["sorted"] + rounded(pairs * 4)
    layout["operands"] = layout["place_of"] + rounded(pairs * 4)
    layout["gate_up"] = layout["operands"] + rounded(2 * pairs * hidden * 2)
    layout["down"] = layout["gate_up"] + rounded(2 * pairs * intermediate * 4)
    layout["total"] = layout["down"] + rounded(pairs * hidden * 4)
    return layout


def exl3_tc_workspace_bytes(pairs, hidden, intermediate):
    align = lambda n: (n + 255) // 256 * 256
    return (align(2 * pairs * hidden * 2) + align(EXL3_TC_GATE_UP_SLICES * 2 * pairs * intermediate * 4) +
            align(EXL3_TC_DOWN_SLICES * pairs * hidden * 4))


class Card:
    """One open card: its arena, a staging block for copies, and a bump allocator over the arena."""

    def __init__(self, arena_bytes, index=0, staging_bytes=64 << 20):
        self.lib = library()
        if card_count() <= index:
            raise AnemoneError("no card %d on this machine" % index, STATUS_UNSUPPORTED)
        self.arena_bytes = int(arena_bytes)
        self.handle = C.c_void_p()
        check(self.lib.backend_hip_card_open(index, self.arena_bytes, C.byref(self.handle)), "card_open")
        self.staging = C.c_void_p()
        self.staging_bytes = int(staging_bytes)
        check(self.lib.backend_hip_staging_allocate(self.staging_bytes, C.byref(self.staging)), "staging_allocate")
        self.staging_view = np.ctypeslib.as_array(C.cast(self.staging, C.POINTER(u8)), shape=(self.staging_bytes,))
        self.cursor = 256

    def close(self):
        if self.handle:
            self.lib.backend_hip_card_close(self.handle, 10 * SECOND)
            self.lib.backend_hip_staging_free(self.staging)
            self.handle = C.c_void_p()

    def describe(self, index=0):
        description = CardDescription()
        check(self.lib.backend_hip_card_describe(index, C.byref(description)), "card_describe")
        return description

    def reserve(self, byte_count, alignment=256):
        """A range of the arena: the planner's job in the reference, a bump allocation here."""
        offset = (self.cursor + alignment - 1) // alignment * alignment
        if offset + byte_count > self.arena_bytes:
            raise AnemoneError("the arena is full", STATUS_OUT_OF_MEMORY)
        self.cursor = offset + int(byte_count)
        return offset

    def upload(self, offset, array):
        data = np.ascontiguousarray(array).view(np.uint8).reshape(-1)
        ticket = u64(0)
        for start in range(0, data.size, self.staging_bytes):
            piece = data[start:start + self.staging_bytes]
            self.staging_view[:piece.size] = piece
            check(self.lib.backend_hip_upload_begin(self.handle, offset + start, self.staging, piece.size, C.byref(ticket)), "upload_begin")
            check(self.lib.backend_hip_upload_wait(self.handle, ticket, 60 * SECOND), "upload_wait")

    def place(self, array, alignment=256):
        array = np.ascontiguousarray(array)
        offset = self.reserve(array.nbytes, alignment)
        self.upload(offset, array)
        return offset

    def download(self, offset, byte_count, dtype=np.uint8):
        out = np.empty(int(byte_count), dtype=np.uint8)
        ticket = u64(0)
        for start in range(0, out.size, self.staging_bytes):
            size = min(self.staging_bytes, out.size - start)
            check(self.lib.backend_hip_download_begin(self.handle, offset + start, self.staging, size, C.byref(ticket)), "download_begin")
            check(self.lib.backend_hip_upload_wait(self.handle, ticket, 60 * SECOND), "download wait")
            out[start:start + size] = self.staging_view[:size]
        return out.view(dtype)

    def kernel(self, file, function, record_bytes):
        handle = u32(BACKEND_NO_KERNEL)
        check(self.lib.backend_hip_kernel_prepare(self.handle, file.encode(), function.encode(), record_bytes, C.byref(handle)),
              "kernel_prepare %s" % function)
        return handle.value

    def run(self, launches, wait=True):
        array = launches if isinstance(launches, C.Array) else (KernelLaunch * len(launches))(*launches)
        check(self.lib.backend_hip_launch_run(self.handle, array, len(array)), "launch_run")
        if wait:
            self.wait()

    def wait(self, seconds=60):
        check(self.lib.backend_hip_launch_wait(self.handle, seconds * SECOND), "launch_wait")

    def run_timed(self, launches):
        array = launches if isinstance(launches, C.Array) else (KernelLaunch * len(launches))(*launches)
        out = (C.c_double * len(array))()
        check(self.lib.backend_hip_launch_run_timed(self.handle, array, len(array), out), "launch_run_timed")
        return list(out)

    def capture(self, launches):
        array = launches if isinstance(launches, C.Array) else (KernelLaunch * len(launches))(*launches)
        graph = u32(0)
        check(self.lib.backend_hip_graph_capture(self.handle, array, len(array), C.byref(graph)), "graph_capture")
        return graph.value

    def run_graph(self, graph, wait=True):
        check(self.lib.backend_hip_graph_run(self.handle, graph), "graph_run")
        if wait:
            self.wait()

    def measure(self, body):
        """Device microseconds of whatever `body()` queues on the card."""
        check(self.lib.backend_hip_measure_begin(self.handle), "measure_begin")
        body()
        check(self.lib.backend_hip_measure_end(self.handle), "measure_end")
        out = C.c_double(0)
        check(self.lib.backend_hip_measure_elapsed_us(self.handle, 120 * SECOND, C.byref(out)), "measure_elapsed_us")
        return out.value


def step_block(live_rows):
    """struct step_block {u64 sequence; u32 row_count; u32 flags} as bytes."""
    return np.frombuffer(np.array([0], dtype="<u8").tobytes() + np.array([live_rows, 0], dtype="<u4").tobytes(), dtype=np.uint8)


def launches_of(count):
    return (KernelLaunch * count)()


WIDE_PAIR_DTYPE = np.dtype([("pair_index", "<u4"), ("route_weight", "<f4")])
WIDE_RUN_DTYPE = np.dtype([("first_pair", "<u4"), ("pair_count", "<u4")])
WIDE_TILE_DTYPE = np.dtype([("gate_offset", "<u8"), ("up_offset", "<u8"), ("down_offset", "<u8"), ("first_pair", "<u4"),
                            ("pair_count", "<u4")])


def wide_tile_count(rows, picks, experts):
    return (rows * picks + 63) // 64 + experts


def wide_job_count(rows, picks, experts):
    return min(rows * picks, (rows * picks + 7 * experts) // 8)


class WideRouter:
    """The wide select of a layer already laid out in a card's arena (its offsets table, bias, scores and step block):
    reserves the picks, counts, sorted pairs, runs, tiles and the job table of `rows` rows, and prepares the four
    launches."""

    def __init__(self, layer, rows, weight_format, gate_up_shape, down_shape, widths=None, order=0):
        card = layer.card
        self.layer, self.card, self.rows = layer, card, rows
        E, P = layer.E, layer.P
        self.tile_count, self.job_count = wide_tile_count(rows, P, E), wide_job_count(rows, P, E)
        sizes = {"picks": rows * P * 8, "counts": (rows + ROUTER_SORT_ROWS - 1) // ROUTER_SORT_ROWS * E * 4,
                 "pairs": rows * P * 8, "runs": E * 8, "tiles": self.tile_count * 32, "jobs": self.job_count * 96}
        self.ranges = {name: Range(card.reserve(size), size) for name, size in sizes.items()}
        d = RouterWideDescription()
        d.expert_offsets = layer.expert_offsets.ctypes.data_as(C.POINTER(u64))
        self._widths = None if widths is None else np.ascontiguousarray(widths, dtype=np.uint32)
        d.expert_widths = None if widths is None else self._widths.ctypes.data_as(C.POINTER(u32))
        d.step, d.scores = Range(layer.step_offset, 16), Range(layer.scores_offset, rows * E * 4)
        d.bias, d.offsets = Range(layer.bias_offset, E * 4), Range(layer.offsets_offset, E * 24)
        d.expert_weights = Range(layer.weights_offset, layer.weights_bytes)
        d.affinities = Range(layer.affinities_offset, rows * E * 4)
        for name, value in self.ranges.items():
            setattr(d, name, value)
        d.gate_up_shape, d.down_shape, d.weight_format, d.order = gate_up_shape, down_shape, weight_format, order
        d.row_count, d.expert_count, d.pick_count = rows, E, P
        d.affinity_kind, d.route_scale = layer.affinity_kind, layer.route_scale
        self.description = d

    def launches(self, small=False):
        """The four launches of any row count; small: the two of at most ROUTER_SORT_ROWS rows (select, router_wide_small)."""
        launches = launches_of(2 if small else 4)
        prepare = self.card.lib.router_wide_small_prepare if small else self.card.lib.router_wide_prepare
        check(prepare(C.byref(self.description), self.card.arena_bytes, C.byref(self.layer.router_kernels), launches),
              "router_wide_small_prepare" if small else "router_wide_prepare")
        return launches

    def read(self, name, dtype):
        r = self.ranges[name]
        return self.card.download(r.byte_offset, r.byte_count).view(dtype)


class Exl3Layer:
    """One EXL3 MoE layer laid out in a card's arena the way the reference's loader lays one out: the experts'
    stored matrices, the [E][3] offsets table, an optional per-matrix widths table, the router's weights and bias;
    and the scratch ranges of a step of at most `rows` rows. Builds the prepared launches through the library's
    prepare functions."""

    def __init__(self, card, hidden, inner, expert_count, picks, rows, matrices, widths, router_weights_bf16=None,
                 bias=None, affinity_kind=AFFINITY_SIGMOID, route_scale=1.5, limit=10.0, host_experts=()):
        """host_experts: the experts kept in host memory (not on the card): the job table names them by tags and
        run_pause() puts them into the card's slots (one slot a pair of a step) ahead of the experts' launches."""
        self.card, self.H, self.I, self.E, self.P, self.rows = card, hidden, inner, expert_count, picks, rows
        self.limit, self.affinity_kind, self.route_scale = limit, affinity_kind, route_scale
        self.pairs = rows * picks
        lib = card.lib
        widths = np.asarray(widths, dtype=np.uint32).reshape(expert_count, 3)
        self.widths = widths
        self.uniform_width = int(widths[0, 0]) if np.all(widths == widths[0, 0]) else 0
        host_experts = list(host_experts)
        aligned = lambda n: (n + 255) // 256 * 256
        part_bytes = [aligned(max(matrices[e][m].nbytes for e in host_experts)) for m in range(3)] if host_experts else [0, 0, 0]
        slot_bytes = sum(part_bytes)
        total = aligned(sum(m.nbytes + 64 for e, trio in enumerate(matrices) if e not in host_experts for m in trio) + 256)
        self.weights_offset = card.reserve(total + self.pairs * slot_bytes, 256)
        offsets = np.zeros((expert_count, 3), dtype=np.uint64)
        cursor = self.weights_offset
        blob = np.zeros(total, dtype=np.uint8)
        for e, trio in enumerate(matrices):
            if e in host_experts: # a tag: the same for the three matrices
                offsets[e, :] = self.weights_offset + total + 16 * host_experts.index(e)
                continue
            for m, matrix in enumerate(trio):
                cursor = (cursor + 63) // 64 * 64
                offsets[e, m] = cursor
                blob[cursor - self.weights_offset:cursor - self.weights_offset + matrix.nbytes] = matrix
                cursor += matrix.nbytes
        self.weights_bytes = total + self.pairs * slot_bytes
        card.upload(self.weights_offset, blob)
        if host_experts:
            self.pause = ExpertPause()
            self.pause.slots_offset, self.pause.slot_byte_count, self.pause.expert_byte_count = self.weights_offset + total, slot_bytes, slot_bytes
            self.pause.matrix_offsets[0], self.pause.matrix_offsets[1], self.pause.matrix_offsets[2] = 0, part_bytes[0], part_bytes[0] + part_bytes[1]
            self.pause.first_host_expert, self.pause.host_expert_count = 0, len(host_experts)
            self.pause.jobs_per_row, self.pause.slot_count = picks, self.pairs
            # the layer's host arena: every host expert's three matrices at the pause's matrix offsets; the page-locked copies
            # the pauses upload from are the library's to make (expert_host_copies_attach)
            host_arena = np.zeros(len(host_experts) * slot_bytes, dtype=np.uint8)
            for i, e in enumerate(host_experts):
                for m in range(3):
                    at = i * slot_bytes + int(self.pause.matrix_offsets[m])
                    host_arena[at:at + matrices[e][m].nbytes] = matrices[e][m].view(np.uint8).reshape(-1)
            host_offsets = (np.arange(len(host_experts), dtype=np.uint64) * np.uint64(slot_bytes))
            self.host_copies, pause_offsets = ExpertHostCopies(), (u64 * 1)()
            check(lib.expert_host_copies_attach(backend_table(), C.byref(self.pause), 1, host_offsets.ctypes.data_as(C.POINTER(u64)), len(host_experts),
                                                host_arena.ctypes.data, host_arena.nbytes, self.pairs * 96, 64 << 30, C.byref(self.host_copies),
                                                pause_offsets), "expert_host_copies_attach")
            base = C.cast(self.host_copies.block, C.c_void_p).value
            self.pause_copies = C.c_void_p(base + int(pause_offsets[0]))
            self.pause_table_staging = C.c_void_p(base + int(self.host_copies.table_staging_offset))
            self.slot_fields = np.zeros(2 * self.pairs, dtype=np.uint64)
            self.slots = ExpertSlots(self.slot_fields.ctypes.data_as(C.POINTER(u64)), 0, self.pairs, 0)
        self.expert_offsets = offsets
        self.offsets_offset = card.place(offsets)
        packed = (widths[:, 0] | (widths[:, 1] << 8) | (widths[:, 2] << 16)).astype(np.uint32)
        self.packed_widths = packed
        self.widths_offset = card.place(packed) if self.uniform_width == 0 else 0
        self.step_offset = card.place(step_block(rows))
        self.x_offset = card.reserve(rows * hidden * 2)
        self.scores_offset = card.reserve(rows * expert_count * 4)
        self.affinities_offset = card.reserve(rows * expert_count * 4)
        self.bias_offset = card.place(np.zeros(expert_count, dtype=np.float32) if bias is None else np.asarray(bias, dtype=np.float32))
        self.router_offset = card.place(router_weights_bf16) if router_weights_bf16 is not None else 0
        self.jobs_offset = card.reserve(self.pairs * 96)
        self.out_offset = card.reserve(rows * hidden * 4)
        if rows <= 64:  # the chain's scratch and the fused decode's workspace: steps of decode size
            self.scratch_offset = card.reserve(int(lib.exl3_scratch_byte_count(self.pairs, hidden)))
            self.hidden_offset = card.reserve(self.pairs * inner * 2)
            self.workspace_offset = card.reserve(exl3_tc_workspace_bytes(self.pairs, hidden, inner))
        self.tcp_workspace_offset = None
        self.kernels = RouterKernels()
        check(lib.router_kernels_prepare(backend_table(), card.handle, C.byref(self.kernels)), "router_kernels_prepare")
        self.router_kernels = self.kernels

    def set_rows(self, x_bf16, live_rows=None):
        self.card.upload(self.x_offset, x_bf16)
        live = self.rows if live_rows is None else live_rows
        self.card.upload(self.step_offset, step_block(live))

    def release_host_experts(self):
        """Gives the page-locked copies back (expert_host_copies_detach): after the last pause's uploads have retired."""
        self.card.lib.expert_host_copies_detach(backend_table(), C.byref(self.host_copies))

    def run_pause(self):
        """The layer's expert pause behind its select (expert_pause_run): the experts uploaded."""
        self.pause.jobs_offset = self.jobs_offset
        uploaded = u32(0)
        check(self.card.lib.expert_pause_run(backend_table(), self.card.handle, C.byref(self.pause), self.rows, C.byref(self.slots),
                                             self.pause_table_staging, self.pause_copies, 60 * SECOND, C.byref(uploaded)), "expert_pause_run")
        return uploaded.value

    def experts_description(self):
        d = RoutedExpertsDescription()
        d.jobs = Range(self.jobs_offset, self.pairs * 96)
        d.expert_weights = Range(self.weights_offset, self.weights_bytes)
        width = self.uniform_width if self.uniform_width else int(self.widths.max())
        d.gate_up_shape = Shape(self.I, self.H, width, 0)
        d.down_shape = Shape(self.H, self.I, width, 0)
        d.weight_format = WEIGHT_FORMAT_EXL3
        d.job_count, d.row_count, d.pairs_per_row = self.pairs, self.rows, self.P
        d.activation_limit = self.limit
        return d

    def projection_launch(self):
        d = RouterProjectionDescription(Range(self.router_offset, self.E * self.H * 2), Range(self.x_offset, self.rows * self.H * 2),
                                        Range(self.scores_offset, self.rows * self.E * 4), self.rows, self.H, self.E, 0)
        launch = launches_of(1)
        check(self.card.lib.router_projection_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.kernels), launch), "router_projection_prepare")
        return launch

    def select_launch(self, order=0):
        experts = self.experts_description()
        d = RouterDescription()
        d.experts = C.pointer(experts)
        d.expert_offsets = self.expert_offsets.ctypes.data_as(C.POINTER(u64))
        d.expert_widths = self.packed_widths.ctypes.data_as(C.POINTER(u32)) if self.uniform_width == 0 else None
        d.step = Range(self.step_offset, 16)
        d.scores = Range(self.scores_offset, self.rows * self.E * 4)
        d.bias = Range(self.bias_offset, self.E * 4)
        d.offsets = Range(self.offsets_offset, self.E * 24)
        d.affinities = Range(self.affinities_offset, self.rows * self.E * 4)
        d.order, d.expert_count, d.pick_count = order, self.E, self.P
        d.affinity_kind, d.route_scale = self.affinity_kind, self.route_scale
        launch = launches_of(1)
        check(self.card.lib.router_select_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.kernels), launch), "router_select_prepare")
        return launch

    def chain_record(self):
        r = Exl3ExpertRecord()
        r.jobs_offset, r.input_offset = self.jobs_offset, self.x_offset
        r.operands_offset = self.scratch_offset
        r.products_offset = self.scratch_offset + self.pairs * self.H * 4
        r.output_offset = r.products_offset
        r.hidden_offset = self.hidden_offset
        r.input_size, r.inner_size, r.pair_count, r.pairs_per_row = self.H, self.I, self.pairs, self.P
        r.job_count = self.pairs
        r.bits_per_weight = self.uniform_width if self.uniform_width else 4
        r.activation_limit = self.limit
        r.widths_offset = self.widths_offset
        return r

    def chain_launches(self):
        """The reference's seven launches behind the select: five of the chain, then the row sum."""
        record = self.chain_record()
        launches = launches_of(EXL3_EXPERT_LAUNCHES + 1)
        check(self.card.lib.exl3_experts_prepare(C.byref(record), self.card.arena_bytes, backend_table(), self.card.handle,
                                                 ARITHMETIC_CLASS_GFX950, launches), "exl3_experts_prepare")
        row_sum = RowSumArguments(record.output_offset, self.out_offset, self.H, self.P)
        one = launches_of(1)
        check(self.card.lib.exl3_row_sum_prepare(C.byref(row_sum), self.rows, self.card.arena_bytes, backend_table(),
                                                 self.card.handle, one), "exl3_row_sum_prepare")
        launches[EXL3_EXPERT_LAUNCHES] = one[0]
        return launches

    def tc_record(self):
        r = Exl3TcRecord()
        r.jobs_offset, r.hidden_offset = self.jobs_offset, self.x_offset
        r.workspace_offset, r.output_offset = self.workspace_offset, self.out_offset
        r.row_count, r.job_capacity, r.intermediate = self.rows, self.pairs, self.I
        r.bits_x2 = {2: 4, 3: 6, 4: 8, 40: 5}.get(self.uniform_width, 8)
        r.activation_limit = self.limit
        r.widths_offset, r.hidden, r.pairs_per_row = self.widths_offset, self.H, self.P
        r.expert_count = self.E if self.widths_offset else 0
        return r

    def tc_launches(self, shared_offset=None):
        """The fused decode's launches; with shared_offset the combine adds each row's sum to the shared expert's
        bfloat16 rows there, in place, and leaves the float32 output alone."""
        record = self.tc_record()
        if shared_offset is not None:
            record.shared_sum, record.shared_offset = 1, shared_offset
        launches = launches_of(EXL3_TC_LAUNCHES)
        check(self.card.lib.exl3_tc_prepare(C.byref(record), self.card.arena_bytes, backend_table(), self.card.handle, launches), "exl3_tc_prepare")
        return launches

    def wide_router(self):
        width = self.uniform_width if self.uniform_width else int(self.widths.max())
        return WideRouter(self, self.rows, WEIGHT_FORMAT_EXL3, Shape(self.I, self.H, width, 0), Shape(self.H, self.I, width, 0),
                          widths=None if self.uniform_width else self.packed_widths)

    def tcp_record(self, picks_offset):
        if self.tcp_workspace_offset is None:
            self.tcp_layout = exl3_tcp_layout(self.rows, self.P, self.E, self.H, self.I)
            self.tcp_workspace_offset = self.card.reserve(self.tcp_layout["total"], 256)
        r = Exl3TcpRecord()
        r.picks_offset, r.expert_offsets_offset, r.hidden_offset = picks_offset, self.offsets_offset, self.x_offset
        r.workspace_offset, r.output_offset = self.tcp_workspace_offset, self.out_offset
        r.row_count, r.intermediate = self.rows, self.I
        r.bits_x2 = {2: 4, 3: 6, 4: 8, 40: 5}.get(self.uniform_width, 8)
        r.activation_limit = self.limit
        r.widths_offset, r.hidden, r.pairs_per_row, r.expert_count = self.widths_offset, self.H, self.P, self.E
        return r

    def tcp_launches(self, picks_offset):
        """The prefill form: seven launches from the picks [rows][P] of a wide select (or any table of that form)."""
        record = self.tcp_record(picks_offset)
        launches, count = launches_of(8), u32(0)
        check(self.card.lib.exl3_tcp_prepare(C.byref(record), self.card.arena_bytes, backend_table(), self.card.handle, launches,
                                             C.byref(count)), "exl3_tcp_prepare")
        return (KernelLaunch * count.value)(*[launches[i] for i in range(count.value)])

    def jobs(self):
        return self.card.download(self.jobs_offset, self.pairs * 96).view(JOB_DTYPE)

    def output(self):
        return self.card.download(self.out_offset, self.rows * self.H * 4, np.float32).reshape(self.rows, self.H)


class Fp4Layer:
    """One MoE layer of the original FP4 weights (WEIGHT_FORMAT_E2M1_SCALED; or, with weight_format, of FP8 weights,
    WEIGHT_FORMAT_E4M3_SCALED; stored bytes as the reference's packs hold them; with WEIGHT_FORMAT_E2M1_GFX950,
    WEIGHT_FORMAT_E4M3_GFX950 or WEIGHT_FORMAT_E4M3_BLOCK128_GFX950 the matrices, given in the reference's bytes (in
    E4M3_BLOCK128's for the last), go through the library's load-time re-lay-out first) in a card's arena, with the scratch ranges of a step of at most `rows` rows: the quantizer of the rows,
    the router's select, and the four launches of the routed experts."""

    def __init__(self, card, hidden, inner, expert_count, picks, rows, matrices, router_weights_bf16=None,
                 affinity_kind=AFFINITY_SIGMOID, route_scale=1.5, limit=10.0, gate_up_slices=4, down_slices=2,
                 weight_format=WEIGHT_FORMAT_E2M1_SCALED):
        self.card, self.H, self.I, self.E, self.P, self.rows = card, hidden, inner, expert_count, picks, rows
        self.weight_format = weight_format
        self.bits = 4 if weight_format in (WEIGHT_FORMAT_E2M1_SCALED, WEIGHT_FORMAT_E2M1_GFX950) else 8
        self.native = weight_format in (WEIGHT_FORMAT_E2M1_GFX950, WEIGHT_FORMAT_E4M3_GFX950, WEIGHT_FORMAT_E4M3_BLOCK128_GFX950)
        if self.native:  # a matrix that lies at several experts' places is packed once
            packed = {}
            for trio in matrices:
                for m, matrix in enumerate(trio):
                    if id(matrix) not in packed:
                        packed[id(matrix)] = gfx950_pack(weight_format, *((inner, hidden) if m < 2 else (hidden, inner)), matrix)
            matrices = [[packed[id(matrix)] for matrix in trio] for trio in matrices]
        self.block128 = weight_format in (WEIGHT_FORMAT_E4M3_BLOCK128, WEIGHT_FORMAT_E4M3_BLOCK128_GFX950)
        self.limit, self.affinity_kind, self.route_scale = limit, affinity_kind, route_scale
        self.gate_up_slices, self.down_slices = gate_up_slices, down_slices
        self.pairs = rows * picks
        lib = card.lib
        total = sum(m.nbytes + 64 for trio in matrices for m in trio)
        self.weights_offset, self.weights_bytes = card.reserve(total, 256), total
        offsets = np.zeros((expert_count, 3), dtype=np.uint64)
        cursor, blob = self.weights_offset, np.zeros(total, dtype=np.uint8)
        for e, trio in enumerate(matrices):
            for m, matrix in enumerate(trio):
                cursor = (cursor + 63) // 64 * 64
                offsets[e, m] = cursor
                blob[cursor - self.weights_offset:cursor - self.weights_offset + matrix.nbytes] = matrix
                cursor += matrix.nbytes
        card.upload(self.weights_offset, blob)
        self.expert_offsets = offsets
        self.offsets_offset = card.place(offsets)
        self.step_offset = card.place(step_block(rows))
        self.x_offset = card.reserve(rows * hidden * 2)
        self.scores_offset = card.reserve(rows * expert_count * 4)
        self.affinities_offset = card.reserve(rows * expert_count * 4)
        self.bias_offset = card.place(np.zeros(expert_count, dtype=np.float32))
        self.router_offset = card.place(router_weights_bf16) if router_weights_bf16 is not None else 0
        self.jobs_offset = card.reserve(self.pairs * 96)
        names = {"codes": rows * hidden, "exponents": rows * hidden // 32, "operands": rows * hidden * 2,
                 "hidden": self.pairs * inner * 2, "hidden_codes": self.pairs * inner,
                 "hidden_exponents": self.pairs * inner // 32, "hidden_operands": self.pairs * inner * 2,
                 "pair_output": self.pairs * hidden * 2, "row_output": rows * hidden * 4}
        self.ranges = {name: Range(card.reserve(size), size) for name, size in names.items()}
        self.kernels, self.router_kernels = LinearKernels(), RouterKernels()
        check(lib.linear_kernels_prepare(backend_table(), card.handle, ARITHMETIC_CLASS_GFX950, C.byref(self.kernels)), "linear_kernels_prepare")
        check(lib.router_kernels_prepare(backend_table(), card.handle, C.byref(self.router_kernels)), "router_kernels_prepare")

    def set_rows(self, x_bf16, live_rows=None):
        self.card.upload(self.x_offset, x_bf16)
        self.card.upload(self.step_offset, step_block(self.rows if live_rows is None else live_rows))

    def experts_description(self, wide=None):
        """wide: a WideRouter whose job table the experts read instead of the select's."""
        d = RoutedExpertsDescription()
        d.jobs = Range(self.jobs_offset, self.pairs * 96) if wide is None else wide.ranges["jobs"]
        d.expert_weights = Range(self.weights_offset, self.weights_bytes)
        for name, value in self.ranges.items():
            setattr(d, name, value)
        d.gate_up_shape, d.down_shape = Shape(self.I, self.H, self.bits, 0), Shape(self.H, self.I, self.bits, 0)
        d.weight_format = self.weight_format
        d.job_count, d.row_count, d.pairs_per_row = self.pairs if wide is None else wide.job_count, self.rows, self.P
        d.gate_up_slice_count, d.down_slice_count = self.gate_up_slices, self.down_slices
        d.activation_limit = self.limit
        return d

    def quantize_launch(self):
        d = QuantizeDescription(Range(self.x_offset, self.rows * self.H * 2), self.ranges["codes"], self.ranges["exponents"],
                                self.ranges["operands"], self.H, self.rows)
        launch = launches_of(1)
        prepare = self.card.lib.linear_quantize_128_prepare if self.block128 else self.card.lib.linear_quantize_prepare
        check(prepare(C.byref(d), self.card.arena_bytes, C.byref(self.kernels), launch), "linear_quantize_prepare")
        return launch

    def projection_launch(self):
        d = RouterProjectionDescription(Range(self.router_offset, self.E * self.H * 2), Range(self.x_offset, self.rows * self.H * 2),
                                        Range(self.scores_offset, self.rows * self.E * 4), self.rows, self.H, self.E, 0)
        launch = launches_of(1)
        check(self.card.lib.router_projection_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.router_kernels), launch), "router_projection_prepare")
        return launch

    def select_launch(self, order=0):
        experts = self.experts_description()
        d = RouterDescription()
        d.experts = C.pointer(experts)
        d.expert_offsets = self.expert_offsets.ctypes.data_as(C.POINTER(u64))
        d.expert_widths = None
        d.step, d.scores = Range(self.step_offset, 16), Range(self.scores_offset, self.rows * self.E * 4)
        d.bias, d.offsets = Range(self.bias_offset, self.E * 4), Range(self.offsets_offset, self.E * 24)
        d.affinities = Range(self.affinities_offset, self.rows * self.E * 4)
        d.order, d.expert_count, d.pick_count = order, self.E, self.P
        d.affinity_kind, d.route_scale = self.affinity_kind, self.route_scale
        launch = launches_of(1)
        check(self.card.lib.router_select_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.router_kernels), launch), "router_select_prepare")
        return launch

    def wide_router(self):
        return WideRouter(self, self.rows, self.weight_format, Shape(self.I, self.H, self.bits, 0), Shape(self.H, self.I, self.bits, 0))

    def expert_launches(self, wide=None):
        d = self.experts_description(wide)
        launches = launches_of(4)
        check(self.card.lib.linear_routed_experts_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.kernels), launches), "linear_routed_experts_prepare")
        return launches

    def wide_expert_launches(self, wide):
        """The wide form over the tiles and sorted pairs of a WideRouter: gate/up with the quantization, down, row sum."""
        if not hasattr(self, "wide_kernels"):
            self.wide_kernels = LinearWideKernels()
            check(self.card.lib.linear_wide_kernels_prepare(backend_table(), self.card.handle, ARITHMETIC_CLASS_GFX950,
                                                            C.byref(self.wide_kernels)), "linear_wide_kernels_prepare")
        d = LinearWideExpertsDescription()
        d.experts = self.experts_description(wide)
        d.experts.gate_up_slice_count = d.experts.down_slice_count = 1
        d.tiles, d.pairs, d.tile_count = wide.ranges["tiles"], wide.ranges["pairs"], wide.tile_count
        if self.native:
            if not hasattr(self, "native_kernels"):
                self.native_kernels = LinearNativeKernels()
                check(self.card.lib.linear_native_kernels_prepare(backend_table(), self.card.handle, ARITHMETIC_CLASS_GFX950,
                                                                  C.byref(self.native_kernels)), "linear_native_kernels_prepare")
            launches = launches_of(4 if self.block128 else 3)
            check(self.card.lib.linear_native_experts_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.kernels), C.byref(self.native_kernels),
                                                              launches), "linear_native_experts_prepare")
            return launches
        launches = launches_of(4 if self.block128 else 3)
        prepare = self.card.lib.linear_wide_experts_block128_prepare if self.block128 else self.card.lib.linear_wide_experts_prepare
        check(prepare(C.byref(d), self.card.arena_bytes, C.byref(self.kernels), C.byref(self.wide_kernels), launches), "linear_wide_experts_prepare")
        return launches

    def producer_launch(self):
        """One launch in place of the first two of expert_launches(): gate with up, and the hidden vectors' quantization."""
        if not hasattr(self, "fused_kernels"):
            self.fused_kernels = ExpertFusedKernels()
            check(self.card.lib.expert_fused_kernels_prepare(backend_table(), self.card.handle, ARITHMETIC_CLASS_GFX950,
                                                             C.byref(self.fused_kernels)), "expert_fused_kernels_prepare")
            size = self.pairs * (self.I // 32) * 4
            self.arrivals = Range(self.card.place(np.zeros(size, dtype=np.uint8)), size)
        d = self.experts_description()
        launch = launches_of(1)
        check(self.card.lib.expert_producer_prepare(C.byref(d), self.arrivals, self.card.arena_bytes, C.byref(self.kernels),
                                                    C.byref(self.fused_kernels), launch), "expert_producer_prepare")
        return launch

    def read(self, name, dtype=np.uint8):
        r = self.ranges[name]
        return self.card.download(r.byte_offset, r.byte_count, dtype)

    def jobs(self):
        return self.card.download(self.jobs_offset, self.pairs * 96).view(JOB_DTYPE)


LINEAR_WIDE_GROUP_BLOCKS, LINEAR_WIDE_TILE_BLOCKS, LINEAR_INTERLEAVED_CHUNK_BLOCKS, LINEAR_INTERLEAVED_TILE_BLOCKS = 0, 1, 2, 3
LINEAR_MAXIMUM_ROWS = 8
MODEL_STREAMS = 4


DENSE_BFLOAT16, DENSE_FLOAT32, DENSE_ROW_SCALE = 0, 1, 1
MODEL_MIXES, MODEL_NORM_EPSILON = 24, 1e-20
SITE_FRONT_SCRATCH_BYTES, SITE_FRONT_MOST_WIDTH = 7184, 5120
SITE_FRONT_KIND_SITE, SITE_FRONT_KIND_FFN, SITE_FRONT_KIND_INPUT, SITE_FRONT_KIND_COEFFICIENTS = 0, 1, 2, 3


class SiteFront:
    """The step ahead of a layer's routed experts, as the launches the reference's fused site front stands for: the mix
    project (the dense product of the site's float32 mix weights [24][4 width] with the streams as its rows, scaled by
    the row's reciprocal root mean square), the mix finish (pre, post and comb by Sinkhorn, the collapse of the streams
    with the carried pre and its norm: the sublayer's input) and, behind the sublayer, the post. The router's scores in
    the dense product's order are scores_launch. Arrays live in the arena of `card`."""

    def __init__(self, card, rows, width, mix_weights, scale, base, norm_weight_bf16, hidden_range=None):
        self.card, self.rows, self.width = card, rows, width
        self.constants = {"mix_weights": np.ascontiguousarray(mix_weights, dtype=np.float32), "scale": np.ascontiguousarray(scale, dtype=np.float32),
                          "base": np.ascontiguousarray(base, dtype=np.float32), "norm_weight": np.ascontiguousarray(norm_weight_bf16, dtype=np.uint16)}
        assert self.constants["mix_weights"].shape == (MODEL_MIXES, MODEL_STREAMS * width)
        self.ranges = {name: Range(card.place(array, 256), array.nbytes) for name, array in self.constants.items()}
        sizes = {"streams": rows * MODEL_STREAMS * width * 2, "carried_pre": rows * MODEL_STREAMS * 4, "mixes": rows * MODEL_MIXES * 4,
                 "post": rows * MODEL_STREAMS * 4, "comb": rows * MODEL_STREAMS * MODEL_STREAMS * 4, "output": rows * width * 2,
                 "routed_sums": rows * width * 4}
        if hidden_range is None:
            sizes["hidden"] = rows * width * 2
        else:
            self.ranges["hidden"] = hidden_range
        self.ranges.update({name: Range(card.reserve(size), size) for name, size in sizes.items()})
        self.dense_kernels, self.hyper_kernels = DenseLinearKernels(), HyperKernelsRecord()
        check(card.lib.dense_linear_kernels_prepare(backend_table(), card.handle, C.byref(self.dense_kernels)), "dense_linear_kernels_prepare")
        check(card.lib.hyper_kernels_prepare(backend_table(), card.handle, C.byref(self.hyper_kernels)), "hyper_kernels_prepare")

    def set_streams(self, streams_bf16, carried_pre):
        self.card.upload(self.ranges["streams"].byte_offset, np.ascontiguousarray(streams_bf16, dtype=np.uint16))
        self.card.upload(self.ranges["carried_pre"].byte_offset, np.ascontiguousarray(carried_pre, dtype=np.float32))

    def dense_launch(self, weights, rows_range, output, output_size, input_size, weight_type, output_type=DENSE_FLOAT32, flags=0, scale=1.0,
                     epsilon=0.0, rows=None):
        d = DenseLinearDescription()
        d.weights, d.rows, d.output, d.step = weights, rows_range, output, Range(0, 0)
        d.output_size, d.input_size, d.row_count = output_size, input_size, self.rows if rows is None else rows
        d.weight_type, d.output_type, d.flags, d.output_scale, d.epsilon = weight_type, output_type, flags, scale, epsilon
        launch = launches_of(1)
        check(self.card.lib.dense_linear_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.dense_kernels), launch), "dense_linear_prepare")
        return launch

    def mix_project_launch(self, rows=None):
        return self.dense_launch(self.ranges["mix_weights"], self.ranges["streams"], self.ranges["mixes"], MODEL_MIXES, MODEL_STREAMS * self.width,
                                 DENSE_FLOAT32, DENSE_FLOAT32, DENSE_ROW_SCALE, 1.0, MODEL_NORM_EPSILON, rows)

    def site_launches(self, rows=None, combined=False):
        """[the mix finish, the post] (hyper_site_prepare)."""
        d = HyperSiteDescription()
        for name in ("streams", "carried_pre", "mixes", "scale", "base", "norm_weight", "post", "comb", "hidden", "output"):
            setattr(d, name, self.ranges[name])
        d.routed_sums = self.ranges["routed_sums"] if combined else Range(0, 0)
        d.row_count, d.reserved_zero = self.rows if rows is None else rows, self.width
        launches = launches_of(2)
        check(self.card.lib.hyper_site_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.hyper_kernels), launches), "hyper_site_prepare")
        return launches

    def front_description(self, rows=None, layer=None, order=0, kind=None):
        """The description of the fused front of `rows` rows (site_front_prepare); with `layer` (an Exl3Layer or Fp4Layer
        whose rows are this front's hidden range) the FFN front, whose select is the layer's. Keeps what it points at."""
        if "scratch" not in self.ranges:
            sizes = {"codes": self.rows * self.width, "exponents": self.rows * self.width // 32, "operands": self.rows * self.width * 2,
                     "scratch": SITE_FRONT_SCRATCH_BYTES}
            self.ranges.update({name: Range(self.card.reserve(size), size) for name, size in sizes.items()})
            self.card.upload(self.ranges["scratch"].byte_offset, np.zeros(SITE_FRONT_SCRATCH_BYTES, np.uint8))
            self.front_kernels = SiteFrontKernels()
            check(self.card.lib.site_front_kernels_prepare(backend_table(), self.card.handle, C.byref(self.front_kernels)), "site_front_kernels_prepare")
        d = SiteFrontDescription()
        for name in ("streams", "carried_pre", "mix_weights", "scale", "base", "norm_weight", "post", "comb", "hidden", "codes", "exponents",
                     "operands", "scratch"):
            setattr(d, name, self.ranges[name])
        d.kind = (SITE_FRONT_KIND_SITE if layer is None else SITE_FRONT_KIND_FFN) if kind is None else kind
        d.row_count, d.reserved_zero = self.rows if rows is None else rows, self.width
        keep = [d]
        if layer is not None:
            experts = layer.experts_description()
            r = RouterDescription()
            r.experts = C.pointer(experts)
            r.expert_offsets = layer.expert_offsets.ctypes.data_as(C.POINTER(u64))
            packed = getattr(layer, "packed_widths", None)
            r.expert_widths = packed.ctypes.data_as(C.POINTER(u32)) if packed is not None and getattr(layer, "uniform_width", 1) == 0 else None
            r.step, r.scores = Range(layer.step_offset, 16), Range(layer.scores_offset, layer.rows * layer.E * 4)
            r.bias, r.offsets = Range(layer.bias_offset, layer.E * 4), Range(layer.offsets_offset, layer.E * 24)
            r.affinities = Range(layer.affinities_offset, layer.rows * layer.E * 4)
            r.order, r.expert_count, r.pick_count = order, layer.E, layer.P
            r.affinity_kind, r.route_scale = layer.affinity_kind, layer.route_scale
            d.router = C.pointer(r)
            d.router_weights = Range(layer.router_offset, layer.E * layer.H * 2)
            keep += [experts, r]
        self.kept = keep
        return d

    def front_launch(self, rows=None, layer=None, order=0, kind=None):
        """ONE launch for the mix project, the mix finish, (with `layer`: the router's scores and its select) and the
        quantization of the sublayer's input; with kind SITE_FRONT_KIND_INPUT or _COEFFICIENTS one of the two launches
        the site front may be cut in (the input front first)."""
        d = self.front_description(rows, layer, order, kind)
        router_kernels = None if layer is None else C.byref(layer.router_kernels)
        launch = launches_of(1)
        check(self.card.lib.site_front_prepare(C.byref(d), self.card.arena_bytes, router_kernels, C.byref(self.front_kernels), launch),
              "site_front_prepare")
        return launch

    def read(self, name, dtype=np.uint8):
        return self.card.download(self.ranges[name].byte_offset, self.ranges[name].byte_count, dtype)


class SharedExpert:
    """The step behind a layer's routed experts: the shared expert (three WEIGHT_FORMAT_E4M3_SCALED matrices applied to
    every row: gate with up, the hidden step, the quantizer, down) and the FFN site's join (a row's routed sum, the
    shared expert's output added to it, the post of the four residual streams). Reads the rows' codes and the pair
    outputs of `layer` (an Fp4Layer); holds its own scratch, the streams, post and comb in the layer's arena."""

    def __init__(self, layer, matrices, gate_up_slices=1, down_slices=1, wide_form=LINEAR_INTERLEAVED_CHUNK_BLOCKS, inner=None):
        self.layer, self.card = layer, layer.card
        card, rows, hidden = layer.card, layer.rows, layer.H
        self.inner = inner = layer.I if inner is None else inner
        self.gate_up_slices, self.down_slices, self.wide_form = gate_up_slices, down_slices, wide_form
        self.matrix_ranges = [Range(card.place(matrix, 256), matrix.nbytes) for matrix in matrices]
        names = {"gate_output": rows * inner * 2, "up_output": rows * inner * 2, "hidden": rows * inner * 2,
                 "hidden_codes": rows * inner, "hidden_exponents": rows * inner // 32, "hidden_operands": rows * inner * 2,
                 "output": rows * hidden * 2, "streams": rows * MODEL_STREAMS * hidden * 2, "post": rows * MODEL_STREAMS * 4,
                 "comb": rows * MODEL_STREAMS * MODEL_STREAMS * 4, "row_sums": rows * hidden * 4}
        self.ranges = {name: Range(card.reserve(size), size) for name, size in names.items()}
        self.fused_kernels = ExpertFusedKernels()
        check(card.lib.expert_fused_kernels_prepare(backend_table(), card.handle, ARITHMETIC_CLASS_GFX950, C.byref(self.fused_kernels)),
              "expert_fused_kernels_prepare")

    def matrix(self, index, slices):
        outputs, inputs = (self.layer.H, self.inner) if index == 2 else (self.inner, self.layer.H)
        return LinearMatrix(self.matrix_ranges[index], Shape(outputs, inputs, 8, 0), WEIGHT_FORMAT_E4M3_SCALED, slices, self.wide_form, 0)

    def set_site(self, streams_bf16, post, comb):
        self.card.upload(self.ranges["streams"].byte_offset, streams_bf16)
        self.card.upload(self.ranges["post"].byte_offset, np.ascontiguousarray(post, dtype=np.float32))
        self.card.upload(self.ranges["comb"].byte_offset, np.ascontiguousarray(comb, dtype=np.float32))

    def description(self, rows=None):
        d = SharedExpertDescription()
        d.gate, d.up, d.down = self.matrix(0, self.gate_up_slices), self.matrix(1, self.gate_up_slices), self.matrix(2, self.down_slices)
        d.codes, d.exponents, d.operands = (self.layer.ranges[name] for name in ("codes", "exponents", "operands"))
        for name in ("gate_output", "up_output", "hidden", "hidden_codes", "hidden_exponents", "hidden_operands", "output"):
            setattr(d, name, self.ranges[name])
        d.row_count, d.activation_limit = self.layer.rows if rows is None else rows, self.layer.limit
        return d

    def launches(self, rows=None):
        """The shared expert's four launches: gate with up, the hidden step, the quantizer, down."""
        d = self.description(rows)
        launches = launches_of(4)
        check(self.card.lib.linear_shared_expert_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.layer.kernels), launches),
              "linear_shared_expert_prepare")
        return launches

    def join_description(self, rows=None, row_sums=True):
        d = ExpertJoinDescription()
        d.pair_output, d.shared_output = self.layer.ranges["pair_output"], self.ranges["output"]
        d.streams, d.post, d.comb = self.ranges["streams"], self.ranges["post"], self.ranges["comb"]
        d.row_sums = self.ranges["row_sums"] if row_sums else Range(0, 0)
        d.pairs_per_row, d.row_count, d.width = self.layer.P, self.layer.rows if rows is None else rows, self.layer.H
        return d

    def join_launch(self, rows=None, row_sums=True):
        d = self.join_description(rows, row_sums)
        launch = launches_of(1)
        check(self.card.lib.expert_join_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.fused_kernels), launch), "expert_join_prepare")
        return launch

    def post_launch(self, rows=None):
        """hyper_post_entry with the combine, reading the layer's row outputs (what expert_row_sum_entry, the last of the
        routed experts' launches, wrote): the second of the two launches a join stands for."""
        d = self.join_description(rows, True)
        d.row_sums = self.layer.ranges["row_output"]
        launch = launches_of(1)
        check(self.card.lib.expert_post_prepare(C.byref(d), self.card.arena_bytes, self.fused_kernels.post, launch), "expert_post_prepare")
        return launch

    def shared_join_launch(self, rows=None, row_sums=True):
        """The shared expert's down and the join in one launch (at most LINEAR_MAXIMUM_ROWS rows)."""
        d = ExpertSharedJoinDescription()
        d.down = self.matrix(2, self.down_slices)
        d.codes, d.exponents, d.operands = self.ranges["hidden_codes"], self.ranges["hidden_exponents"], self.ranges["hidden_operands"]
        d.join = self.join_description(rows, row_sums)
        launch = launches_of(1)
        check(self.card.lib.expert_shared_join_prepare(C.byref(d), self.card.arena_bytes, C.byref(self.layer.kernels),
                                                       C.byref(self.fused_kernels), launch), "expert_shared_join_prepare")
        return launch

    def read(self, name, dtype=np.uint8):
        r = self.ranges[name]
        return self.card.download(r.byte_offset, r.byte_count, dtype)
